#!/usr/bin/env python3
"""Extract the golden vectors the reference's own tests hold for the attention
path into small fixtures next to this script.  Only DATA is read (a text file
of expected outputs and the literal arrays of an inline known-answer test);
no reference code is imported or executed.

Sources (relative to the reference checkout):
  serenitymojo/ops/parity/sdpa_math_ref.txt        tags dh128 [1,8,32,128], dh512 [1,64,1,512]
      inputs are the closed forms of ops/parity/sdpa_math_parity.mojo:32-50
  serenitymojo/ops/parity/sdpa_bwd_ref.txt         gradients dq/dk/dv for tags dh128 [1,8,32,128], dh64 [1,8,8,64]
      inputs are the closed forms of ops/parity/sdpa_bwd_parity.mojo:44-65
  serenitymojo/ops_smoke2.mojo:239-278              q/k/v/out literals, [1,4,2,8], scale 0.35355339
  serenitymojo/ops_smoke.mojo:78-96                 rms_norm x[3,6], g[6], eps 1e-6 -> y[3,6]
  serenitymojo/ops_smoke2.mojo:92-120               rope x[3,8], cos/sin[3,4] -> interleaved y[3,8], half-split y[3,8]

Run once where the reference is mounted:  python tests/golden/make_fixtures.py [/root/reference]
"""
import json
import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    with open(os.path.join(ref, "serenitymojo/ops/parity/sdpa_math_ref.txt")) as f:
        for line in f:
            parts = line.split()
            if parts:
                out[parts[0]] = np.array([float(x) for x in parts[1:]], dtype=np.float64)
    assert out["dh128"].size == 1 * 8 * 32 * 128 and out["dh512"].size == 1 * 64 * 1 * 512
    np.savez_compressed(os.path.join(HERE, "sdpa_math_ref.npz"), dh128=out["dh128"], dh512=out["dh512"])

    bwd = {}
    with open(os.path.join(ref, "serenitymojo/ops/parity/sdpa_bwd_ref.txt")) as f:
        for line in f:
            parts = line.split()
            if parts:
                bwd[parts[0]] = np.array([float(x) for x in parts[1:]], dtype=np.float64)
    for tag, n in (("dh128", 1 * 8 * 32 * 128), ("dh64", 1 * 8 * 8 * 64)):
        for g in ("dq", "dk", "dv"):
            assert bwd[tag + "_" + g].size == n, (tag, g)
    np.savez_compressed(os.path.join(HERE, "sdpa_bwd_ref.npz"), **bwd)

    with open(os.path.join(ref, "serenitymojo/ops_smoke2.mojo")) as f:
        lines = f.read().split("\n")
    text = "\n".join(lines[238:278])           # lines 239..278, 1-based
    kat = {}
    for name in ("q_sdpa", "k_sdpa", "v_sdpa", "out_sdpa_ref"):
        m = re.search(r"var %s = _lf\((.*?)\n\s*\)" % name, text, re.S)
        vals = [float(x) for x in re.findall(r"-?\d+\.\d+", m.group(1))]
        assert len(vals) == 64, (name, len(vals))
        kat[name] = vals
    kat["shape_bshd"] = [1, 4, 2, 8]
    kat["scale"] = 0.35355339
    with open(os.path.join(HERE, "ops_smoke2_sdpa_kat.json"), "w") as f:
        json.dump(kat, f, indent=0)

    def literals(text, name, count):
        m = re.search(r"var %s = _lf\((.*?)\n\s*\)" % name, text, re.S)
        vals = [float(x) for x in re.findall(r"-?\d+\.\d+", m.group(1))]
        assert len(vals) == count, (name, len(vals))
        return vals

    pre = {}
    with open(os.path.join(ref, "serenitymojo/ops_smoke.mojo")) as f:
        text = "\n".join(f.read().split("\n")[77:96])
    pre["rms_x"] = literals(text, "x_rms", 18)
    pre["rms_g"] = literals(text, "g_rms", 6)
    pre["rms_y"] = literals(text, "y_rms_ref", 18)
    pre["rms_eps"] = 1e-6
    text = "\n".join(lines[91:120])
    pre["rope_x"] = literals(text, "x_rope", 24)
    pre["rope_cos"] = literals(text, "cos_rope", 12)
    pre["rope_sin"] = literals(text, "sin_rope", 12)
    pre["rope_y_interleaved"] = literals(text, "y_int_ref", 24)
    pre["rope_y_halfsplit"] = literals(text, "y_half_ref", 24)
    with open(os.path.join(HERE, "ops_smoke_rmsnorm_rope_kat.json"), "w") as f:
        json.dump(pre, f, indent=0)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
