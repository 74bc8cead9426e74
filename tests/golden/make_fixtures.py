#!/usr/bin/env python3
"""Extract the golden vectors the reference's own tests hold for the attention
path into small fixtures next to this script.  Only DATA is read (a text file
of expected outputs and the literal arrays of an inline known-answer test);
no reference code is imported or executed.

Sources (relative to the reference checkout):
  serenitymojo/ops/parity/sdpa_math_ref.txt        tags dh128 [1,8,32,128], dh512 [1,64,1,512]
      inputs are the closed forms of ops/parity/sdpa_math_parity.mojo:32-50
  serenitymojo/ops_smoke2.mojo:239-278              q/k/v/out literals, [1,4,2,8], scale 0.35355339

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
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
