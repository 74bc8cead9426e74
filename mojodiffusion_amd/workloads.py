"""Synthetic attention workloads of the DiT shapes this library is measured on.

Each workload fixes the tensor shape, the quantization recipe and the input
statistics (K carries a per-channel offset or a few outlier channels, which is
what K-mean smoothing exists for).  Inputs are generated on the host with
numpy's PCG64 so that every consumer (tests, bench, CPU checker) sees the same
bits for a given seed:

    seed = 1000 * workload_id + {0: q, 1: k, 2: v, 3: offset / outlier choice}

Values are drawn in logical [B, H, S, D] order, rounded to bf16 with
round-to-nearest-even and returned in the caller layout [B, S, H, D] as uint16
bit patterns.  "N(0, 2)" / "N(0, 4)" offsets are read as standard deviation 2 / 4.
"""
from dataclasses import dataclass, replace

import numpy as np


@dataclass(frozen=True)
class Workload:
    wid: int
    name: str
    B: int
    H: int
    S: int
    D: int
    variant: int            # 0: INT8 QK / FP16 PV, 1: INT8 QK / FP8-e4m3 PV
    blkq: int               # tokens per Q scale block
    blkk: int               # tokens per K scale block
    k_offset_std: float     # per-(b,h,d) additive K offset, 0 = none
    k_outlier_frac: float   # fraction of K channels multiplied by k_outlier_gain
    k_outlier_gain: float = 8.0

    @property
    def scale(self):
        return float(1.0 / np.sqrt(self.D))

    @property
    def ops(self):
        """Effective attention operations: QK^T and PV, 2*S*S*D each per head."""
        return 4 * self.B * self.H * self.S * self.S * self.D

    def scaled(self, **kw):
        """Same statistics and recipe at another size (for quick parity cases)."""
        return replace(self, **kw)


WORKLOADS = {
    1: Workload(1, "c1_small_B1_H8_S1024_D64", 1, 8, 1024, 64, 0, 64, 64, 2.0, 0.0),
    2: Workload(2, "c2_flux_klein_joint_B1_H24_S4608_D128", 1, 24, 4608, 128, 0, 128, 64, 4.0, 0.0),
    3: Workload(3, "c3_zimage_B2_H30_S4352_D128", 2, 30, 4352, 128, 0, 128, 64, 0.0, 0.01),
    4: Workload(4, "c4_sage2_2048px_B1_H24_S16896_D128", 1, 24, 16896, 128, 1, 32, 64, 4.0, 0.0),
    5: Workload(5, "c5_video_B1_H40_S32760_D128", 1, 40, 32760, 128, 1, 128, 64, 4.0, 0.0),
}


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def _normal_bhsd(seed, w):
    return np.random.default_rng(seed).standard_normal((w.B, w.H, w.S, w.D), dtype=np.float32)


def make_inputs(w):
    """Returns (q, k, v) as uint16 bf16 bit patterns, each [B, S, H, D]."""
    base = 1000 * w.wid
    out = []
    for t in range(3):
        x = _normal_bhsd(base + t, w)
        if t == 1:
            rng = np.random.default_rng(base + 3)
            if w.k_offset_std > 0:
                off = rng.standard_normal((w.B, w.H, 1, w.D), dtype=np.float32) * np.float32(w.k_offset_std)
                x = x + off                      # fp32 add before the bf16 rounding
            if w.k_outlier_frac > 0:
                n_out = int(np.ceil(w.k_outlier_frac * w.D))
                for b in range(w.B):
                    for h in range(w.H):
                        ch = rng.choice(w.D, size=n_out, replace=False)
                        x[b, h, :, ch] *= np.float32(w.k_outlier_gain)
        out.append(np.ascontiguousarray(f32_to_bf16_bits(x).transpose(0, 2, 1, 3)))
        del x
    return tuple(out)


def device_inputs(w, seed):
    """(q, k, v) bf16 torch tensors [B, S, H, D] on the GPU with the workload's statistics, drawn by
    torch's device generator: for full-size runs that need no bit-reproducible host copy (the
    largest workload takes minutes to draw on the host)."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    shape = (w.B, w.S, w.H, w.D)
    q = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    k = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if w.k_offset_std > 0:
        k += w.k_offset_std * torch.randn((w.B, 1, w.H, w.D), generator=g, device="cuda", dtype=torch.float32)
    if w.k_outlier_frac > 0:
        n = int(np.ceil(w.k_outlier_frac * w.D))
        gain = torch.ones((w.B, 1, w.H, w.D), device="cuda")
        for b in range(w.B):
            for h in range(w.H):
                idx = torch.randperm(w.D, generator=g, device="cuda")[:n]
                gain[b, 0, h, idx] = w.k_outlier_gain
        k *= gain
    k = k.to(torch.bfloat16)
    v = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    return q, k, v
