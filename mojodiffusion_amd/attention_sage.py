"""Host side of the quantized-SDPA path: the serenitymojo attention call surface
bound to libmi355_sage.so.

Function names, argument meaning and error behaviour follow
serenitymojo/ops/attention_flash.mojo (sdpa_flash_train_fwd :149-202, _rect
:205-264, sdpa_flash_fwd_padmask :267-342, sdpa_flash_train_fwd_f32 :457-475) and
serenitymojo/ops/attention.mojo (sdpa :1596-1647, sdpa_chunked :1650-1687,
sdpa_nomask :1690-1718, sdpa_nomask_tiled :1762-1787, sdpa_qwen_keymask :1790-1857,
sdpa_cross_nomask :1860-1894, sdpa_cross_masked :1897-1936, sdpa_nomask_slab
:2144-2169), and the math-mode backward surface of serenitymojo/ops/attention_backward.mojo
(sdpa_backward :435, _masked :566, _rect :928, _scratch :1099, _rect_slab :1477, _slab :1641) with
its shape dispatchers (autograd_v2/ops_record.mojo:165, :463; attention_flash.mojo:610) and the
recorded attention node (autograd_v2/ops_record.mojo:329-352).  Tensors are [B, S, H, Dh]; torch is
used only to own device memory and the stream.  What differs from the cuDNN path:
no 128-padding copies are needed (ragged S is handled in the kernels), so the
`*_pad` members of the result alias the caller's tensors.
"""
from dataclasses import dataclass

import torch

from . import _lib

PV_FP16 = 0
PV_FP8 = 1


class Error(RuntimeError):
    """Counterpart of Mojo's `raise Error(...)`."""


@dataclass
class SdpaFlashFwd:
    """serenitymojo/ops/attention_flash.mojo:108-135."""
    o: torch.Tensor
    o_pad: torch.Tensor
    q_pad: torch.Tensor
    k_pad: torch.Tensor
    v_pad: torch.Tensor
    stats: torch.Tensor


_workspaces = {}


def _workspace(nbytes, device):
    """Caller-side workspace reuse: one growing buffer per (device, stream), so steady-state
    calls allocate nothing and calls on different streams never share scratch memory.  A
    buffer that is replaced stays alive for the work already queued on its stream: torch's
    allocator hands its memory out again only to that same stream."""
    stream = torch.cuda.current_stream(device)
    key = (device.type, device.index, stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _require_bf16(name, *ts):
    for t in ts:
        if t.dtype != torch.bfloat16:
            raise Error("%s: q/k/v must be BF16" % name)


def _require_cuda(name, *ts):
    for t in ts:
        if not t.is_cuda:
            raise Error("%s: tensors must live on the GPU (no CPU fallback exists)" % name)
        if not t.is_contiguous():
            raise Error("%s: tensors must be contiguous [B,S,H,Dh]" % name)


def _call_train_fwd(name, q, k, v, scale, real_q, real_kv, variant, want_stats, mask=None):
    B, Sq, H, Dh = q.shape
    Skv = k.shape[1]
    L = _lib.lib()
    o = torch.empty_like(q)
    stats = torch.empty((B, H, Sq, 1), dtype=torch.float32, device=q.device) if want_stats else None
    nbytes = L.mi355_sage_workspace_bytes(B, H, Sq, Skv, Dh, variant)
    ws = _workspace(max(nbytes, 256), q.device)
    qs = _lib.strides_bhnd(Sq, H, Dh)
    ks = _lib.strides_bhnd(Skv, H, Dh)
    stream = torch.cuda.current_stream(q.device).cuda_stream
    if mask is not None:
        rc = L.mi355_sage_sdpa_bf16_keymask(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), stats.data_ptr() if want_stats else None,
            B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, 0, 0, 0, 0, 0,
            mask[0], mask[1], stream, variant, ws.data_ptr(), ws.numel())
    elif want_stats:
        rc = L.mi355_sage_sdpa_bf16_train_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), stats.data_ptr(),
            B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, 0, 0, 0, 0, 0,
            0, real_q, real_kv, stream, variant, ws.data_ptr(), ws.numel())
    else:
        rc = L.mi355_sage_sdpa_bf16(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
            B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, 0, 0, 0, 0,
            0, stream, variant, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: shim rc=%d (B=%d Sq=%d Skv=%d H=%d Dh=%d)" % (name, rc, B, Sq, Skv, H, Dh))
    return o, stats


def _check_shapes(name, q, k, v, square):
    if q.dim() != 4:
        raise Error("%s: q must be rank-4 [B,S,H,Dh]" % name)
    if k.shape != v.shape or k.dim() != 4:
        raise Error("%s: k/v shape mismatch" % name)
    if q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2] or q.shape[3] != k.shape[3]:
        raise Error("%s: q and k/v disagree on B/H/Dh" % name)
    if square and q.shape[1] != k.shape[1]:
        raise Error("%s: k/v shape does not match q [B,S,H,Dh]" % name)


def sdpa_flash_train_fwd(q, k, v, scale, variant=PV_FP16):
    """Forward on [B,S,H,Dh] BF16 (no mask, non-causal); returns O and the
    log-sum-exp Stats [B,H,S,1].  Fails loudly on any non-zero return code."""
    _require_bf16("sdpa_flash_train_fwd", q, k, v)
    _check_shapes("sdpa_flash_train_fwd", q, k, v, True)
    _require_cuda("sdpa_flash_train_fwd", q, k, v)
    o, stats = _call_train_fwd("sdpa_flash_train_fwd", q, k, v, scale, q.shape[1], k.shape[1], variant, True)
    return SdpaFlashFwd(o, o, q, k, v, stats)


def sdpa_flash_train_fwd_rect(q, k, v, scale, variant=PV_FP16):
    """Rectangular no-mask attention: q [B,Sq,H,Dh], k/v [B,Skv,H,Dh]."""
    _require_bf16("sdpa_flash_train_fwd_rect", q, k, v)
    _check_shapes("sdpa_flash_train_fwd_rect", q, k, v, False)
    _require_cuda("sdpa_flash_train_fwd_rect", q, k, v)
    o, stats = _call_train_fwd("sdpa_flash_train_fwd_rect", q, k, v, scale, q.shape[1], k.shape[1], variant, True)
    return SdpaFlashFwd(o, o, q, k, v, stats)


def sdpa_flash_fwd_padmask(q, k, v, real_len, scale, variant=PV_FP16):
    """Pre-padded [B,S_BUF,H,Dh] buffers whose first real_len positions are real:
    keys at and beyond real_len are excluded from every query; query rows there
    are garbage the caller discards."""
    _require_bf16("sdpa_flash_fwd_padmask", q, k, v)
    _check_shapes("sdpa_flash_fwd_padmask", q, k, v, True)
    s_buf = q.shape[1]
    if s_buf % 128 != 0:
        raise Error("sdpa_flash_fwd_padmask: S_BUF must be 128-aligned")
    if real_len < 1 or real_len > s_buf:
        raise Error("sdpa_flash_fwd_padmask: real_len out of [1, S_BUF]")
    _require_cuda("sdpa_flash_fwd_padmask", q, k, v)
    o, stats = _call_train_fwd("sdpa_flash_fwd_padmask", q, k, v, scale, real_len, real_len, variant, True)
    return SdpaFlashFwd(o, o, q, k, v, stats)


def sdpa_flash_train_fwd_f32(q, k, v, scale, variant=PV_FP16):
    """F32 activations: cast to BF16 at the boundary, attend, cast back
    (attention_flash.mojo:457-475).  Returns (att_f32, SdpaFlashFwd of the bf16 run)."""
    fwd = sdpa_flash_train_fwd(q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16), scale, variant)
    return fwd.o.to(torch.float32), fwd


@dataclass
class SdpaFlashGrads:
    """serenitymojo/ops/attention_flash.mojo:138-146."""
    d_q: torch.Tensor
    d_k: torch.Tensor
    d_v: torch.Tensor


def _call_bwd(name, q, k, v, o, d_out, stats, scale, real_q, real_kv):
    B, Sq, H, Dh = q.shape
    Skv = k.shape[1]
    L = _lib.lib()
    d_q, d_k, d_v = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws = _workspace(max(L.mi355_sage_bwd_workspace_bytes(B, H, Sq, Skv, Dh), 256), q.device)
    qs = _lib.strides_bhnd(Sq, H, Dh)
    ks = _lib.strides_bhnd(Skv, H, Dh)
    stream = torch.cuda.current_stream(q.device).cuda_stream
    rc = L.mi355_sage_sdpa_bwd_bf16(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_out.data_ptr(), stats.data_ptr(),
        d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(),
        B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, qs, qs, ks, ks,
        0, 0, 0, 0, 0, 0, 0, 0, 0,
        0, real_q, real_kv, stream, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: shim rc=%d (B=%d Sq=%d Skv=%d H=%d Dh=%d)" % (name, rc, B, Sq, Skv, H, Dh))
    return SdpaFlashGrads(d_q, d_k, d_v)


def sdpa_flash_backward(fwd, d_out, scale, real_len=None):
    """dQ/dK/dV [B,S,H,Dh] BF16 from the saved train-forward set and the upstream d_out
    (attention_flash.mojo:345-433).  The reference pads the sequence to 128 around its call; the
    kernels here take any length, so the saved tensors are used as they are.  real_len: the valid
    length of a sdpa_flash_fwd_padmask forward (rows and keys at and beyond it get zero gradients)."""
    name = "sdpa_flash_backward"
    _require_bf16(name, fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad)
    if d_out.dtype != torch.bfloat16:
        raise Error("%s: d_out must be BF16" % name)
    if d_out.shape != fwd.o_pad.shape:
        raise Error("%s: d_out shape does not match the forward output" % name)
    _require_cuda(name, fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, d_out, fwd.stats)
    rq = fwd.q_pad.shape[1] if real_len is None else real_len
    rk = fwd.k_pad.shape[1] if real_len is None else real_len
    return _call_bwd(name, fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, d_out, fwd.stats, scale, rq, rk)


def sdpa_flash_backward_f32(q_bf, k_bf, v_bf, o_bf, stats, d_att, scale):
    """F32 gradient in and out around the bf16 backward (attention_flash.mojo:478-535): d_att F32
    -> bf16, dQ/dK/dV bf16 -> F32.  The reference accepts 128-aligned S only on this path."""
    name = "sdpa_flash_backward_f32"
    if q_bf.shape[1] % 128 != 0:
        raise Error("%s: S must be 128-aligned" % name)
    _require_bf16(name, q_bf, k_bf, v_bf, o_bf)
    do_bf = d_att.to(torch.bfloat16)
    _require_cuda(name, q_bf, k_bf, v_bf, o_bf, do_bf, stats)
    g = _call_bwd(name, q_bf, k_bf, v_bf, o_bf, do_bf, stats, scale, q_bf.shape[1], k_bf.shape[1])
    return SdpaFlashGrads(g.d_q.to(torch.float32), g.d_k.to(torch.float32), g.d_v.to(torch.float32))


def sdpa_flash_backward_raw(q_pad, k_pad, v_pad, o_pad, stats, d_out, scale):
    """bf16 in and out on the saved set of the graph path (attention_flash.mojo:538-607)."""
    name = "sdpa_flash_backward_raw"
    _require_bf16(name, q_pad, k_pad, v_pad, o_pad)
    if d_out.dtype != torch.bfloat16:
        raise Error("%s: d_out must be BF16" % name)
    _require_cuda(name, q_pad, k_pad, v_pad, o_pad, d_out, stats)
    return _call_bwd(name, q_pad, k_pad, v_pad, o_pad, d_out, stats, scale, q_pad.shape[1], k_pad.shape[1])


def sdpa_flash_backward_dispatch(q_pad, k_pad, v_pad, o_pad, stats, d_out, scale, B, S, H, Dh):
    """attention_flash.mojo:610-633: the autograd engine's entry, runtime dims in.  The reference
    looks the dims up in a table of compiled instantiations and raises for the others; the kernels
    here take their dims at run time, so every shape the saved tensors really have is served."""
    name = "sdpa_flash_backward_dispatch"
    if tuple(q_pad.shape) != (B, S, H, Dh):
        raise Error("%s: no bucket (B,S,H,Dh)=(%d,%d,%d,%d)" % (name, B, S, H, Dh))
    return sdpa_flash_backward_raw(q_pad, k_pad, v_pad, o_pad, stats, d_out, scale)


@dataclass
class SdpaGrads:
    """serenitymojo/ops/attention_backward.mojo:56-66."""
    d_q: torch.Tensor
    d_k: torch.Tensor
    d_v: torch.Tensor


class ScratchRingMark:
    """serenitymojo/scratch_ring.mojo:20-25 (front positions only: nothing here allocates from the back)."""

    def __init__(self, slab_index, offset):
        self.slab_index = slab_index
        self.offset = offset


class ScratchRingAllocator:
    """Counterpart of serenitymojo/scratch_ring.mojo:27-215: frame-scoped scratch in slabs the
    caller owns.  alloc() bumps through the slabs (a new slab when the current one is full),
    mark() / rewind() give the memory back in stack order; the caller rewinds only when nothing
    queued later on another stream still reads what was allocated since the mark."""

    def __init__(self, slab_bytes, device="cuda", alignment=256):
        self.slab_bytes = int(slab_bytes)
        self.device = device
        self.alignment = alignment
        self.slabs = []
        self.slab_index = 0
        self.offset = 0

    def capacity_bytes(self):
        return self.slab_bytes * len(self.slabs)

    def used_bytes(self):
        return self.slab_index * self.slab_bytes + self.offset

    def mark(self):
        return ScratchRingMark(self.slab_index, self.offset)

    def reset(self):
        self.slab_index = 0
        self.offset = 0

    def rewind(self, mark):
        if (mark.slab_index, mark.offset) > (self.slab_index, self.offset):
            raise Error("ScratchRingAllocator: rewind mark is ahead of the allocator")
        self.slab_index = mark.slab_index
        self.offset = mark.offset

    def alloc(self, nbytes):
        nbytes = int(nbytes)
        if nbytes > self.slab_bytes:
            raise Error("ScratchRingAllocator: request %d exceeds the slab size %d" % (nbytes, self.slab_bytes))
        while True:
            if self.slab_index == len(self.slabs):
                self.slabs.append(torch.empty(self.slab_bytes, dtype=torch.uint8, device=self.device))
            slab = self.slabs[self.slab_index]
            base = slab.data_ptr()
            start = (base + self.offset + self.alignment - 1) // self.alignment * self.alignment - base
            if start + nbytes <= self.slab_bytes:
                self.offset = start + nbytes
                return slab[start:start + nbytes]
            self.slab_index += 1
            self.offset = 0


def _math_bwd(name, q, k, v, d_out, scale, variant, alloc, out_alloc=None):
    """The decomposed backward's contract on the flash kernels: the forward is recomputed by the
    quantized kernel (its O and log-sum-exp), the gradients by the bf16 backward.  `alloc(nbytes)`
    provides every intermediate (workspaces, O, Stats, bf16 staging); the three results, in q's
    dtype, are fresh tensors, or come from `out_alloc(nbytes)` when that is given."""
    if q.dtype != k.dtype or q.dtype != v.dtype or q.dtype != d_out.dtype:
        raise Error("%s: q/k/v/d_out dtype mismatch" % name)
    _require_cuda(name, q, k, v, d_out)
    B, Sq, H, Dh = q.shape
    Skv = k.shape[1]
    if Dh not in (64, 128):
        raise Error("%s: Dh=%d is not supported by the backward kernels (64 or 128)" % (name, Dh))
    L = _lib.lib()
    dev = q.device
    stream = torch.cuda.current_stream(dev).cuda_stream

    def staged(t):
        if t.dtype == torch.bfloat16:
            return t
        out = alloc(t.numel() * 2).view(torch.bfloat16).view(t.shape)
        out.copy_(t)
        return out

    qb, kb, vb, gb = staged(q), staged(k), staged(v), staged(d_out)
    o = alloc(q.numel() * 2).view(torch.bfloat16).view(q.shape)
    stats = alloc(B * H * Sq * 4).view(torch.float32).view(B, H, Sq, 1)
    nfw = max(L.mi355_sage_workspace_bytes(B, H, Sq, Skv, Dh, variant), 256)
    nbw = max(L.mi355_sage_bwd_workspace_bytes(B, H, Sq, Skv, Dh), 256)
    ws = alloc(max(nfw, nbw))            # the forward is finished with it before the backward starts (one stream)
    qs = _lib.strides_bhnd(Sq, H, Dh)
    ks = _lib.strides_bhnd(Skv, H, Dh)
    rc = L.mi355_sage_sdpa_bf16_train_fwd(
        qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), o.data_ptr(), stats.data_ptr(),
        B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, 0, 0, 0, 0, 0,
        0, Sq, Skv, stream, variant, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: forward shim rc=%d (B=%d Sq=%d Skv=%d H=%d Dh=%d)" % (name, rc, B, Sq, Skv, H, Dh))
    same = q.dtype == torch.bfloat16

    def result_like(t):
        if out_alloc is None:
            return torch.empty_like(t)
        return out_alloc(t.numel() * t.element_size()).view(t.dtype).view(t.shape)

    dq = result_like(q) if same else alloc(q.numel() * 2).view(torch.bfloat16).view(q.shape)
    dk = result_like(k) if same else alloc(k.numel() * 2).view(torch.bfloat16).view(k.shape)
    dv = result_like(v) if same else alloc(v.numel() * 2).view(torch.bfloat16).view(v.shape)
    rc = L.mi355_sage_sdpa_bwd_bf16(
        qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), o.data_ptr(), gb.data_ptr(), stats.data_ptr(),
        dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
        B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, qs, qs, qs, ks, ks,
        0, 0, 0, 0, 0, 0, 0, 0, 0,
        0, Sq, Skv, stream, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: backward shim rc=%d (B=%d Sq=%d Skv=%d H=%d Dh=%d)" % (name, rc, B, Sq, Skv, H, Dh))
    if same:
        return SdpaGrads(dq, dk, dv)
    outs = []
    for g, like in ((dq, q), (dk, k), (dv, v)):
        r = result_like(like)
        r.copy_(g)
        outs.append(r)
    return SdpaGrads(*outs)


def _torch_alloc(device):
    return lambda nbytes: torch.empty(int(nbytes), dtype=torch.uint8, device=device)


def _check_bwd_rect(name, q, k, v, d_out):
    """Shape checks in the order and with the messages of attention_backward.mojo:947-958."""
    if q.dim() != 4:
        raise Error("%s: q shape != [B,Sq,H,Dh]" % name)
    B, Sq, H, Dh = q.shape
    if k.dim() != 4 or k.shape[0] != B or k.shape[2] != H or k.shape[3] != Dh:
        raise Error("%s: k shape != [B,Skv,H,Dh]" % name)
    if v.shape != k.shape:
        raise Error("%s: v shape != [B,Skv,H,Dh]" % name)
    if d_out.shape != q.shape:
        raise Error("%s: d_out shape != [B,Sq,H,Dh]" % name)


def sdpa_backward_rect(q, k, v, d_out, scale, variant=PV_FP16):
    """attention_backward.mojo:928-1096: gradients of full attention wrt q [B,Sq,H,Dh] and k, v
    [B,Skv,H,Dh] from the inputs and the upstream gradient alone (no saved forward), in q's dtype."""
    name = "sdpa_backward_rect"
    if q.dtype != k.dtype or q.dtype != v.dtype or q.dtype != d_out.dtype:
        raise Error("%s: q/k/v/d_out dtype mismatch" % name)
    _check_bwd_rect(name, q, k, v, d_out)
    return _math_bwd(name, q, k, v, d_out, scale, variant, _torch_alloc(q.device))


def _check_bwd_square(name, q, k, v, d_out):
    if q.dtype != k.dtype or q.dtype != v.dtype or q.dtype != d_out.dtype:
        raise Error("%s: q/k/v/d_out dtype mismatch" % name)
    if q.dim() != 4:
        raise Error("%s: q shape != compile-time [B,S,H,Dh]" % name)
    if k.shape != q.shape or v.shape != q.shape or d_out.shape != q.shape:
        raise Error("%s: k/v/d_out shape does not match q [B,S,H,Dh]" % name)


def sdpa_backward(q, k, v, d_out, scale, variant=PV_FP16):
    """attention_backward.mojo:435-563: the square case."""
    _check_bwd_square("sdpa_backward", q, k, v, d_out)
    return _math_bwd("sdpa_backward", q, k, v, d_out, scale, variant, _torch_alloc(q.device))


def sdpa_backward_masked(q, k, v, mask_f32, d_out, scale):
    """attention_backward.mojo:566-740 takes an additive mask into the recomputed softmax.  The
    backward kernels here know valid lengths only, so this call is refused instead of answered
    without the mask."""
    raise Error("sdpa_backward_masked: an additive mask is not supported by the backward kernels")


def sdpa_backward_scratch(q, k, v, d_out, scale, scratch, variant=PV_FP16):
    """attention_backward.mojo:1099-1268: the intermediates come from the caller's scratch ring
    and are given back before the call returns; the three gradients are fresh tensors."""
    mark = scratch.mark()
    try:
        _check_bwd_square("sdpa_backward_scratch", q, k, v, d_out)
        g = _math_bwd("sdpa_backward_scratch", q, k, v, d_out, scale, variant, scratch.alloc)
        # (results that were staged in the ring have been converted into fresh tensors by now)
        return g
    finally:
        scratch.rewind(mark)


def sdpa_backward_rect_slab(q, k, v, d_out, scale, slab, variant=PV_FP16):
    """attention_backward.mojo:1477-1638: `sdpa_backward_rect` with every intermediate taken
    from the step's slab (nothing is given back before the step's reset)."""
    name = "sdpa_backward_rect"
    if q.dtype != k.dtype or q.dtype != v.dtype or q.dtype != d_out.dtype:
        raise Error("%s: q/k/v/d_out dtype mismatch" % name)
    _check_bwd_rect(name, q, k, v, d_out)
    return _math_bwd(name, q, k, v, d_out, scale, variant, slab.alloc, slab.alloc)


def sdpa_backward_slab(q, k, v, d_out, scale, slab, variant=PV_FP16):
    """attention_backward.mojo:1641-1768."""
    _check_bwd_square("sdpa_backward", q, k, v, d_out)
    return _math_bwd("sdpa_backward", q, k, v, d_out, scale, variant, slab.alloc, slab.alloc)


def sdpa_backward_dispatch(q, k, v, d_out, scale, B, S, H, Dh, variant=PV_FP16):
    """autograd_v2/ops_record.mojo:165-216: runtime dims -> instantiation.  No table here: the
    dims only have to be the tensors' own."""
    if tuple(q.shape) != (B, S, H, Dh):
        raise Error("sdpa_backward_dispatch: no comptime bucket for (B,S,H,Dh)=(%d,%d,%d,%d)" % (B, S, H, Dh))
    return sdpa_backward(q, k, v, d_out, scale, variant)


def sdpa_backward_dispatch_slab(q, k, v, d_out, scale, B, S, H, Dh, slab, variant=PV_FP16):
    """autograd_v2/ops_record.mojo:463-510."""
    if tuple(q.shape) != (B, S, H, Dh):
        raise Error("sdpa_backward_dispatch: no comptime bucket for (B,S,H,Dh)=(%d,%d,%d,%d)" % (B, S, H, Dh))
    return sdpa_backward_slab(q, k, v, d_out, scale, slab, variant)


class _SdpaNode(torch.autograd.Function):
    """The OPK_SDPA node of the reference's autograd engine in its flash recording
    (serenitymojo/autograd_v2/ops_record.mojo:329-352 records q, k, v and — with the flash arm —
    the forward's saved set; autograd_v2/engine.mojo:236-252 feeds that set and the upstream
    gradient, cast to BF16, to sdpa_flash_backward_dispatch and casts the three gradients back)."""

    @staticmethod
    def forward(ctx, q, k, v, scale, variant):
        if q.dtype != k.dtype or q.dtype != v.dtype:
            raise Error("sdpa_nomask: q/k/v dtype mismatch")
        fwd = sdpa_flash_train_fwd(q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16), scale, variant)
        ctx.save_for_backward(fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, fwd.stats)
        ctx.scale = float(scale)
        return fwd.o.to(q.dtype)

    @staticmethod
    def backward(ctx, g):
        q, k, v, o, stats = ctx.saved_tensors
        B, S, H, Dh = q.shape
        g_bf = g.to(torch.bfloat16).contiguous()
        fb = sdpa_flash_backward_dispatch(q, k, v, o, stats, g_bf, ctx.scale, B, S, H, Dh)
        return fb.d_q.to(g.dtype), fb.d_k.to(g.dtype), fb.d_v.to(g.dtype), None, None


def record_sdpa(q, k, v, scale, variant=PV_FP16):
    """att = sdpa_nomask(q, k, v, scale) recorded for backpropagation
    (serenitymojo/autograd_v2/ops_record.mojo:329-352): the result carries a node whose backward
    yields d_q, d_k, d_v.  torch's autograd graph stands in for the reference's `Graph`."""
    return _SdpaNode.apply(q, k, v, scale, variant)


def sdpa_nomask(q, k, v, scale, variant=PV_FP16):
    """Full attention without a mask tensor (attention.mojo:1690-1718): the entry
    every DiT sampler uses.  Output has q's dtype; F32/F16 storage is cast to
    BF16 at the boundary as the reference's per-model dispatchers do
    (models/zimage/lora_block.mojo:99-123)."""
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("sdpa_nomask: q/k/v dtype mismatch")
    _check_shapes("sdpa_nomask", q, k, v, True)
    _require_cuda("sdpa_nomask", q, k, v)
    if q.dtype == torch.bfloat16:
        o, _ = _call_train_fwd("sdpa_nomask", q, k, v, scale, q.shape[1], k.shape[1], variant, False)
        return o
    o, _ = _call_train_fwd("sdpa_nomask", q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16),
                           scale, q.shape[1], k.shape[1], variant, False)
    return o.to(q.dtype)


def _nomask(name, q, k, v, scale, variant, square, mask=None):
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("%s: q/k/v dtype mismatch" % name)
    _check_shapes(name, q, k, v, square)
    _require_cuda(name, q, k, v)
    if q.dtype == torch.bfloat16:
        return _call_train_fwd(name, q, k, v, scale, q.shape[1], k.shape[1], variant, False, mask)[0]
    o = _call_train_fwd(name, q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16),
                        scale, q.shape[1], k.shape[1], variant, False, mask)[0]
    return o.to(q.dtype)


def sdpa_nomask_tiled(q, k, v, scale, variant=PV_FP16):
    """attention.mojo:1762-1787: the long-sequence entry (video DiTs).  The
    quantized kernel never materialises scores, so it is the same kernel."""
    return _nomask("sdpa_nomask_tiled", q, k, v, scale, variant, True)


def sdpa_qwen_keymask(q, k, v, n_txt, real_txt_len, scale, variant=PV_FP16):
    """attention.mojo:1790-1857: joint attention, tokens ordered TXT then IMG; text keys
    [0, real_txt_len) and image keys [n_txt, S) are kept, the padded text keys
    [real_txt_len, n_txt) are masked.  n_txt is the reference's compile-time N_TXT."""
    if n_txt > q.shape[1] if q.dim() == 4 else False:
        raise Error("sdpa_qwen_keymask: N_TXT must be <= S")
    if real_txt_len < 0 or real_txt_len > n_txt:
        raise Error("sdpa_qwen_keymask: real_txt_len out of range")
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("sdpa_qwen_keymask: q/k/v dtype mismatch")
    if q.dim() != 4:
        raise Error("sdpa_qwen_keymask: q must be rank-4 [B,S,H,Dh]")
    if k.shape != q.shape or v.shape != q.shape:
        raise Error("sdpa_qwen_keymask: k/v shape mismatch")
    return _nomask("sdpa_qwen_keymask", q, k, v, scale, variant, True, (real_txt_len, n_txt))


def sdpa_cross_nomask(q, k, v, scale, variant=PV_FP16):
    """attention.mojo:1860-1894: rectangular Sq != Skv, no mask."""
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("sdpa_cross_nomask: q/k/v dtype mismatch")
    _check_shapes("sdpa_cross_nomask", q, k, v, False)
    _require_cuda("sdpa_cross_nomask", q, k, v)
    if q.dtype == torch.bfloat16:
        return _call_train_fwd("sdpa_cross_nomask", q, k, v, scale, q.shape[1], k.shape[1], variant, False)[0]
    o = _call_train_fwd("sdpa_cross_nomask", q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16),
                        scale, q.shape[1], k.shape[1], variant, False)[0]
    return o.to(q.dtype)


def _masked(name, q, k, v, mask, scale, variant, square):
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("%s: q/k/v dtype mismatch" % name)
    if q.dtype != mask.dtype:
        raise Error("%s: q/mask dtype mismatch" % name)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise Error("%s: q must be rank-4 [B,S,H,Dh]" % name if square else "%s: q/k/v must be rank-4 [B,S,H,Dh]" % name)
    _check_shapes(name, q, k, v, square)
    B, Sq, H, Dh = q.shape
    Skv = k.shape[1]
    if tuple(mask.shape) != (B, H, Sq, Skv):
        raise Error("%s: mask must be [B,H,S,S]" % name if square else "%s: mask must be [B,H,Sq,Skv]" % name)
    _require_cuda(name, q, k, v)
    if not mask.is_cuda:
        raise Error("%s: tensors must live on the GPU (no CPU fallback exists)" % name)
    out_dtype = q.dtype
    if q.dtype != torch.bfloat16:
        q, k, v, mask = (t.to(torch.bfloat16) for t in (q, k, v, mask))
    if mask.stride(3) != 1 or any(st % 4 for st in mask.stride()[:3]):
        mask = mask.contiguous()
        if Skv % 4:                                   # rows of the bias must start 8-byte aligned
            padded = torch.zeros((B, H, Sq, (Skv + 3) // 4 * 4), dtype=mask.dtype, device=mask.device)
            padded[..., :Skv] = mask
            mask = padded
    L = _lib.lib()
    o = torch.empty_like(q)
    ws = _workspace(max(L.mi355_sage_workspace_bytes(B, H, Sq, Skv, Dh, variant), 256), q.device)
    qs, ks = _lib.strides_bhnd(Sq, H, Dh), _lib.strides_bhnd(Skv, H, Dh)
    ms = (_lib.ctypes.c_int64 * 4)(*mask.stride())
    rc = L.mi355_sage_sdpa_bf16_mask(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), o.data_ptr(),
                                     B, H, Sq, Skv, Dh, float(scale), qs, ks, ks, ms, qs, 0, 0, 0, 0, 0,
                                     torch.cuda.current_stream(q.device).cuda_stream, variant, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: shim rc=%d (B=%d Sq=%d Skv=%d H=%d Dh=%d)" % (name, rc, B, Sq, Skv, H, Dh))
    return o.to(out_dtype)


def sdpa(q, k, v, mask, scale, variant=PV_FP16):
    """attention.mojo:1596-1647: full attention with an additive score bias.  q, k, v:
    [B,S,H,Dh]; mask: [B,H,S,S] of q's dtype (zeros = full attention); returns [B,S,H,Dh] in
    q's dtype."""
    return _masked("sdpa", q, k, v, mask, scale, variant, True)


def sdpa_chunked(q, k, v, mask, scale, variant=PV_FP16):
    """attention.mojo:1650-1687: the reference's head-chunked variant of `sdpa` (same result,
    smaller score slab).  This kernel never holds a score slab, so it is the same call."""
    return _masked("sdpa_chunked", q, k, v, mask, scale, variant, True)


def sdpa_tiled(q, k, v, mask, scale, variant=PV_FP16):
    """attention.mojo:1721-1759: the reference's online-softmax variant of `sdpa` for large S
    (same contract and result; never holds the [S,S] scores).  This kernel is that already."""
    return _masked("sdpa_tiled", q, k, v, mask, scale, variant, True)


def sdpa_cross_masked(q, k, v, mask, scale, variant=PV_FP16):
    """attention.mojo:1897-1936: rectangular attention with an additive bias [B,H,Sq,Skv]."""
    return _masked("sdpa_cross_masked", q, k, v, mask, scale, variant, False)


class StepSlab:
    """Counterpart of serenitymojo/autograd_v2/step_slab.mojo:39-90: a bump allocator over one
    device buffer owned by the caller's step.  alloc() hands out 256-byte-aligned views and never
    touches the device allocator; reset() rewinds (host bookkeeping only)."""

    def __init__(self, slab_bytes, device="cuda", alignment=256):
        self.buf = torch.empty(int(slab_bytes), dtype=torch.uint8, device=device)
        self.alignment = alignment
        self.used = 0
        self.peak = 0
        self.n_allocs = 0

    def alloc(self, nbytes):
        base = self.buf.data_ptr()
        start = (base + self.used + self.alignment - 1) // self.alignment * self.alignment - base
        if start + nbytes > self.buf.numel():
            raise Error("StepSlab: out of space (%d + %d > %d)" % (start, nbytes, self.buf.numel()))
        self.used = start + nbytes
        self.peak = max(self.peak, self.used)
        self.n_allocs += 1
        return self.buf[start:start + nbytes]

    def reset(self):
        self.used = 0

    def peak_bytes(self):
        return self.peak

    def capacity_bytes(self):
        return self.buf.numel()

    def used_bytes(self):
        return self.used


def sdpa_nomask_slab(q, k, v, scale, slab, variant=PV_FP16):
    """attention.mojo:2144-2169: `sdpa_nomask` with every allocation (the output and the
    intermediates) taken from the caller's StepSlab instead of the device allocator — the form a
    captured step uses.  BF16 only (the reference's slab path converts nothing either)."""
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise Error("sdpa_nomask: q/k/v dtype mismatch")
    _check_shapes("sdpa_nomask", q, k, v, True)
    _require_bf16("sdpa_nomask_slab", q, k, v)
    _require_cuda("sdpa_nomask", q, k, v)
    B, S, H, Dh = q.shape
    L = _lib.lib()
    o = slab.alloc(q.numel() * 2).view(torch.bfloat16).view(q.shape)
    nws = max(L.mi355_sage_workspace_bytes(B, H, S, S, Dh, variant), 256)
    ws = slab.alloc(nws)
    st = _lib.strides_bhnd(S, H, Dh)
    rc = L.mi355_sage_sdpa_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, S, S, Dh, float(scale),
                                st, st, st, st, 0, 0, 0, 0, 0, torch.cuda.current_stream(q.device).cuda_stream,
                                variant, ws.data_ptr(), nws)
    if rc != 0:
        raise Error("sdpa_nomask: shim rc=%d (B=%d S=%d H=%d Dh=%d)" % (rc, B, S, H, Dh))
    return o


def _norm_rope_args(name, q_pre, k_pre, v, q_norm, k_norm, cos, sin, halfsplit=False, full_row=False):
    _check_shapes(name, q_pre, k_pre, v, True)
    _require_bf16(name, q_pre, k_pre, v)
    _require_cuda(name, q_pre, k_pre, v)
    B, S, H, Dh = q_pre.shape
    cols = H * Dh if full_row else Dh
    if q_norm.numel() != cols or k_norm.numel() != cols:
        raise Error("%s: weight must be [%d]" % (name, cols))
    flags = (_lib.ROPE_HALFSPLIT if halfsplit else 0) | (_lib.NORM_FULL_ROW if full_row else 0)
    gq = q_norm.to(device=q_pre.device, dtype=torch.bfloat16).contiguous()
    gk = k_norm.to(device=q_pre.device, dtype=torch.bfloat16).contiguous()
    batch_rows = 0
    if (cos is None) != (sin is None):
        raise Error("%s: cos and sin come together" % name)
    if cos is not None:
        if cos.dtype != sin.dtype or cos.dtype not in (torch.float32, torch.bfloat16):
            raise Error("%s: cos/sin tables must be F32 (or both BF16)" % name)
        if cos.dtype == torch.bfloat16:
            flags |= _lib.ROPE_TABLES_BF16
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != Dh // 2:
            raise Error("%s: cos/sin must be [rows, D/2]" % name)
        if cos.shape[0] == B * S * H and B > 1:
            batch_rows = S * H
        elif cos.shape[0] != S * H:
            raise Error("%s: cos/sin rows must be S*H (or B*S*H)" % name)
        cos, sin = cos.contiguous(), sin.contiguous()
    return gq, gk, cos, sin, batch_rows, flags


def qk_norm_rope_sdpa_nomask(q_pre, k_pre, v, q_norm, k_norm, eps, cos, sin, scale, variant=PV_FP16,
                             blkq=None, blkk=64, k_flags=_lib.K_SMOOTH | _lib.K_BALANCE, halfsplit=False,
                             full_row=False):
    """The attention block of a DiT layer from the projections on, in one call:

        q = rope_interleaved(rms_norm(q_pre, q_norm, eps), cos, sin)
        k = rope_interleaved(rms_norm(k_pre, k_norm, eps), cos, sin)
        att = sdpa_nomask(q, k, v, scale)

    (serenitymojo/models/klein/single_block.mojo:977-982) with the norm and the rotation fused
    into the quantizers.  q_pre/k_pre/v: BF16 [B,S,H,Dh]; q_norm/k_norm: [Dh] (cast to BF16 like
    ops/norm.mojo:170-172 does when the gain's dtype differs); cos/sin: F32 [S*H, Dh/2]
    (sampling/klein_sampler.mojo:305-307) or [B*S*H, Dh/2], or None for norm only.
    halfsplit: rope_halfsplit instead of rope_interleaved (ops/rope.mojo:10-13; the per-head norm +
    half-split rotation of models/anima/block.mojo:360-366).  full_row: the RMSNorm runs over the
    whole inner dim, q_norm/k_norm are [H*Dh] (rms_norm on [S, H*Dh] before the reshape to heads,
    models/ltx2/ltx2_block.mojo:419-432, whose tables are BF16 — also accepted)."""
    name = "qk_norm_rope_sdpa_nomask"
    gq, gk, cos, sin, batch_rows, flags = _norm_rope_args(name, q_pre, k_pre, v, q_norm, k_norm, cos, sin, halfsplit, full_row)
    B, S, H, Dh = q_pre.shape
    L = _lib.lib()
    o = torch.empty_like(q_pre)
    nbytes = L.mi355_sage_workspace_bytes(B, H, S, S, Dh, variant)
    ws = _workspace(max(nbytes, 256), q_pre.device)
    st = _lib.strides_bhnd(S, H, Dh)
    if blkq is None:
        blkq = 32 if variant == PV_FP8 else 128
    rc = L.mi355_sage_sdpa_bf16_norm_rope(
        q_pre.data_ptr(), k_pre.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, S, S, Dh, float(scale),
        st, st, st, st, 0, 0, 0, 0, 0, torch.cuda.current_stream(q_pre.device).cuda_stream,
        variant, blkq, blkk, int(k_flags), gq.data_ptr(), gk.data_ptr(), float(eps),
        cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None, batch_rows,
        flags, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: shim rc=%d (B=%d S=%d H=%d Dh=%d)" % (name, rc, B, S, H, Dh))
    return o


def qk_norm_rope_sdpa_flash_train_fwd(q_pre, k_pre, v, q_norm, k_norm, eps, cos, sin, scale, variant=PV_FP16,
                                      halfsplit=False, full_row=False):
    """The same block where the caller keeps the attention statistics for a backward pass:
    rms_norm / rope_interleaved followed by sdpa_flash_train_fwd
    (serenitymojo/ops/attention_flash.mojo:149-202).  Returns an SdpaFlashFwd whose stats are the
    log-sum-exp of the normalised, rotated Q and K."""
    name = "qk_norm_rope_sdpa_flash_train_fwd"
    gq, gk, cos, sin, batch_rows, flags = _norm_rope_args(name, q_pre, k_pre, v, q_norm, k_norm, cos, sin, halfsplit, full_row)
    B, S, H, Dh = q_pre.shape
    L = _lib.lib()
    o = torch.empty_like(q_pre)
    stats = torch.empty((B, H, S, 1), dtype=torch.float32, device=q_pre.device)
    nbytes = L.mi355_sage_workspace_bytes(B, H, S, S, Dh, variant)
    ws = _workspace(max(nbytes, 256), q_pre.device)
    st = _lib.strides_bhnd(S, H, Dh)
    rc = L.mi355_sage_sdpa_bf16_norm_rope_train_fwd(
        q_pre.data_ptr(), k_pre.data_ptr(), v.data_ptr(), o.data_ptr(), stats.data_ptr(), B, H, S, S, Dh, float(scale),
        st, st, st, st, 0, 0, 0, 0, 0, 0, S, S, torch.cuda.current_stream(q_pre.device).cuda_stream,
        variant, gq.data_ptr(), gk.data_ptr(), float(eps),
        cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None, batch_rows,
        flags, ws.data_ptr(), ws.numel())
    if rc != 0:
        raise Error("%s: shim rc=%d (B=%d S=%d H=%d Dh=%d)" % (name, rc, B, S, H, Dh))
    return SdpaFlashFwd(o, o, q_pre, k_pre, v, stats)
