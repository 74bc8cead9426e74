// mi355_sage_host.hpp — the serenitymojo attention call surface for compiled (C++) callers,
// header-only, on top of the C ABI in mi355_sage.h.
//
// The reference's host code is Mojo: Tensor = a device buffer + shape + dtype
// (serenitymojo/tensor.mojo:33-62), operators are free functions that validate, allocate their
// results, call the native library through FFI and `raise Error(...)` on a non-zero return code
// (serenitymojo/ops/attention_flash.mojo:149-202).  This header restates that surface one to
// one — same function names, argument order and meaning, same error texts — for a host that
// has no Mojo toolchain:
//
//   sdpa_flash_train_fwd, _rect, sdpa_flash_fwd_padmask      attention_flash.mojo:149, :205, :267
//   sdpa_flash_backward, sdpa_flash_backward_raw, _dispatch  attention_flash.mojo:345, :538, :610
//   sdpa_nomask, sdpa_nomask_tiled, sdpa_cross_nomask        ops/attention.mojo:1690, :1762, :1860
//   sdpa_qwen_keymask                                        ops/attention.mojo:1790
//   sdpa, sdpa_cross_masked                                  ops/attention.mojo:1596, :1897
//
// What differs from the cuDNN bridge: no padding of the sequence to 128 is needed (ragged lengths
// are handled in the kernels), so the `*_pad` members of a forward result share the caller's
// buffers.  BF16 only: the F32 / F16 boundary casts of the reference's dispatchers are the
// caller's (they are elementwise kernels of the framework, not of this library).
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "mi355_sage.h"

namespace mi355_sage_host {

// Counterpart of Mojo's `raise Error(...)`.
struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// serenitymojo/io/dtype.mojo:39-57 (the three storage types the attention surface meets).
enum class STDtype { BF16, F16, F32 };
inline size_t dtype_bytes(STDtype d) { return d == STDtype::F32 ? 4 : 2; }

// serenitymojo's DeviceContext as far as this surface uses it: the stream the work is queued on.
struct DeviceContext {
    hipStream_t stream = nullptr;
    void synchronize() const {
        if (hipStreamSynchronize(stream) != hipSuccess) throw Error("DeviceContext: synchronize failed");
    }
};

// A device buffer + shape + dtype (serenitymojo/tensor.mojo:33-62).  Movable; copying shares the
// buffer (the reference's ArcPointer[Tensor] / zero-copy views), it never copies device memory.
class Tensor {
  public:
    Tensor() = default;
    Tensor(std::vector<int64_t> shape, STDtype dtype) : shape_(std::move(shape)), dtype_(dtype) {
        void* p = nullptr;
        const size_t n = nbytes();
        if (hipMalloc(&p, n ? n : 1) != hipSuccess) throw Error("Tensor: device allocation of " + std::to_string(n) + " bytes failed");
        buf_ = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
    }
    // A view of `other`'s buffer with another shape (no copy).
    Tensor(const Tensor& other, std::vector<int64_t> shape) : buf_(other.buf_), shape_(std::move(shape)), dtype_(other.dtype_) {}
    const std::vector<int64_t>& shape() const { return shape_; }
    STDtype dtype() const { return dtype_; }
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape_) n *= d;
        return n;
    }
    size_t nbytes() const { return (size_t)numel() * dtype_bytes(dtype_); }
    void* unsafe_ptr() const { return buf_.get(); }      // the raw device address handed to native code
    bool defined() const { return buf_ != nullptr; }

  private:
    std::shared_ptr<void> buf_;
    std::vector<int64_t> shape_;
    STDtype dtype_ = STDtype::BF16;
};

// attention_flash.mojo:108-135.
struct SdpaFlashFwd {
    Tensor o, o_pad, q_pad, k_pad, v_pad, stats;
};
// attention_flash.mojo:138-146.
struct SdpaFlashGrads {
    Tensor d_q, d_k, d_v;
};

namespace detail {

// attention_flash.mojo:46-54: logical [B,H,N,D] over [B,N,H,Dh] memory.
struct Strides {
    int64_t s[4];
    Strides(int64_t n, int64_t h, int64_t dh) : s{n * h * dh, dh, h * dh, 1} {}
};

inline std::string dims(int B, int Sq, int Skv, int H, int Dh) {
    return " (B=" + std::to_string(B) + " Sq=" + std::to_string(Sq) + " Skv=" + std::to_string(Skv) +
           " H=" + std::to_string(H) + " Dh=" + std::to_string(Dh) + ")";
}

inline void require_bf16(const char* name, std::initializer_list<const Tensor*> ts) {
    for (const Tensor* t : ts)
        if (t->dtype() != STDtype::BF16) throw Error(std::string(name) + ": q/k/v must be BF16");
}

inline void check_shapes(const char* name, const Tensor& q, const Tensor& k, const Tensor& v, bool square) {
    const std::string n(name);
    if (q.shape().size() != 4) throw Error(n + ": q must be rank-4 [B,S,H,Dh]");
    if (k.shape() != v.shape() || k.shape().size() != 4) throw Error(n + ": k/v shape mismatch");
    if (q.shape()[0] != k.shape()[0] || q.shape()[2] != k.shape()[2] || q.shape()[3] != k.shape()[3])
        throw Error(n + ": q and k/v disagree on B/H/Dh");
    if (square && q.shape()[1] != k.shape()[1]) throw Error(n + ": k/v shape does not match q [B,S,H,Dh]");
}

// One growing workspace per (device, stream), kept for the life of the process (the library's own policy for
// a NULL workspace, spelled out on the caller's side so that steady-state calls allocate nothing).
inline void* workspace(size_t nbytes, hipStream_t stream, size_t* have) {
    struct Slot { int dev; hipStream_t stream; void* p; size_t bytes; };
    static std::vector<Slot> slots;
    static std::mutex guard;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) throw Error("workspace: no current device");
    std::lock_guard<std::mutex> lock(guard);
    for (Slot& s : slots)
        if (s.dev == dev && s.stream == stream) {
            if (s.bytes < nbytes) {
                void* p = nullptr;
                const size_t want = nbytes > 2 * s.bytes ? nbytes : 2 * s.bytes;
                if (hipMalloc(&p, want) != hipSuccess) throw Error("workspace allocation failed");
                s.p = p;                 // the old buffer stays allocated: queued work may still use it
                s.bytes = want;
            }
            *have = s.bytes;
            return s.p;
        }
    void* p = nullptr;
    if (hipMalloc(&p, nbytes) != hipSuccess) throw Error("workspace allocation failed");
    slots.push_back(Slot{dev, stream, p, nbytes});
    *have = nbytes;
    return p;
}

struct Call {
    int B, Sq, Skv, H, Dh;
    Call(const Tensor& q, const Tensor& k)
        : B((int)q.shape()[0]), Sq((int)q.shape()[1]), Skv((int)k.shape()[1]), H((int)q.shape()[2]), Dh((int)q.shape()[3]) {}
};

// The train-forward / plain / key-range-mask call with freshly allocated results.
inline std::pair<Tensor, Tensor> forward(const char* name, const Tensor& q, const Tensor& k, const Tensor& v, float scale,
                                         int real_q, int real_kv, int variant, bool want_stats, const DeviceContext& ctx,
                                         int mask_lo = 0, int mask_hi = 0, bool keymask = false) {
    const Call c(q, k);
    Tensor o(q.shape(), STDtype::BF16);
    Tensor stats;
    if (want_stats) stats = Tensor({c.B, c.H, c.Sq, 1}, STDtype::F32);
    size_t have = 0;
    size_t need = mi355_sage_workspace_bytes(c.B, c.H, c.Sq, c.Skv, c.Dh, variant);
    void* ws = workspace(need < 256 ? 256 : need, ctx.stream, &have);
    const Strides qs(c.Sq, c.H, c.Dh), ks(c.Skv, c.H, c.Dh);
    int rc;
    if (keymask)
        rc = mi355_sage_sdpa_bf16_keymask(q.unsafe_ptr(), k.unsafe_ptr(), v.unsafe_ptr(), o.unsafe_ptr(),
                                          want_stats ? stats.unsafe_ptr() : nullptr, c.B, c.H, c.Sq, c.Skv, c.Dh, scale,
                                          qs.s, ks.s, ks.s, qs.s, 0, 0, 0, 0, 0, mask_lo, mask_hi, ctx.stream, variant, ws, have);
    else if (want_stats)
        rc = mi355_sage_sdpa_bf16_train_fwd(q.unsafe_ptr(), k.unsafe_ptr(), v.unsafe_ptr(), o.unsafe_ptr(), stats.unsafe_ptr(),
                                            c.B, c.H, c.Sq, c.Skv, c.Dh, scale, qs.s, ks.s, ks.s, qs.s, 0, 0, 0, 0, 0,
                                            0, real_q, real_kv, ctx.stream, variant, ws, have);
    else
        rc = mi355_sage_sdpa_bf16(q.unsafe_ptr(), k.unsafe_ptr(), v.unsafe_ptr(), o.unsafe_ptr(), c.B, c.H, c.Sq, c.Skv, c.Dh,
                                  scale, qs.s, ks.s, ks.s, qs.s, 0, 0, 0, 0, 0, ctx.stream, variant, ws, have);
    if (rc != 0) throw Error(std::string(name) + ": shim rc=" + std::to_string(rc) + dims(c.B, c.Sq, c.Skv, c.H, c.Dh));
    return {o, stats};
}

inline SdpaFlashGrads backward(const char* name, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& o,
                               const Tensor& d_out, const Tensor& stats, float scale, int real_q, int real_kv,
                               const DeviceContext& ctx) {
    const Call c(q, k);
    SdpaFlashGrads g{Tensor(q.shape(), STDtype::BF16), Tensor(k.shape(), STDtype::BF16), Tensor(v.shape(), STDtype::BF16)};
    size_t have = 0;
    size_t need = mi355_sage_bwd_workspace_bytes(c.B, c.H, c.Sq, c.Skv, c.Dh);
    void* ws = workspace(need < 256 ? 256 : need, ctx.stream, &have);
    const Strides qs(c.Sq, c.H, c.Dh), ks(c.Skv, c.H, c.Dh);
    const int rc = mi355_sage_sdpa_bwd_bf16(q.unsafe_ptr(), k.unsafe_ptr(), v.unsafe_ptr(), o.unsafe_ptr(), d_out.unsafe_ptr(),
                                            stats.unsafe_ptr(), g.d_q.unsafe_ptr(), g.d_k.unsafe_ptr(), g.d_v.unsafe_ptr(),
                                            c.B, c.H, c.Sq, c.Skv, c.Dh, scale, qs.s, ks.s, ks.s, qs.s, qs.s, qs.s, ks.s, ks.s,
                                            0, 0, 0, 0, 0, 0, 0, 0, 0, 0, real_q, real_kv, ctx.stream, ws, have);
    if (rc != 0) throw Error(std::string(name) + ": shim rc=" + std::to_string(rc) + dims(c.B, c.Sq, c.Skv, c.H, c.Dh));
    return g;
}

}  // namespace detail

constexpr int PV_FP16 = MI355_SAGE_PV_FP16;
constexpr int PV_FP8 = MI355_SAGE_PV_FP8;

// attention_flash.mojo:149-202: training forward on [B,S,H,Dh] BF16 — O and the softmax Stats
// (natural-log log-sum-exp, [B,H,S,1] F32) the flash backward needs.
inline SdpaFlashFwd sdpa_flash_train_fwd(const Tensor& q, const Tensor& k, const Tensor& v, float scale,
                                         const DeviceContext& ctx, int variant = PV_FP16) {
    const char* name = "sdpa_flash_train_fwd";
    detail::require_bf16(name, {&q, &k, &v});
    detail::check_shapes(name, q, k, v, true);
    auto r = detail::forward(name, q, k, v, scale, (int)q.shape()[1], (int)k.shape()[1], variant, true, ctx);
    return SdpaFlashFwd{r.first, r.first, q, k, v, r.second};
}

// attention_flash.mojo:205-264: S_q != S_kv.
inline SdpaFlashFwd sdpa_flash_train_fwd_rect(const Tensor& q, const Tensor& k, const Tensor& v, float scale,
                                              const DeviceContext& ctx, int variant = PV_FP16) {
    const char* name = "sdpa_flash_train_fwd_rect";
    detail::require_bf16(name, {&q, &k, &v});
    detail::check_shapes(name, q, k, v, false);
    auto r = detail::forward(name, q, k, v, scale, (int)q.shape()[1], (int)k.shape()[1], variant, true, ctx);
    return SdpaFlashFwd{r.first, r.first, q, k, v, r.second};
}

// attention_flash.mojo:267-342: buffers of S_BUF tokens of which the first real_len are real; keys
// beyond it get no weight.  Rows beyond it are computed and meaningless, as in the reference.
inline SdpaFlashFwd sdpa_flash_fwd_padmask(const Tensor& q, const Tensor& k, const Tensor& v, int real_len, float scale,
                                           const DeviceContext& ctx, int variant = PV_FP16) {
    const char* name = "sdpa_flash_fwd_padmask";
    detail::require_bf16(name, {&q, &k, &v});
    detail::check_shapes(name, q, k, v, true);
    const int S_BUF = (int)q.shape()[1];
    if (S_BUF % 128 != 0) throw Error(std::string(name) + ": S_BUF must be 128-aligned");
    if (real_len < 1 || real_len > S_BUF) throw Error(std::string(name) + ": real_len out of [1, S_BUF]");
    auto r = detail::forward(name, q, k, v, scale, real_len, real_len, variant, true, ctx);
    return SdpaFlashFwd{r.first, r.first, q, k, v, r.second};
}

// attention_flash.mojo:345-433: dQ, dK, dV [B,S,H,Dh] BF16 from the saved forward set.
inline SdpaFlashGrads sdpa_flash_backward(const SdpaFlashFwd& fwd, const Tensor& d_out, float scale, const DeviceContext& ctx,
                                          int real_len = 0) {
    const char* name = "sdpa_flash_backward";
    detail::require_bf16(name, {&fwd.q_pad, &fwd.k_pad, &fwd.v_pad, &fwd.o_pad});
    if (d_out.dtype() != STDtype::BF16) throw Error(std::string(name) + ": d_out must be BF16");
    if (d_out.shape() != fwd.o_pad.shape()) throw Error(std::string(name) + ": d_out shape does not match the forward output");
    const int rq = real_len > 0 ? real_len : (int)fwd.q_pad.shape()[1];
    const int rk = real_len > 0 ? real_len : (int)fwd.k_pad.shape()[1];
    return detail::backward(name, fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, d_out, fwd.stats, scale, rq, rk, ctx);
}

// attention_flash.mojo:538-607: the same on the saved tensors of the graph path.
inline SdpaFlashGrads sdpa_flash_backward_raw(const Tensor& q_pad, const Tensor& k_pad, const Tensor& v_pad, const Tensor& o_pad,
                                              const Tensor& stats, const Tensor& d_out, float scale, const DeviceContext& ctx) {
    const char* name = "sdpa_flash_backward_raw";
    detail::require_bf16(name, {&q_pad, &k_pad, &v_pad, &o_pad});
    if (d_out.dtype() != STDtype::BF16) throw Error(std::string(name) + ": d_out must be BF16");
    return detail::backward(name, q_pad, k_pad, v_pad, o_pad, d_out, stats, scale, (int)q_pad.shape()[1], (int)k_pad.shape()[1], ctx);
}

// attention_flash.mojo:610-633: runtime dims in; every shape the tensors really have is served
// (the reference looks them up in a table of compiled instantiations).
inline SdpaFlashGrads sdpa_flash_backward_dispatch(const Tensor& q_pad, const Tensor& k_pad, const Tensor& v_pad, const Tensor& o_pad,
                                                   const Tensor& stats, const Tensor& d_out, float scale, int B, int S, int H, int Dh,
                                                   const DeviceContext& ctx) {
    if (q_pad.shape() != std::vector<int64_t>{B, S, H, Dh})
        throw Error("sdpa_flash_backward_dispatch: no bucket (B,S,H,Dh)=(" + std::to_string(B) + "," + std::to_string(S) + "," +
                    std::to_string(H) + "," + std::to_string(Dh) + ")");
    return sdpa_flash_backward_raw(q_pad, k_pad, v_pad, o_pad, stats, d_out, scale, ctx);
}

// ops/attention.mojo:1690-1718: full attention without a mask tensor, the entry of every DiT sampler.
inline Tensor sdpa_nomask(const Tensor& q, const Tensor& k, const Tensor& v, float scale, const DeviceContext& ctx,
                          int variant = PV_FP16) {
    const char* name = "sdpa_nomask";
    if (q.dtype() != k.dtype() || q.dtype() != v.dtype()) throw Error("sdpa_nomask: q/k/v dtype mismatch");
    detail::check_shapes(name, q, k, v, true);
    detail::require_bf16(name, {&q, &k, &v});
    return detail::forward(name, q, k, v, scale, 0, 0, variant, false, ctx).first;
}

// ops/attention.mojo:1762-1787: the long-sequence entry; the same kernel here.
inline Tensor sdpa_nomask_tiled(const Tensor& q, const Tensor& k, const Tensor& v, float scale, const DeviceContext& ctx,
                                int variant = PV_FP16) {
    const char* name = "sdpa_nomask_tiled";
    if (q.dtype() != k.dtype() || q.dtype() != v.dtype()) throw Error("sdpa_nomask_tiled: q/k/v dtype mismatch");
    detail::check_shapes(name, q, k, v, true);
    detail::require_bf16(name, {&q, &k, &v});
    return detail::forward(name, q, k, v, scale, 0, 0, variant, false, ctx).first;
}

// ops/attention.mojo:1860-1894: rectangular attention.
inline Tensor sdpa_cross_nomask(const Tensor& q, const Tensor& k, const Tensor& v, float scale, const DeviceContext& ctx,
                                int variant = PV_FP16) {
    const char* name = "sdpa_cross_nomask";
    if (q.dtype() != k.dtype() || q.dtype() != v.dtype()) throw Error("sdpa_cross_nomask: q/k/v dtype mismatch");
    detail::check_shapes(name, q, k, v, false);
    detail::require_bf16(name, {&q, &k, &v});
    return detail::forward(name, q, k, v, scale, 0, 0, variant, false, ctx).first;
}

// ops/attention.mojo:1790-1857: joint text + image sequence whose text part holds n_txt tokens of
// which the first real_txt_len are real; keys [real_txt_len, n_txt) get no weight.
inline Tensor sdpa_qwen_keymask(const Tensor& q, const Tensor& k, const Tensor& v, int n_txt, int real_txt_len, float scale,
                                const DeviceContext& ctx, int variant = PV_FP16) {
    const char* name = "sdpa_qwen_keymask";
    if (q.shape().size() == 4 && n_txt > q.shape()[1]) throw Error("sdpa_qwen_keymask: N_TXT must be <= S");
    if (real_txt_len < 0 || real_txt_len > n_txt) throw Error("sdpa_qwen_keymask: real_txt_len out of range");
    if (q.dtype() != k.dtype() || q.dtype() != v.dtype()) throw Error("sdpa_qwen_keymask: q/k/v dtype mismatch");
    detail::check_shapes(name, q, k, v, true);
    detail::require_bf16(name, {&q, &k, &v});
    return detail::forward(name, q, k, v, scale, 0, 0, variant, false, ctx, real_txt_len, n_txt, true).first;
}

namespace detail {
inline Tensor masked(const char* name, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& mask, float scale,
                     const DeviceContext& ctx, int variant, bool square) {
    const std::string n(name);
    if (q.dtype() != k.dtype() || q.dtype() != v.dtype()) throw Error(n + ": q/k/v dtype mismatch");
    if (q.dtype() != mask.dtype()) throw Error(n + ": q/mask dtype mismatch");
    check_shapes(name, q, k, v, square);
    require_bf16(name, {&q, &k, &v});
    const Call c(q, k);
    if (mask.shape() != std::vector<int64_t>{c.B, c.H, c.Sq, c.Skv})
        throw Error(n + (square ? ": mask must be [B,H,S,S]" : ": mask must be [B,H,Sq,Skv]"));
    if (c.Skv % 4 != 0) throw Error(n + ": rows of the mask must start 8-byte aligned (S_kv a multiple of 4, or pad the rows)");
    Tensor o(q.shape(), STDtype::BF16);
    size_t have = 0;
    size_t need = mi355_sage_workspace_bytes(c.B, c.H, c.Sq, c.Skv, c.Dh, variant);
    void* ws = workspace(need < 256 ? 256 : need, ctx.stream, &have);
    const Strides qs(c.Sq, c.H, c.Dh), ks(c.Skv, c.H, c.Dh);
    const int64_t ms[4] = {(int64_t)c.H * c.Sq * c.Skv, (int64_t)c.Sq * c.Skv, c.Skv, 1};
    const int rc = mi355_sage_sdpa_bf16_mask(q.unsafe_ptr(), k.unsafe_ptr(), v.unsafe_ptr(), mask.unsafe_ptr(), o.unsafe_ptr(),
                                             c.B, c.H, c.Sq, c.Skv, c.Dh, scale, qs.s, ks.s, ks.s, ms, qs.s, 0, 0, 0, 0, 0,
                                             ctx.stream, variant, ws, have);
    if (rc != 0) throw Error(n + ": shim rc=" + std::to_string(rc) + dims(c.B, c.Sq, c.Skv, c.H, c.Dh));
    return o;
}
}  // namespace detail

// ops/attention.mojo:1596-1647: attention with an additive mask [B,H,S,S] in q's dtype.
inline Tensor sdpa(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& mask, float scale, const DeviceContext& ctx,
                   int variant = PV_FP16) {
    return detail::masked("sdpa", q, k, v, mask, scale, ctx, variant, true);
}

// ops/attention.mojo:1897-1936: rectangular, mask [B,H,Sq,Skv].
inline Tensor sdpa_cross_masked(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& mask, float scale,
                                const DeviceContext& ctx, int variant = PV_FP16) {
    return detail::masked("sdpa_cross_masked", q, k, v, mask, scale, ctx, variant, false);
}

}  // namespace mi355_sage_host
