// sage_api.hip — the C ABI of libmi355_sage.so (declared in include/mi355_sage.h).
// Host-side only: argument checks, workspace carving, kernel sequencing.
#include "../../include/mi355_sage.h"
#include "sage_internal.h"

#include <cstdio>
#include <mutex>

using namespace sage;

namespace {

constexpr size_t kAlign = 256;
inline size_t align_up(size_t x) { return (x + kAlign - 1) / kAlign * kAlign; }

#define SAGE_LOG(...)                              \
    do {                                           \
        std::fprintf(stderr, "[mi355_sage] ");     \
        std::fprintf(stderr, __VA_ARGS__);         \
        std::fprintf(stderr, "\n");                \
    } while (0)

#define SAGE_HIP(expr)                                                              \
    do {                                                                            \
        hipError_t e_ = (expr);                                                     \
        if (e_ != hipSuccess) {                                                     \
            SAGE_LOG("%s failed: %s", #expr, hipGetErrorString(e_));                \
            return (int)e_;                                                         \
        }                                                                           \
    } while (0)

bool dims_ok(int D) { return D == 64 || D == 128; }

// Row starts must be 16-byte aligned and the head dim contiguous.
int check_view(const char* name, const void* p, const int64_t* s, int64_t off) {
    if (s[3] != 1) {
        SAGE_LOG("%s: innermost stride %lld != 1", name, (long long)s[3]);
        return MI355_SAGE_EUNSUPPORTED;
    }
    const uintptr_t a = reinterpret_cast<uintptr_t>(p) + (uintptr_t)(off * 2);
    if ((a & 15) || (s[0] & 7) || (s[1] & 7) || (s[2] & 7)) {
        SAGE_LOG("%s: rows are not 16-byte aligned", name);
        return MI355_SAGE_EUNSUPPORTED;
    }
    return 0;
}

View make_view(const void* p, const int64_t* s, int64_t off) {
    return View{static_cast<const uint16_t*>(p) + off, s[0], s[1], s[2]};
}

bool blk_ok(int blk) { return blk == 32 || blk == 64 || blk == 128; }

// The attention kernel keeps one head's K scales in LDS.
int check_kv_len(int N_kv, int blkk) {
    if (pad_to(N_kv, kPadKV) / blkk > kMaxKScales) {
        SAGE_LOG("N_kv=%d with %d-token K blocks exceeds %d scale blocks per head", N_kv, blkk, kMaxKScales);
        return MI355_SAGE_EUNSUPPORTED;
    }
    return 0;
}

// Workspace layout of the one-shot calls.
struct Carve {
    size_t q8, k8, vq, qscale, kscale, kmean, vscale, partial, qshift, total;
};

Carve carve(int B, int H, int Nq, int Nkv, int D, int variant) {
    const size_t bh = (size_t)B * H;
    const size_t nqp = (size_t)pad_to(Nq, kTileQ), nkp = (size_t)pad_to(Nkv, kPadKV);
    Carve c{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
    c.q8 = take(bh * nqp * D);
    c.k8 = take(bh * nkp * D);
    c.vq = take(bh * nkp * D * (variant == MI355_SAGE_PV_FP16 ? 2 : 1));
    c.qscale = take(bh * (nqp / 32) * sizeof(float));      // smallest block is 32 tokens
    c.kscale = take(bh * (nkp / 32) * sizeof(float));
    c.kmean = take(bh * D * sizeof(float));
    c.vscale = take(bh * D * sizeof(float));
    c.partial = take(bh * ((Nkv + kGroup - 1) / kGroup) * D * sizeof(double));
    c.qshift = take(bh * nqp * sizeof(float));
    c.total = off;
    return c;
}

// Internal workspace: one buffer per device, grown on demand, never freed
// while the process lives (same lifetime as the cuDNN shim's per-graph workspace).
std::mutex g_ws_mutex;
struct DevWs { void* p = nullptr; size_t bytes = 0; };
DevWs g_ws[64];

int internal_workspace(size_t need, void** out) {
    int dev = 0;
    SAGE_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return MI355_SAGE_EUNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DevWs& w = g_ws[dev];
    if (w.bytes < need) {
        // The old buffer may still be in use by work queued earlier; wait before freeing.
        if (w.p) {
            SAGE_HIP(hipDeviceSynchronize());
            SAGE_HIP(hipFree(w.p));
            w.p = nullptr;
            w.bytes = 0;
        }
        SAGE_HIP(hipMalloc(&w.p, need));
        w.bytes = need;
    }
    *out = w.p;
    return 0;
}

// The optional ops in front of the quantizers (RMSNorm + interleaved RoPE of Q and of K).
struct Pre {
    PreOp q{}, k{};
};

// q_gain / k_gain null together = nothing to do.  Tables are optional on top of the gains.
int make_pre(const void* q_gain, const void* k_gain, float eps, const void* rope_cos, const void* rope_sin,
             int64_t rope_batch_rows, Pre* out) {
    *out = Pre{};
    if (!q_gain && !k_gain && !rope_cos && !rope_sin) return 0;
    if (!q_gain || !k_gain) { SAGE_LOG("RMSNorm gains must be given for both Q and K"); return MI355_SAGE_EINVAL; }
    if ((rope_cos == nullptr) != (rope_sin == nullptr)) return MI355_SAGE_EINVAL;
    if (!(eps >= 0.0f) || rope_batch_rows < 0) return MI355_SAGE_EINVAL;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q_gain) | reinterpret_cast<uintptr_t>(k_gain) |
                           reinterpret_cast<uintptr_t>(rope_cos) | reinterpret_cast<uintptr_t>(rope_sin);
    if (bits & 15) { SAGE_LOG("gains and RoPE tables must be 16-byte aligned"); return MI355_SAGE_EUNSUPPORTED; }
    out->q = PreOp{static_cast<const uint16_t*>(q_gain), eps, static_cast<const float*>(rope_cos),
                   static_cast<const float*>(rope_sin), rope_batch_rows};
    out->k = out->q;
    out->k.gain = static_cast<const uint16_t*>(k_gain);
    return 0;
}

int quant_qk(const View& q, const View& k, int B, int H, int Nq, int Nkv, int D, float scale,
             int blkq, int blkk, int smooth_k, int8_t* q8, float* qscale, int8_t* k8, float* kscale,
             float* kmean, double* partial, float* qshift, const Pre& pre, hipStream_t st) {
    const float cmul = (float)((double)scale * 1.4426950408889634074);   // scale*log2(e), rounded once
    if (smooth_k) SAGE_HIP(launch_kmean(k, B, H, Nkv, D, partial, kmean, pre.k, st));
    SAGE_HIP(launch_quant_i8(q, B, H, Nq, D, pad_to(Nq, kTileQ), blkq, false, cmul, kmean, q8, qscale,
                             smooth_k ? qshift : nullptr, pre.q, st));
    SAGE_HIP(launch_quant_i8(k, B, H, Nkv, D, pad_to(Nkv, kPadKV), blkk, true, 0.0f,
                             smooth_k ? kmean : nullptr, k8, kscale, nullptr, pre.k, st));
    return 0;
}

int sdpa_impl(const void* Q, const void* K, const void* V, void* O, void* Stats,
              int B, int H, int N_q, int N_kv, int D, float scale,
              const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
              int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t stats_off,
              int causal, int real_N_kv, void* stream,
              int variant, int blkq, int blkk, int smooth_k, void* workspace, size_t workspace_bytes,
              const Pre& pre = Pre{}) {
    // argument checks in the order of serenitymojo/ops/cshim/cudnn_sdpa.cpp:391-393
    if (!Q || !K || !V || !O) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!qs || !ks || !vs || !os) return MI355_SAGE_EINVAL;
    if (causal) { SAGE_LOG("causal attention is not supported"); return MI355_SAGE_EUNSUPPORTED; }
    if (!dims_ok(D)) { SAGE_LOG("head dim %d not supported (64 or 128)", D); return MI355_SAGE_EUNSUPPORTED; }
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (!blk_ok(blkq) || !blk_ok(blkk)) { SAGE_LOG("block sizes must be 32, 64 or 128"); return MI355_SAGE_EUNSUPPORTED; }
    int rc;
    if ((rc = check_kv_len(N_kv, blkk))) return rc;
    if ((rc = check_view("Q", Q, qs, q_off)) || (rc = check_view("K", K, ks, k_off)) ||
        (rc = check_view("V", V, vs, v_off)) || (rc = check_view("O", O, os, o_off)))
        return rc;
    // Keys past the real length are excluded from the statistics and the scores alike:
    // the quantizers see only the first kv tokens.
    const int kv = (real_N_kv > 0 && real_N_kv < N_kv) ? real_N_kv : N_kv;

    const Carve c = carve(B, H, N_q, kv, D, variant);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    if (ws) {
        if (workspace_bytes < c.total) {
            SAGE_LOG("workspace too small: %zu < %zu", workspace_bytes, c.total);
            return MI355_SAGE_EWORKSPACE;
        }
        if (reinterpret_cast<uintptr_t>(ws) & (kAlign - 1)) return MI355_SAGE_EUNSUPPORTED;
    } else {
        void* p = nullptr;
        if ((rc = internal_workspace(c.total, &p))) return rc;
        ws = static_cast<uint8_t*>(p);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    int8_t* q8 = reinterpret_cast<int8_t*>(ws + c.q8);
    int8_t* k8 = reinterpret_cast<int8_t*>(ws + c.k8);
    void* vq = ws + c.vq;
    float* qscale = reinterpret_cast<float*>(ws + c.qscale);
    float* kscale = reinterpret_cast<float*>(ws + c.kscale);
    float* kmean = reinterpret_cast<float*>(ws + c.kmean);
    float* vscale = reinterpret_cast<float*>(ws + c.vscale);
    double* partial = reinterpret_cast<double*>(ws + c.partial);
    float* qshift = Stats ? reinterpret_cast<float*>(ws + c.qshift) : nullptr;

    const View q = make_view(Q, qs, q_off), k = make_view(K, ks, k_off), v = make_view(V, vs, v_off);
    const int64_t nkp = pad_to(kv, kPadKV);
    if (variant == MI355_SAGE_PV_FP16 && !Stats) {
        // two launches: {Q quantize, V repack, K-mean group sums} then {K mean + K quantize}
        const float cmul = (float)((double)scale * 1.4426950408889634074);   // scale*log2(e), rounded once
        SAGE_HIP(launch_prep_fused(q, k, v, B, H, N_q, kv, D, pad_to(N_q, kTileQ), nkp, cmul, blkq, smooth_k != 0,
                                   q8, qscale, static_cast<uint16_t*>(vq), partial, pre.q, pre.k, st));
        SAGE_HIP(launch_kquant_fused(k, B, H, kv, D, nkp, blkk, smooth_k ? partial : nullptr, kmean, k8, kscale,
                                     pre.k, st));
    } else {
        // Stats needs <q, kmean> per row, i.e. the mean before the Q quantizer; the e4m3 V path
        // has its own three launches
        if ((rc = quant_qk(q, k, B, H, N_q, kv, D, scale, blkq, blkk, smooth_k, q8, qscale, k8, kscale,
                           kmean, partial, qshift, pre, st)))
            return rc;
        if (variant == MI355_SAGE_PV_FP16)
            SAGE_HIP(launch_quant_v_f16(v, B, H, kv, D, nkp, static_cast<uint16_t*>(vq), st));
        else
            SAGE_HIP(launch_quant_v_fp8(v, B, H, kv, D, nkp, static_cast<uint8_t*>(vq), vscale, st));
    }

    AttnArgs a{};
    a.q8 = q8; a.qscale = qscale; a.blkq = blkq;
    a.k8 = k8; a.kscale = kscale; a.blkk = blkk;
    a.vq = vq; a.vscale = vscale; a.qshift = smooth_k ? qshift : nullptr;
    a.variant = variant;
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = kv; a.kv_valid = kv; a.D = D;
    a.nq_pad = pad_to(N_q, kTileQ); a.nkv_pad = nkp;
    a.o = static_cast<uint16_t*>(O) + o_off; a.osb = os[0]; a.osh = os[1]; a.osn = os[2];
    a.stats = Stats ? static_cast<float*>(Stats) + stats_off : nullptr;
    SAGE_HIP(launch_attn(a, st));
    return MI355_SAGE_OK;
}

}  // namespace

extern "C" {

const char* mi355_sage_version(void) { return "mi355_sage 0.1 gfx950"; }

int64_t mi355_sage_pad_q(int64_t n) { return pad_to(n, kTileQ); }
int64_t mi355_sage_pad_kv(int64_t n) { return pad_to(n, kPadKV); }

int mi355_sage_v_slot(int key_in_tile, int variant) {
    if (key_in_tile < 0 || key_in_tile >= kTileKV) return -1;
    return variant == MI355_SAGE_PV_FP16 ? v_slot_f16(key_in_tile) : v_slot_fp8(key_in_tile);
}

size_t mi355_sage_workspace_bytes(int B, int H, int N_q, int N_kv, int D, int variant) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || !dims_ok(D)) return 0;
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return 0;
    return carve(B, H, N_q, N_kv, D, variant).total;
}

size_t mi355_sage_quant_scratch_bytes(int B, int H, int N_kv, int D) {
    if (B <= 0 || H <= 0 || N_kv <= 0 || D <= 0) return 0;
    return align_up((size_t)B * H * ((N_kv + kGroup - 1) / kGroup) * D * sizeof(double));
}

int mi355_sage_sdpa_bf16(const void* Q, const void* K, const void* V, void* O,
                         int B, int H, int N_q, int N_kv, int D, float scale,
                         const int64_t* q_strides, const int64_t* k_strides,
                         const int64_t* v_strides, const int64_t* o_strides,
                         int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                         int causal, void* stream,
                         int variant, void* workspace, size_t workspace_bytes) {
    const int blkq = variant == MI355_SAGE_PV_FP8 ? 32 : 128;
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, blkq, 64, 1,
                     workspace, workspace_bytes);
}

int mi355_sage_sdpa_bf16_ex(const void* Q, const void* K, const void* V, void* O,
                            int B, int H, int N_q, int N_kv, int D, float scale,
                            const int64_t* q_strides, const int64_t* k_strides,
                            const int64_t* v_strides, const int64_t* o_strides,
                            int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                            int causal, void* stream,
                            int variant, int blkq, int blkk, int smooth_k,
                            void* workspace, size_t workspace_bytes) {
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, blkq, blkk,
                     smooth_k ? 1 : 0, workspace, workspace_bytes);
}

int mi355_sage_sdpa_bf16_train_fwd(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                   int B, int H, int N_q, int N_kv, int D, float scale,
                                   const int64_t* q_strides, const int64_t* k_strides,
                                   const int64_t* v_strides, const int64_t* o_strides,
                                   int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                   int64_t stats_off, int causal, int real_N_q, int real_N_kv,
                                   void* stream, int variant, void* workspace, size_t workspace_bytes) {
    if (!Stats) return MI355_SAGE_EINVAL;              // cudnn_sdpa.cpp:485
    (void)real_N_q;                                    // padded query rows are computed and ignored
    const int blkq = variant == MI355_SAGE_PV_FP8 ? 32 : 128;
    return sdpa_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, stats_off, causal, real_N_kv, stream, variant,
                     blkq, 64, 1, workspace, workspace_bytes);
}

int mi355_sage_quant_qk_bf16(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                             float scale, const int64_t* q_strides, const int64_t* k_strides,
                             int64_t q_off, int64_t k_off, int blkq, int blkk, int smooth_k,
                             void* q8, void* qscale, void* k8, void* kscale, void* kmean,
                             void* scratch, size_t scratch_bytes, void* stream) {
    if (!Q || !K || !q8 || !qscale || !k8 || !kscale) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!q_strides || !k_strides) return MI355_SAGE_EINVAL;
    if (smooth_k && (!kmean || !scratch)) return MI355_SAGE_EINVAL;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk)) return MI355_SAGE_EUNSUPPORTED;
    if (smooth_k && scratch_bytes < mi355_sage_quant_scratch_bytes(B, H, N_kv, D)) return MI355_SAGE_EWORKSPACE;
    int rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("K", K, k_strides, k_off))) return rc;
    return quant_qk(make_view(Q, q_strides, q_off), make_view(K, k_strides, k_off), B, H, N_q, N_kv, D,
                    scale, blkq, blkk, smooth_k, static_cast<int8_t*>(q8), static_cast<float*>(qscale),
                    static_cast<int8_t*>(k8), static_cast<float*>(kscale), static_cast<float*>(kmean),
                    static_cast<double*>(scratch), nullptr, Pre{}, static_cast<hipStream_t>(stream));
}

int mi355_sage_quant_qk_norm_rope_bf16(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                                       float scale, const int64_t* q_strides, const int64_t* k_strides,
                                       int64_t q_off, int64_t k_off,
                                       const void* q_gain, const void* k_gain, float eps,
                                       const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows,
                                       int blkq, int blkk, int smooth_k,
                                       void* q8, void* qscale, void* k8, void* kscale, void* kmean,
                                       void* scratch, size_t scratch_bytes, void* stream) {
    if (!Q || !K || !q8 || !qscale || !k8 || !kscale) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!q_strides || !k_strides) return MI355_SAGE_EINVAL;
    if (smooth_k && (!kmean || !scratch)) return MI355_SAGE_EINVAL;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk)) return MI355_SAGE_EUNSUPPORTED;
    if (smooth_k && scratch_bytes < mi355_sage_quant_scratch_bytes(B, H, N_kv, D)) return MI355_SAGE_EWORKSPACE;
    int rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("K", K, k_strides, k_off))) return rc;
    Pre pre;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    return quant_qk(make_view(Q, q_strides, q_off), make_view(K, k_strides, k_off), B, H, N_q, N_kv, D,
                    scale, blkq, blkk, smooth_k, static_cast<int8_t*>(q8), static_cast<float*>(qscale),
                    static_cast<int8_t*>(k8), static_cast<float*>(kscale), static_cast<float*>(kmean),
                    static_cast<double*>(scratch), nullptr, pre, static_cast<hipStream_t>(stream));
}

int mi355_sage_sdpa_bf16_norm_rope(const void* Q, const void* K, const void* V, void* O,
                                   int B, int H, int N_q, int N_kv, int D, float scale,
                                   const int64_t* q_strides, const int64_t* k_strides,
                                   const int64_t* v_strides, const int64_t* o_strides,
                                   int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                   int causal, void* stream,
                                   int variant, int blkq, int blkk, int smooth_k,
                                   const void* q_gain, const void* k_gain, float eps,
                                   const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows,
                                   void* workspace, size_t workspace_bytes) {
    Pre pre;
    int rc;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, blkq, blkk,
                     smooth_k ? 1 : 0, workspace, workspace_bytes, pre);
}

int mi355_sage_sdpa_bf16_norm_rope_train_fwd(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                             int B, int H, int N_q, int N_kv, int D, float scale,
                                             const int64_t* q_strides, const int64_t* k_strides,
                                             const int64_t* v_strides, const int64_t* o_strides,
                                             int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                             int64_t stats_off, int causal, int real_N_q, int real_N_kv,
                                             void* stream, int variant,
                                             const void* q_gain, const void* k_gain, float eps,
                                             const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows,
                                             void* workspace, size_t workspace_bytes) {
    if (!Stats) return MI355_SAGE_EINVAL;
    (void)real_N_q;
    Pre pre;
    int rc;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    const int blkq = variant == MI355_SAGE_PV_FP8 ? 32 : 128;
    return sdpa_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, stats_off, causal, real_N_kv, stream, variant,
                     blkq, 64, 1, workspace, workspace_bytes, pre);
}

int mi355_sage_quant_v_f16(const void* V, int B, int H, int N_kv, int D, const int64_t* v_strides,
                           int64_t v_off, void* v16, void* stream) {
    if (!V || !v16 || !v_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!dims_ok(D)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_view("V", V, v_strides, v_off))) return rc;
    SAGE_HIP(launch_quant_v_f16(make_view(V, v_strides, v_off), B, H, N_kv, D, pad_to(N_kv, kPadKV),
                                static_cast<uint16_t*>(v16), static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

int mi355_sage_quant_v_fp8(const void* V, int B, int H, int N_kv, int D, const int64_t* v_strides,
                           int64_t v_off, void* v8, void* vscale, void* stream) {
    if (!V || !v8 || !vscale || !v_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!dims_ok(D)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_view("V", V, v_strides, v_off))) return rc;
    SAGE_HIP(launch_quant_v_fp8(make_view(V, v_strides, v_off), B, H, N_kv, D, pad_to(N_kv, kPadKV),
                                static_cast<uint8_t*>(v8), static_cast<float*>(vscale),
                                static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

int mi355_sage_attn_fwd(const void* q8, const void* qscale, int blkq, const void* k8, const void* kscale,
                        int blkk, const void* vq, const void* vscale, int variant, int B, int H, int N_q,
                        int N_kv, int kv_valid, int D, void* O, const int64_t* o_strides, int64_t o_off,
                        void* stats, void* stream) {
    if (!q8 || !qscale || !k8 || !kscale || !vq || !O || !o_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (kv_valid <= 0 || kv_valid > N_kv) return MI355_SAGE_EINVAL;
    if (variant == MI355_SAGE_PV_FP8 && !vscale) return MI355_SAGE_EINVAL;
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_kv_len(N_kv, blkk))) return rc;
    if ((rc = check_view("O", O, o_strides, o_off))) return rc;
    AttnArgs a{};
    a.q8 = static_cast<const int8_t*>(q8); a.qscale = static_cast<const float*>(qscale); a.blkq = blkq;
    a.k8 = static_cast<const int8_t*>(k8); a.kscale = static_cast<const float*>(kscale); a.blkk = blkk;
    a.vq = vq; a.vscale = static_cast<const float*>(vscale); a.qshift = nullptr;
    a.variant = variant;
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = N_kv; a.kv_valid = kv_valid; a.D = D;
    a.nq_pad = pad_to(N_q, kTileQ); a.nkv_pad = pad_to(N_kv, kPadKV);
    a.o = static_cast<uint16_t*>(O) + o_off; a.osb = o_strides[0]; a.osh = o_strides[1]; a.osn = o_strides[2];
    a.stats = static_cast<float*>(stats);
    SAGE_HIP(launch_attn(a, static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

}  // extern "C"
