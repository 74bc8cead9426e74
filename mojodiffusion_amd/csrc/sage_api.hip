// sage_api.hip — the C ABI of libmi355_sage.so (declared in include/mi355_sage.h).
// Host-side only: argument checks, workspace carving, kernel sequencing.
#include "../../include/mi355_sage.h"
#include "../../include/mi355_sage_test.h"
#include "sage_internal.h"

#include <cstdio>
#include <mutex>
#include <vector>

using namespace sage;

// Scratch of mi355_sage_sdpa_bf16_static: device memory that belongs to the loaded library, so
// that entry point never allocates.  Each GPU the library runs on holds its own copy of the
// array, at its own address, until the process ends.  In host code the array's NAME is only a
// handle for hipGetSymbolAddress; the address that call returns is what kernels are given.
constexpr size_t kStaticScratchBytes = 16u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

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

// Forward: 64, 128 and (four-wave workgroups, no fused pre-ops) 256 channels per head; backward: 64, 128.
bool dims_ok(int D) { return D == 64 || D == 128 || D == 256; }
bool bwd_dims_ok(int D) { return D == 64 || D == 128; }

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
int check_kv_len(int N_kv, int blkk, int D) {
    (void)blkk;
    if (pad_to(N_kv, kPadKV) > max_keys(D)) {
        SAGE_LOG("N_kv=%d exceeds the %d keys per head the attention kernel takes", N_kv, max_keys(D));
        return MI355_SAGE_EUNSUPPORTED;
    }
    return 0;
}

// Workspace layout of the one-shot calls.
struct Carve {
    size_t q8, k8, vq, qscale, kscale, kmean, qmul, kmul, vscale, kpart_sum, kpart_mm, vpart, qshift, rowinv_q, rowinv_k, split, total;
};

Carve carve(int B, int H, int Nq, int Nkv, int D, int variant) {
    const size_t bh = (size_t)B * H;
    const size_t nqp = (size_t)pad_to(Nq, kTileQ), nkp = (size_t)pad_to(Nkv, kPadKV);
    const size_t ng = (size_t)((Nkv + kGroup - 1) / kGroup);
    Carve c{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
    c.q8 = take(bh * nqp * D);
    c.k8 = take(bh * nkp * D);
    c.vq = take(bh * nkp * D * (variant == MI355_SAGE_PV_FP16 ? 2 : 1));
    c.qscale = take(bh * (nqp / 32) * sizeof(float));      // smallest block is 32 tokens
    c.kscale = take(bh * (nkp / 32) * sizeof(float));
    c.kmean = take(bh * D * sizeof(float));
    c.qmul = take(bh * D * sizeof(float));
    c.kmul = take(bh * D * sizeof(float));
    c.vscale = take(bh * D * sizeof(float));
    c.kpart_sum = take(bh * ng * D * sizeof(double));
    c.kpart_mm = take(bh * ng * D * 2 * sizeof(float));
    c.vpart = take(variant == MI355_SAGE_PV_FP16 ? 0 : bh * ng * D * sizeof(float));
    c.qshift = take(bh * nqp * sizeof(float));
    c.rowinv_q = take((size_t)B * Nq * sizeof(float));        // whole-row RMSNorm statistic per token (optional pre-op)
    c.rowinv_k = take((size_t)B * Nkv * sizeof(float));
    // hand-over slots of the attention kernel's split scheduling, for the shapes that qualify
    c.split = take(attn_split_bytes(attn_split_rule(B, H, Nq, Nkv, D, variant), D));
    c.total = off;
    return c;
}

// Scratch of the stage quantizers: K group sums and minima / maxima, V group maxima.
struct ScratchCarve {
    size_t kpart_sum, kpart_mm, vpart, rowinv_q, rowinv_k, total;
};
ScratchCarve scratch_carve(int B, int H, int Nkv, int D) {
    const size_t n = (size_t)B * H * ((Nkv + kGroup - 1) / kGroup) * D;
    ScratchCarve c{};
    c.kpart_sum = 0;
    c.kpart_mm = align_up(n * sizeof(double));
    c.vpart = c.kpart_mm + align_up(n * 2 * sizeof(float));
    // whole-row RMSNorm statistics (that pre-op needs N_q == N_kv)
    c.rowinv_q = c.vpart + align_up(n * sizeof(float));
    c.rowinv_k = c.rowinv_q + align_up((size_t)B * Nkv * sizeof(float));
    c.total = c.rowinv_k + align_up((size_t)B * Nkv * sizeof(float));
    return c;
}

// Internal workspaces (workspace == NULL): one buffer per (device, stream), so calls on
// different streams never share one.  A buffer that has become too small is replaced by a
// larger one and kept allocated until the process ends: work queued earlier may still be
// using it, and waiting for that work would make the call synchronise.  Sizes at least double,
// so the retired buffers of a stream add up to less than its current one.  Allocation is not
// possible while the stream is being captured into a graph: such a call fails with
// MI355_SAGE_EWORKSPACE unless the buffer is already large enough.
std::mutex g_ws_mutex;
struct StreamWs { int dev; hipStream_t stream; void* p; size_t bytes; };
std::vector<StreamWs> g_ws;          // one-shot calls
std::vector<StreamWs> g_split_ws;    // hand-over slots of mi355_sage_attn_fwd, which takes no workspace

int internal_workspace(std::vector<StreamWs>& registry, size_t need, hipStream_t stream, void** out) {
    int dev = 0;
    SAGE_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    StreamWs* w = nullptr;
    for (auto& e : registry)
        if (e.dev == dev && e.stream == stream) { w = &e; break; }
    if (w == nullptr || w->bytes < need) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            SAGE_LOG("the internal workspace would have to grow to %zu bytes while the stream is being captured; "
                     "pass a workspace or run the call once before capturing", need);
            return MI355_SAGE_EWORKSPACE;
        }
        const size_t bytes = w ? (need > 2 * w->bytes ? need : 2 * w->bytes) : need;
        void* p = nullptr;
        SAGE_HIP(hipMalloc(&p, bytes));
        if (w == nullptr) {
            registry.push_back(StreamWs{dev, stream, p, bytes});
            w = &registry.back();
        } else {
            w->p = p;              // the old buffer stays allocated (see above)
            w->bytes = bytes;
        }
    }
    *out = w->p;
    return 0;
}

// The optional ops in front of the quantizers (RMSNorm + interleaved RoPE of Q and of K).
struct Pre {
    PreOp q{}, k{};
    bool full_row = false;      // RMSNorm over all H*D channels of a token (gains of H*D entries)
};

// q_gain / k_gain null together = nothing to do.  Tables are optional on top of the gains.
int make_pre(const void* q_gain, const void* k_gain, float eps, const void* rope_cos, const void* rope_sin,
             int64_t rope_batch_rows, int rope_layout, Pre* out) {
    *out = Pre{};
    if (!q_gain && !k_gain && !rope_cos && !rope_sin) return 0;
    if (!q_gain || !k_gain) { SAGE_LOG("RMSNorm gains must be given for both Q and K"); return MI355_SAGE_EINVAL; }
    if ((rope_cos == nullptr) != (rope_sin == nullptr)) return MI355_SAGE_EINVAL;
    if (!(eps >= 0.0f) || rope_batch_rows < 0) return MI355_SAGE_EINVAL;
    if (rope_layout & ~(MI355_SAGE_ROPE_HALFSPLIT | MI355_SAGE_ROPE_TABLES_BF16 | MI355_SAGE_NORM_FULL_ROW)) return MI355_SAGE_EINVAL;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q_gain) | reinterpret_cast<uintptr_t>(k_gain) |
                           reinterpret_cast<uintptr_t>(rope_cos) | reinterpret_cast<uintptr_t>(rope_sin);
    if (bits & 15) { SAGE_LOG("gains and RoPE tables must be 16-byte aligned"); return MI355_SAGE_EUNSUPPORTED; }
    out->q = PreOp{static_cast<const uint16_t*>(q_gain), eps, static_cast<const float*>(rope_cos),
                   static_cast<const float*>(rope_sin), rope_batch_rows, (rope_layout & MI355_SAGE_ROPE_HALFSPLIT) ? 1 : 0,
                   (rope_layout & MI355_SAGE_ROPE_TABLES_BF16) ? 1 : 0, nullptr, 0};
    out->full_row = (rope_layout & MI355_SAGE_NORM_FULL_ROW) != 0;
    out->k = out->q;
    out->k.gain = static_cast<const uint16_t*>(k_gain);
    return 0;
}

// Device address of `scratch` on the current device, looked up once per device.
std::mutex g_static_mutex;
void* g_static_ptr[64] = {};

int static_scratch(void** out) {
    int dev = 0;
    SAGE_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return MI355_SAGE_EUNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_static_ptr[dev] == nullptr) {
        void* p = nullptr;
        SAGE_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & (kAlign - 1))) return MI355_SAGE_EUNSUPPORTED;
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return 0;
}

float cmul_of(float scale) { return (float)((double)scale * 1.4426950408889634074); }   // scale*log2(e), rounded once

// Clips the masked key range to [0, n) and counts the keys that remain.
int clip_mask(int n, int mask_lo, int mask_hi, KeyMask* km) {
    int lo = mask_lo < 0 ? 0 : mask_lo, hi = mask_hi > n ? n : mask_hi;
    if (hi <= lo) lo = hi = 0;
    *km = KeyMask{lo, hi};
    return n - (hi - lo);
}

struct QuantOut {
    int8_t* q8; float* qscale; int8_t* k8; float* kscale;
    float *kmean, *qmul, *kmul;
    double* kpart_sum; float* kpart_mm;
    float* rowdot;
    float *rowinv_q, *rowinv_k;       // whole-row RMSNorm statistics (only with that pre-op)
};

// K statistics + Q / K encoders (+ the V passes when vq is given): launches 1-3.
int quantize(const View& q, const View& k, const View* v, int B, int H, int Nq, int Nkv, int D, float scale,
             int blkq, int blkk, int k_flags, const KeyMask& km, int kept, const QuantOut& o,
             int variant, void* vq, float* vscale, float* vpart, const Pre& pre_in, hipStream_t st) {
    Pre pre = pre_in;
    if (pre.full_row) {
        SAGE_HIP(launch_row_inv(q, k, B, H, Nq, Nkv, D, pre.q.eps, o.rowinv_q, o.rowinv_k, st));
        pre.q.row_inv = o.rowinv_q; pre.q.row_n = Nq;
        pre.k.row_inv = o.rowinv_k; pre.k.row_n = Nkv;
    }
    const float cmul = cmul_of(scale);
    const int64_t nqp = pad_to(Nq, kTileQ), nkp = pad_to(Nkv, kPadKV);
    const bool kstats = (k_flags & 3) != 0;
    PrepArgs p{};
    p.k = k; p.H = H; p.Nkv = Nkv; p.nkv_pad = nkp; p.km = km; p.pre_k = pre.k;
    p.vmode = 2;
    if (v != nullptr && variant != MI355_SAGE_PV_FP16) {
        p.v = *v;
        p.vmode = 1;                       // (the fp16 repack needs no statistics: it goes with launch 3)
        p.vpart = vpart;
    }
    p.kpart_sum = kstats ? o.kpart_sum : nullptr;
    p.kpart_mm = o.kpart_mm;
    SAGE_HIP(launch_prep(p, B, D, st));

    FinalArgs f{};
    f.total = (int64_t)B * H * D; f.D = D; f.ngroups = (Nkv + kGroup - 1) / kGroup; f.kept = kept;
    f.flags = k_flags; f.cmul = cmul;
    f.kpart_sum = p.kpart_sum; f.kpart_mm = o.kpart_mm;
    f.kmean = o.kmean; f.qmul = o.qmul; f.kmul = o.kmul;
    f.vpart = vpart; f.vscale = p.vmode == 1 ? vscale : nullptr;
    SAGE_HIP(launch_stats_final(f, st));

    QuantArgs a{};
    a.q = q; a.k = k; a.H = H; a.Nq = Nq; a.Nkv = Nkv; a.nq_pad = nqp; a.nkv_pad = nkp; a.km = km;
    a.blkq = blkq; a.blkk = blkk; a.cmul = cmul;
    a.kmean = o.kmean; a.qmul = o.qmul; a.kmul = o.kmul; a.vscale = vscale;
    a.q8 = o.q8; a.qscale = o.qscale; a.rowdot = o.rowdot; a.k8 = o.k8; a.kscale = o.kscale;
    if (p.vmode == 1) { a.v = *v; a.v8 = static_cast<uint8_t*>(vq); }
    else if (v != nullptr) { a.v = *v; a.v16 = static_cast<uint16_t*>(vq); }
    a.pre_q = pre.q; a.pre_k = pre.k;
    SAGE_HIP(launch_quant(a, B, D, st));
    return 0;
}

struct MaskArgs {
    int lo = 0, hi = 0;                // keys lo <= s < hi are masked
    const void* add = nullptr;         // additive bias, bf16, logical [B,H,N_q,N_kv]
    const int64_t* add_strides = nullptr;
    int64_t add_off = 0;
};

int sdpa_impl(const void* Q, const void* K, const void* V, void* O, void* Stats,
              int B, int H, int N_q, int N_kv, int D, float scale,
              const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
              int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t stats_off,
              int causal, int real_N_kv, void* stream,
              int variant, int blkq, int blkk, int k_flags, void* workspace, size_t workspace_bytes,
              const Pre& pre = Pre{}, const MaskArgs& mask = MaskArgs{}) {
    // argument checks in the order of serenitymojo/ops/cshim/cudnn_sdpa.cpp:391-393
    if (!Q || !K || !V || !O) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!qs || !ks || !vs || !os) return MI355_SAGE_EINVAL;
    if (!dims_ok(D)) { SAGE_LOG("head dim %d not supported (64, 128 or 256)", D); return MI355_SAGE_EUNSUPPORTED; }
    if (D == 256 && pre.q.gain != nullptr) { SAGE_LOG("the fused RMSNorm / RoPE are built for head dims 64 and 128"); return MI355_SAGE_EUNSUPPORTED; }
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (!blk_ok(blkq) || !blk_ok(blkk)) { SAGE_LOG("block sizes must be 32, 64 or 128"); return MI355_SAGE_EUNSUPPORTED; }
    if (k_flags & ~3) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_kv_len(N_kv, blkk, D))) return rc;
    if ((rc = check_view("Q", Q, qs, q_off)) || (rc = check_view("K", K, ks, k_off)) ||
        (rc = check_view("V", V, vs, v_off)) || (rc = check_view("O", O, os, o_off)))
        return rc;
    if (pre.q.gain != nullptr && (pre.q.cos != nullptr || pre.full_row) && N_q != N_kv) {
        SAGE_LOG("fused RoPE / whole-row RMSNorm are self-attention pre-ops: N_q must equal N_kv");
        return MI355_SAGE_EUNSUPPORTED;
    }
    if (mask.add != nullptr) {
        const int64_t* ms = mask.add_strides;
        if (!ms) return MI355_SAGE_EINVAL;
        const uintptr_t a = reinterpret_cast<uintptr_t>(mask.add) + (uintptr_t)(mask.add_off * 2);
        if (ms[3] != 1 || (a & 7) || (ms[0] & 3) || (ms[1] & 3) || (ms[2] & 3)) {
            SAGE_LOG("mask: key stride must be 1 and every row 8-byte aligned");
            return MI355_SAGE_EUNSUPPORTED;
        }
    }
    // Keys past the real length are excluded from the statistics and the scores alike:
    // the quantizers see only the first kv tokens.
    const int kv = (real_N_kv > 0 && real_N_kv < N_kv) ? real_N_kv : N_kv;
    KeyMask km;
    const int kept = clip_mask(kv, mask.lo, mask.hi, &km);
    if (kept <= 0) { SAGE_LOG("every key is masked"); return MI355_SAGE_EINVAL; }

    hipStream_t st = static_cast<hipStream_t>(stream);
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
        if ((rc = internal_workspace(g_ws, c.total, st, &p))) return rc;
        ws = static_cast<uint8_t*>(p);
    }
    // (one decision for carving and launching; slots the caller's workspace was not sized for — a
    // forced schedule of the test switch — come from the library's per-stream buffer)
    const int split_wgs = causal ? 0 : attn_split_workgroups(B, H, N_q, kv, D, variant);
    // The plain forward leaves Q to the attention kernel, which encodes its own rows (same codes and
    // scales): the quantize stage then neither reads Q nor writes its codes.
    const bool q_in_kernel = Stats == nullptr && mask.add == nullptr && pre.q.gain == nullptr && D <= 128 && split_wgs == 0;
    QuantOut o{};
    o.q8 = q_in_kernel ? nullptr : reinterpret_cast<int8_t*>(ws + c.q8);
    o.k8 = reinterpret_cast<int8_t*>(ws + c.k8);
    o.qscale = reinterpret_cast<float*>(ws + c.qscale);
    o.kscale = reinterpret_cast<float*>(ws + c.kscale);
    o.kmean = reinterpret_cast<float*>(ws + c.kmean);
    o.qmul = reinterpret_cast<float*>(ws + c.qmul);
    o.kmul = reinterpret_cast<float*>(ws + c.kmul);
    o.kpart_sum = reinterpret_cast<double*>(ws + c.kpart_sum);
    o.kpart_mm = reinterpret_cast<float*>(ws + c.kpart_mm);
    o.rowinv_q = reinterpret_cast<float*>(ws + c.rowinv_q);
    o.rowinv_k = reinterpret_cast<float*>(ws + c.rowinv_k);
    // Stats needs <q, kmean> per row: K smoothing lowers every score of a row by it
    float* qshift = (Stats && (k_flags & MI355_SAGE_K_SMOOTH)) ? reinterpret_cast<float*>(ws + c.qshift) : nullptr;
    o.rowdot = qshift;
    void* vq = ws + c.vq;
    float* vscale = reinterpret_cast<float*>(ws + c.vscale);
    float* vpart = reinterpret_cast<float*>(ws + c.vpart);

    const View q = make_view(Q, qs, q_off), k = make_view(K, ks, k_off), v = make_view(V, vs, v_off);
    if ((rc = quantize(q, k, &v, B, H, N_q, kv, D, scale, blkq, blkk, k_flags, km, kept, o, variant, vq, vscale,
                       vpart, pre, st)))
        return rc;

    AttnArgs a{};
    a.q8 = o.q8; a.qscale = o.qscale; a.blkq = blkq;
    a.k8 = o.k8; a.kscale = o.kscale; a.blkk = blkk;
    a.vq = vq; a.vscale = vscale; a.qshift = qshift;
    a.variant = variant;
    a.km = km;
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = kv; a.kv_valid = kv; a.D = D;
    a.causal = causal ? 1 : 0;
    a.nq_pad = pad_to(N_q, kTileQ); a.nkv_pad = pad_to(kv, kPadKV);
    a.o = static_cast<uint16_t*>(O) + o_off; a.osb = os[0]; a.osh = os[1]; a.osn = os[2];
    a.stats = Stats ? static_cast<float*>(Stats) + stats_off : nullptr;
    if (mask.add != nullptr) {
        a.amask = static_cast<const uint16_t*>(mask.add) + mask.add_off;
        a.amb = mask.add_strides[0]; a.amh = mask.add_strides[1]; a.amn = mask.add_strides[2];
    }
    if (q_in_kernel) {
        a.q_src = q.p; a.qsb = q.sb; a.qsh = q.sh; a.qsn = q.sn;
        a.qmul = o.qmul;
    }
    a.split_wgs = split_wgs;
    if (a.split_wgs > 0) {
        if (attn_split_bytes(a.split_wgs, D) <= attn_split_bytes(attn_split_rule(B, H, N_q, kv, D, variant), D)) a.split = ws + c.split;
        else if ((rc = internal_workspace(g_split_ws, attn_split_bytes(a.split_wgs, D), st, &a.split))) return rc;
    }
    SAGE_HIP(launch_attn(a, st));
    return MI355_SAGE_OK;
}

int default_blkq(int variant) { return variant == MI355_SAGE_PV_FP8 ? 32 : 128; }
constexpr int kDefaultFlags = MI355_SAGE_K_SMOOTH | MI355_SAGE_K_BALANCE;

}  // namespace

extern "C" {

const char* mi355_sage_version(void) { return "mi355_sage 0.2 gfx950"; }

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
    return scratch_carve(B, H, N_kv, D).total;
}

int mi355_sage_sdpa_bf16(const void* Q, const void* K, const void* V, void* O,
                         int B, int H, int N_q, int N_kv, int D, float scale,
                         const int64_t* q_strides, const int64_t* k_strides,
                         const int64_t* v_strides, const int64_t* o_strides,
                         int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                         int causal, void* stream,
                         int variant, void* workspace, size_t workspace_bytes) {
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, default_blkq(variant), 64,
                     kDefaultFlags, workspace, workspace_bytes);
}

int mi355_sage_sdpa_bf16_static(const void* Q, const void* K, const void* V, void* O,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides,
                                const int64_t* v_strides, const int64_t* o_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                int causal, void* stream, int variant) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!dims_ok(D) || (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8)) return MI355_SAGE_EUNSUPPORTED;
    const size_t need = carve(B, H, N_q, N_kv, D, variant).total;
    if (need > kStaticScratchBytes) {
        SAGE_LOG("mi355_sage_sdpa_bf16_static: this problem needs %zu bytes of scratch, the built-in buffer holds %zu; "
                 "use mi355_sage_sdpa_bf16 with a workspace", need, kStaticScratchBytes);
        return MI355_SAGE_EWORKSPACE;
    }
    // Nothing in the buffer has to start at zero: every byte a kernel of the path reads was
    // written by an earlier kernel of the same call (pad rows and pad blocks included).
    void* p = nullptr;
    int rc;
    if ((rc = static_scratch(&p))) return rc;
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, default_blkq(variant), 64,
                     kDefaultFlags, p, kStaticScratchBytes);
}

size_t mi355_sage_static_scratch_bytes(void) { return kStaticScratchBytes; }

int mi355_sage_sdpa_bf16_ex(const void* Q, const void* K, const void* V, void* O,
                            int B, int H, int N_q, int N_kv, int D, float scale,
                            const int64_t* q_strides, const int64_t* k_strides,
                            const int64_t* v_strides, const int64_t* o_strides,
                            int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                            int causal, void* stream,
                            int variant, int blkq, int blkk, int k_flags,
                            void* workspace, size_t workspace_bytes) {
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, blkq, blkk,
                     k_flags, workspace, workspace_bytes);
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
    return sdpa_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, stats_off, causal, real_N_kv, stream, variant,
                     default_blkq(variant), 64, kDefaultFlags, workspace, workspace_bytes);
}

int mi355_sage_sdpa_bf16_keymask(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                 int B, int H, int N_q, int N_kv, int D, float scale,
                                 const int64_t* q_strides, const int64_t* k_strides,
                                 const int64_t* v_strides, const int64_t* o_strides,
                                 int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                 int64_t stats_off, int mask_lo, int mask_hi,
                                 void* stream, int variant, void* workspace, size_t workspace_bytes) {
    if (mask_lo < 0 || mask_hi < mask_lo || mask_hi > N_kv) return MI355_SAGE_EINVAL;
    MaskArgs m;
    m.lo = mask_lo; m.hi = mask_hi;
    return sdpa_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, stats_off, 0, 0, stream, variant,
                     default_blkq(variant), 64, kDefaultFlags, workspace, workspace_bytes, Pre{}, m);
}

int mi355_sage_sdpa_bf16_mask(const void* Q, const void* K, const void* V, const void* Mask, void* O,
                              int B, int H, int N_q, int N_kv, int D, float scale,
                              const int64_t* q_strides, const int64_t* k_strides,
                              const int64_t* v_strides, const int64_t* mask_strides, const int64_t* o_strides,
                              int64_t q_off, int64_t k_off, int64_t v_off, int64_t mask_off, int64_t o_off,
                              void* stream, int variant, void* workspace, size_t workspace_bytes) {
    if (!Mask || !mask_strides) return MI355_SAGE_EINVAL;
    MaskArgs m;
    m.add = Mask; m.add_strides = mask_strides; m.add_off = mask_off;
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, 0, 0, stream, variant,
                     default_blkq(variant), 64, kDefaultFlags, workspace, workspace_bytes, Pre{}, m);
}

static int quant_qk_entry(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                          float scale, const int64_t* q_strides, const int64_t* k_strides,
                          int64_t q_off, int64_t k_off, const Pre& pre, int blkq, int blkk, int k_flags,
                          int mask_lo, int mask_hi,
                          void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
                          void* scratch, size_t scratch_bytes, void* stream) {
    if (!Q || !K || !q8 || !qscale || !k8 || !kscale || !kmean || !qmul || !kmul) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!q_strides || !k_strides) return MI355_SAGE_EINVAL;
    if ((k_flags & 3) && !scratch) return MI355_SAGE_EINVAL;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk) || (k_flags & ~3)) return MI355_SAGE_EUNSUPPORTED;
    if (D == 256 && pre.q.gain != nullptr) return MI355_SAGE_EUNSUPPORTED;
    const ScratchCarve sc = scratch_carve(B, H, N_kv, D);
    if ((k_flags & 3) && scratch_bytes < sc.total) return MI355_SAGE_EWORKSPACE;
    if (pre.q.gain != nullptr && (pre.q.cos != nullptr || pre.full_row) && N_q != N_kv) return MI355_SAGE_EUNSUPPORTED;
    if (pre.full_row && (!scratch || scratch_bytes < sc.total)) return MI355_SAGE_EWORKSPACE;
    int rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("K", K, k_strides, k_off))) return rc;
    KeyMask km;
    const int kept = clip_mask(N_kv, mask_lo, mask_hi, &km);
    if (kept <= 0) return MI355_SAGE_EINVAL;
    QuantOut o{};
    o.q8 = static_cast<int8_t*>(q8); o.qscale = static_cast<float*>(qscale);
    o.k8 = static_cast<int8_t*>(k8); o.kscale = static_cast<float*>(kscale);
    o.kmean = static_cast<float*>(kmean); o.qmul = static_cast<float*>(qmul); o.kmul = static_cast<float*>(kmul);
    o.kpart_sum = reinterpret_cast<double*>(static_cast<uint8_t*>(scratch) + sc.kpart_sum);
    o.kpart_mm = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + sc.kpart_mm);
    o.rowinv_q = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + sc.rowinv_q);
    o.rowinv_k = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + sc.rowinv_k);
    return quantize(make_view(Q, q_strides, q_off), make_view(K, k_strides, k_off), nullptr, B, H, N_q, N_kv, D,
                    scale, blkq, blkk, k_flags, km, kept, o, 0, nullptr, nullptr, nullptr, pre,
                    static_cast<hipStream_t>(stream));
}

int mi355_sage_quant_qk_bf16(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                             float scale, const int64_t* q_strides, const int64_t* k_strides,
                             int64_t q_off, int64_t k_off, int blkq, int blkk, int k_flags,
                             int mask_lo, int mask_hi,
                             void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
                             void* scratch, size_t scratch_bytes, void* stream) {
    return quant_qk_entry(Q, K, B, H, N_q, N_kv, D, scale, q_strides, k_strides, q_off, k_off, Pre{}, blkq, blkk,
                          k_flags, mask_lo, mask_hi, q8, qscale, k8, kscale, kmean, qmul, kmul, scratch,
                          scratch_bytes, stream);
}

int mi355_sage_quant_qk_norm_rope_bf16(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                                       float scale, const int64_t* q_strides, const int64_t* k_strides,
                                       int64_t q_off, int64_t k_off,
                                       const void* q_gain, const void* k_gain, float eps,
                                       const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
                                       int blkq, int blkk, int k_flags,
                                       void* q8, void* qscale, void* k8, void* kscale,
                                       void* kmean, void* qmul, void* kmul,
                                       void* scratch, size_t scratch_bytes, void* stream) {
    Pre pre;
    int rc;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, rope_layout, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    return quant_qk_entry(Q, K, B, H, N_q, N_kv, D, scale, q_strides, k_strides, q_off, k_off, pre, blkq, blkk,
                          k_flags, 0, 0, q8, qscale, k8, kscale, kmean, qmul, kmul, scratch, scratch_bytes, stream);
}

int mi355_sage_sdpa_bf16_norm_rope(const void* Q, const void* K, const void* V, void* O,
                                   int B, int H, int N_q, int N_kv, int D, float scale,
                                   const int64_t* q_strides, const int64_t* k_strides,
                                   const int64_t* v_strides, const int64_t* o_strides,
                                   int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                   int causal, void* stream,
                                   int variant, int blkq, int blkk, int k_flags,
                                   const void* q_gain, const void* k_gain, float eps,
                                   const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
                                   void* workspace, size_t workspace_bytes) {
    Pre pre;
    int rc;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, rope_layout, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    return sdpa_impl(Q, K, V, O, nullptr, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, 0, causal, 0, stream, variant, blkq, blkk,
                     k_flags, workspace, workspace_bytes, pre);
}

int mi355_sage_sdpa_bf16_norm_rope_train_fwd(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                             int B, int H, int N_q, int N_kv, int D, float scale,
                                             const int64_t* q_strides, const int64_t* k_strides,
                                             const int64_t* v_strides, const int64_t* o_strides,
                                             int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off,
                                             int64_t stats_off, int causal, int real_N_q, int real_N_kv,
                                             void* stream, int variant,
                                             const void* q_gain, const void* k_gain, float eps,
                                             const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
                                             void* workspace, size_t workspace_bytes) {
    if (!Stats) return MI355_SAGE_EINVAL;
    (void)real_N_q;
    Pre pre;
    int rc;
    if ((rc = make_pre(q_gain, k_gain, eps, rope_cos, rope_sin, rope_batch_rows, rope_layout, &pre))) return rc;
    if (!pre.q.gain) return MI355_SAGE_EINVAL;
    return sdpa_impl(Q, K, V, O, Stats, B, H, N_q, N_kv, D, scale, q_strides, k_strides, v_strides,
                     o_strides, q_off, k_off, v_off, o_off, stats_off, causal, real_N_kv, stream, variant,
                     default_blkq(variant), 64, kDefaultFlags, workspace, workspace_bytes, pre);
}

int mi355_sage_quant_qkv_bf16(const void* Q, const void* K, const void* V, int B, int H, int N_q, int N_kv, int D,
                              float scale, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                              int64_t q_off, int64_t k_off, int64_t v_off,
                              int variant, int blkq, int blkk, int k_flags, int mask_lo, int mask_hi,
                              void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
                              void* vq, void* vscale, void* scratch, size_t scratch_bytes, void* stream) {
    if (!Q || !K || !V || !k8 || !kscale || !kmean || !qmul || !kmul || !vq || !scratch) return MI355_SAGE_EINVAL;
    if ((q8 == nullptr) != (qscale == nullptr)) return MI355_SAGE_EINVAL;      // both NULL: Q is left to mi355_sage_attn_fwd_q16
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!q_strides || !k_strides || !v_strides) return MI355_SAGE_EINVAL;
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (variant == MI355_SAGE_PV_FP8 && !vscale) return MI355_SAGE_EINVAL;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk) || (k_flags & ~3)) return MI355_SAGE_EUNSUPPORTED;
    const ScratchCarve sc = scratch_carve(B, H, N_kv, D);
    if (scratch_bytes < sc.total) return MI355_SAGE_EWORKSPACE;
    int rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("K", K, k_strides, k_off)) ||
        (rc = check_view("V", V, v_strides, v_off)))
        return rc;
    KeyMask km;
    const int kept = clip_mask(N_kv, mask_lo, mask_hi, &km);
    if (kept <= 0) return MI355_SAGE_EINVAL;
    uint8_t* scr = static_cast<uint8_t*>(scratch);
    QuantOut o{};
    o.q8 = static_cast<int8_t*>(q8); o.qscale = static_cast<float*>(qscale);
    o.k8 = static_cast<int8_t*>(k8); o.kscale = static_cast<float*>(kscale);
    o.kmean = static_cast<float*>(kmean); o.qmul = static_cast<float*>(qmul); o.kmul = static_cast<float*>(kmul);
    o.kpart_sum = reinterpret_cast<double*>(scr + sc.kpart_sum);
    o.kpart_mm = reinterpret_cast<float*>(scr + sc.kpart_mm);
    o.rowinv_q = reinterpret_cast<float*>(scr + sc.rowinv_q);
    o.rowinv_k = reinterpret_cast<float*>(scr + sc.rowinv_k);
    const View v = make_view(V, v_strides, v_off);
    return quantize(make_view(Q, q_strides, q_off), make_view(K, k_strides, k_off), &v, B, H, N_q, N_kv, D, scale,
                    blkq, blkk, k_flags, km, kept, o, variant, vq, static_cast<float*>(vscale),
                    reinterpret_cast<float*>(scr + sc.vpart), Pre{}, static_cast<hipStream_t>(stream));
}

int mi355_sage_quant_v_f16(const void* V, int B, int H, int N_kv, int D, const int64_t* v_strides,
                           int64_t v_off, int mask_lo, int mask_hi, void* v16, void* stream) {
    if (!V || !v16 || !v_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!dims_ok(D)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_view("V", V, v_strides, v_off))) return rc;
    PrepArgs p{};
    p.v = make_view(V, v_strides, v_off); p.H = H; p.Nkv = N_kv; p.nkv_pad = pad_to(N_kv, kPadKV);
    clip_mask(N_kv, mask_lo, mask_hi, &p.km);
    p.vmode = 0; p.v16 = static_cast<uint16_t*>(v16);
    SAGE_HIP(launch_prep(p, B, D, static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

int mi355_sage_quant_v_fp8(const void* V, int B, int H, int N_kv, int D, const int64_t* v_strides,
                           int64_t v_off, int mask_lo, int mask_hi, void* v8, void* vscale,
                           void* scratch, size_t scratch_bytes, void* stream) {
    if (!V || !v8 || !vscale || !v_strides || !scratch) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!dims_ok(D)) return MI355_SAGE_EUNSUPPORTED;
    const ScratchCarve sc = scratch_carve(B, H, N_kv, D);
    if (scratch_bytes < sc.total) return MI355_SAGE_EWORKSPACE;
    int rc;
    if ((rc = check_view("V", V, v_strides, v_off))) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    PrepArgs p{};
    p.v = make_view(V, v_strides, v_off); p.H = H; p.Nkv = N_kv; p.nkv_pad = pad_to(N_kv, kPadKV);
    if (clip_mask(N_kv, mask_lo, mask_hi, &p.km) <= 0) return MI355_SAGE_EINVAL;
    p.vmode = 1; p.vpart = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + sc.vpart);
    SAGE_HIP(launch_prep(p, B, D, st));
    FinalArgs f{};
    f.total = (int64_t)B * H * D; f.D = D; f.ngroups = (N_kv + kGroup - 1) / kGroup;
    f.vpart = p.vpart; f.vscale = static_cast<float*>(vscale);
    SAGE_HIP(launch_stats_final(f, st));
    QuantArgs a{};
    a.v = p.v; a.H = H; a.Nkv = N_kv; a.nkv_pad = p.nkv_pad; a.km = p.km; a.blkq = 32; a.blkk = 32;
    a.vscale = f.vscale; a.v8 = static_cast<uint8_t*>(v8);
    SAGE_HIP(launch_quant(a, B, D, st));
    return MI355_SAGE_OK;
}

int mi355_sage_attn_fwd(const void* q8, const void* qscale, int blkq, const void* k8, const void* kscale,
                        int blkk, const void* vq, const void* vscale, int variant, int B, int H, int N_q,
                        int N_kv, int kv_valid, int mask_lo, int mask_hi, int D,
                        void* O, const int64_t* o_strides, int64_t o_off,
                        const void* qshift, void* stats, void* stream) {
    if (!q8 || !qscale || !k8 || !kscale || !vq || !O || !o_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (kv_valid <= 0 || kv_valid > N_kv) return MI355_SAGE_EINVAL;
    if (variant == MI355_SAGE_PV_FP8 && !vscale) return MI355_SAGE_EINVAL;
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (!dims_ok(D) || !blk_ok(blkq) || !blk_ok(blkk)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_kv_len(N_kv, blkk, D))) return rc;
    if ((rc = check_view("O", O, o_strides, o_off))) return rc;
    AttnArgs a{};
    a.q8 = static_cast<const int8_t*>(q8); a.qscale = static_cast<const float*>(qscale); a.blkq = blkq;
    a.k8 = static_cast<const int8_t*>(k8); a.kscale = static_cast<const float*>(kscale); a.blkk = blkk;
    a.vq = vq; a.vscale = static_cast<const float*>(vscale); a.qshift = static_cast<const float*>(qshift);
    a.variant = variant;
    if (clip_mask(kv_valid, mask_lo, mask_hi, &a.km) <= 0) return MI355_SAGE_EINVAL;
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = N_kv; a.kv_valid = kv_valid; a.D = D;
    a.nq_pad = pad_to(N_q, kTileQ); a.nkv_pad = pad_to(N_kv, kPadKV);
    a.o = static_cast<uint16_t*>(O) + o_off; a.osb = o_strides[0]; a.osh = o_strides[1]; a.osn = o_strides[2];
    a.stats = static_cast<float*>(stats);
    // Same scheduling, hence the same bits, as the one-shot calls: shapes that are split over a
    // fixed number of workgroups need hand-over slots, kept per (device, stream) by the library.
    a.split_wgs = attn_split_workgroups(B, H, N_q, kv_valid, D, variant);
    const size_t split_bytes = attn_split_bytes(a.split_wgs, D);
    if (split_bytes > 0 && (rc = internal_workspace(g_split_ws, split_bytes, static_cast<hipStream_t>(stream), &a.split))) return rc;
    SAGE_HIP(launch_attn(a, static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

int mi355_sage_attn_fwd_q16(const void* Q, const int64_t* q_strides, int64_t q_off, const void* qmul, int blkq,
                            const void* k8, const void* kscale, int blkk, const void* vq, const void* vscale, int variant,
                            int B, int H, int N_q, int N_kv, int kv_valid, int mask_lo, int mask_hi, int D,
                            void* O, const int64_t* o_strides, int64_t o_off, void* stream) {
    if (!Q || !q_strides || !qmul || !k8 || !kscale || !vq || !O || !o_strides) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (kv_valid <= 0 || kv_valid > N_kv) return MI355_SAGE_EINVAL;
    if (variant == MI355_SAGE_PV_FP8 && !vscale) return MI355_SAGE_EINVAL;
    if (variant != MI355_SAGE_PV_FP16 && variant != MI355_SAGE_PV_FP8) return MI355_SAGE_EUNSUPPORTED;
    if (!dims_ok(D) || D > 128 || !blk_ok(blkq) || !blk_ok(blkk)) return MI355_SAGE_EUNSUPPORTED;
    int rc;
    if ((rc = check_kv_len(N_kv, blkk, D))) return rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("O", O, o_strides, o_off))) return rc;
    // (shapes of the split schedule keep the encoded-Q form: the one-shot calls do the same)
    if (attn_split_workgroups(B, H, N_q, kv_valid, D, variant) > 0) return MI355_SAGE_EUNSUPPORTED;
    AttnArgs a{};
    const View q = make_view(Q, q_strides, q_off);
    a.q_src = q.p; a.qsb = q.sb; a.qsh = q.sh; a.qsn = q.sn; a.qmul = static_cast<const float*>(qmul); a.blkq = blkq;
    a.k8 = static_cast<const int8_t*>(k8); a.kscale = static_cast<const float*>(kscale); a.blkk = blkk;
    a.vq = vq; a.vscale = static_cast<const float*>(vscale);
    a.variant = variant;
    if (clip_mask(kv_valid, mask_lo, mask_hi, &a.km) <= 0) return MI355_SAGE_EINVAL;
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = N_kv; a.kv_valid = kv_valid; a.D = D;
    a.nq_pad = pad_to(N_q, kTileQ); a.nkv_pad = pad_to(N_kv, kPadKV);
    a.o = static_cast<uint16_t*>(O) + o_off; a.osb = o_strides[0]; a.osh = o_strides[1]; a.osn = o_strides[2];
    SAGE_HIP(launch_attn(a, static_cast<hipStream_t>(stream)));
    return MI355_SAGE_OK;
}

int mi355_sage_attn_split_faults(int reset) { return attn_split_faults(reset); }

// (declared in include/mi355_sage_test.h: switches for the library's own tests)
int mi355_sage_attn_split_rule(int B, int H, int N_q, int N_kv, int D, int variant) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0) return 0;
    return attn_split_rule(B, H, N_q, N_kv, D, variant);
}

int mi355_sage_set_attn_split(int mode) {
    if (mode < -1 || mode > kSplitMaxWorkgroups || (mode > 0 && (mode & 7))) return MI355_SAGE_EINVAL;
    attn_split_override(mode);
    return MI355_SAGE_OK;
}

int mi355_sage_set_attn_split_wait(int polls) {
    if (polls < -(1 << 24) || polls > (1 << 24)) return MI355_SAGE_EINVAL;
    attn_split_wait(polls);
    return MI355_SAGE_OK;
}

// ---- backward ---------------------------------------------------------------------------------
struct BwdCarve { size_t kT, qT, doT, lse2, delta, kcen, total; };
static BwdCarve bwd_carve(int B, int H, int Nq, int Nkv, int D) {
    const size_t bh = (size_t)B * H;
    const size_t nqp = (size_t)pad_to(Nq, 64), nkp = (size_t)pad_to(Nkv, 64);
    BwdCarve c{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
    c.kT = take(bh * nkp * D * 2);
    c.qT = take(bh * nqp * D * 2);
    c.doT = take(bh * nqp * D * 2);
    c.lse2 = take(bh * nqp * sizeof(float));
    c.delta = take(bh * nqp * sizeof(float));
    c.kcen = take(bh * D * sizeof(float));
    c.total = off;
    return c;
}

size_t mi355_sage_bwd_workspace_bytes(int B, int H, int N_q, int N_kv, int D) {
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || !bwd_dims_ok(D)) return 0;
    return bwd_carve(B, H, N_q, N_kv, D).total;
}

int mi355_sage_sdpa_bwd_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                             const void* Stats, void* dQ, void* dK, void* dV,
                             int B, int H, int N_q, int N_kv, int D, float scale,
                             const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                             const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                             const int64_t* dk_strides, const int64_t* dv_strides,
                             int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                             int64_t stats_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                             int causal, int real_N_q, int real_N_kv, void* stream,
                             void* workspace, size_t workspace_bytes) {
    // same order as serenitymojo/ops/cshim/cudnn_sdpa_bwd.cpp:348-352
    if (!Q || !K || !V || !O || !dO || !Stats) return MI355_SAGE_EINVAL;
    if (!dQ || !dK || !dV) return MI355_SAGE_EINVAL;
    if (B <= 0 || H <= 0 || N_q <= 0 || N_kv <= 0 || D <= 0) return MI355_SAGE_EINVAL;
    if (!q_strides || !k_strides || !v_strides || !o_strides || !do_strides || !dq_strides || !dk_strides || !dv_strides)
        return MI355_SAGE_EINVAL;
    if (causal) { SAGE_LOG("causal attention is not supported"); return MI355_SAGE_EUNSUPPORTED; }
    if (!bwd_dims_ok(D)) { SAGE_LOG("backward: head dim %d is not supported (64 or 128)", D); return MI355_SAGE_EUNSUPPORTED; }
    int rc;
    if ((rc = check_view("Q", Q, q_strides, q_off)) || (rc = check_view("K", K, k_strides, k_off)) ||
        (rc = check_view("V", V, v_strides, v_off)) || (rc = check_view("O", O, o_strides, o_off)) ||
        (rc = check_view("dO", dO, do_strides, do_off)) || (rc = check_view("dQ", dQ, dq_strides, dq_off)) ||
        (rc = check_view("dK", dK, dk_strides, dk_off)) || (rc = check_view("dV", dV, dv_strides, dv_off)))
        return rc;
    // the tile copies address a head's rows with 32-bit byte offsets
    auto span_ok = [&](const char* name, int N, const int64_t* s) {
        if (s[2] < 0 || (uint64_t)(N - 1) * (uint64_t)s[2] * 2 + (uint64_t)D * 2 > 0xFFFFFFFFull) {
            SAGE_LOG("%s: a head's rows span more than 4 GiB (or the row stride is negative)", name);
            return false;
        }
        return true;
    };
    if (!span_ok("Q", N_q, q_strides) || !span_ok("dO", N_q, do_strides) || !span_ok("K", N_kv, k_strides) ||
        !span_ok("V", N_kv, v_strides))
        return MI355_SAGE_EUNSUPPORTED;

    const BwdCarve c = bwd_carve(B, H, N_q, N_kv, D);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (workspace == nullptr) {
        if ((rc = internal_workspace(g_ws, c.total, st, &workspace))) return rc;
    } else if (workspace_bytes < c.total || (reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1))) {
        SAGE_LOG("backward workspace: %zu bytes at a 256-byte boundary needed, %zu given", c.total, workspace_bytes);
        return MI355_SAGE_EWORKSPACE;
    }
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    BwdArgs a{};
    a.q = make_view(Q, q_strides, q_off);
    a.k = make_view(K, k_strides, k_off);
    a.v = make_view(V, v_strides, v_off);
    a.o = make_view(O, o_strides, o_off);
    a.dout = make_view(dO, do_strides, do_off);
    a.stats = static_cast<const float*>(Stats) + stats_off;
    a.dq = static_cast<uint16_t*>(dQ) + dq_off; a.dq_sb = dq_strides[0]; a.dq_sh = dq_strides[1]; a.dq_sn = dq_strides[2];
    a.dk = static_cast<uint16_t*>(dK) + dk_off; a.dk_sb = dk_strides[0]; a.dk_sh = dk_strides[1]; a.dk_sn = dk_strides[2];
    a.dv = static_cast<uint16_t*>(dV) + dv_off; a.dv_sb = dv_strides[0]; a.dv_sh = dv_strides[1]; a.dv_sn = dv_strides[2];
    a.B = B; a.H = H; a.Nq = N_q; a.Nkv = N_kv; a.D = D;
    a.valid_q = real_N_q > 0 && real_N_q < N_q ? real_N_q : N_q;          // cudnn_sdpa_bwd.cpp:362-363
    a.valid_kv = real_N_kv > 0 && real_N_kv < N_kv ? real_N_kv : N_kv;
    a.scale = scale;
    a.kT = reinterpret_cast<uint16_t*>(ws + c.kT);
    a.qT = reinterpret_cast<uint16_t*>(ws + c.qT);
    a.doT = reinterpret_cast<uint16_t*>(ws + c.doT);
    a.lse2 = reinterpret_cast<float*>(ws + c.lse2);
    a.delta = reinterpret_cast<float*>(ws + c.delta);
    a.kcen = reinterpret_cast<float*>(ws + c.kcen);
    a.nq_pad = pad_to(N_q, 64);
    a.nkv_pad = pad_to(N_kv, 64);
    SAGE_HIP(launch_bwd(a, st));
    return 0;
}

}  // extern "C"
