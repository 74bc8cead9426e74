// sage_internal.h — shared declarations of the kernels' launchers (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

namespace sage {

// Tile geometry of the attention kernel; the quantized layouts are padded to it.
constexpr int kTileQ  = 256;   // query rows per workgroup (8 waves x 32 rows)
constexpr int kTileKV = 64;    // keys per main-loop iteration
constexpr int kPadKV  = 128;   // key tokens are padded to this (every scale-block size divides it)
constexpr int kLeaf   = 16;    // tokens per leaf of the K-mean summation tree
constexpr int kGroup  = 256;   // tokens per group (16 leaves)
constexpr int kMaxKScales = 1024;   // K scale blocks per head the attention kernel stages in LDS

inline int64_t pad_to(int64_t n, int64_t m) { return (n + m - 1) / m * m; }

// Logical [B,H,N,D] view of a bf16 tensor.
struct View {
    const uint16_t* p;       // base + element offset
    int64_t sb, sh, sn;      // element strides (D stride is 1)
};

// RMSNorm over D (+ interleaved RoPE) applied to the rows of Q or K as the quantizers load
// them: what serenitymojo/ops/norm.mojo:81-114 and ops/rope.mojo:104-122 leave in memory as
// bf16 tensors, computed on the fly.  gain == null: rows are used as they are.
struct PreOp {
    const uint16_t* gain;        // bf16 [D]
    float eps;
    const float* cos;            // fp32 [rows, D/2], row = n*H + h (+ b*batch_rows); null = no rotation
    const float* sin;
    int64_t batch_rows;          // 0: all batches share the table
};

// ---- quantize kernels (sage_quant.hip) -------------------------------------
// Q (is_k = false): x = f32(q)*cmul.  K (is_k = true): x = f32(k) - mean (mean may be null).
// rowdot (Q only, may be null): [B,H,n_pad] <pre-scaled q row, mean>, needed for the
// log-sum-exp output when K is smoothed.
hipError_t launch_quant_i8(const View& x, int B, int H, int N, int D, int64_t n_pad,
                           int blk, bool is_k, float cmul, const float* mean,
                           int8_t* codes, float* scales, float* rowdot, const PreOp& pre, hipStream_t st);

// K mean: group partials (double, [B,H,ngroups,D]) then the final mean.
hipError_t launch_kmean(const View& k, int B, int H, int N, int D,
                        double* group_partials, float* kmean, const PreOp& pre, hipStream_t st);

// One-shot path: Q quantizer + V fp16 repack + K-mean group sums in one launch, then the
// K quantizer that finishes the mean from the group partials itself (partial == null: no
// smoothing).  Same arithmetic, bit for bit, as the separate launches above.
hipError_t launch_prep_fused(const View& q, const View& k, const View& v, int B, int H, int Nq, int Nkv, int D,
                             int64_t nq_pad, int64_t nkv_pad, float cmul, int blkq, bool smooth_k,
                             int8_t* q8, float* qscale, uint16_t* v16, double* partial,
                             const PreOp& pre_q, const PreOp& pre_k, hipStream_t st);
hipError_t launch_kquant_fused(const View& k, int B, int H, int N, int D, int64_t n_pad, int blk,
                               const double* partial, float* kmean, int8_t* codes, float* scales,
                               const PreOp& pre, hipStream_t st);

hipError_t launch_quant_v_f16(const View& v, int B, int H, int N, int D, int64_t n_pad,
                              uint16_t* v16, hipStream_t st);

hipError_t launch_quant_v_fp8(const View& v, int B, int H, int N, int D, int64_t n_pad,
                              uint8_t* v8, float* vscale, hipStream_t st);

// ---- attention kernel (sage_attn.hip) --------------------------------------
struct AttnArgs {
    const int8_t* q8;  const float* qscale;  int blkq;
    const int8_t* k8;  const float* kscale;  int blkk;
    const void* vq;    const float* vscale;  const float* qshift;  // qshift [B,H,nq_pad], stats only
    int variant;
    int B, H, Nq, Nkv, kv_valid, D;
    int64_t nq_pad, nkv_pad;
    uint16_t* o; int64_t osb, osh, osn;
    float* stats;            // [B,H,Nq] or null
};
hipError_t launch_attn(const AttnArgs& a, hipStream_t st);

// Key k of a 64-key tile is stored at this slot of the V tile (host + device).
__host__ __device__ inline int v_slot_f16(int k) {
    // 16-key groups; inside a group the quads of 4 keys are ordered 0,2,1,3 so that
    // each half-wave finds the 8 keys its score registers hold in one 16-byte run.
    int g = k >> 4, r = k & 15, quad = r >> 2, w = r & 3;
    return (g << 4) | ((quad & 1) << 3) | ((quad >> 1) << 2) | w;
}
__host__ __device__ inline int v_slot_fp8(int k) {
    // whole 64-key tile: half-wave h holds keys with bit 2 == h; its 32 keys are
    // ordered by (32-key block, row group of 8, key within quad).
    int kb = k >> 5, r = k & 31, grp = r >> 3, half = (r >> 2) & 1, w = r & 3;
    return (half << 5) | (kb << 4) | (grp << 2) | w;
}

}  // namespace sage
