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
// The attention kernel stages one head's K scales in LDS, one entry per 32 keys: keys per head it takes
// (256 channels: the tile rings leave room for a quarter as many entries).
__host__ __device__ constexpr int max_keys(int D) { return (D > 128 ? 2048 : 8192) * 32; }

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
    int halfsplit;               // 0: pairs (2i, 2i+1) (ops/rope.mojo:7-9); 1: pairs (i, i + D/2) (ops/rope.mojo:10-13)
    int tables_bf16;             // the tables hold bf16 instead of fp32
    const float* row_inv;        // [B, row_n]: 1/sqrt(mean over all H*D channels + eps) per token; null: the
    int64_t row_n;               //   statistic is taken per head over D.  With it the gain has H*D entries.
};

// Keys lo <= s < hi take no part (statistics, scale blocks, scores); lo >= hi: no such range.
struct KeyMask {
    int lo, hi;
};

// ---- quantize kernels (sage_quant.hip): three launches --------------------------------
// Launch 1: passes over V and K whose results the later launches need.
struct PrepArgs {
    View k, v;
    int H, Nkv;
    int64_t nkv_pad;
    KeyMask km;
    int vmode;                       // 0: fp16 repack into v16; 1: channel maxima per group into vpart; 2: no V pass
    uint16_t* v16;
    float* vpart;                    // [B,H,ngroups,D]
    double* kpart_sum;               // [B,H,ngroups,D] group sums; null: no K pass
    float* kpart_mm;                 // [B,H,ngroups,D,2] group minima / maxima
    PreOp pre_k;
    int ngroups, nk_wg, nv_units, n_bh;    // filled by the launcher
};
hipError_t launch_prep(const PrepArgs& a, int B, int D, hipStream_t st);

// Launch 0 (only with a whole-row RMSNorm in front): 1/sqrt(mean(x^2) + eps) over all H*D channels
// of every token of Q (rows [0, B*Nq)) and K (the rows after them), squares added in the order of
// serenitymojo/ops/norm.mojo:56-72.
hipError_t launch_row_inv(const View& q, const View& k, int B, int H, int Nq, int Nkv, int D, float eps,
                          float* inv_q, float* inv_k, hipStream_t st);

// Launch 2: per (b,h,channel) K mean and balancing factor, V scale.
struct FinalArgs {
    int64_t total;                   // B*H*D
    int D, ngroups, kept, flags;     // kept = number of keys that count; flags: bit 0 smoothing, bit 1 balancing
    float cmul;                      // fp32(scale*log2(e))
    const double* kpart_sum;         // null: no K statistics (mean 0, factor 1)
    const float* kpart_mm;
    float *kmean, *qmul, *kmul;      // [B,H,D] each; kmean null: K outputs are skipped
    const float* vpart;
    float* vscale;                   // null: V output is skipped
};
hipError_t launch_stats_final(const FinalArgs& a, hipStream_t st);

// Launch 3: the encoders.  q8 / k8 / v8 null: that role is skipped.
struct QuantArgs {
    View q, k, v;
    int H, Nq, Nkv;
    int64_t nq_pad, nkv_pad;
    KeyMask km;
    int blkq, blkk;
    float cmul;
    const float *kmean, *qmul, *kmul, *vscale;
    int8_t* q8;
    float* qscale;
    float* rowdot;                   // [B,H,nq_pad] <f32(q)*cmul, kmean>, or null
    int8_t* k8;
    float* kscale;
    uint8_t* v8;                     // e4m3 V tiles (needs vscale), or
    uint16_t* v16;                   // fp16 V tiles (the repack needs no statistics; it rides here so that launch 1 is short)
    PreOp pre_q, pre_k;
    int nq_blk, nk_blk, nv_tile, n_bh;     // filled by the launcher
};
hipError_t launch_quant(const QuantArgs& a, int B, int D, hipStream_t st);

// ---- attention kernel (sage_attn.hip) --------------------------------------
// rint(x / sc) for |x / sc| <= ~127 without paying a full IEEE divide per element: x * (1/sc)
// is within 2^-15 of the correctly rounded quotient (both below 128), so whenever it lies at
// least 2^-12 away from a rounding tie it rounds to the same integer; the few elements near
// a tie (and any non-finite case) take the true divide.  `fast` is false when sc is so small
// or large that 1/sc is not a normal number.
__device__ __forceinline__ float rint_quotient(float x, float sc, float rinv, bool fast) {
    const float q = x * rinv;
    float n = rintf(q);
    if (!fast || !(fabsf(q - n) <= 0.5f - 0x1p-12f)) n = rintf(x / sc);
    return n;
}

struct AttnArgs {
    const int8_t* q8;  const float* qscale;  int blkq;
    const int8_t* k8;  const float* kscale;  int blkk;
    const void* vq;    const float* vscale;  const float* qshift;  // qshift [B,H,nq_pad], stats only
    int variant;
    KeyMask km;
    int B, H, Nq, Nkv, kv_valid, D;
    int causal;              // 1: query i sees keys j <= i only (never together with the split schedule)
    int64_t nq_pad, nkv_pad;
    uint16_t* o; int64_t osb, osh, osn;
    float* stats;            // [B,H,Nq] or null
    const uint16_t* amask;   // additive bias, bf16, base + offset; null = none
    int64_t amb, amh, amn;   // its element strides for batch, head, query (key stride 1)
    // Q taken as bf16 and encoded by the attention kernel itself (q8 / qscale unused then): base + offset,
    // element strides of batch, head and token, and the channel multipliers [B,H,D] of the quantize stage.
    // Only without Stats, additive bias and split schedule, at up to 128 channels.
    const uint16_t* q_src;   // null: q8 / qscale are read
    int64_t qsb, qsh, qsn;
    const float* qmul;
    int split_wgs;           // workgroups of the split schedule (attn_split_workgroups), 0: one workgroup per item
    void* split;             // attn_split_bytes(split_wgs, D) bytes, 256-byte aligned (null when 0)
};
hipError_t launch_attn(const AttnArgs& a, hipStream_t st);
// Shapes whose items do not fill whole rounds of workgroups are spread evenly over a fixed number
// of workgroups that hand partial results to each other through `split`.
// attn_split_rule: the number of workgroups (a multiple of 8) the shape alone asks for, or 0 for one
// workgroup per item — what workspaces are sized by.
// attn_split_workgroups: what a launch on the current device uses: the rule where the device deals
// workgroup ids round-robin to 8 XCDs of 32 compute units (else 0), or what the test switch forces.
int attn_split_rule(int B, int H, int Nq, int kv_valid, int D, int variant);
int attn_split_workgroups(int B, int H, int Nq, int kv_valid, int D, int variant);
size_t attn_split_bytes(int workgroups, int D);
constexpr size_t kSplitFlagBytes = 4096;     // one int per workgroup in front of the state slots
constexpr int kSplitMaxWorkgroups = 1024;
void attn_split_override(int mode);          // 0: by shape and device (default); -1: never; n > 0 (multiple of 8): always n
void attn_split_wait(int polls);             // bound of the hand-over wait; 0: default; < 0: test mode (no flag is raised)
int attn_split_faults(int reset);            // workgroups that gave up on the current device since the last reset; < 0: -hipError_t

// ---- backward (sage_bwd.hip) -------------------------------------------------
// bf16 flash backward: Q, K, V, O, dO and the forward's log-sum-exp in, dQ, dK, dV out.
struct BwdArgs {
    View q, k, v, o, dout;
    const float* stats;                          // [B,H,Nq] contiguous, natural log
    uint16_t *dq, *dk, *dv;
    int64_t dq_sb, dq_sh, dq_sn, dk_sb, dk_sh, dk_sn, dv_sb, dv_sh, dv_sn;
    int B, H, Nq, Nkv, D;
    int valid_q, valid_kv;                       // rows / keys past these are padding
    float scale;
    // workspace
    uint16_t *kT, *qT, *doT;                     // [B,H,n_pad/64,D,64] bf16, rows in v_slot_f16 order, zero past valid
    float *lse2, *delta;                         // [B,H,nq_pad]: Stats*log2(e) (+inf past valid), rowsum(dO*O)
    float* kcen;                                 // [B,H,D]: a vector close to the mean key (see sage_bwd.hip)
    int64_t nq_pad, nkv_pad;                     // multiples of 64
};
hipError_t launch_bwd(const BwdArgs& a, hipStream_t st);

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
