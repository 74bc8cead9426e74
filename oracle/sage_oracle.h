/*
 * sage_oracle.h — CPU oracle for the quantized-SDPA hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker: tests, the smoke
 * check and the bench's cpu_baseline leg may call it; the product library
 * (libmi355_sage.so) never links, loads or falls back to it.
 *
 * Every tensor is addressed as logical [B, H, N, D] through four ELEMENT
 * strides, the convention of the reference's native attention seam
 * (serenitymojo/ops/cshim/cudnn_sdpa.cpp:375-387; the Mojo caller describes
 * its [B,S,H,Dh] memory as {S*H*Dh, Dh, H*Dh, 1},
 * serenitymojo/ops/attention_flash.mojo:46-54).
 *
 * Pinning status (what fixes each function independently of this file):
 *   sage_oracle_sdpa_f32 / _online_f32 ... reference golden vectors
 *       (ops/parity/sdpa_math_ref.txt, ops_smoke2.mojo:239-278) + closed forms.
 *   bf16 / fp16 / e4m3 codecs ............. reference KATs
 *       (ops/tests/fp8_quant_smoke.mojo:108-143) + torch / numpy library codecs.
 *   sage_oracle_rms_norm_f32 / _rope_interleaved_f32 ... reference vectors
 *       (ops_smoke.mojo:78-96, ops_smoke2.mojo:95-120) + the closed form of
 *       ops_smoke2.mojo:372-403.  The squares are added in the order the reference's kernel
 *       spells out (ops/norm.mojo:56-72).  sage_oracle_norm_rope_bf16 composes the two with RNE
 *       bf16 stores; whether the reference's compiler contracts the products of the rotation
 *       into fused multiply-adds is the one thing its text cannot pin (PARITY UNPINNED there;
 *       this file uses separately rounded products).
 *   sage_oracle_sdpa_f32_ex (key range mask, additive mask) ... reduces to sage_oracle_sdpa_f32
 *       on the kept keys / with a zero mask; float64 brute force (tests/).
 *   sage_oracle_quant_q* / _kstats / _kmean / _quant_k* / _quant_v_* , sage_oracle_attn*:
 *       PARITY UNPINNED by the reference — it holds no INT8 / SageAttention
 *       code, test or vector.  They are pinned only by closed forms, invariants
 *       and an independent numpy restatement (tests/), never by reference data.
 */
#ifndef SAGE_ORACLE_H
#define SAGE_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar codecs ------------------------------------------------------ */
float    sage_oracle_bf16_to_f32(uint16_t b);
uint16_t sage_oracle_f32_to_bf16(float f);   /* RNE, ops/torch_bf16.mojo:27-60 */
float    sage_oracle_f16_to_f32(uint16_t h);
uint16_t sage_oracle_f32_to_f16(float f);    /* RNE, finite overflow saturates to 65504 */
float    sage_oracle_e4m3_to_f32(uint8_t b); /* ops/fp8.mojo:60-78 */
uint8_t  sage_oracle_f32_to_e4m3(float f);   /* RNE + saturate, ops/fp8_quant.mojo:61-93 */

/* vector forms for the tests */
void sage_oracle_f32_to_bf16_n(const float* x, uint16_t* y, int64_t n);
void sage_oracle_f32_to_f16_n(const float* x, uint16_t* y, int64_t n);
void sage_oracle_f32_to_e4m3_n(const float* x, uint8_t* y, int64_t n);
void sage_oracle_e4m3_to_f32_n(const uint8_t* x, float* y, int64_t n);

/* ---- full-precision SDPA (the referee) ---------------------------------- */
/* Exact two-pass softmax attention, double accumulation.  Restates
 * serenitymojo/ops/attention.mojo:18-27 and the numpy generator
 * ops/parity/sdpa_math_oracle.py:39-52.  Returns 0, or -1 on bad arguments
 * (same checks as cudnn_sdpa.cpp:391-393). */
int sage_oracle_sdpa_f32(const float* q, const float* k, const float* v, float* o,
                         int B, int H, int Nq, int Nkv, int D, float scale,
                         const int64_t* qs, const int64_t* ks,
                         const int64_t* vs, const int64_t* os);

/* The same with keys [mask_lo, mask_hi) left out (what serenitymojo/ops/attention.mojo:1790-1857
 * does with a -1e4 bias), an optional additive bias in natural-log units, contiguous
 * [B,H,Nq,Nkv] (attention.mojo:1596-1647, :1897-1936), and an optional log-sum-exp output
 * stats [B,H,Nq] (natural log, of the scaled and biased scores). */
int sage_oracle_sdpa_f32_ex(const float* q, const float* k, const float* v, float* o,
                            int B, int H, int Nq, int Nkv, int D, float scale,
                            const int64_t* qs, const int64_t* ks,
                            const int64_t* vs, const int64_t* os,
                            int mask_lo, int mask_hi, const float* addmask, float* stats);

/* One-key-at-a-time online-softmax recurrence in fp32, restating
 * serenitymojo/ops/attention.mojo:744-801 (m starts at -3e38, natural exp). */
int sage_oracle_sdpa_online_f32(const float* q, const float* k, const float* v, float* o,
                                int B, int H, int Nq, int Nkv, int D, float scale,
                                const int64_t* qs, const int64_t* ks,
                                const int64_t* vs, const int64_t* os);

/* ---- backward of the full-precision SDPA ------------------------------------ */
/* Decomposed backward in double precision, restating serenitymojo/ops/attention_backward.mojo:12-19.
 * o == stats == NULL: probabilities recomputed from q, k (the torch.autograd reference of
 * ops/parity/sdpa_bwd_oracle.py:56-63).  Both given: the flash interface of
 * ops/cshim/cudnn_sdpa_bwd.cpp:325-347 — attn = exp(score - stats[row]) and the softmax-backward
 * row term is rowsum(dO * O), and dQ is taken with the keys centred on their mean (a row of dS sums
 * to zero for consistent O and stats, so this changes nothing then; it keeps a small inconsistency
 * of a lower-precision forward from being multiplied by the keys' common offset).
 * stats contiguous [B,H,Nq] (natural log).  Rows >= real_nq and keys
 * >= real_nkv (0: all) are padding; their gradients are zero.  Pinned by the reference's golden
 * gradients ops/parity/sdpa_bwd_ref.txt, torch.autograd in float64, central differences, and the
 * invariance of attention to a common shift of all keys (sum over keys of dK is zero). */
int sage_oracle_sdpa_bwd_f32(const float* q, const float* k, const float* v, const float* o,
                             const float* dout, const float* stats,
                             float* dq, float* dk, float* dv,
                             int B, int H, int Nq, int Nkv, int D, float scale,
                             const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                             const int64_t* dos, const int64_t* dqs, const int64_t* dks, const int64_t* dvs,
                             int real_nq, int real_nkv);

/* ---- the two ops in front of the path (fused into the quantizers by the product) ---- */
/* RMSNorm rows x cols in fp32: serenitymojo/ops/norm.mojo:47-79.  Pinned by the reference's
 * vector serenitymojo/ops_smoke.mojo:78-96 and the closed form of ops_smoke2.mojo:372-403;
 * the squares are added in the order of the reference's kernel (norm.mojo:56-72). */
int sage_oracle_rms_norm_f32(const float* x, const float* g, int64_t rows, int cols, float eps, float* out);
/* Interleaved RoPE in fp32: serenitymojo/ops/rope.mojo:7-9.  Pinned by ops_smoke2.mojo:95-120. */
int sage_oracle_rope_interleaved_f32(const float* x, const float* cs, const float* sn,
                                     int64_t rows, int D, float* out);
/* Half-split RoPE in fp32 (pairs x[i], x[i + D/2]): serenitymojo/ops/rope.mojo:10-13.  Pinned by
 * the reference's vector ops_smoke2.mojo:113-132 (y_half_ref). */
int sage_oracle_rope_halfsplit_f32(const float* x, const float* cs, const float* sn,
                                   int64_t rows, int D, float* out);
/* The bf16 pipeline rms_norm -> (bf16) -> rope_interleaved -> (bf16) of
 * serenitymojo/models/klein/single_block.mojo:977-981 on a strided [B,H,N,D] view; output
 * contiguous [B,N,H,D].  Tables [.., D/2] fp32 with row n*H + h (+ b*table_batch_rows);
 * cs == NULL: no rotation.  The bf16 roundings are RNE (ops/torch_bf16.mojo:27-60). */
int sage_oracle_norm_rope_bf16(const uint16_t* x, int B, int H, int N, int D, const int64_t* st,
                               const uint16_t* gain, float eps, const float* cs, const float* sn,
                               int64_t table_batch_rows, uint16_t* y);
/* The same with options, pre_flags: bit 0 half-split pairing (rope.mojo:10-13; the per-head
 * rms_norm -> rope_halfsplit sequence of serenitymojo/models/anima/block.mojo:360-366); bit 1 bf16
 * tables (cs / sn point at uint16); bit 2 RMSNorm over the whole row of H*D channels with a gain
 * of H*D entries (serenitymojo/models/ltx2/ltx2_block.mojo:419-432: rms_norm on [S, H*D], then
 * the reshape to heads).  Wide rows accumulate `local += v*v` per thread (norm.mojo:62-65); whether
 * the reference's compiler fuses that multiply-add is not visible in its text: parity unpinned
 * for that bit, separately rounded here. */
int sage_oracle_norm_rope_bf16_ex(const uint16_t* x, int B, int H, int N, int D, const int64_t* st,
                                  const uint16_t* gain, float eps, const void* cs, const void* sn,
                                  int64_t table_batch_rows, int pre_flags, uint16_t* y);

/* ---- quantizers --------------------------------------------------------- */
/* Padded token count used by every quantized tensor: N rounded up to `mult`. */
int64_t sage_oracle_pad(int64_t n, int64_t mult);

/* Q: qs = f32(bf16) * c, c = fp32(scale*log2(e)) (rounded once from double);
 * per (b,h,block of blkq tokens): amax -> sc = amax/127 (1.0 if amax==0),
 * code = clamp(rne(qs/sc), -127, 127).  q8: [B,H,Npad,D] contiguous (pad rows 0),
 * qscale: [B,H,ceil(N/blkq)].  Npad = pad(N, npad_mult). */
int sage_oracle_quant_q(const uint16_t* q, int B, int H, int N, int D,
                        const int64_t* strides, float scale, int blkq, int npad_mult,
                        int8_t* q8, float* qscale);

/* Per-channel K statistics over the kept keys (token s is kept unless mask_lo <= s < mask_hi),
 * per (b,h,d):
 *   mean  (flags & 1): the summation tree of sage_oracle_kmean below with masked tokens adding
 *         +0.0, divided by the number of kept keys; 0 when the flag is clear.
 *   s_d   (flags & 2): sqrtf(max over kept keys of |f32(k) - mean|) (1 when that maximum is 0);
 *         1 when the flag is clear.  This balances the channels between K and Q: K is divided
 *         and Q multiplied by s_d, which leaves every score unchanged in real arithmetic and
 *         takes the square root of a channel's excess range out of each side.
 *   kmul = 1.0f / s_d,  qmul = c * s_d  with c = fp32(scale*log2(e)).
 * kmean, qmul, kmul: [B,H,D].  Returns -1 when no key is kept. */
int sage_oracle_kstats(const uint16_t* k, int B, int H, int N, int D, const int64_t* strides,
                       float scale, int flags, int mask_lo, int mask_hi,
                       float* kmean, float* qmul, float* kmul);

/* Q with a per-channel multiplier: x = f32(bf16) * qmul[b,h,d] (qmul NULL: the scalar c),
 * then the per-block INT8 rule of sage_oracle_quant_q. */
int sage_oracle_quant_q_ch(const uint16_t* q, int B, int H, int N, int D,
                           const int64_t* strides, float scale, const float* qmul, int blkq, int npad_mult,
                           int8_t* q8, float* qscale);

/* K with mean and per-channel multiplier: x = (f32(bf16) - kmean[b,h,d]) * kmul[b,h,d] (two
 * fp32 operations; either pointer may be NULL), then the per-block INT8 rule.  Masked tokens
 * do not count for their block's maximum and get code 0. */
int sage_oracle_quant_k_ch(const uint16_t* k, int B, int H, int N, int D,
                           const int64_t* strides, const float* kmean, const float* kmul,
                           int mask_lo, int mask_hi, int blkk, int npad_mult,
                           int8_t* k8, float* kscale);

/* K mean over tokens per (b,h,d) with a fixed summation tree in double:
 * 16-token leaves (tokens ascending), groups of 16 leaves (ascending), groups
 * ascending; the total is divided by N in double and rounded once to fp32.
 * (Sums of bf16 values in double are exact unless one column spans more than
 * ~2^40 in magnitude, so in practice any order gives these bits; the tree is
 * what holds when it does not.)  kmean: [B,H,D]. */
int sage_oracle_kmean(const uint16_t* k, int B, int H, int N, int D,
                      const int64_t* strides, float* kmean);

/* K: ks = f32(bf16) - kmean[b,h,d] (kmean may be NULL = no smoothing), then
 * the same per-block INT8 rule with blocks of blkk tokens. */
int sage_oracle_quant_k(const uint16_t* k, int B, int H, int N, int D,
                        const int64_t* strides, const float* kmean, int blkk, int npad_mult,
                        int8_t* k8, float* kscale);

/* V variant 0: fp16 RNE of the bf16 value; plain [B,H,Npad,D], pad rows 0. */
int sage_oracle_quant_v_f16(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* strides, int npad_mult, uint16_t* v16);

/* V variant 1: per (b,h,d) amax over tokens -> vscale = amax/448 (1.0 if 0),
 * byte = e4m3(v / vscale).  v8 plain [B,H,Npad,D], vscale [B,H,D]. */
int sage_oracle_quant_v_fp8(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* strides, int npad_mult,
                            uint8_t* v8, float* vscale);

/* The same with masked rows (mask_lo <= s < mask_hi) left 0. */
int sage_oracle_quant_v_f16_masked(const uint16_t* v, int B, int H, int N, int D,
                                   const int64_t* strides, int mask_lo, int mask_hi, int npad_mult, uint16_t* v16);

/* The same with the channel maximum taken over the kept keys only and masked rows left 0. */
int sage_oracle_quant_v_fp8_masked(const uint16_t* v, int B, int H, int N, int D,
                                   const int64_t* strides, int mask_lo, int mask_hi, int npad_mult,
                                   uint8_t* v8, float* vscale);

/* ---- quantized attention ------------------------------------------------ */
/* s[i,j] = float(sum_d q8*k8) * (qscale*kscale)   (log2 domain)
 * variant 0: p = exp2(s - max_j s), P16 = f16(p), O = sum P16*V16 / sum p
 * variant 1: p = exp2(s - ceil(max_j s)), P8 = e4m3(p*448), O = sum P8*V8 * vscale / sum P8
 *            (an integer reference: shifting it by a whole number only moves the exponent of
 *            every probability, so their e4m3 significands do not depend on which integer an
 *            implementation that walks the keys in tiles happens to hold)
 * O -> bf16 RNE in the caller's strides; o_f32 (optional, same strides) gets
 * the unrounded value.  Padded tensors as produced by the quantizers above
 * with token pads NqPad / NkvPad. */
int sage_oracle_attn(const int8_t* q8, const float* qscale, int blkq, int64_t NqPad,
                     const int8_t* k8, const float* kscale, int blkk, int64_t NkvPad,
                     const void* vq, const float* vscale, int variant,
                     int B, int H, int Nq, int Nkv, int D,
                     uint16_t* o_bf16, float* o_f32, const int64_t* os);

/* The same with keys [mask_lo, mask_hi) masked, an optional additive bias (natural-log units,
 * contiguous [B,H,Nq,Nkv], converted to the log2 domain with one fp32 multiply and added to the
 * dequantised score), qshift [B,H,NqPad] (log2 units, may be NULL) and an optional stats output
 * [B,H,Nq]: (reference + log2(sum p) + qshift) * ln 2. */
int sage_oracle_attn_ex(const int8_t* q8, const float* qscale, int blkq, int64_t NqPad,
                        const int8_t* k8, const float* kscale, int blkk, int64_t NkvPad,
                        const void* vq, const float* vscale, int variant,
                        int B, int H, int Nq, int Nkv, int D,
                        int mask_lo, int mask_hi, const float* addmask, const float* qshift,
                        uint16_t* o_bf16, float* o_f32, const int64_t* os, float* stats);

/* Whole path on bf16 inputs (quantize + attention), the CPU baseline's unit
 * of work.  Allocates its own temporaries.  k_flags: bit 0 = K mean smoothing, bit 1 =
 * per-channel Q/K balancing. */
int sage_oracle_sdpa_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                          uint16_t* o, float* o_f32,
                          int B, int H, int Nq, int Nkv, int D, float scale,
                          const int64_t* qs, const int64_t* ks,
                          const int64_t* vs, const int64_t* os,
                          int variant, int blkq, int blkk, int k_flags);
int sage_oracle_sdpa_bf16_ex(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                             uint16_t* o, float* o_f32, float* stats,
                             int B, int H, int Nq, int Nkv, int D, float scale,
                             const int64_t* qs, const int64_t* ks,
                             const int64_t* vs, const int64_t* os,
                             int variant, int blkq, int blkk, int k_flags,
                             int mask_lo, int mask_hi, const float* addmask);

int sage_oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
