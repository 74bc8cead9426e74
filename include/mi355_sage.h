/*
 * mi355_sage.h — C ABI of libmi355_sage.so: SageAttention-style quantized
 * scaled-dot-product attention for AMD MI355X (gfx950), hand-written HIP.
 *
 * The library sits behind the same seam as the reference's native attention
 * shim: raw device pointers, dims, four ELEMENT strides per tensor describing
 * the memory as logical [B, H, N, D], element offsets, a stream, an int return
 * code.  Work is enqueued on the caller's stream; no call waits for the device.
 *
 * Conventions shared by every entry point
 *   - tensors are caller-allocated device memory; stride arrays are host
 *     memory read during the call only
 *     (serenitymojo/ops/attention_flash.mojo:177-193);
 *   - q/k/v/o are bf16; the innermost (D) stride must be 1 and every row start
 *     must be 16-byte aligned (callers hand out 16-byte-aligned scratch views,
 *     serenitymojo/scratch_ring.mojo:49);
 *   - D is 64, 128 or — forward only and without the fused RMSNorm / RoPE, as the reference's
 *     Ideogram-4 arm uses it (serenitymojo/models/dit/ideogram4_dit.mojo:29-49) — 256;
 *     attention is full and non-causal; trailing keys (real_N_kv) or one range of keys
 *     (_keymask) can be masked; N_q may differ from N_kv;
 *   - return 0 on success; -1 for a null pointer, a non-positive dimension or
 *     null strides (serenitymojo/ops/cshim/cudnn_sdpa.cpp:391-393); -2 for an
 *     unsupported configuration; -3 for a workspace that is too small; a
 *     positive value is a hipError_t.  Diagnostics go to stderr tagged
 *     [mi355_sage].
 */
#ifndef MI355_SAGE_H
#define MI355_SAGE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_SAGE_OK            0
#define MI355_SAGE_EINVAL      (-1)
#define MI355_SAGE_EUNSUPPORTED (-2)
#define MI355_SAGE_EWORKSPACE  (-3)

/* P*V arithmetic. */
#define MI355_SAGE_PV_FP16 0   /* INT8 QK^T, FP16 P*V              */
#define MI355_SAGE_PV_FP8  1   /* INT8 QK^T, FP8-e4m3 P*V, per-channel V scales */

/* Quantization recipe flags (k_flags). */
#define MI355_SAGE_K_SMOOTH  1   /* subtract the per-channel mean of K over the keys          */
#define MI355_SAGE_ROPE_INTERLEAVED 0   /* pairs (x[2i], x[2i+1]): serenitymojo/ops/rope.mojo:7-9 (FLUX, Klein, Z-Image) */
#define MI355_SAGE_ROPE_HALFSPLIT   1   /* pairs (x[i], x[i+D/2]): serenitymojo/ops/rope.mojo:10-13 (Anima, Hunyuan, LTX-2 ...) */
/* two more bits of the same argument (rope_layout): */
#define MI355_SAGE_ROPE_TABLES_BF16 2   /* rope_cos / rope_sin hold bf16 (rope.mojo:147-165 casts them to fp32) */
#define MI355_SAGE_NORM_FULL_ROW    4   /* the RMSNorm runs over all H*D channels of a token, q_gain / k_gain have H*D
                                           entries (channel h*D + d): rms_norm on [S, H*D] before the reshape to heads,
                                           serenitymojo/models/ltx2/ltx2_block.mojo:419-432 */
#define MI355_SAGE_K_BALANCE 2   /* per channel d: K / s_d, Q * s_d with s_d = sqrt(max|K - mean|)
                                    over the keys: scores are unchanged, and a channel whose
                                    range is r times the others' costs each side sqrt(r), not
                                    one side r, of its INT8 resolution                         */

/* ------------------------------------------------------------------------
 * One-shot drop-in.
 * Replaces flame_cudnn_sdpa_bf16 (serenitymojo/ops/cshim/cudnn_sdpa.cpp:375-387):
 * the parameter list up to `stream` is identical; `variant`, `workspace` and
 * `workspace_bytes` are appended.  Quantizes Q/K (K mean-smoothed, Q and K
 * channel-balanced, Q in 128-token blocks for variant 0 and 32-token blocks for
 * variant 1, K in 64-token blocks), repacks or quantizes V, runs the attention
 * kernel and writes bf16 O in the caller's strides.
 *
 * workspace == NULL: the library keeps one internal device buffer per (device,
 * stream), grown on demand and never freed (the counterpart of the reference
 * shim's lazily allocated, never-freed workspace, cudnn_sdpa.cpp:218-231); a call
 * that does not grow it allocates nothing, and a call that would have to grow it
 * while its stream is being captured into a graph returns -3.  Otherwise
 * workspace_bytes must be at least mi355_sage_workspace_bytes(...) and the
 * pointer 256-byte aligned; calls that share one workspace must be ordered on one
 * stream.  `causal` != 0 (cudnn_sdpa.cpp:190-192, cuDNN's set_causal_mask): query i sees keys j <= i only,
 * aligned at the top left when N_q != N_kv; the key tiles past a workgroup's last row are never read.
 * ---------------------------------------------------------------------- */
int mi355_sage_sdpa_bf16(
    const void* Q, const void* K, const void* V, void* O,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int causal,
    void* stream,
    int variant, void* workspace, size_t workspace_bytes);

/* mi355_sage_sdpa_bf16 for callers that cannot allocate device memory and hold no workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments and result as mi355_sage_sdpa_bf16; the
 * intermediate tensors live in a buffer of mi355_sage_static_scratch_bytes() bytes (16 MiB) that is
 * part of the loaded library on every GPU, so the call allocates nothing.  A problem whose
 * workspace (mi355_sage_workspace_bytes) exceeds that returns -3.  All calls on one GPU share the
 * buffer: calls that overlap in time on one GPU (different streams, or threads) race. */
int mi355_sage_sdpa_bf16_static(
    const void* Q, const void* K, const void* V, void* O,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int causal,
    void* stream,
    int variant);
size_t mi355_sage_static_scratch_bytes(void);

/* Same with the quantization recipe spelled out: blkq / blkk = tokens per Q / K
 * scale block (32, 64 or 128 each), k_flags = MI355_SAGE_K_SMOOTH | MI355_SAGE_K_BALANCE
 * or a subset. */
int mi355_sage_sdpa_bf16_ex(
    const void* Q, const void* K, const void* V, void* O,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int causal,
    void* stream,
    int variant, int blkq, int blkk, int k_flags,
    void* workspace, size_t workspace_bytes);

/* mi355_sage_sdpa_bf16_ex on the PRE-norm projections: Q and K rows are RMS-normalised with
 * their gains and rotated (interleaved RoPE) on the way into the quantizers, i.e. the three
 * calls rms_norm / rope_interleaved / sdpa of serenitymojo/models/klein/single_block.mojo:977-982
 * in one, with the arithmetic of serenitymojo/ops/norm.mojo:81-114 and ops/rope.mojo:104-122
 * (bf16 stores between the steps included).  Arguments of the fused ops as in
 * mi355_sage_quant_qk_norm_rope_bf16.  V is used as it is.  With tables N_q must equal N_kv
 * (one table row per position, shared by Q and K); otherwise -2. */
int mi355_sage_sdpa_bf16_norm_rope(
    const void* Q, const void* K, const void* V, void* O,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int causal,
    void* stream,
    int variant, int blkq, int blkk, int k_flags,
    const void* q_gain, const void* k_gain, float eps,
    const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
    void* workspace, size_t workspace_bytes);

/* Replaces flame_cudnn_sdpa_bf16_train_fwd (cudnn_sdpa.cpp:470-484), the symbol
 * every Mojo caller binds (serenitymojo/ops/attention_flash.mojo:182-192): same
 * parameter list plus the three trailing arguments.  Stats receives the fp32
 * natural-log log-sum-exp of the scaled scores, layout [B,H,N_q,1] with strides
 * {H*N_q, N_q, 1, 1} (cudnn_sdpa.cpp:304-312).  real_N_kv in (0, N_kv) masks
 * the keys at and beyond it (the padding mask of attention_flash.mojo:275-287);
 * query rows at and beyond real_N_q are computed but carry no meaning. */
int mi355_sage_sdpa_bf16_train_fwd(
    const void* Q, const void* K, const void* V, void* O, void* Stats,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int64_t stats_offset_elems,
    int causal,
    int real_N_q, int real_N_kv,
    void* stream,
    int variant, void* workspace, size_t workspace_bytes);

/* Joint text + image attention with padded text keys masked: replaces sdpa_qwen_keymask
 * (serenitymojo/ops/attention.mojo:1790-1857, kernel :804-870), which keeps the text keys
 * [0, real_txt_len), masks [real_txt_len, N_TXT) and keeps the image keys [N_TXT, S): pass
 * mask_lo = real_txt_len, mask_hi = N_TXT (0 <= mask_lo <= mask_hi <= N_kv; equal = no mask).
 * Masked keys are left out of the scores, of the K statistics and scale blocks, and of the V
 * scales.  Stats may be NULL.  Default recipe of mi355_sage_sdpa_bf16. */
int mi355_sage_sdpa_bf16_keymask(
    const void* Q, const void* K, const void* V, void* O, void* Stats,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems,
    int64_t stats_offset_elems,
    int mask_lo, int mask_hi,
    void* stream,
    int variant, void* workspace, size_t workspace_bytes);

/* Attention with an additive score bias: the native path behind sdpa / sdpa_chunked
 * (serenitymojo/ops/attention.mojo:1596-1647, :1650-1687; mask [B,H,S,S]) and sdpa_cross_masked
 * (:1897-1936; mask [B,H,Sq,Skv]).  Mask: bf16 (the dtype of q, as the reference requires),
 * logical [B,H,N_q,N_kv] through four element strides — the key stride must be 1, rows 8-byte
 * aligned; a stride of 0 broadcasts over batch or head.  The bias is in the units of the scaled
 * scores (softmax(scale * q.k + mask)); -inf (or the reference's -1e4) removes a key for a row.
 * Default recipe of mi355_sage_sdpa_bf16; the K statistics do not look at the mask. */
int mi355_sage_sdpa_bf16_mask(
    const void* Q, const void* K, const void* V, const void* Mask, void* O,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* mask_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t mask_offset_elems, int64_t o_offset_elems,
    void* stream,
    int variant, void* workspace, size_t workspace_bytes);

/* mi355_sage_sdpa_bf16_train_fwd on the pre-norm projections (default recipe: Q blocks of 128
 * tokens, 32 for the e4m3 variant; K blocks of 64; K smoothing and balancing on), for the blocks that run
 * rms_norm / rope_interleaved in front of sdpa_flash_train_fwd
 * (serenitymojo/models/klein/single_block.mojo:977-982 with the flash arm of :102).  Stats is the
 * log-sum-exp of the scores of the normalised, rotated Q and K. */
int mi355_sage_sdpa_bf16_norm_rope_train_fwd(
    const void* Q, const void* K, const void* V, void* O, void* Stats,
    int B, int H, int N_q, int N_kv, int D,
    float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    const int64_t* v_strides, const int64_t* o_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int64_t v_offset_elems, int64_t o_offset_elems, int64_t stats_offset_elems,
    int causal, int real_N_q, int real_N_kv,
    void* stream,
    int variant,
    const void* q_gain, const void* k_gain, float eps,
    const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
    void* workspace, size_t workspace_bytes);

/* Bytes of workspace the one-shot calls need for this problem (0 on bad
 * arguments).  No counterpart in the reference, whose shim sizes its own. */
size_t mi355_sage_workspace_bytes(int B, int H, int N_q, int N_kv, int D, int variant);

/* ------------------------------------------------------------------------
 * Stage entry points (no counterpart in the reference, which has no quantized
 * attention): each kernel of the path in isolation, so that the INT8 codes and
 * fp32 scales can be compared bit-for-bit with a CPU restatement.
 *
 * Quantized tensor layouts (device memory, caller-allocated):
 *   q8      int8  [B, H, pad_q(N_q),  D]   pad rows are 0
 *   qscale  fp32  [B, H, pad_q(N_q)/blkq]  pad blocks are 1.0
 *   k8      int8  [B, H, pad_kv(N_kv), D]   pad rows and masked keys are 0
 *   kscale  fp32  [B, H, pad_kv(N_kv)/blkk]
 *   kmean, qmul, kmul  fp32 [B, H, D]       per-channel mean of K (0 without smoothing) and
 *                                           the multipliers of Q and K (scale*log2(e) and 1
 *                                           without balancing)
 *   v16     fp16  [B, H, pad_kv/64, D, 64]  64-key tiles, channel-major inside a
 *                                           tile, key k of a tile stored at slot
 *                                           mi355_sage_v_slot(k, PV_FP16); masked keys 0
 *   v8      e4m3  [B, H, pad_kv/64, D, 64]  same with mi355_sage_v_slot(k, PV_FP8)
 *   vscale  fp32  [B, H, D]
 * mask_lo / mask_hi: keys mask_lo <= s < mask_hi take no part (0, 0 = none).
 * ---------------------------------------------------------------------- */
int64_t mi355_sage_pad_q(int64_t n);    /* query tokens round up to the query tile  */
int64_t mi355_sage_pad_kv(int64_t n);   /* key tokens round up to 128               */
int     mi355_sage_v_slot(int key_in_tile, int variant);

/* Bytes of scratch mi355_sage_quant_qk_bf16 / _quant_v_fp8 need (per-group partial results). */
size_t mi355_sage_quant_scratch_bytes(int B, int H, int N_kv, int D);

/* Per channel over the kept keys: mean (K_SMOOTH), s_d = sqrt(max|f32(k) - mean|) (K_BALANCE;
 * 1 when that maximum is 0), kmul = 1/s_d, qmul = fp32(scale*log2(e)) * s_d.
 * Q: x = f32(q) * qmul;  K: x = (f32(k) - kmean) * kmul.
 * Per block: amax -> s = amax/127 (1.0 when 0) -> code = clamp(rne(x/s), +-127).
 * kmean, qmul and kmul are always written. */
int mi355_sage_quant_qk_bf16(
    const void* Q, const void* K,
    int B, int H, int N_q, int N_kv, int D, float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    int blkq, int blkk, int k_flags, int mask_lo, int mask_hi,
    void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
    void* scratch, size_t scratch_bytes, void* stream);

/* The same with the two ops the callers run in front of attention fused in: every Q and K row
 * goes through RMSNorm over D with a bf16 gain (serenitymojo/ops/norm.mojo:81-114,
 * out = bf16(x * 1/sqrt(mean(x^2)+eps) * g), squares added in the order of norm.mojo:56-72) and,
 * when tables are given, interleaved RoPE with fp32 tables (serenitymojo/ops/rope.mojo:104-122,
 * pairs (2i, 2i+1), result bf16) before it is quantized — the call order of
 * serenitymojo/models/klein/single_block.mojo:977-981, without the two bf16 round trips through
 * memory.  q_gain, k_gain: bf16 [D].  rope_cos / rope_sin: fp32 [rows, D/2], row = n*H + h
 * (serenitymojo/sampling/klein_sampler.mojo:305-307), batch b starting at row
 * b*rope_batch_rows (0 = one table for all batches); both NULL = norm only.  Q rows and K rows
 * use the same table (self-attention positions), so with tables N_q must equal N_kv (-2
 * otherwise).  rope_layout: MI355_SAGE_ROPE_INTERLEAVED, or MI355_SAGE_ROPE_HALFSPLIT for the
 * pairing (i, i + D/2) of rope_halfsplit (serenitymojo/ops/rope.mojo:147-165; per-head norm +
 * half-split rotation as in serenitymojo/models/anima/block.mojo:360-366), optionally ORed with
 * MI355_SAGE_ROPE_TABLES_BF16 and MI355_SAGE_NORM_FULL_ROW (LTX-2's sequence: RMSNorm over the whole
 * inner dim, half-split rotation with bf16 tables; that statistic takes one more launch and, like
 * the tables, needs N_q == N_kv).  Gains and tables must be 16-byte aligned. */
int mi355_sage_quant_qk_norm_rope_bf16(
    const void* Q, const void* K,
    int B, int H, int N_q, int N_kv, int D, float scale,
    const int64_t* q_strides, const int64_t* k_strides,
    int64_t q_offset_elems, int64_t k_offset_elems,
    const void* q_gain, const void* k_gain, float eps,
    const void* rope_cos, const void* rope_sin, int64_t rope_batch_rows, int rope_layout,
    int blkq, int blkk, int k_flags,
    void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
    void* scratch, size_t scratch_bytes, void* stream);

/* Q, K and V in the three launches the one-shot calls use (V repack or V channel maxima ride
 * with the K statistics, the e4m3 V encode with the Q / K encoders): same outputs, bit for bit, as
 * mi355_sage_quant_qk_bf16 followed by mi355_sage_quant_v_f16 / _fp8, which take five.  vq is v16
 * or v8 by `variant`; vscale is written for MI355_SAGE_PV_FP8 only (may be NULL otherwise).
 * q8 == qscale == NULL: Q is not encoded here (mi355_sage_attn_fwd_q16 does it); qmul is still written.
 * scratch as for mi355_sage_quant_qk_bf16. */
int mi355_sage_quant_qkv_bf16(
    const void* Q, const void* K, const void* V,
    int B, int H, int N_q, int N_kv, int D, float scale,
    const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
    int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
    int variant, int blkq, int blkk, int k_flags, int mask_lo, int mask_hi,
    void* q8, void* qscale, void* k8, void* kscale, void* kmean, void* qmul, void* kmul,
    void* vq, void* vscale,
    void* scratch, size_t scratch_bytes, void* stream);

/* V -> fp16 (round-to-nearest-even, finite overflow saturates), tiled layout. */
int mi355_sage_quant_v_f16(
    const void* V, int B, int H, int N_kv, int D,
    const int64_t* v_strides, int64_t v_offset_elems, int mask_lo, int mask_hi,
    void* v16, void* stream);

/* V -> e4m3 with per-(b,h,channel) scale amax/448 over the kept keys (1.0 when 0), tiled layout. */
int mi355_sage_quant_v_fp8(
    const void* V, int B, int H, int N_kv, int D,
    const int64_t* v_strides, int64_t v_offset_elems, int mask_lo, int mask_hi,
    void* v8, void* vscale, void* scratch, size_t scratch_bytes, void* stream);

/* Attention on the quantized tensors.  kv_valid = number of real keys (<= N_kv); keys beyond
 * it and keys in [mask_lo, mask_hi) are masked.  stats may be NULL; with stats, qshift
 * ([B,H,pad_q(N_q)] fp32, log2 units, may be NULL) is added to every row's log-sum-exp: the
 * amount K smoothing lowered that row's scores by. */
int mi355_sage_attn_fwd(
    const void* q8, const void* qscale, int blkq,
    const void* k8, const void* kscale, int blkk,
    const void* vq, const void* vscale, int variant,
    int B, int H, int N_q, int N_kv, int kv_valid, int mask_lo, int mask_hi, int D,
    void* O, const int64_t* o_strides, int64_t o_offset_elems,
    const void* qshift, void* stats, void* stream);

/* The attention stage as the plain forward (no Stats, no additive mask) runs it: Q comes as bf16
 * (any [B,H,N,D] view with 16-byte aligned rows) together with the channel multipliers `qmul`
 * [B,H,D] of the quantize stage, and the kernel encodes its own rows while its first K / V tiles
 * are on their way — the same codes and scales mi355_sage_quant_qkv_bf16 writes, so O has the
 * same bits as mi355_sage_attn_fwd on that stage's q8 / qscale.  mi355_sage_quant_qkv_bf16 with
 * q8 == qscale == NULL is the quantize stage that goes with it (K and V only, qmul still written).
 * Head dims 64 and 128; a shape that the split schedule takes returns -2 (use mi355_sage_attn_fwd).
 * The rest of the arguments as in mi355_sage_attn_fwd.  (A stage of this library's own; the
 * reference's boundary is the one-shot call, serenitymojo/ops/cshim/cudnn_sdpa.cpp:370-393.) */
int mi355_sage_attn_fwd_q16(
    const void* Q, const int64_t* q_strides, int64_t q_offset_elems, const void* qmul, int blkq,
    const void* k8, const void* kscale, int blkk, const void* vq, const void* vscale, int variant,
    int B, int H, int N_q, int N_kv, int kv_valid, int mask_lo, int mask_hi, int D,
    void* O, const int64_t* o_strides, int64_t o_offset_elems, void* stream);

/* Scheduling of the attention kernel (no counterpart in the reference).
 * One workgroup computes 256 query rows of one head against all keys.  A shape whose row tiles
 * leave the last round of the 256 compute units at most half full (more than 256 tiles, 16 % or
 * more of the launch idle; fp16 variant, head dim up to 128) is instead cut into equal shares of
 * (row tile, key tile) steps for exactly 256 workgroups, which hand unnormalised partial results to
 * each other inside the launch.  The choice depends on the shape only, so all entry points give the
 * same bits for the same problem; outputs of the two schedules differ by rounding (the probabilities
 * of a row are rounded against a different running maximum).  The hand-over relies on workgroup ids
 * being dealt round-robin to 8 XCDs of 32 compute units, so the schedule is used only on a device
 * that reports exactly that (hipDeviceAttributeNumberOfXccs == 8, 256 compute units); on any other
 * partitioning every shape takes one workgroup per row tile.  Its hand-over slots are part of
 * mi355_sage_workspace_bytes for the shapes that qualify (whatever the device); mi355_sage_attn_fwd,
 * which takes no workspace, keeps its slots in a library-owned per-stream buffer (allocated on the
 * first such call of a stream, never while that stream is being captured).
 *
 * A workgroup that does not find a partial result it waits for (a bounded wait: the launch never
 * hangs), or finds it written on another XCD, writes NaN into its rows AND counts a fault on the
 * device.  mi355_sage_attn_split_faults returns the number of such workgroups on the current device
 * since the last reset (0 in a healthy run; negative: a HIP error), and clears the count when
 * `reset` is non-zero.  It copies one word from the device with the blocking HIP call: synchronise
 * the streams whose launches are to be covered first.  No attention call checks the count itself,
 * so none of them synchronises. */
int mi355_sage_attn_split_faults(int reset);

/* Backward.  Replaces flame_cudnn_sdpa_bwd_bf16 (serenitymojo/ops/cshim/cudnn_sdpa_bwd.cpp:325-347;
 * Mojo callers ops/attention_flash.mojo:345-433, :478-535, :538-607): identical parameter list up
 * to `stream`, then the workspace pair.  Q, K, V, O, dO bf16 and dQ, dK, dV bf16, each a logical
 * [B,H,N,D] view through 4 element strides + an element offset; Stats fp32 contiguous [B,H,N_q]
 * (natural-log log-sum-exp, as the train-forward entry points write it).  Computes, without ever
 * storing an N_q x N_kv matrix,
 *     P = exp(scale * Q K^T - Stats),  dV = P^T dO,  dS = P * (dO V^T - rowsum(dO * O)),
 *     dQ = scale * dS K,  dK = scale * dS^T Q
 * in bf16 matrix instructions with fp32 accumulation (no quantization: gradients keep bf16
 * operands).  real_N_q / real_N_kv (0 or >= N: all) are the valid lengths; padding rows and keys
 * take no part and their gradient rows are written as zeros.  causal must be 0.
 * Workspace: mi355_sage_bwd_workspace_bytes(...) bytes, 256-byte aligned, or NULL for the
 * library's per-stream buffer (same rules as the forward).  Unlike the pair handed to cuDNN, O and
 * Stats may come from the quantized forward: the probabilities recomputed here are then not quite
 * the ones O and Stats belong to, and a row of dS no longer sums to zero exactly.  dQ is therefore
 * taken as scale * (dS K - rowsum(dS) c) with c close to the mean key — the same value for a
 * consistent forward, and free of the keys' common offset times that row sum otherwise. */
size_t mi355_sage_bwd_workspace_bytes(int B, int H, int N_q, int N_kv, int D);
int mi355_sage_sdpa_bwd_bf16(
    const void* Q, const void* K, const void* V, const void* O, const void* dO, const void* Stats,
    void* dQ, void* dK, void* dV,
    int B, int H, int N_q, int N_kv, int D, float scale,
    const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
    const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
    const int64_t* dk_strides, const int64_t* dv_strides,
    int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems, int64_t o_offset_elems,
    int64_t do_offset_elems, int64_t stats_offset_elems, int64_t dq_offset_elems,
    int64_t dk_offset_elems, int64_t dv_offset_elems,
    int causal, int real_N_q, int real_N_kv, void* stream,
    void* workspace, size_t workspace_bytes);

/* Library identification: "mi355_sage <version> gfx950". */
const char* mi355_sage_version(void);

#ifdef __cplusplus
}
#endif
#endif
