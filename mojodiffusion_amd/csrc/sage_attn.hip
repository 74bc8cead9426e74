// sage_attn.hip — flash-style attention on quantized operands for gfx950.
//
// One workgroup (8 waves) owns 256 query rows of one (batch, head); wave w owns
// rows 32w..32w+31.  The kernel works on the TRANSPOSED problem so that no
// cross-lane data movement is needed between the two matrix products:
//
//   S^T = K . Q^T      v_mfma_i32_32x32x32_i8   A = K tile (LDS), B = Q^T (registers)
//   O^T = V^T . P^T    v_mfma_f32_32x32x16_f16  A = V^T tile (LDS), B = P^T (registers)
//                      v_mfma_f32_32x32x64_f8f6f4 for the e4m3 variant
//
// In the 32x32 accumulator layout lane l holds column (l & 31) — one query —
// and 16 rows (keys, or output channels) selected by (l >> 5).  Softmax
// statistics, the rescale factor and the normaliser are therefore plain
// per-lane scalars, and the exponentiated scores a lane holds are exactly the
// B-operand fragment of the second product once V^T is stored with its keys in
// the matching slot order (v_slot_f16 / v_slot_fp8).
//
// Pipeline.  K and V^T tiles of 64 keys travel global -> LDS with register-
// bypassing copies (global_load_lds_dwordx4) into rings (K: 4 slots, V^T: 4), two
// iterations ahead of their use; the 16-byte-chunk XOR swizzle is applied on the source
// side of the copy.  Iteration t computes
// the scores of tile t, then interleaves — one matrix instruction, then the
// exponentials of two scores, in program order — the softmax of tile t with
// P.V of tile t-1, so the matrix pipe and the vector ALU of a SIMD run
// together inside one wave; the second wave on the SIMD covers what is left.
// Scores are in the log2 domain (scale*log2(e) is folded into the Q
// quantizer), so the exponential is a bare v_exp_f32.
#include "sage_internal.h"

#include <hip/hip_fp16.h>

#include <atomic>
#include <type_traits>

// Measurement builds only (`make parts`, never part of the library): SAGE_LOOP_PART is a mask of
// parts of the main loop to leave out, so that what each is worth can be read off the kernel's own
// clock stamps (bench.py --clock-probe --probe-lib ...).  Results are wrong by design; every kernel
// still runs to its end (no address and no trip count depends on what is left out).
//   1 no tile copies in the loop   2 no workgroup barrier in the loop   4 no LDS fragment reads
#ifndef SAGE_LOOP_PART
#define SAGE_LOOP_PART 0
#endif
namespace sage {
constexpr int kLoopPart = SAGE_LOOP_PART;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// Byte offset of 16-byte chunk L of a tile.  Chunks are grouped into 128-byte super-rows
// (8 chunks); the chunk position inside a super-row is XORed with bits of the index of
// the PAIR of super-rows it belongs to, so that the 16 lanes the 64-bank LDS serves per
// cycle (16 consecutive rows, one logical column) land in 16 different 16-byte bank groups.
__device__ __forceinline__ int swz(int L) { return (((L >> 3) << 3) | ((L & 7) ^ ((L >> 4) & 7))) << 4; }

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at
// lds_base + 16*l.  Written as assembly on purpose: the compiler then keeps no record of
// an outstanding LDS write and does not put a full vector-memory wait in front of every
// later LDS read; completion is awaited explicitly (dma_wait) before the workgroup
// barrier that publishes the tile.
__device__ __forceinline__ void dma16(const void* gbase_uniform, uint32_t goff, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base_uniform), "v"(goff), "s"(gbase_uniform)
                 : "memory");      // (m0 cannot be named as a clobber: to this compiler it is a reserved register — it
                                   // warns that "clobbering them may lead to undefined behaviour" — which it never
                                   // keeps a value in across statements; its own uses set m0 right before the use)
}
// Wait until at most N of this wave's copies are still in flight (they complete in order).
template <int N> __device__ __forceinline__ void dma_wait() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

// The int32 score accumulators start at the bit pattern of the float 1/(2*pi) instead of 0.
// That pattern is 2^-3 * (1 + 2292099 * 2^-23), so adding an integer dot with
// |dot| < 2292099 (the largest possible |dot| is 128*127*127 = 2064512) changes only the
// mantissa: a finished accumulator, read as fp32, IS the float 1/(2*pi) + dot * 2^-26.  No
// int->float conversion is needed and dequantisation, max subtraction and the exponent
// argument collapse into one FMA per score (the scale carries the factor 2^26).
constexpr int kMagicI = 0x3E22F983;
constexpr float kMagicF = 0.15915494309189532f;        // the same 32 bits
constexpr float kMagicUnit = 67108864.0f;               // 2^26: accumulator-as-float steps per integer
// With 256 channels |dot| can reach 256*127*127 = 4129024, more than the mantissa of 1/(2*pi) has
// room for below it.  0.1875 = 2^-3 * (1 + 2^22 * 2^-23) leaves 2^22 = 4194304 either way at the
// same step of 2^-26.
constexpr int kMagicWideI = 0x3E400000;
constexpr float kMagicWideF = 0.1875f;
// e4m3 variant: a wave whose bias * f can exceed this takes the bias off its accumulators (see exact_bias).
constexpr float kExactBias = 4096.0f;
template <int D> struct Magic {
    static constexpr int I = D > 128 ? kMagicWideI : kMagicI;
    static constexpr float F = D > 128 ? kMagicWideF : kMagicF;
};

// First matrix instruction of a score chain: accumulator input = the constant above, held in 16
// registers for the whole kernel (behind an empty statement, or the compiler re-creates the 16
// copies for every chain).  The instruction could take 1/(2*pi) as an inline operand, but only
// written as assembly, and then the compiler does not know that a matrix instruction is writing
// those registers: it neither keeps the wait states before the first other instruction that
// touches them — a spill store two instructions later wrote the old contents — nor can it be told.
template <int D>
__device__ __forceinline__ v16i magic_splat() {
    constexpr int M = Magic<D>::I;
    v16i c = {M, M, M, M, M, M, M, M, M, M, M, M, M, M, M, M};
    asm volatile("" : "+v"(c));
    return c;
}

// A row's reference maximum is only refreshed (and the accumulators rescaled) when a tile
// exceeds it by more than tau powers of two; until then p = exp2(s - m_used) may reach
// 2^tau.  fp16 P holds 2^8 without loss.  The e4m3 variant maps p = 2^tau to the format
// maximum 448, i.e. it stores e4m3(p * 448 / 2^tau); the factor cancels against the
// normaliser, which sums the same scaled values.  Its reference is always a whole number
// (the maximum rounded up): a probability's e4m3 significand then depends on the fractional
// part of its score only, not on which whole number the reference happens to be, so the
// stored probabilities are those of a softmax taken against ceil(row maximum) up to a power
// of two, and the rescale factors are exact.
template <int VARIANT> struct Lazy {
    static constexpr float tau = VARIANT == 0 ? 8.0f : 1.0f;
    static constexpr float log2_pscale = VARIANT == 0 ? 0.0f : 7.807354922057604f;     // log2(448 / 2)
    static constexpr bool integer_ref = VARIANT == 1;
};

// ADDMASK: an additive score bias (natural-log units, bf16, logical [B,H,Nq,Nkv] through element
// strides with the key stride 1) is added to the dequantised scores.  That instantiation looks
// for every tile's maximum on the biased scores (no optimistic tiles) and lets its ordinary
// global loads share the vector-memory counter with the tile copies, i.e. it waits for all of
// them at the midpoint: it is bound by the N_q x N_kv bias it has to read, not by the copies.
// Workgroups of the split schedule that gave up on a hand-over (see the kernel's fold-in part).
static __device__ unsigned int g_split_faults;

// QF: the kernel takes Q as bf16 (q_src, strides; q8 / qscale unread) and encodes its own 32 rows per
// wave in the prologue — the quantize stage's arithmetic (quant_i8_block), so the codes and scales
// are the ones that stage would have written — which saves the stage a read of Q and a write and
// this kernel's read of the codes.
template <int D, int VARIANT, bool STATS, bool ADDMASK, bool SPLIT, bool QF = false>
__global__ __launch_bounds__(D > 128 ? 256 : 512) void sage_attn_kernel(
    const int8_t* __restrict__ q8, const float* __restrict__ qscale, int blkq,
    const uint16_t* __restrict__ q_src, int64_t qsb, int64_t qsh, int64_t qsn, const float* __restrict__ qmul,
    const int8_t* __restrict__ k8, const float* __restrict__ kscale, int blkk,
    const uint8_t* __restrict__ vq, const float* __restrict__ vscale,
    const float* __restrict__ qshift,
    int H, int Nq, int kv_valid_all, int mask_lo, int mask_hi, int causal, int64_t nq_pad, int64_t nkv_pad,
    uint16_t* __restrict__ o, int64_t osb, int64_t osh, int64_t osn,
    float* __restrict__ stats, int n_qtiles, int total_wg,
    const uint16_t* __restrict__ amask, int64_t amb, int64_t amh, int64_t amn,
    int split_groups, float* split_part, int* split_flags, int split_wait) {
    constexpr int KS_OFF = VARIANT == 0 ? 3 : 2;        // see lds_ks
    constexpr int VB = (VARIANT == 0) ? 2 : 1;          // bytes per V element
    constexpr int KSTEPS = D / 32;                      // int8 MFMA steps over the head dim
    constexpr int DB = D / 32;                          // 32-channel output blocks
    constexpr int K_BYTES = kTileKV * D;                // K tile
    constexpr int V_BYTES = D * kTileKV * VB;           // V^T tile
    // 256 channels: the output accumulators alone take 128 registers per lane, so a wave gets a SIMD
    // to itself (up to 512 registers) and a workgroup is 4 waves = 128 query rows.
    constexpr int NW = D > 128 ? 4 : 8;                 // waves per workgroup
    constexpr int THREADS = NW * 64;
    constexpr int ROWS_WG = NW * 32;                    // query rows per workgroup
    constexpr int K_NCH = K_BYTES / 1024, V_NCH = V_BYTES / 1024;      // 1 KiB copies per tile
    constexpr int K_CH = (K_NCH + NW - 1) / NW;         // copies per wave (short tiles: some waves repeat a copy)
    constexpr int V_CH = (V_NCH + NW - 1) / NW;
    constexpr int LEAD = D > 128 ? 1 : 2;               // tile copies run this many iterations ahead (LDS: 160 KiB)
    // ring depths: the tile in use, LEAD tiles published or in flight, and the slot the next copy
    // goes to — for K the tile whose scores are being computed is t+1, for V^T the tile in use is t-1.
    // (Up to 128 channels that is four slots each, so slot numbers are a mask away.)
    constexpr int NSK = LEAD + 2, NSV = LEAD + 2;
    constexpr int K_CPR = D / 16;                       // chunks per K row
    constexpr int V_CPR = kTileKV * VB / 16;            // chunks per V^T row
    constexpr int VROW = kTileKV * VB;                  // bytes per V^T row
    constexpr int JS = VARIANT == 0 ? 4 : 1;            // PV steps over the 64 keys of a tile
    constexpr int NUNIT = JS * DB;                      // PV matrix instructions per tile
    constexpr int EPU = 32 / NUNIT;                     // scores exponentiated per PV instruction
    constexpr int FPU = VARIANT == 0 ? 1 : 2;           // 16-byte V fragments per PV instruction
    constexpr int PD = VARIANT == 0 ? 2 : 1;            // V fragment prefetch distance (units)
    constexpr int PW = VARIANT == 0 ? 16 : 8;           // dwords of packed P per tile
    static_assert(32 % NUNIT == 0 && (EPU % 2 == 0 || EPU == 1), "unit split");

    __shared__ __attribute__((aligned(1024))) uint8_t lds_k[NSK][K_BYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_v[NSV][V_BYTES];
    __shared__ __attribute__((aligned(16))) float lds_ks[max_keys(D) / 32 + 4];
    __shared__ float lds_qmax[QF ? 8 : 1];              // QF: largest |pre-scaled q| of each wave's 32 rows
    static_assert(!QF || (D <= 128 && !STATS && !ADDMASK && !SPLIT), "Q is encoded in the kernel only in the plain forward");

    // Work items are (q tile, b*h) pairs, `total_wg` of them; an item takes `ntiles` steps (key
    // tiles).  Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; each XCD gets a
    // contiguous range of items, so the workgroups sharing one head's K/V also share one L2.
    //
    // split_groups == 0: one workgroup per item.  Otherwise the XCD's steps, laid end to end, are
    // cut into split_groups equal spans, one per workgroup of that XCD, so that every compute unit
    // gets the same number of steps whatever the item count.  A span covers the tail of one item,
    // whole items, and the head of another.  The workgroup that holds an item's last key tile
    // writes the item's output; the others leave their unnormalised accumulators, reference
    // maxima and row sums in split_part and raise their flag.  A workgroup walks its span from
    // the back, so what it leaves for others it leaves first, and the only workgroups it ever
    // waits for are ones with a lower id in the same XCD — dispatched before it, and not waiting
    // for anybody when they produce what it needs.
    const int bid = blockIdx.x;
    const int xcd = bid & 7, wg_j = bid >> 3;
    const int items_per = (total_wg + 7) >> 3;
    const int xcd_full = total_wg - (items_per - 1) * 8;        // XCDs that own `items_per` items (1..8)
    const int n_items = xcd < xcd_full ? items_per : items_per - 1;
    const int item0 = xcd < xcd_full ? xcd * items_per : xcd_full * items_per + (xcd - xcd_full) * (items_per - 1);
    const int ntiles_item = (kv_valid_all + kTileKV - 1) / kTileKV;
    // (the launcher has checked that steps x workgroups stays inside 32 bits)
    const uint32_t xcd_steps = (uint32_t)n_items * (uint32_t)ntiles_item;
    auto span_lo = [&](int j) -> int {
        return SPLIT ? (int)(xcd_steps * (uint32_t)j / (uint32_t)split_groups) : min(j, n_items) * ntiles_item;
    };
    const int span_begin = span_lo(wg_j);
    int span_end = span_lo(wg_j + 1);

#ifdef SAGE_CLOCK_PROBE
    // Measurement build only (libmi355_sage_probe.so): shader cycles and constant-rate time of
    // this workgroup, written behind the [B,H,Nq] Stats output (the caller sizes the buffer).
    const unsigned long long probe_r0 = __builtin_amdgcn_s_memrealtime();
    const unsigned long long probe_t0 = __builtin_readcyclecounter();
#endif
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- one segment = key tiles [t_off, t_off + ntiles) of one item, last segment of the span first
    // (the instantiation without splitting is straight-line code: one segment, the whole item)
    if (SPLIT && span_end <= span_begin) return;        // an empty span
    do {
    // (divisors through an empty statement: a few divisions per segment are cheaper than their
    // reciprocals kept in registers across the main loop)
    int ntiles_div = ntiles_item, qtiles_div = n_qtiles, heads_div = H;
    if constexpr (SPLIT) asm volatile("" : "+s"(ntiles_div), "+s"(qtiles_div), "+s"(heads_div));
    const int item_local = SPLIT ? (int)((uint32_t)(span_end - 1) / (uint32_t)ntiles_div) : wg_j;
    const int item_base = item_local * ntiles_item;
    const int t_off = SPLIT ? max(span_begin, item_base) - item_base : 0;
    const int wg = item0 + item_local;
    const int qt = (int)((uint32_t)wg % (uint32_t)qtiles_div);
    // Causal (query i sees keys j <= i, cuDNN's top-left alignment): the keys past this workgroup's last
    // row are masked for every one of its rows — they are treated as the ragged end, so their tiles are
    // never copied — and the steps on a wave's diagonal mask key > row element by element (below).
    const int kv_valid = (!SPLIT && causal) ? min(kv_valid_all, (qt + 1) * ROWS_WG) : kv_valid_all;
    const int ntiles = SPLIT ? span_end - item_base - t_off : (kv_valid + kTileKV - 1) / kTileKV;
    const bool seg_finishes = !SPLIT || t_off + ntiles == ntiles_item;   // holds the item's last key tile: writes the output
    span_end = item_base + t_off;
    const int64_t bh = (uint32_t)wg / (uint32_t)qtiles_div;
    const int b = (int)((uint32_t)bh / (uint32_t)heads_div), h = (int)((uint32_t)bh % (uint32_t)heads_div);
    // (through an empty statement: what is derived from the lane number — row addresses, fragment
    // and copy offsets — is formed in the segment that uses it instead of being carried in registers
    // from before the loop over the segments and across the hand-over code at its end)
    int lane = tid & 63;
    if constexpr (SPLIT) asm volatile("" : "+v"(lane));
    const int l32 = lane & 31, half = lane >> 5;
    const int row_in_tile = wave * 32 + l32;
    const int qrow = qt * ROWS_WG + row_in_tile;        // this lane's query (padded index)
    const int wave_row0 = qt * ROWS_WG + wave * 32;     // the wave's first query (the same for all its lanes)
    if constexpr (SPLIT) __syncthreads();               // every wave has left the previous segment's LDS

    // Q^T fragments: 16 bytes of the head dim per step, resident for the whole kernel.
    v4i qf[KSTEPS];
    float sq;
    if constexpr (!QF) {
        const int8_t* qp = q8 + (bh * nq_pad + qrow) * D + half * 16;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) qf[s] = *reinterpret_cast<const v4i*>(qp + s * 32);
        sq = qscale[bh * (nq_pad / blkq) + qrow / blkq] * kMagicUnit;
    }
    // QF: this lane's 16 channels of every 32 (its half of the row), rows past N_q as zeros, and the
    // channel multipliers that go with them
    u32x4 rw[QF ? KSTEPS : 1][2];
    v4f qm[QF ? KSTEPS : 1][4];
    if constexpr (QF) {
        {
            const float* mp = qmul + bh * D + half * 16;
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
#pragma unroll
                for (int j = 0; j < 4; j++) qm[s][j] = *reinterpret_cast<const v4f*>(mp + s * 32 + j * 4);
        }
        {
            const uint16_t* qp = q_src + b * qsb + h * qsh + (int64_t)qrow * qsn + half * 16;
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    rw[s][j] = u32x4{0u, 0u, 0u, 0u};
                    if (qrow < Nq) rw[s][j] = *reinterpret_cast<const u32x4*>(qp + s * 32 + j * 8);
                }
        }
        // (the arithmetic follows further down, behind the first tile copies: their latency and this
        // one's then run side by side)
    }
    // this lane's row of the additive bias (padding rows read the last real row; their output is dropped)
    const uint16_t* mrow = ADDMASK ? amask + b * amb + h * amh + (int64_t)min(qrow, Nq - 1) * amn : nullptr;

    // K scales of this head are staged in LDS once: a global load inside the main loop
    // would make the compiler wait for ALL outstanding vector-memory operations, i.e. for the
    // tile copies that are meant to stay in flight.
    const float* ksc = kscale + bh * (nkv_pad / blkk);
    const int ush = blkk == 32 ? 0 : (blkk == 64 ? 1 : 2);      // log2(32-key blocks per scale block)
    // (staged per 32-key block, KS_OFF entries in: the main loop fetches the eight entries of one trip
    // with two 16-byte reads, and its first entry then sits on a 16-byte boundary)
    for (int i = tid; i < (int)(nkv_pad / 32); i += THREADS) lds_ks[KS_OFF + i] = ksc[i >> ush];
    auto kscale_of = [&](int u32blk) -> float { return lds_ks[KS_OFF + u32blk]; };

    // tile indices below are relative to the segment's first tile
    const uint8_t* kg = reinterpret_cast<const uint8_t*>(k8) + bh * nkv_pad * D + (int64_t)t_off * K_BYTES;
    const uint8_t* vg = vq + bh * nkv_pad * D * VB + (int64_t)t_off * V_BYTES;
    const int last = ntiles - 1;

    // Tile-relative LDS byte offsets of this lane's MFMA A-operand fragments.  Rows
    // 32 apart keep the same swizzle, so the 32-row blocks are plain constant offsets.
    // (held as complete LDS addresses — ring base included — behind an empty statement: a ring slot,
    // key block or channel block is then an immediate offset of the read instruction, at most 61 440,
    // where the compiler, left to fold the bases itself, re-forms addresses past 65 535 in the loop)
    uint32_t koff[KSTEPS], voff[JS * FPU];
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) koff[s] = lds_addr(&lds_k[0][0]) + swz(l32 * K_CPR + s * 2 + half);
    if constexpr (VARIANT == 0) {
#pragma unroll
        for (int j = 0; j < JS; j++) voff[j] = lds_addr(&lds_v[0][0]) + swz(l32 * V_CPR + j * 2 + half);
    } else {
        voff[0] = lds_addr(&lds_v[0][0]) + swz(l32 * V_CPR + half * 2);
        voff[1] = lds_addr(&lds_v[0][0]) + swz(l32 * V_CPR + half * 2 + 1);
    }
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) asm volatile("" : "+v"(koff[s]));
#pragma unroll
    for (int j = 0; j < JS * FPU; j++) asm volatile("" : "+v"(voff[j]));
    typedef const __attribute__((address_space(3))) v4i* lds_v4i_ptr;
    auto k_frag = [&](int slot, int st, int kb) -> v4i { return *reinterpret_cast<lds_v4i_ptr>(koff[st] + (uint32_t)(slot * K_BYTES + kb * 32 * D)); };
    auto v_frag = [&](int slot, int jx, int d) -> v4i { return *reinterpret_cast<lds_v4i_ptr>(voff[jx] + (uint32_t)(slot * V_BYTES + d * 32 * VROW)); };

    // Copy i of wave w fills the 1 KiB run c = (i*8 + w) mod (copies per tile) of a tile (short
    // tiles are covered twice with identical data, which keeps every wave's copy count equal);
    // the lane that fills physical chunk P fetches logical chunk swz^-1(P) (the XOR is its own
    // inverse).
    int ksrc[K_CH], vsrc[V_CH];
    uint32_t kdst[K_CH], vdst[V_CH];
#pragma unroll
    for (int i = 0; i < K_CH; i++) {
        const int c = (i * NW + wave) % K_NCH;
        ksrc[i] = swz(c * 64 + lane);
        kdst[i] = lds_addr(&lds_k[0][0]) + c * 1024;
    }
#pragma unroll
    for (int i = 0; i < V_CH; i++) {
        const int c = (i * NW + wave) % V_NCH;
        vsrc[i] = swz(c * 64 + lane);
        vdst[i] = lds_addr(&lds_v[0][0]) + c * 1024;
    }
    auto dma_k_at = [&](const uint8_t* g, int slot) {
#pragma unroll
        for (int i = 0; i < K_CH; i++) dma16(g, ksrc[i], __builtin_amdgcn_readfirstlane(kdst[i] + slot * K_BYTES));
    };
    auto dma_v_at = [&](const uint8_t* g, int slot) {
#pragma unroll
        for (int i = 0; i < V_CH; i++) dma16(g, vsrc[i], __builtin_amdgcn_readfirstlane(vdst[i] + slot * V_BYTES));
    };
    auto dma_k = [&](int t, int slot) { dma_k_at(kg + (int64_t)t * K_BYTES, slot); };
    auto dma_v = [&](int t, int slot) { dma_v_at(vg + (int64_t)t * V_BYTES, slot); };

    v16f oacc[DB];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[d][i] = 0.0f;
    // reference maximum the exponentials are taken against (log2 domain); finite from the start
    // so that a tile whose keys are all masked (every score -inf) still yields p = 0, not NaN
    float m_used = -3.0e38f;
    float l_run = 0.0f;            // fp16 variant: this lane's share of the row sum
    // e4m3 variant: the row sum is taken over the ROUNDED probabilities, on the matrix pipe — one
    // more product per tile against a tile of ones (e4m3 1.0 = 0x38) gives every lane the sum over
    // all 64 keys of its query, in every accumulator element; element 0 is the one that is kept
    // to scale.  It is rescaled together with the output accumulators.
    v16f lacc;
#pragma unroll
    for (int i = 0; i < 16; i++) lacc[i] = 0.0f;
    const v8i ones8 = {0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838};

    // The main loop advances in STEPS of SK keys: 32 for the fp16 variant (one P.V matrix
    // instruction covers 16 keys), 64 for the e4m3 variant (its matrix instruction covers 64).  A
    // 64-key tile in LDS holds SPT = 64 / SK steps.  Step h is NM matrix-instruction slots: the
    // P.V instructions of step h-1 and the score instructions of step h+1, dealt evenly (fp16:
    // P.V, score, P.V, ...; e4m3: score, score, P.V, ...), each followed by its share of the vector
    // work of step h's softmax.  Every matrix instruction then has independent vector instructions
    // behind it in program order, and the vector ALU never meets a run of matrix instructions with
    // nothing of its own to do (measured on the instruction mix alone, two waves per SIMD:
    // 2060 clocks per 64 keys with the score instructions in a block of their own, 1680 dealt
    // out like this).  Three steps are in flight per wave, yet the scores (two buffers of SK keys)
    // and the packed probabilities (two buffers) take no more registers than one 64-key tile did.
    constexpr int SK = VARIANT == 0 ? 32 : 64;          // keys per step
    constexpr int SKB = SK / 32;                        // 32-key blocks per step
    constexpr int SPT = kTileKV / SK;                   // steps per tile
    constexpr int NQ = KSTEPS * SKB;                    // score matrix instructions per step
    constexpr int NPV = NUNIT / SPT;                    // P.V matrix instructions per step
    constexpr int NM = NQ + NPV;                        // slots per step
    constexpr int OPP = VARIANT == 0 ? 7 : 5;           // vector operations per pair of scores (see vop)
    constexpr int NP = 8 * SKB;                         // pairs of scores per lane and step
    constexpr int NV = NP * OPP;                        // vector operations of a step's softmax
    constexpr int PWS = PW / SPT;                       // dwords of packed P per step
    constexpr int PDS = 2;      // operand fragments are requested this many slots ahead
    constexpr int KOFF = SPT == 1 ? 2 : 1;              // the barrier of tile t publishes K(t + KOFF) and V(t)
    constexpr int PERIOD = 4 * SPT;                     // steps after which ring slots and parity repeat
    // GRP == 3: the operands of three slots are requested together, three to five slots ahead and in
    // reverse order, so that the first of the three matrix instructions waits for the request made
    // last — LDS answers in order — and the other two need no wait instruction at all.
    constexpr int GRP = VARIANT == 0 ? 3 : 1;
    constexpr int PF = GRP > 1 ? GRP : PDS;             // slots whose operands a step finds requested on entry
    static_assert(NM % 3 == 0 && NM / 3 == KSTEPS && PDS <= NM / 2 && (GRP == 1 || GRP == 3), "slot pattern");
    auto slot_is_qk = [](int m) { return VARIANT == 0 ? m % 3 == 1 : m % 3 != 2; };
    // number of the score instruction or of the P.V unit (within the step) in slot m
    auto slot_index = [](int m) {
        if (VARIANT == 0) return m % 3 == 1 ? m / 3 : 2 * (m / 3) + (m % 3) / 2;
        return m % 3 == 2 ? m / 3 : 2 * (m / 3) + m % 3;
    };

    // Loop-carried: the operand fragments of the first PDS slots, the scores of two steps and the
    // packed probabilities of two steps (by parity of the step).
    v4i fr[NM][FPU];
    v16i s[2][SKB];
    const v16i smagic = magic_splat<D>();
    uint32_t p[2][PWS];

    // Operands of slot m of a step whose score instructions read key block `kbq` (fp16 variant; the
    // e4m3 variant reads both blocks) of the K tile in `kslot` and whose P.V instructions read the
    // steps `sub` of the V^T tile in `vslot`.
    auto fetch = [&](int m, int kslot, int kbq, int vslot, int sub) {
        if (kLoopPart & 4) { asm volatile("" : "+v"(fr[m][0])); return; }
        if (slot_is_qk(m)) {
            const int n = slot_index(m), st = SKB == 1 ? n : n >> 1, kb = SKB == 1 ? kbq : n & 1;
            fr[m][0] = k_frag(kslot, st, kb);
        } else {
            const int u = slot_index(m), j = VARIANT == 0 ? 2 * sub + u / DB : 0, d = u % DB;
#pragma unroll
            for (int x = 0; x < FPU; x++)
                fr[m][x] = v_frag(vslot, j * FPU + x, d);
        }
    };
    auto qk_step = [&](int sb, int n, const v4i& a) {
        const int st = SKB == 1 ? n : n >> 1, kb = SKB == 1 ? 0 : n & 1;
        s[sb][kb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qf[st], st == 0 ? smagic : s[sb][kb], 0, 0, 0);
    };
    auto pv_unit = [&](int pb, int u, const v4i (&a)[FPU]) {
        const int jj = u / DB, d = u % DB;
        if constexpr (VARIANT == 0) {
            const v4i pw = {(int)p[pb][jj * 4], (int)p[pb][jj * 4 + 1], (int)p[pb][jj * 4 + 2], (int)p[pb][jj * 4 + 3]};
            oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a[0]),
                                                             __builtin_bit_cast(v8h, pw), oacc[d], 0, 0, 0);
        } else {
            const v8i a8 = {a[0].x, a[0].y, a[0].z, a[0].w, a[1].x, a[1].y, a[1].z, a[1].w};
            const v8i pw = {(int)p[pb][0], (int)p[pb][1], (int)p[pb][2], (int)p[pb][3],
                            (int)p[pb][4], (int)p[pb][5], (int)p[pb][6], (int)p[pb][7]};
            oacc[d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, pw, oacc[d], 0, 0, 0, 0, 0, 0);
            if (u == NPV - 1) lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones8, pw, lacc, 0, 0, 0, 0, 0, 0);
        }
    };

    // ---- prologue: K(0) (.. K(KOFF-1)), then K(x + KOFF), V(x) for x < LEAD into the rings; scores of step 0
    // (tile indices past the end are clamped: the extra copies are in bounds and unused)
#pragma unroll
    for (int x = 0; x < KOFF; x++) dma_k(min(x, last), x % NSK);
#pragma unroll
    for (int x = 0; x < LEAD; x++) {
        dma_k(min(x + KOFF, last), (x + KOFF) % NSK);
        dma_v(min(x, last), x % NSV);
    }
    if constexpr (QF) {
        // ---- Q of this wave's 32 rows -> int8 codes and scale (quant_i8_block's arithmetic)
        float x[KSTEPS][16];
        float am = 0.0f;
        {
#pragma unroll
            for (int s = 0; s < KSTEPS; s++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const v4f m0 = qm[s][2 * j], m1 = qm[s][2 * j + 1];
                    const float m[8] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        x[s][j * 8 + 2 * e] = __uint_as_float(rw[s][j][e] << 16) * m[2 * e];
                        x[s][j * 8 + 2 * e + 1] = __uint_as_float(rw[s][j][e] & 0xFFFF0000u) * m[2 * e + 1];
                        am = fmaxf(fmaxf(am, fabsf(x[s][j * 8 + 2 * e])), fabsf(x[s][j * 8 + 2 * e + 1]));
                    }
                }
        }
        // the row's other half, then the wave's 32 rows, then the waves that share a scale block
        {
            const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(am), __float_as_uint(am), false, false);
            am = fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
        }
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) am = fmaxf(am, __shfl_xor(am, off, 64));
        if (blkq > 32) {
            if (lane == 0) lds_qmax[wave] = am;
            __syncthreads();
            const int nwv = blkq >> 5, w0 = wave & ~(nwv - 1);
            am = lds_qmax[w0];
            for (int w = 1; w < nwv; w++) am = fmaxf(am, lds_qmax[w0 + w]);
        }
        const float sc = am > 0.0f ? am / 127.0f : 1.0f;
        const bool fast = sc >= 0x1p-100f && sc <= 0x1p100f;
        const float rinv = 1.0f / sc;
        float kRound = 12582912.0f, rv = rinv;             // (see quant_i8_block)
        asm volatile("" : "+v"(rv), "+v"(kRound));
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            uint32_t tb[16], wd[4];
            float dm = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float t0 = fmaf(x[s][e], rv, kRound), t1 = fmaf(x[s][e + 1], rv, kRound);
                const float d0 = fmaf(x[s][e], rv, -(t0 - kRound)), d1 = fmaf(x[s][e + 1], rv, -(t1 - kRound));
                dm = fmaxf(fmaxf(dm, fabsf(d0)), fabsf(d1));
                tb[e] = __float_as_uint(t0);
                tb[e + 1] = __float_as_uint(t1);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t lo = __builtin_amdgcn_perm(tb[4 * j + 1], tb[4 * j], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm(tb[4 * j + 3], tb[4 * j + 2], 0x0c0c0400u);
                wd[j] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
            }
            if (__builtin_expect(!fast || __any(!(dm <= 0.5f - 0x1p-16f)), 0)) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int j = 0; j < 4; j++) wd[j] = 0u;
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    float r = rint_quotient(x[s][e], sc, rinv, fast);
                    r = r > 127.0f ? 127.0f : r;
                    r = r < -127.0f ? -127.0f : r;
                    wd[e >> 2] |= ((uint32_t)((int)r) & 0xFFu) << ((e & 3) * 8);
                }
            }
            qf[s] = v4i{(int)wd[0], (int)wd[1], (int)wd[2], (int)wd[3]};
        }
        sq = sc * kMagicUnit;
    }
    dma_wait<LEAD*(K_CH + V_CH)>();
    __syncthreads();
    // The exponent argument is score * f + c0 with c0 = -(bias * f + reference): the constant carries
    // the accumulators' bias times f, and its rounding (half an ulp at that magnitude) shifts every
    // exponent argument of a key block by the same small amount.  An e4m3 probability next to a
    // rounding boundary then lands on the other side of it.  On the workloads' statistics the shift
    // is ~1e-5 and harmless; a wave whose largest bias * f (its rows' Q scale times the largest K
    // scale) would bring it to 1e-4 takes the bias off its accumulators first, in every step (exact:
    // both are multiples of 2^-26 below 2^-2), and its constant is the reference alone.
    bool exact_bias = false;
    if constexpr (VARIANT == 1 && !ADDMASK) {
        float ks_max = 0.0f;
        for (int i = lane; i < (int)(nkv_pad / 32); i += 64) ks_max = fmaxf(ks_max, lds_ks[KS_OFF + i]);
        exact_bias = __any(Magic<D>::F * sq * ks_max > kExactBias);
    }
    {
        v4i k0[NQ];
#pragma unroll
        for (int n = 0; n < NQ; n++) {
            const int st = SKB == 1 ? n : n >> 1, kb = SKB == 1 ? 0 : n & 1;
            k0[n] = k_frag(0, st, kb);
        }
#pragma unroll
        for (int n = 0; n < NQ; n++) qk_step(0, n, k0[n]);
    }
    const int last_step = ntiles * SPT - 1;
#pragma unroll
    for (int m = PF - 1; m >= 0; m--)
        if (slot_is_qk(m)) fetch(m, (1 / SPT) % NSK, 1 % SPT, 0, 0);

    // Step h (X = h & 1, tile t = h / SPT).  On entry: s[X] = scores of step h; (h > 0) p[X^1] = P(h-1);
    // fr[0..PDS) = the first slots' operands; the tiles the step reads are published.  The step
    // computes the scores of step h+1 into s[X^1], adds P(h-1).V(h-1) to the output and turns s[X]
    // into p[X].  The first step of a tile holds the tile's barrier.
    //
    // OPT (fp16 variant, interior steps): the exponentials are taken against the reference
    // maximum as it stands, without looking for the step's maximum first — that removes the
    // max / compare / cross-lane chain from the common path.  A reference that has become too
    // low shows up as a large sum (every p is non-negative, so sum <= 2^12 bounds each
    // p, far inside fp16 range); then the step is redone the careful way.
    //
    // HT >= 0: h modulo 4 * SPT as a compile-time number (both rings have four slots then), so that
    // every ring slot and key block below is a constant and the LDS addresses are register + immediate.
    // HT < 0: h is known at run time only, but for its position in the tile, -1 - HT.
    float kst[8];       // K scales of the eight 32-key blocks of one trip of the main loop
    const uint8_t *kg_trip = kg, *vg_trip = vg;          // K and V^T tile of the trip's first step
    auto step = [&](int h, auto x_tag, auto h_tag, auto first_tag, auto qk_tag) {
        constexpr int X = decltype(x_tag)::value;            // h & 1: selects the score / probability buffers
        constexpr int HT = decltype(h_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;
        constexpr bool DOQK = decltype(qk_tag)::value;       // false in the last step
        constexpr bool OPT = VARIANT == 0 && !FIRST && !ADDMASK;
        constexpr bool TRIP = HT >= 0 && !FIRST;             // a step of the main loop: no masked keys, scales in kst
        static_assert(HT < 0 || (NSK == 4 && NSV == 4), "constant slots need four-slot rings");
        constexpr int SUB = HT >= 0 ? HT % SPT : -1 - HT;    // step within its tile
        static_assert(SUB >= 0 && SUB < SPT, "position in the tile");
        static_assert((SPT == 1 || X == SUB) && (HT < 0 || X == (HT & 1)), "parity of the step");
        const int t = SPT == 2 ? h >> 1 : h;
        // tiles: score operands of step h+1, and of step h+2 (requested at the end of this step);
        // V^T of step h-1, and of step h
        const int tq = (h + 1) / SPT, tq2 = (h + 2) / SPT, tv = (h + SPT - 1) / SPT - 1, tv2 = h / SPT;
        const int slot_kq = HT >= 0 ? ((HT + 1) / SPT) & 3 : tq % NSK, slot_kq2 = HT >= 0 ? ((HT + 2) / SPT) & 3 : tq2 % NSK;
        const int slot_vp = HT >= 0 ? ((HT + 4 * SPT - 1) / SPT) & 3 : (tv + NSV) % NSV, slot_vp2 = HT >= 0 ? (HT / SPT) & 3 : tv2 % NSV;
        constexpr int kbq = (SUB + 1) % SPT, kbq2 = SUB % SPT;            // key block of the scores (fp16 variant)
        constexpr int subv = (SUB + SPT - 1) % SPT, subv2 = SUB;          // step of the V^T tile
        const int slot_kcopy = HT >= 0 ? (HT / SPT + KOFF + LEAD) & 3 : (t + KOFF + LEAD) % NSK;
        const int slot_vcopy = HT >= 0 ? (HT / SPT + LEAD) & 3 : (t + LEAD) % NSV;

        float f[SKB], c0[SKB];
#pragma unroll
        for (int kb = 0; kb < SKB; kb++)
            f[kb] = sq * (TRIP ? kst[((HT + PERIOD - 1) % PERIOD) * SKB + kb] : kscale_of(t_off * 2 + h * SKB + kb));
        // Steps that hold masked keys (the ragged end, the masked range) are rare: a real branch.
        // A masked score becomes -inf (as an integer: below every real accumulator), which the
        // exponent path below turns into p = 0 without any further test.
        const int key0 = t_off * kTileKV + h * SK;
        if (!TRIP && __builtin_expect(key0 + SK > kv_valid || (key0 < mask_hi && key0 + SK > mask_lo) ||
                                      (causal && key0 + SK - 1 > wave_row0), 0)) {
            asm volatile("" ::: "memory");
#pragma unroll
            for (int kb = 0; kb < SKB; kb++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = key0 + kb * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                    if (key >= kv_valid || (key >= mask_lo && key < mask_hi) || (causal && key > qrow)) s[X][kb][i] = (int)0xFF800000;
                }
        }
        // biased scores in the log2 domain, without the reference maximum (ADDMASK only)
        float xs[SKB][ADDMASK ? 16 : 1];
        if constexpr (ADDMASK) {
#pragma unroll
            for (int kb = 0; kb < SKB; kb++) {
                // (the bias of the accumulators is taken off before the multiplication: exact, where
                // folding it into the multiply-add's constant would cost the constant's rounding)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int key = key0 + kb * 32 + g * 8 + half * 4;
                    uint32_t w0 = 0u, w1 = 0u;
                    if (key + 4 <= kv_valid) {
                        const u32x2 w = *reinterpret_cast<const u32x2*>(mrow + key);
                        w0 = w.x; w1 = w.y;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (key + e < kv_valid) (e < 2 ? w0 : w1) |= (uint32_t)mrow[key + e] << ((e & 1) * 16);
                    }
                    const float mv[4] = {__uint_as_float(w0 << 16), __uint_as_float(w0 & 0xFFFF0000u),
                                         __uint_as_float(w1 << 16), __uint_as_float(w1 & 0xFFFF0000u)};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float sdq = (__int_as_float(s[X][kb][g * 4 + e]) - Magic<D>::F) * f[kb];
                        xs[kb][g * 4 + e] = fmaf(mv[e], 1.4426950408889634f, sdq);
                    }
                }
            }
        }
        float corr = 1.0f;
        bool refresh = false;
        // the step's maximum on the raw accumulators (monotone in the score since f > 0), refresh decision
        auto decide = [&](float tau) {
            float mt = -INFINITY;
            if constexpr (ADDMASK) {
#pragma unroll
                for (int kb = 0; kb < SKB; kb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) mt = fmaxf(mt, xs[kb][i]);
            } else
#pragma unroll
            for (int kb = 0; kb < SKB; kb++) {
                int ma = max(max(s[X][kb][0], s[X][kb][1]), s[X][kb][2]);
                int mb = max(max(s[X][kb][3], s[X][kb][4]), s[X][kb][5]);
#pragma unroll
                for (int i = 6; i < 14; i += 4) {
                    ma = max(max(ma, s[X][kb][i]), s[X][kb][i + 1]);
                    mb = max(max(mb, s[X][kb][i + 2]), s[X][kb][i + 3]);
                }
                const int mi = max(max(ma, mb), max(s[X][kb][14], s[X][kb][15]));
                const float mk = mi < 0 ? -INFINITY : (float)(mi - Magic<D>::I) * (f[kb] * (1.0f / kMagicUnit));
                mt = fmaxf(mt, mk);
            }
            const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(mt), __float_as_uint(mt), false, false);
            mt = fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
            refresh = __any(mt > m_used + tau);
            float m_new = m_used;
            if (refresh) m_new = Lazy<VARIANT>::integer_ref ? ceilf(fmaxf(m_used, mt)) : fmaxf(m_used, mt);
            corr = __builtin_amdgcn_exp2f(m_used - m_new);           // 1 when nothing changed
            m_used = m_new;
            l_run *= corr;             // already includes step h-1's probabilities
        };
        if (!OPT) decide(Lazy<VARIANT>::tau);
#pragma unroll
        for (int kb = 0; kb < SKB; kb++) {
            c0[kb] = Lazy<VARIANT>::log2_pscale - fmaf(Magic<D>::F, f[kb], m_used);
        }
        // (e4m3 variant, score scales beyond anything the workloads show: see `exact_bias`; such a wave
        // takes none of its steps through the main loop)
        if constexpr (VARIANT == 1 && !ADDMASK && !TRIP) {
            if (__builtin_expect(exact_bias, 0)) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int kb = 0; kb < SKB; kb++) {
#pragma unroll
                    for (int i = 0; i < 16; i++) s[X][kb][i] = __float_as_int(__int_as_float(s[X][kb][i]) - Magic<D>::F);
                    c0[kb] = Lazy<VARIANT>::log2_pscale - m_used;
                }
            }
        }
        const float l_before = l_run;

        // The softmax of the step as NV single vector operations, so that they can be dealt out over
        // the slots.  Pair k = scores 2k, 2k+1 of this lane (k counts through the key block, then the
        // accumulator element); its operations: exponent argument of either score, the two exponentials,
        // the packing and (fp16 variant) the two additions to the lane's share of the row sum.  The sum
        // is taken over the unrounded probabilities with plain fp32 additions: v_dot2c_f32_f16 on the
        // packed pair would do it in one instruction, but that instruction does not start while a
        // matrix instruction is executing (measured: matrix instruction + two of them = 57 clocks,
        // + two of any other vector instruction = 33), so each one would cost the matrix pipe a bubble.
        float ea[NP][2];
        // Order: the two exponent arguments of pair 0; then per pair k its two exponentials, the
        // exponent arguments of pair k+1, its packing and its additions — an exponential's result is
        // first read two instructions later (read right away it costs a wait state and the latency).
        auto vop = [&](int n) {
            int k, r;
            if (n < 2) { k = 0; r = n; }
            else {
                const int mm = n - 2, kblk = mm / OPP < NP - 1 ? mm / OPP : NP - 1, q = mm - kblk * OPP;
                if (q < 2) { k = kblk; r = 2 + q; }
                else if (kblk < NP - 1) {
                    if (q < 4) { k = kblk + 1; r = q - 2; }
                    else { k = kblk; r = q; }
                } else { k = kblk; r = q + 2; }
            }
            const int kb = k >> 3, i = (2 * k) & 15;
            if (r < 2) {
                if constexpr (ADDMASK) ea[k][r] = xs[kb][i + r] - (m_used - Lazy<VARIANT>::log2_pscale);
                else ea[k][r] = fmaf(__int_as_float(s[X][kb][i + r]), f[kb], c0[kb]);
            } else if (r < 4) {
                ea[k][r - 2] = __builtin_amdgcn_exp2f(ea[k][r - 2]);
            } else if (r == 4) {
                if constexpr (VARIANT == 0) {
                    const v2h pr = {(_Float16)ea[k][0], (_Float16)ea[k][1]};
                    p[X][k] = __builtin_bit_cast(uint32_t, pr);
                    // (pinned: left alone, the compiler moves every conversion of the step behind the
                    // check at its end and keeps all the exponentials in registers until then)
                    asm volatile("" : "+v"(p[X][k]));
                } else {
                    const int w = k >> 1;
                    if (k & 1) p[X][w] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(ea[k][0], ea[k][1], (int)p[X][w], true);
                    else p[X][w] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(ea[k][0], ea[k][1], 0, false);
                    asm volatile("" : "+v"(p[X][w]));
                }
            } else {
                l_run += ea[k][r - 5];
            }
        };

        // At the barrier every wave has finished the previous tile's steps completely, so the ring
        // slots they read are free: publish K(t + KOFF) / V(t), start the copies of K(t + KOFF + LEAD)
        // and V(t + LEAD).
        auto midpoint = [&]() {
            dma_wait<ADDMASK ? 0 : (LEAD - 1) * (K_CH + V_CH)>();
            if (!(kLoopPart & 2)) __syncthreads();
            if (!(kLoopPart & 1)) {
            if constexpr (TRIP) {
                // (the main loop stops early enough that these tiles exist; their addresses are the
                // trip's base plus a constant)
                constexpr int dt = ((HT + PERIOD - 1) % PERIOD + 1 % SPT) / SPT;       // tiles since the trip's first step
                dma_k_at(kg_trip + (dt + KOFF + LEAD) * K_BYTES, slot_kcopy);
                dma_v_at(vg_trip + (dt + LEAD) * V_BYTES, slot_vcopy);
            } else {
                dma_k(min(t + KOFF + LEAD, last), slot_kcopy);
                dma_v(min(t + LEAD, last), slot_vcopy);
            }
            }
        };

#pragma unroll
        for (int m = 0; m < NM; m++) {
            // operands of the slots ahead (past the end: of the next step's first slots)
            auto fetch_slot = [&](int mf) {
                if (mf < NM) {
                    if (slot_is_qk(mf) ? DOQK : !FIRST) fetch(mf, slot_kq, kbq, slot_vp, subv);
                } else {
                    if (!slot_is_qk(mf - NM) || DOQK) fetch(mf - NM, slot_kq2, kbq2, slot_vp2, subv2);
                }
            };
            if constexpr (GRP == 1) {
                fetch_slot(m + PDS);
            } else if (m % GRP == 0) {
#pragma unroll
                for (int g = GRP - 1; g >= 0; g--) fetch_slot(m + GRP + g);
            }
            if (slot_is_qk(m)) {
                if (DOQK) qk_step(X ^ 1, slot_index(m), fr[m][0]);
            } else if (!FIRST) {
                pv_unit(X ^ 1, slot_index(m), fr[m]);
            }
#pragma unroll
            for (int n = m * NV / NM; n < (m + 1) * NV / NM; n++) vop(n);
            if (SUB == 0 && m == NM / 2 - 1) midpoint();
            __builtin_amdgcn_sched_barrier(0);
        }
        if (OPT) {
            // !(x <= bound) also catches an infinite or NaN sum
            if (__builtin_expect(__any(!(l_run - l_before <= 4096.0f)), 0)) {
                l_run = l_before;
                decide(0.0f);
#pragma unroll
                for (int kb = 0; kb < SKB; kb++) c0[kb] = Lazy<VARIANT>::log2_pscale - fmaf(Magic<D>::F, f[kb], m_used);
#pragma unroll
                for (int n = 0; n < NV; n++) vop(n);
            }
        }
        if (!FIRST && __builtin_expect(refresh, 0)) {
            // the accumulators include step h-1 at the old reference; move them to the new one
            // (the empty volatile statement keeps this rare block a real branch)
            asm volatile("" ::: "memory");
#pragma unroll
            for (int d = 0; d < DB; d++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[d][i] *= corr;
            lacc[0] *= corr;
        }
    };

    using T = std::true_type;
    using F = std::false_type;
    using X0 = std::integral_constant<int, 0>;
    using X1 = std::integral_constant<int, 1>;
    using R0 = std::integral_constant<int, -1>;                         // ring slots from h at run time; first step of a tile
    using R1 = std::integral_constant<int, SPT == 2 ? -2 : -1>;         // ... the step of odd h
    // The last step computes no further scores.  (With a single step the first one is also the last;
    // it computes the scores of the clamped copy and nobody reads them.)
    int hs = 1;
    // (the split instantiations sit at the register limit and keep their slots in registers; so do the
    // ones with an additive mask, whose time goes into reading the mask anyway)
    if constexpr (NSK == 4 && NSV == 4 && !SPLIT && !ADDMASK) {
        step(0, X0{}, std::integral_constant<int, 0>{}, T{}, T{});
        // The main loop takes the steps in front of the first masked key (the ragged end, the masked
        // range) without looking for masked keys; the steps after that go through the loop below.
        int clean = (kv_valid - t_off * kTileKV) / SK;
        if (mask_hi > mask_lo && t_off * kTileKV < mask_hi) clean = min(clean, max(mask_lo - t_off * kTileKV, 0) / SK);
        if (exact_bias) clean = 0;
        if (causal) clean = min(clean, (wave_row0 + 1) / SK);       // steps whose every key is <= the wave's first row
        // (... and in front of the last tiles, so that the copies a trip starts need no clamping)
        const int trip_end = min(last_step - SPT * (KOFF + LEAD) + (SPT - 1), clean);
        for (; hs + PERIOD <= trip_end; hs += PERIOD) {
            kg_trip = kg + (int64_t)(hs / SPT) * K_BYTES;
            vg_trip = vg + (int64_t)(hs / SPT) * V_BYTES;
            {
                const v4f* kp = reinterpret_cast<const v4f*>(&lds_ks[KS_OFF + t_off * 2 + hs * SKB]);
                const v4f k0 = kp[0], k1 = kp[1];
                kst[0] = k0.x; kst[1] = k0.y; kst[2] = k0.z; kst[3] = k0.w;
                kst[4] = k1.x; kst[5] = k1.y; kst[6] = k1.z; kst[7] = k1.w;
            }
            step(hs, X1{}, std::integral_constant<int, 1 % PERIOD>{}, F{}, T{});
            step(hs + 1, X0{}, std::integral_constant<int, 2 % PERIOD>{}, F{}, T{});
            step(hs + 2, X1{}, std::integral_constant<int, 3 % PERIOD>{}, F{}, T{});
            step(hs + 3, X0{}, std::integral_constant<int, 4 % PERIOD>{}, F{}, T{});
            if constexpr (PERIOD == 8) {
                step(hs + 4, X1{}, std::integral_constant<int, 5>{}, F{}, T{});
                step(hs + 5, X0{}, std::integral_constant<int, 6>{}, F{}, T{});
                step(hs + 6, X1{}, std::integral_constant<int, 7>{}, F{}, T{});
                step(hs + 7, X0{}, std::integral_constant<int, 0>{}, F{}, T{});
            }
        }
    } else {
        step(0, X0{}, R0{}, T{}, T{});
    }
    // the remaining steps, ring slots from the step number (hs is odd here)
    for (; hs + 1 < last_step; hs += 2) {
        step(hs, X1{}, R1{}, F{}, T{});
        step(hs + 1, X0{}, R0{}, F{}, T{});
    }
    if (hs == last_step) {
        step(hs, X1{}, R1{}, F{}, F{});
    } else if constexpr (SPT == 1) {                    // (with two steps per tile the last step is an odd one)
        if (hs + 1 == last_step) {
            step(hs, X1{}, R1{}, F{}, T{});
            step(hs + 1, X0{}, R0{}, F{}, F{});
        }
    }
    // ---- drain: P.V of the last step ------------------------------------------------------
    auto drain = [&](auto x_tag) {
        constexpr int X = decltype(x_tag)::value;
        v4i vd[NPV][FPU];
        auto read_vd = [&](int u) {
            const int j = VARIANT == 0 ? 2 * (SPT - 1) + u / DB : 0, d = u % DB;
#pragma unroll
            for (int x = 0; x < FPU; x++)
                vd[u][x] = v_frag(last % NSV, j * FPU + x, d);
        };
#pragma unroll
        for (int u = 0; u < PD && u < NPV; u++) read_vd(u);
#pragma unroll
        for (int u = 0; u < NPV; u++) {
            if (u + PD < NPV) read_vd(u + PD);
            pv_unit(X, u, vd[u]);
        }
    };
    if (SPT == 2 || (last_step & 1)) drain(X1{});
    else drain(X0{});

    // Hand-over between workgroups of ONE XCD goes through that XCD's L2, which every compute unit
    // of the XCD reads and writes: the producer only has to wait until its stores have left the
    // compute unit (the vector L1 writes through), the consumer reads past its own L1.  No L2
    // write-back or invalidation — device-scope fences would throw the K/V tiles out of the L2 for
    // everybody.  That both sides sit on the same XCD follows from the round-robin placement of
    // workgroup ids; the flag carries the producer's XCD number so that the consumer can check.
    constexpr int PART_FLOATS = (DB * 16 + 2) * THREADS;    // one workgroup's slot of split_part
    const int my_xcd = SPLIT ? (int)__builtin_amdgcn_s_getreg(20 | (3 << 11)) : 0;     // XCC_ID, bits 3:0
    if (SPLIT && !seg_finishes) {
        // ---- this item ends in another workgroup's span: hand over the running state ----------
        float* part = split_part + (int64_t)bid * PART_FLOATS;
        // (taken through an empty statement so that the store addresses are formed here, not kept
        // in registers from before the loop)
        uint32_t lane_off = (uint32_t)tid;
        asm volatile("" : "+v"(lane_off));
#pragma unroll
        for (int d = 0; d < DB; d++) {
#pragma unroll
            for (int i = 0; i < 16; i++) part[(d * 16 + i) * THREADS + lane_off] = oacc[d][i];
            __builtin_amdgcn_sched_barrier(0);          // one block at a time (keeps the live registers down)
        }
        part[DB * 16 * THREADS + lane_off] = m_used;
        part[DB * 16 * THREADS + THREADS + lane_off] = VARIANT == 0 ? l_run : lacc[0];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // (split_wait < 0: a test of the bounded wait below, in which nobody raises a flag)
        if (tid == 0 && split_wait > 0) __hip_atomic_store(split_flags + bid, 1 + my_xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        continue;
    }
    float poison = 0.0f;
    if (SPLIT && t_off > 0) {
        // ---- fold in what the workgroups before this one computed for the item's earlier tiles
        int need = item_base + t_off;                   // steps [need, end of item) are accounted for
        uint32_t lane_off = (uint32_t)tid;
        asm volatile("" : "+v"(lane_off));
        for (int jp = wg_j - 1; need > item_base && jp >= 0; jp--) {
            const int ps0 = span_lo(jp), ps1 = span_lo(jp + 1);
            if (ps1 <= ps0) continue;                   // an empty span
            const int pb = jp * 8 + xcd;
            // Bounded wait.  The producer runs this part first and waits for nobody, so the flag
            // is normally up long before; if it never comes, or comes from another XCD, the rows
            // are poisoned with NaN rather than left to hang or to read stale data.
            int spins = 0, flag;
            while ((flag = __hip_atomic_load(split_flags + pb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) == 0) {
                if (++spins > (split_wait < 0 ? -split_wait : split_wait)) break;
                __builtin_amdgcn_s_sleep(16);
            }
            asm volatile("" ::: "memory");
            if (flag != 1 + my_xcd) {
                poison = __builtin_nanf("");
                if (tid == 0) atomicAdd(&g_split_faults, 1u);       // what mi355_sage_attn_split_faults reports
            }
            const float* part = split_part + (int64_t)pb * PART_FLOATS;
            auto peer = [&](int idx) { return __hip_atomic_load(part + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
            const float m_p = peer(DB * 16 * THREADS + lane_off), l_p = peer(DB * 16 * THREADS + THREADS + lane_off);
            const float m_new = fmaxf(m_used, m_p);
            const float ca = __builtin_amdgcn_exp2f(m_used - m_new), cb = __builtin_amdgcn_exp2f(m_p - m_new);
            if constexpr (VARIANT == 0) l_run = l_run * ca + l_p * cb;
            else lacc[0] = lacc[0] * ca + l_p * cb;
#pragma unroll
            for (int d = 0; d < DB; d++) {
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[d][i] = oacc[d][i] * ca + peer((d * 16 + i) * THREADS + lane_off) * cb;
                __builtin_amdgcn_sched_barrier(0);
            }
            m_used = m_new;
            need = ps0;
        }
    }

    // ---- epilogue: normalise, bf16 round-to-nearest-even, caller's strides ---------
    float l_tot;
    if constexpr (VARIANT == 0) {
        const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        l_tot = __uint_as_float(r.x) + __uint_as_float(r.y);
    } else {
        l_tot = lacc[0];
    }
    const float inv = 1.0f / l_tot + poison;      // l carries pscale, which cancels the pscale in P
    if (qrow < Nq) {
        uint16_t* op = o + b * osb + h * osh + (int64_t)qrow * osn;
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int ch = d * 32 + g * 8 + half * 4;
                float x[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    x[e] = oacc[d][g * 4 + e];
                    if (VARIANT == 1) x[e] = x[e] * vscale[bh * D + ch + e];
                    x[e] *= inv;
                }
                u32x2 pk;
                pk.x = f32_to_bf16_rne(x[0]) | ((uint32_t)f32_to_bf16_rne(x[1]) << 16);
                pk.y = f32_to_bf16_rne(x[2]) | ((uint32_t)f32_to_bf16_rne(x[3]) << 16);
                *reinterpret_cast<u32x2*>(op + ch) = pk;
            }
        if (STATS && half == 0) {
            // natural-log log-sum-exp of the scaled scores.  With K smoothing every score
            // of a row was lowered by <q, mean>, which the Q quantizer recorded per row.
            const float shift = qshift != nullptr ? qshift[bh * nq_pad + qrow] : 0.0f;
            stats[bh * Nq + qrow] = (m_used + __builtin_amdgcn_logf(l_tot) - Lazy<VARIANT>::log2_pscale + shift) * 0.6931471805599453f;
        }
    }
    } while (SPLIT && span_end > span_begin);       // segments
#ifdef SAGE_CLOCK_PROBE
    if (STATS) {
        __syncthreads();
        const unsigned long long probe_t1 = __builtin_readcyclecounter();
        const unsigned long long probe_r1 = __builtin_amdgcn_s_memrealtime();
        if (tid == 0) {
            float* probe = stats + (int64_t)(total_wg / n_qtiles) * Nq + blockIdx.x * 2;
            probe[0] = (float)(probe_t1 - probe_t0);          // shader clocks
            probe[1] = (float)(probe_r1 - probe_r0);          // 100 MHz ticks
        }
    }
#endif
}

// Polls of a hand-over flag before a workgroup gives up and poisons its rows (about a microsecond
// each: a third of a second, where the longest legitimate wait is a few milliseconds).  Negative:
// test mode — producers raise no flags, consumers give up after that many polls.
static std::atomic<int> g_split_wait{1 << 18};
void attn_split_wait(int polls) { g_split_wait.store(polls == 0 ? (1 << 18) : polls); }

__global__ void split_clear_kernel(int* flags, int n) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) flags[i] = 0;
}

template <int D, int VARIANT>
static hipError_t launch_attn_dv(const AttnArgs& a, hipStream_t st) {
    constexpr int kThreads = D > 128 ? 256 : 512;             // 32 query rows per wave
    const int n_qtiles = (int)(a.nq_pad / (kThreads / 2));
    const int64_t total = (int64_t)n_qtiles * a.B * a.H;
    if (total <= 0 || total > 0x7FFFFFFF) return hipErrorInvalidValue;
    const int split = (D <= 128 && VARIANT == 0 && !a.causal) ? a.split_wgs : 0;
    int* flags = nullptr;
    float* part = nullptr;
    if (split > 0) {
        if (a.split == nullptr || (split & 7)) return hipErrorInvalidValue;
        flags = static_cast<int*>(a.split);
        part = reinterpret_cast<float*>(static_cast<uint8_t*>(a.split) + kSplitFlagBytes);
        // (a kernel, not a memset: the call may be recorded into a graph)
        hipLaunchKernelGGL(split_clear_kernel, dim3(1), dim3(256), 0, st, flags, split);
    }
    dim3 grid((unsigned)(split > 0 ? split : total)), block(kThreads);
#define SAGE_LAUNCH_ATTN2(STATS, ADDMASK, SPLIT)                                                                         \
    hipLaunchKernelGGL((sage_attn_kernel<D, VARIANT, STATS, ADDMASK, SPLIT>), grid, block, 0, st, a.q8, a.qscale, a.blkq, \
                       a.q_src, a.qsb, a.qsh, a.qsn, a.qmul, a.k8, a.kscale, a.blkk, (const uint8_t*)a.vq, a.vscale, a.qshift, a.H, a.Nq, a.kv_valid,          \
                       a.km.lo, a.km.hi, a.causal, a.nq_pad, a.nkv_pad, a.o, a.osb, a.osh, a.osn, a.stats, n_qtiles,               \
                       (int)total, a.amask, a.amb, a.amh, a.amn, split >> 3, part, flags, g_split_wait.load())
#define SAGE_LAUNCH_ATTN(STATS, ADDMASK)                                  \
    do {                                                                  \
        if constexpr (D <= 128 && VARIANT == 0) {                         \
            if (split > 0) SAGE_LAUNCH_ATTN2(STATS, ADDMASK, true);       \
            else SAGE_LAUNCH_ATTN2(STATS, ADDMASK, false);                \
        } else {                                                          \
            SAGE_LAUNCH_ATTN2(STATS, ADDMASK, false);                     \
        }                                                                 \
    } while (0)
    if (a.q_src != nullptr) {
        // Q encoded by the kernel: the plain forward only
        if constexpr (D <= 128) {
            if (a.amask != nullptr || a.stats != nullptr || split > 0 || a.qmul == nullptr) return hipErrorInvalidValue;
            hipLaunchKernelGGL((sage_attn_kernel<D, VARIANT, false, false, false, true>), grid, block, 0, st, nullptr, nullptr, a.blkq,
                               a.q_src, a.qsb, a.qsh, a.qsn, a.qmul, a.k8, a.kscale, a.blkk, (const uint8_t*)a.vq, a.vscale, nullptr,
                               a.H, a.Nq, a.kv_valid, a.km.lo, a.km.hi, a.causal, a.nq_pad, a.nkv_pad, a.o, a.osb, a.osh, a.osn, nullptr,
                               n_qtiles, (int)total, nullptr, 0, 0, 0, 0, nullptr, nullptr, g_split_wait.load());
        } else {
            return hipErrorInvalidValue;
        }
    } else if (a.amask != nullptr) {
        if (a.stats != nullptr) SAGE_LAUNCH_ATTN(true, true);
        else SAGE_LAUNCH_ATTN(false, true);
    } else {
        if (a.stats != nullptr) SAGE_LAUNCH_ATTN(true, false);
        else SAGE_LAUNCH_ATTN(false, false);
    }
#undef SAGE_LAUNCH_ATTN
#undef SAGE_LAUNCH_ATTN2
    return hipGetLastError();
}

// ---- split scheduling: when, and over how many workgroups -------------------------------------
// One workgroup per item runs in ceil(items / 256) rounds on the 256 compute units (a workgroup
// fills one).  When the last round is at most half full and leaves 16 % or more of the launch's
// compute-unit time idle, the steps are spread over exactly 256 workgroups instead.  Measured on
// an MI355X (one-shot call, D = 128): 323 items -13 %, 576 items -11 %, 640 items -5 %, 320 items
// of 32 steps -6 %; under 3 % either way at 400, 432 and 864 items (last round 56 %, 69 %, 38 %
// full) and at 1584 items (seven rounds): a partly filled round runs at a higher clock — the chip
// is power-limited under this kernel — and every hand-over costs a second prologue and 132 KB
// each way.  Twice as many workgroups (two per compute unit, one after the other) were slower
// everywhere but at 1584 items.  The decision depends on the shape only, so every entry point
// produces the same bits for the same problem.
static std::atomic<int> g_split_mode{0};       // 0: by shape and device; -1: never; n > 0: always, over n workgroups

void attn_split_override(int mode) { g_split_mode.store(mode); }

static bool split_fits(int B, int H, int Nq, int kv_valid, int D, int variant) {
    if (D > 128) return false;                 // four-wave workgroups: one per item
    if (variant != 0) return false;            // the e4m3 loop has no registers left for the hand-over
    const int64_t items = pad_to(Nq, kTileQ) / kTileQ * B * H;
    const int64_t ntiles = (kv_valid + kTileKV - 1) / kTileKV;
    return (items / 8 + 1) * ntiles * kSplitMaxWorkgroups < (int64_t)1 << 31;       // 32-bit step arithmetic in the kernel
}

int attn_split_rule(int B, int H, int Nq, int kv_valid, int D, int variant) {
#ifdef SAGE_CLOCK_PROBE
    return 0;                                  // the measurement build reports per-item clocks
#else
    if (!split_fits(B, H, Nq, kv_valid, D, variant)) return 0;
    const int64_t items = pad_to(Nq, kTileQ) / kTileQ * B * H;
    const int64_t ntiles = (kv_valid + kTileKV - 1) / kTileKV;
    constexpr int64_t kUnits = 256;
    if (items <= kUnits) return 0;
    const int64_t rounds = (items + kUnits - 1) / kUnits;
    const int64_t in_last = items - (rounds - 1) * kUnits;     // 1..256 workgroups in the last round
    if (in_last * 2 > kUnits) return 0;                        // more than half full
    if ((kUnits - in_last) * 100 < rounds * kUnits * 16) return 0;     // idle share under 16 %
    if (items * ntiles < kUnits * 16) return 0;                // spans too short to be worth the hand-over
    return (int)kUnits;
#endif
}

// The hand-over goes through one XCD's L2 and relies on workgroup ids being dealt round-robin to 8
// XCDs of 32 compute units: asked of the device once, and the schedule stays off anywhere else.
static bool split_topology_ok() {
    static std::atomic<int> known[64];         // 0: not asked yet, 1: yes, 2: no
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    int k = known[dev].load();
    if (k == 0) {
        int xccs = 0, cus = 0;
        const bool ok = hipDeviceGetAttribute(&xccs, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess &&
                        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
                        xccs == 8 && cus == 256;
        k = ok ? 1 : 2;
        known[dev].store(k);
    }
    return k == 1;
}

int attn_split_workgroups(int B, int H, int Nq, int kv_valid, int D, int variant) {
#ifdef SAGE_CLOCK_PROBE
    return 0;
#else
    const int mode = g_split_mode.load();
    if (mode < 0) return 0;
    if (mode > 0) return split_fits(B, H, Nq, kv_valid, D, variant) ? mode : 0;    // (tests force it whatever the device)
    const int n = attn_split_rule(B, H, Nq, kv_valid, D, variant);
    return n > 0 && split_topology_ok() ? n : 0;
#endif
}

int attn_split_faults(int reset) {
    unsigned n = 0;
    hipError_t e = hipMemcpyFromSymbol(&n, HIP_SYMBOL(g_split_faults), sizeof(n));
    if (e == hipSuccess && reset) {
        const unsigned zero = 0;
        e = hipMemcpyToSymbol(HIP_SYMBOL(g_split_faults), &zero, sizeof(zero));
    }
    if (e != hipSuccess) return -(int)e;
    return n > 0x7FFFFFFFu ? 0x7FFFFFFF : (int)n;
}

size_t attn_split_bytes(int workgroups, int D) {
    if (workgroups <= 0) return 0;
    return kSplitFlagBytes + (size_t)workgroups * ((D / 32) * 16 + 2) * (D > 128 ? 256 : 512) * sizeof(float);
}

hipError_t launch_attn(const AttnArgs& a, hipStream_t st) {
    if (a.nkv_pad > max_keys(a.D)) return hipErrorInvalidValue;      // K scales would not fit the LDS staging
    if (a.D == 128) return a.variant == 0 ? launch_attn_dv<128, 0>(a, st) : launch_attn_dv<128, 1>(a, st);
    if (a.D == 64) return a.variant == 0 ? launch_attn_dv<64, 0>(a, st) : launch_attn_dv<64, 1>(a, st);
    if (a.D == 256) return a.variant == 0 ? launch_attn_dv<256, 0>(a, st) : launch_attn_dv<256, 1>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace sage
