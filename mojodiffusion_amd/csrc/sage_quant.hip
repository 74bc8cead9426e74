// sage_quant.hip — HBM-bound kernels of the quantized-SDPA path (gfx950), three launches:
//
//   prep_kernel         per (b,h), workgroup roles:  V repack to tiled fp16  |  V channel
//                       maxima per 256-token group (e4m3 variant)  |  K channel sums (fp64),
//                       minima and maxima per 256-token group
//   stats_final_kernel  per (b,h,channel): K mean, balancing factor -> kmean, qmul, kmul;
//                       V maxima -> vscale
//   quant_kernel        per (b,h), workgroup roles:  Q blocks -> int8 + scale  |  K blocks ->
//                       int8 + scale  |  V tiles -> e4m3 (e4m3 variant)
//
// Every fp32 step that decides a code is a single IEEE operation (true divide, IEEE sqrt,
// round-half-to-even) and every reduction either has a fixed order (the fp64 sums) or is
// order-free (max / min), so codes, scales and statistics are reproducible bit for bit.
// All kernels read bf16 rows with 16-byte loads (8 channels per lane).
#include "sage_internal.h"

#include <hip/hip_fp16.h>

namespace sage {

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

// Running maximum of the magnitudes of bf16 pairs, as 16-bit integers: of one order with the values
// themselves, infinities and NaNs on top (>= 0x7F80).  One packed instruction per pair.
__device__ __forceinline__ uint32_t bf16_mag_max(uint32_t acc, uint32_t pair) {
    const u16x2 m = __builtin_elementwise_max(__builtin_bit_cast(u16x2, acc), __builtin_bit_cast(u16x2, pair & 0x7FFF7FFFu));
    return __builtin_bit_cast(uint32_t, m);
}
__device__ __forceinline__ bool bf16_mag_finite(uint32_t acc) { return (acc & 0xFFFFu) < 0x7F80u && (acc >> 16) < 0x7F80u; }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

__device__ __forceinline__ void unpack8(const u32x4& w, float* x) {
    x[0] = bf16_lo(w.x); x[1] = bf16_hi(w.x);
    x[2] = bf16_lo(w.y); x[3] = bf16_hi(w.y);
    x[4] = bf16_lo(w.z); x[5] = bf16_hi(w.z);
    x[6] = bf16_lo(w.w); x[7] = bf16_hi(w.w);
}

__device__ __forceinline__ void load8(const float* p, float* x) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x0040u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float round_to_bf16(float f) { return __uint_as_float(f32_to_bf16_rne(f) << 16); }

__device__ __forceinline__ bool key_kept(int s, int N, const KeyMask& m) { return s < N && !(s >= m.lo && s < m.hi); }

// RMSNorm (+ RoPE) of one row, spread over the D/8 consecutive lanes that hold its 16-byte
// chunks: x[0..7] are channels col..col+7.  Every lane of the group must call this (it
// exchanges partial sums); `valid` false = a padding row, which stays zero.
// Arithmetic, step for step (all fp32, no fused multiply-add):
//   the squares are added in the order of serenitymojo/ops/norm.mojo:56-72 — a 256-slot array
//   folded in halves, far pairs first: channel t with t+64 (D = 128), then strides 32, 16 and
//   8, which pair lanes of the row, then 4, 2, 1 inside the lane;
//   inv = 1/sqrt(sum/D + eps); y = bf16((x*inv)*gain); rotation of (y[2i], y[2i+1]) by
//   the table angle with both products rounded before the subtract / add; result bf16.
//   (p.halfsplit: the pairs are (y[i], y[i + D/2]) instead.)
template <int D>
__device__ __forceinline__ void pre_apply(const PreOp& p, int b, int h, int H, int row, int col, bool valid, float* x) {
    constexpr int CPR = D / 8;
    float sq[8];
#pragma unroll
    for (int e = 0; e < 8; e++) sq[e] = x[e] * x[e];
#pragma unroll
    for (int off = CPR / 2; off > 0; off >>= 1)
#pragma unroll
        for (int e = 0; e < 8; e++) sq[e] = sq[e] + __shfl_xor(sq[e], off, 64);
#pragma unroll
    for (int e = 0; e < 4; e++) sq[e] = sq[e] + sq[e + 4];
    sq[0] = sq[0] + sq[2];
    sq[1] = sq[1] + sq[3];
    const float a = sq[0] + sq[1];
    const float mean = a / (float)D;
    float inv = 1.0f / sqrtf(mean + p.eps);
    const uint16_t* gain = p.gain;
    if (p.row_inv != nullptr) {
        // the statistic of the whole token (all heads), computed by launch 0; gain of H*D entries
        inv = valid ? p.row_inv[(int64_t)b * p.row_n + row] : 0.0f;
        gain += h * D;
    }
    const u32x4 gw = *reinterpret_cast<const u32x4*>(gain + col);
    float g[8];
    unpack8(gw, g);
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float t = x[e] * inv;
        y[e] = round_to_bf16(t * g[e]);
    }
    if (p.cos != nullptr && p.halfsplit) {
        // pairs (i, i + D/2): the partner channel sits in the lane CPR/2 further on (or back) among
        // the CPR lanes of this row; both lanes of a pair use table entries (col mod D/2) .. +7
        float yp[8];
#pragma unroll
        for (int e = 0; e < 8; e++) yp[e] = __shfl_xor(y[e], CPR / 2, 64);
        const bool upper = col >= D / 2;
        float cv[8], sv[8];
#pragma unroll
        for (int e = 0; e < 8; e++) cv[e] = 1.0f, sv[e] = 0.0f;
        if (valid) {
            const int64_t trow = (int64_t)b * p.batch_rows + (int64_t)row * H + h;
            const int64_t ti = trow * (D / 2) + (col & (D / 2 - 1));
            if (p.tables_bf16) {
                unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.cos) + ti), cv);
                unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.sin) + ti), sv);
            } else {
                const float* pc = p.cos + ti;
                const float* ps = p.sin + ti;
                const float4 c0 = *reinterpret_cast<const float4*>(pc), c1 = *reinterpret_cast<const float4*>(pc + 4);
                const float4 s0 = *reinterpret_cast<const float4*>(ps), s1 = *reinterpret_cast<const float4*>(ps + 4);
                cv[0] = c0.x; cv[1] = c0.y; cv[2] = c0.z; cv[3] = c0.w; cv[4] = c1.x; cv[5] = c1.y; cv[6] = c1.z; cv[7] = c1.w;
                sv[0] = s0.x; sv[1] = s0.y; sv[2] = s0.z; sv[3] = s0.w; sv[4] = s1.x; sv[5] = s1.y; sv[6] = s1.z; sv[7] = s1.w;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            // lower half: x0*c - x1*s with x0 = own, x1 = partner; upper half: x1*c + x0*s with x1 = own
            const float own = y[e] * cv[e], oth = yp[e] * sv[e];
            x[e] = round_to_bf16(upper ? own + oth : own - oth);
        }
    } else if (p.cos != nullptr) {
        float4 c4 = {1.f, 1.f, 1.f, 1.f}, s4 = {0.f, 0.f, 0.f, 0.f};
        if (valid) {
            const int64_t trow = (int64_t)b * p.batch_rows + (int64_t)row * H + h;
            if (p.tables_bf16) {
                const u32x2 cw = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(p.cos) + trow * (D / 2) + col / 2);
                const u32x2 sw = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(p.sin) + trow * (D / 2) + col / 2);
                c4 = float4{__uint_as_float(cw.x << 16), __uint_as_float(cw.x & 0xFFFF0000u), __uint_as_float(cw.y << 16), __uint_as_float(cw.y & 0xFFFF0000u)};
                s4 = float4{__uint_as_float(sw.x << 16), __uint_as_float(sw.x & 0xFFFF0000u), __uint_as_float(sw.y << 16), __uint_as_float(sw.y & 0xFFFF0000u)};
            } else {
                c4 = *reinterpret_cast<const float4*>(p.cos + trow * (D / 2) + col / 2);
                s4 = *reinterpret_cast<const float4*>(p.sin + trow * (D / 2) + col / 2);
            }
        }
        const float cv[4] = {c4.x, c4.y, c4.z, c4.w}, sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float y0 = y[2 * i], y1 = y[2 * i + 1];
            const float p00 = y0 * cv[i], p11 = y1 * sv[i], p01 = y0 * sv[i], p10 = y1 * cv[i];
            x[2 * i] = round_to_bf16(p00 - p11);
            x[2 * i + 1] = round_to_bf16(p01 + p10);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = y[e];
    }
    if (!valid) {
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = 0.0f;
    }
}

// ---------------------------------------------------------------------------
// Per-block INT8 quantization.  One workgroup (256 threads) per block of BLK tokens of one
// (b,h); the BLK x D tile lives in registers between the absmax pass and the encode pass, so
// HBM sees one read of bf16 and one write of int8.
// ---------------------------------------------------------------------------
// Q (IS_K false): x = f32(q) * chmul[d].  K (IS_K true): x = (f32(k) - mean[d]) * chmul[d];
// tokens that are masked or beyond N count for nothing and get code 0.
// rowdot (Q only, may be null): <f32(q) * cmul, mean> per row.
template <int D, int BLK, bool IS_K, bool PRE, int NT>
__device__ __forceinline__ void quant_i8_block(
    int t, int h, int b, const uint16_t* __restrict__ x, int64_t sb, int64_t sh, int64_t sn,
    int N, int H, int64_t n_pad, const KeyMask& km, const float* __restrict__ mean,
    const float* __restrict__ chmul, float cmul,
    int8_t* __restrict__ codes, float* __restrict__ scales, float* __restrict__ rowdot, float* red,
    const PreOp& pre) {
    constexpr int CPR = D / 8;                 // 16-byte chunks per row
    constexpr int NCH = BLK * CPR / NT;        // chunks per thread
    static_assert(BLK * CPR % NT == 0, "tile must split evenly over the threads");
    static_assert(NT % CPR == 0, "a thread keeps one column group for all its chunks");
    const int tid = threadIdx.x;
    const int r0 = t * BLK;
    const int col = (tid % CPR) * 8;
    const int64_t bh = (int64_t)b * H + h;
    const uint16_t* src = x + b * sb + h * sh;

    u32x4 raw[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int row = r0 + (i * NT + tid) / CPR;
        raw[i] = u32x4{0u, 0u, 0u, 0u};
        if (row < N) raw[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)row * sn + col);
    }
    float mul[8], mu[8];
    load8(chmul + col, mul);
    if (IS_K || rowdot != nullptr) load8(mean + col, mu);

    float v[NCH][8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int row = r0 + (i * NT + tid) / CPR;
        unpack8(raw[i], v[i]);
        if constexpr (PRE) pre_apply<D>(pre, b, h, H, row, col, row < N, v[i]);
        bool counts;
        if (IS_K) {
            counts = key_kept(row, N, km);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float d = v[i][e] - mu[e];
                v[i][e] = d * mul[e];
            }
        } else {
            counts = row < N;
            if (rowdot != nullptr) {
                // <pre-scaled query row, K mean>: the amount K smoothing lowers every score
                // of this row by; the CPR lanes that share a row are adjacent in the wave.
                float dot = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) dot += (v[i][e] * cmul) * mu[e];
#pragma unroll
                for (int off = CPR / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
                if ((tid % CPR) == 0) rowdot[bh * n_pad + row] = dot;
            }
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] *= mul[e];
        }
        if (counts) {
#pragma unroll
            for (int e = 0; e < 8; e += 2) amax = fmaxf(fmaxf(amax, fabsf(v[i][e])), fabsf(v[i][e + 1]));
        }
    }

    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = red[0];
#pragma unroll
    for (int w = 1; w < NT / 64; w++) amax = fmaxf(amax, red[w]);

    const float sc = amax > 0.0f ? amax / 127.0f : 1.0f;      // blocks without a counting token: amax == 0
    if (tid == 0) scales[bh * (n_pad / BLK) + t] = sc;
    const bool fast = sc >= 0x1p-100f && sc <= 0x1p100f;
    const float rinv = 1.0f / sc;

    uint32_t pk[NCH][2];
    float far[NCH] = {};        // per 16-byte chunk: how close the thread's products come to a rounding tie
    bool all_careful = PRE || !fast;
    if constexpr (!PRE) {
        // The common case, three operations per element and no test: t = x * rinv + 1.5 * 2^23 in one
        // fused step IS rint of the exact product p, as an integer in the low bits of t (its lowest
        // byte is the code: |p| <= 127 (1 + 2^-22) for every token that counts, so nothing needs
        // clamping); d = p minus that integer.  p differs from the true quotient by at most
        // 128 * 2^-24 (the rounding of rinv) and the true quotient is itself rounded by at most
        // 2^-18, so wherever |d| <= 1/2 - 2^-16 all three round to the same integer.  The largest
        // |d| of each chunk of eight is looked at after the loop: a chunk in which some lane of the
        // wave comes closer to a tie is encoded again with the true quotient (about one chunk in
        // seventy).  A NaN takes no part in any maximum and ends as code 0 here as there; an infinite
        // input makes the scale infinite, and such a block is encoded with the true quotient throughout.
        float kRound = 12582912.0f;                            // 1.5 * 2^23
        float rv = rinv;
        // (vector registers: the operations below then carry neither a scalar operand nor a literal,
        // and issue at the short rate)
        asm volatile("" : "+v"(rv), "+v"(kRound));
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int row = r0 + (i * NT + tid) / CPR;
            const bool counts = IS_K ? key_kept(row, N, km) : row < N;
            uint32_t tb[8];
            float dm = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const float t0 = fmaf(v[i][e], rv, kRound), t1 = fmaf(v[i][e + 1], rv, kRound);
                const float d0 = fmaf(v[i][e], rv, -(t0 - kRound)), d1 = fmaf(v[i][e + 1], rv, -(t1 - kRound));
                dm = fmaxf(fmaxf(dm, fabsf(d0)), fabsf(d1));
                tb[e] = __float_as_uint(t0);
                tb[e + 1] = __float_as_uint(t1);
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint32_t lo = __builtin_amdgcn_perm(tb[4 * j + 1], tb[4 * j], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm(tb[4 * j + 3], tb[4 * j + 2], 0x0c0c0400u);
                pk[i][j] = counts ? __builtin_amdgcn_perm(hi, lo, 0x05040100u) : 0u;
            }
            far[i] = counts ? dm : 0.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        if (__builtin_expect(all_careful || __any(!(far[i] <= 0.5f - 0x1p-16f)), 0)) {
            asm volatile("" ::: "memory");
            const int row = r0 + (i * NT + tid) / CPR;
            pk[i][0] = pk[i][1] = 0u;
            if (IS_K ? key_kept(row, N, km) : row < N) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    float r = rint_quotient(v[i][e], sc, rinv, fast);
                    r = r > 127.0f ? 127.0f : r;               // (comparisons: a NaN stays one; the conversion instruction makes it 0)
                    r = r < -127.0f ? -127.0f : r;
                    pk[i][e >> 2] |= ((uint32_t)((int)r) & 0xFFu) << ((e & 3) * 8);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int row = r0 + (i * NT + tid) / CPR;
        *reinterpret_cast<u32x2*>(codes + (bh * n_pad + row) * D + col) = u32x2{pk[i][0], pk[i][1]};
    }
}

// ---------------------------------------------------------------------------
// K channel statistics of one group of 256 tokens.  Sums follow a fixed tree, all in fp64:
//   leaf  = 16 consecutive tokens, added in ascending order by one lane
//   group = 16 consecutive leaves, added in ascending order
//   total = groups added in ascending order (stats_final_kernel)
// Tokens that are masked or beyond N add +0.0 and take no part in the minimum / maximum.
// Executed by 16*(D/8) consecutive threads; `tid` is the index among them; g < 0: idle.
// ---------------------------------------------------------------------------
template <int D>
struct KGroupSmem {
    double leafsum[16][D + 2];
    float leafmin[16][D + 1];
    float leafmax[16][D + 1];
};

// D is the number of channels this call covers, starting at channel col0 of a head of DFULL
// channels (the statistics are per channel, so a 256-channel head is done as two windows of 128).
template <int D, bool PRE, int DFULL = D>
__device__ __forceinline__ void kstats_group_body(
    int g, int h, int b, int tid, const uint16_t* __restrict__ k, int64_t sb, int64_t sh, int64_t sn,
    int N, int H, int ngroups, const KeyMask& km, double* __restrict__ part_sum, float* __restrict__ part_mm,
    KGroupSmem<D>& sm, const PreOp& pre, int col0 = 0) {
    static_assert(!PRE || DFULL == D, "the fused pre-ops need the whole row in one call");
    constexpr int CPR = D / 8;
    const int leaf = tid / CPR, col = (tid % CPR) * 8;
    const uint16_t* src = k + b * sb + h * sh + col0 + col;
    const int s0 = g * kGroup + leaf * kLeaf;

    u32x4 w[kLeaf];
#pragma unroll
    for (int i = 0; i < kLeaf; i++) {
        w[i] = u32x4{0u, 0u, 0u, 0u};
        if (g >= 0 && key_kept(s0 + i, N, km)) w[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)(s0 + i) * sn);
    }
    double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float mn[8], mx[8], xprev[8];
#pragma unroll
    for (int e = 0; e < 8; e++) { mn[e] = INFINITY; mx[e] = -INFINITY; xprev[e] = 0.0f; }
    // every token of this leaf counts (no ragged end, no masked range inside it)
    const bool all_kept = g >= 0 && s0 + kLeaf <= N && !(s0 < km.hi && s0 + kLeaf > km.lo);
    static_assert(kLeaf % 2 == 0, "tokens are taken in pairs");
#pragma unroll
    for (int i = 0; i < kLeaf; i++) {
        float x[8];
        unpack8(w[i], x);
        const bool kept = g >= 0 && key_kept(s0 + i, N, km);
        if constexpr (PRE) pre_apply<D>(pre, b, h, H, s0 + i, col, kept, x);
        // tokens that do not count are +0.0 here, which leaves a double sum unchanged
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += (double)x[e];
        if (all_kept) {
            // (the common case, two tokens per three-operand instruction; written as instructions because the
            // compiler puts a canonicalising v_max in front of every operand of fminf / fmaxf that comes out of
            // bit operations — six instructions per element instead of one)
            if (i & 1) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    asm("v_min3_f32 %0, %0, %1, %2" : "+v"(mn[e]) : "v"(xprev[e]), "v"(x[e]));
                    asm("v_max3_f32 %0, %0, %1, %2" : "+v"(mx[e]) : "v"(xprev[e]), "v"(x[e]));
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) xprev[e] = x[e];
            }
        } else if (kept) {
#pragma unroll
            for (int e = 0; e < 8; e++) { mn[e] = fminf(mn[e], x[e]); mx[e] = fmaxf(mx[e], x[e]); }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
        sm.leafsum[leaf][col + e] = acc[e];
        sm.leafmin[leaf][col + e] = mn[e];
        sm.leafmax[leaf][col + e] = mx[e];
    }
    __syncthreads();
    if (tid < D && g >= 0) {
        double gsum = 0.0;
        float gmn = INFINITY, gmx = -INFINITY;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            gsum += sm.leafsum[u][tid];
            gmn = fminf(gmn, sm.leafmin[u][tid]);
            gmx = fmaxf(gmx, sm.leafmax[u][tid]);
        }
        const int64_t o = (((int64_t)b * H + h) * ngroups + g) * DFULL + col0 + tid;
        part_sum[o] = gsum;
        part_mm[2 * o] = gmn;
        part_mm[2 * o + 1] = gmx;
    }
}

// ---------------------------------------------------------------------------
// V repack: bf16 [.., N, D] -> fp16 tiles [.., N/64, D, 64]; key k of a tile goes to slot
// v_slot_f16(k).  One workgroup per (tile, h, b): rows are read coalesced, staged in LDS and
// written back channel-major in 16-byte runs.  Rows that are masked or beyond N become 0.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint16_t f32_to_f16_sat(float x) {
    x = fminf(fmaxf(x, -65504.0f), 65504.0f);
    return __half_as_ushort(__float2half_rn(x));
}

// LDS tile: 64 slots x D halves, unpadded; the 16-byte chunk index of a row is XORed with
// 2*(slot/8) so that both the row-wise 16-byte writes and the column-wise dword reads below
// touch every bank once (D = 128: 16 chunks; D = 64: 8 chunks, XOR with slot/8 instead).
template <int D>
__device__ __forceinline__ int v_tile_chunk(int slot, int chunk) {
    // (D = 256: 32 chunks, XOR with 4*(slot/8))
    return D == 256 ? (chunk ^ (((slot >> 3) & 7) << 2)) : D == 128 ? (chunk ^ (((slot >> 3) & 7) << 1)) : (chunk ^ ((slot >> 3) & 7));
}

template <int D>
__device__ __forceinline__ void quant_v_f16_body(
    int t, int h, int b, const uint16_t* __restrict__ v, int64_t sb, int64_t sh, int64_t sn,
    int N, int H, int64_t n_pad, const KeyMask& km, uint16_t* __restrict__ out, uint16_t* tile) {
    constexpr int CPR = D / 8;
    const int tid = threadIdx.x;
    const uint16_t* src = v + b * sb + h * sh;
    u32x4 raw[64 * CPR / 256];
#pragma unroll
    for (int i = 0; i < 64 * CPR / 256; i++) {
        const int c = i * 256 + tid;
        const int key = c / CPR, col = (c % CPR) * 8;
        const int row = t * 64 + key;
        raw[i] = u32x4{0u, 0u, 0u, 0u};
        if (key_kept(row, N, km)) raw[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)row * sn + col);
    }
#pragma unroll
    for (int i = 0; i < 64 * CPR / 256; i++) {
        const int c = i * 256 + tid;
        const int key = c / CPR, chunk = c % CPR;
        float x[8];
        unpack8(raw[i], x);
        u32x4 o;
        o.x = f32_to_f16_sat(x[0]) | ((uint32_t)f32_to_f16_sat(x[1]) << 16);
        o.y = f32_to_f16_sat(x[2]) | ((uint32_t)f32_to_f16_sat(x[3]) << 16);
        o.z = f32_to_f16_sat(x[4]) | ((uint32_t)f32_to_f16_sat(x[5]) << 16);
        o.w = f32_to_f16_sat(x[6]) | ((uint32_t)f32_to_f16_sat(x[7]) << 16);
        const int slot = v_slot_f16(key);
        *reinterpret_cast<u32x4*>(&tile[slot * D + v_tile_chunk<D>(slot, chunk) * 8]) = o;
    }
    __syncthreads();
    uint16_t* dst = out + ((((int64_t)b * H + h) * (n_pad / 64)) + t) * (int64_t)(D * 64);
    // work item = (channel pair, 8 consecutive slots): eight dword reads, two 16-byte stores
    const uint32_t* tile32 = reinterpret_cast<const uint32_t*>(tile);
#pragma unroll
    for (int i = 0; i < (D / 2) * 8 / 256; i++) {
        const int c = i * 256 + tid;
        const int dp = c >> 3, s0 = (c & 7) * 8;            // channels 2*dp, 2*dp+1
        uint32_t w[8];
#pragma unroll
        for (int e = 0; e < 8; e++)
            w[e] = tile32[(s0 + e) * (D / 2) + v_tile_chunk<D>(s0 + e, dp >> 2) * 4 + (dp & 3)];
        u32x4 lo, hi;
        lo.x = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u); hi.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
        lo.y = __builtin_amdgcn_perm(w[3], w[2], 0x05040100u); hi.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
        lo.z = __builtin_amdgcn_perm(w[5], w[4], 0x05040100u); hi.z = __builtin_amdgcn_perm(w[5], w[4], 0x07060302u);
        lo.w = __builtin_amdgcn_perm(w[7], w[6], 0x05040100u); hi.w = __builtin_amdgcn_perm(w[7], w[6], 0x07060302u);
        *reinterpret_cast<u32x4*>(dst + (2 * dp) * 64 + s0) = lo;
        *reinterpret_cast<u32x4*>(dst + (2 * dp + 1) * 64 + s0) = hi;
    }
}

// ---------------------------------------------------------------------------
// V channel maxima of one group of 256 tokens (e4m3 variant; max is order-free).
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void v_absmax_group_body(
    int g, int h, int b, const uint16_t* __restrict__ v, int64_t sb, int64_t sh, int64_t sn,
    int N, int H, int ngroups, const KeyMask& km, float* __restrict__ part, float (*red)[D + 1]) {
    constexpr int CPR = D / 8;
    constexpr int ROWS = 256 / CPR;                        // rows covered per step
    const int tid = threadIdx.x;
    const int col = (tid % CPR) * 8, r = tid / CPR;
    const uint16_t* src = v + b * sb + h * sh + col;
    float m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 4
    for (int i = 0; i < kGroup / ROWS; i++) {
        const int row = g * kGroup + i * ROWS + r;
        if (key_kept(row, N, km)) {
            u32x4 w = *reinterpret_cast<const u32x4*>(src + (int64_t)row * sn);
            float x[8];
            unpack8(w, x);
#pragma unroll
            for (int e = 0; e < 8; e++) m[e] = fmaxf(m[e], fabsf(x[e]));
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) red[r][col + e] = m[e];
    __syncthreads();
    if (tid < D) {
        float mm = 0.0f;
        for (int i = 0; i < ROWS; i++) mm = fmaxf(mm, red[i][tid]);
        part[(((int64_t)b * H + h) * ngroups + g) * D + tid] = mm;
    }
}

// fp32 -> e4m3fn, round-to-nearest-even, saturating at +-448, NaN -> +-0.
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
    const uint32_t u = __float_as_uint(x);
    const uint32_t sign = (u >> 24) & 0x80u;
    float a = fabsf(x);
    if (!(a == a)) return sign;
    a = fminf(a, 448.0f);
    uint32_t byte;
    if (a < 0.015625f) {                                   // below 2^-6: quantum 2^-9
        byte = (uint32_t)(int)rintf(a * 512.0f);           // 0..8; 8 is exactly code 0x08
    } else {
        const uint32_t au = __float_as_uint(a);
        // keep 3 mantissa bits, round half to even on the 20 dropped bits
        uint32_t r = au + 0x7FFFFu + ((au >> 20) & 1u);
        r >>= 20;                                          // (biased exp << 3) | mant3, carry included
        byte = r - ((127u - 7u) << 3);
        if (byte > 0x7Eu) byte = 0x7Eu;
    }
    return byte | sign;
}

// V tile -> e4m3 with the per-channel scales, tiled layout (slot order v_slot_fp8).
//
// The code of an element is e4m3(RN(x / sc)).  The common case takes neither a divide nor the
// conversion in integer arithmetic: with y = RN(1 / sc) (one true divide per channel and thread),
// q0 = RN(x y), r = x - q0 sc (exact in one fused step) and q1 = RN(q0 + r y), q1 IS the correctly
// rounded quotient (Markstein's correction step; it needs y correctly rounded, q0 within an ulp
// and the significand of sc not all ones), and the conversion instruction rounds to nearest even
// and reaches 448 exactly where the quotient's magnitude is 448 (1 + 2^-23) at most, which the
// scale guarantees.  A wave that sees a non-finite input, or a scale outside the range where none
// of this can underflow, or with an all-ones significand, takes the plain formula.
template <int D, int NT>
__device__ __forceinline__ void quant_v_fp8_body(
    int t, int h, int b, const uint16_t* __restrict__ v, int64_t sb, int64_t sh, int64_t sn,
    int N, int H, int64_t n_pad, const KeyMask& km, const float* __restrict__ vscale,
    uint8_t* __restrict__ out, uint8_t* tile) {
    constexpr int CPR = D / 8;
    constexpr int LD = D + 16;                             // padded row (bytes)
    constexpr int NCH = 64 * CPR / NT;
    static_assert(NT % CPR == 0, "a thread keeps one column group for all its chunks");
    const int tid = threadIdx.x;
    const int64_t bh = (int64_t)b * H + h;
    const uint16_t* src = v + b * sb + h * sh;
    const int col = (tid % CPR) * 8;
    u32x4 w[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int row = t * 64 + (i * NT + tid) / CPR;
        w[i] = u32x4{0u, 0u, 0u, 0u};
        if (key_kept(row, N, km)) w[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)row * sn + col);
    }
    float sc[8], y[8];
    load8(vscale + bh * D + col, sc);
    bool plain = false;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        y[e] = 1.0f / sc[e];
        plain = plain || !(sc[e] >= 0x1p-60f && sc[e] <= 0x1p60f) || (__float_as_uint(sc[e]) & 0x7FFFFFu) == 0x7FFFFFu;
    }
    uint32_t mag = 0u;
#pragma unroll
    for (int i = 0; i < NCH; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) mag = bf16_mag_max(mag, w[i][e]);
    plain = __any(plain || !bf16_mag_finite(mag));
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int key = (i * NT + tid) / CPR;
        float x[8];
        unpack8(w[i], x);
        uint32_t pk[2] = {0u, 0u};
        if (__builtin_expect(plain, 0)) {
#pragma unroll
            for (int e = 0; e < 8; e++) pk[e >> 2] |= f32_to_e4m3(x[e] / sc[e]) << ((e & 3) * 8);
        } else {
            float q[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                // (the residual as -(q0 sc - x): an input of -0 then stays -0 through both steps, as it
                // does through the divide)
                const float q0 = x[e] * y[e];
                q[e] = fmaf(-fmaf(q0, sc[e], -x[e]), y[e], q0);
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                int p2 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j], q[4 * j + 1], 0, false);
                p2 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j + 2], q[4 * j + 3], p2, true);
                pk[j] = (uint32_t)p2;
            }
        }
        *reinterpret_cast<u32x2*>(&tile[v_slot_fp8(key) * LD + col]) = u32x2{pk[0], pk[1]};
    }
    __syncthreads();
    uint8_t* dst = out + ((bh * (n_pad / 64)) + t) * (int64_t)(D * 64);
    // output chunk = (channel d, 16 consecutive slots)
#pragma unroll
    for (int i = 0; i < D * 4 / NT; i++) {
        const int c = i * NT + tid;
        const int d = c >> 2, s0 = (c & 3) * 16;
        uint32_t pk[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int e = 0; e < 16; e++) pk[e >> 2] |= (uint32_t)tile[(s0 + e) * LD + d] << ((e & 3) * 8);
        *reinterpret_cast<u32x4*>(dst + d * 64 + s0) = u32x4{pk[0], pk[1], pk[2], pk[3]};
    }
}

// ---------------------------------------------------------------------------
// Launch 1: independent passes over V and K as workgroup roles of one grid (one launch fills
// the chip where each pass alone is too short to).
// ---------------------------------------------------------------------------
template <int D, bool PRE>
__global__ __launch_bounds__(256) void prep_kernel(PrepArgs a) {
    constexpr int DK = D > 128 ? 128 : D;                 // channels per K statistics call
    constexpr int GPW = 256 / (16 * (DK / 8));            // K groups per workgroup (D = 256: one group, one half of the channels)
    union Smem {
        uint16_t tile[64 * D];
        float red[256 / (D / 8)][D + 1];
        KGroupSmem<DK> kg[GPW];
    };
    __shared__ __attribute__((aligned(16))) Smem sm;
    // Consecutive workgroups take the same unit of consecutive heads: in [.., N, H, D] memory those
    // are neighbours, so the workgroups in flight together read whole DRAM pages between them.  The
    // K-statistics units (longer) are dealt evenly among the V units instead of coming last.
    const int per_bh = a.nv_units + a.nk_wg;
    const int bh = blockIdx.x % a.n_bh, slot = blockIdx.x / a.n_bh;
    const int k_before = (int)(((int64_t)slot * a.nk_wg) / per_bh);
    const bool is_k = (int)(((int64_t)(slot + 1) * a.nk_wg) / per_bh) > k_before;
    const int r = is_k ? a.nv_units + k_before : slot - k_before;
    const int b = bh / a.H, h = bh % a.H;
    if (r < a.nv_units) {
        if (a.vmode == 0)
            quant_v_f16_body<D>(r, h, b, a.v.p, a.v.sb, a.v.sh, a.v.sn, a.Nkv, a.H, a.nkv_pad, a.km, a.v16, sm.tile);
        else
            v_absmax_group_body<D>(r, h, b, a.v.p, a.v.sb, a.v.sh, a.v.sn, a.Nkv, a.H, a.ngroups, a.km, a.vpart, sm.red);
    } else if constexpr (D > 128) {
        const int u = r - a.nv_units;                     // (group, channel half)
        kstats_group_body<DK, false, D>(u >> 1, h, b, threadIdx.x, a.k.p, a.k.sb, a.k.sh, a.k.sn, a.Nkv, a.H, a.ngroups,
                                        a.km, a.kpart_sum, a.kpart_mm, sm.kg[0], a.pre_k, (u & 1) * DK);
    } else {
        const int sub = threadIdx.x / (16 * (D / 8));
        const int g = (r - a.nv_units) * GPW + sub;
        // groups past the end still take part in the barrier inside; they read nothing and
        // store nothing
        kstats_group_body<D, PRE>(g < a.ngroups ? g : -1, h, b, threadIdx.x % (16 * (D / 8)), a.k.p, a.k.sb, a.k.sh,
                                  a.k.sn, a.Nkv, a.H, a.ngroups, a.km, a.kpart_sum, a.kpart_mm, sm.kg[sub], a.pre_k);
    }
}

// ---------------------------------------------------------------------------
// Launch 0: whole-row RMSNorm statistic.  One workgroup of 256 threads per token, exactly the
// reference's reduction (serenitymojo/ops/norm.mojo:56-72): thread t adds the squares of
// channels t, t+256, ... in turn (multiply and add rounded separately), then the 256 partial
// sums fold in halves through LDS, far pairs first.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void row_inv_kernel(View q, View k, int H, int Nq, int Nkv, int D, int rows_q, float eps,
                                                      float* __restrict__ inv_q, float* __restrict__ inv_k) {
    __shared__ float part[256];
    const int tid = threadIdx.x;
    int r = blockIdx.x;
    const bool is_k = r >= rows_q;
    if (is_k) r -= rows_q;
    const View& x = is_k ? k : q;
    const int N = is_k ? Nkv : Nq;
    const int b = r / N, n = r % N;
    const uint16_t* row = x.p + b * x.sb + (int64_t)n * x.sn;
    const int cols = H * D;
    float local = 0.0f;
    for (int c = tid; c < cols; c += 256) {
        const float v = __uint_as_float((uint32_t)row[(int64_t)(c / D) * x.sh + (c % D)] << 16);
        const float sq = v * v;
        local = local + sq;
    }
    part[tid] = local;
    __syncthreads();
    for (int active = 128; active > 0; active >>= 1) {
        if (tid < active) part[tid] = part[tid] + part[tid + active];
        __syncthreads();
    }
    if (tid == 0) {
        const float mean = part[0] / (float)cols;
        (is_k ? inv_k : inv_q)[r] = 1.0f / sqrtf(mean + eps);
    }
}

hipError_t launch_row_inv(const View& q, const View& k, int B, int H, int Nq, int Nkv, int D, float eps,
                          float* inv_q, float* inv_k, hipStream_t st) {
    const int64_t rows_q = (int64_t)B * Nq, rows = rows_q + (int64_t)B * Nkv;
    if (rows > 0x7FFFFFFF) return hipErrorInvalidValue;
    hipLaunchKernelGGL(row_inv_kernel, dim3((unsigned)rows), dim3(256), 0, st, q, k, H, Nq, Nkv, D, (int)rows_q, eps, inv_q, inv_k);
    return hipGetLastError();
}

hipError_t launch_prep(const PrepArgs& a_in, int B, int D, hipStream_t st) {
    PrepArgs a = a_in;
    a.ngroups = (a.Nkv + kGroup - 1) / kGroup;
    // K groups per workgroup: 2 at D = 64, 1 at D = 128; at D = 256 a group takes two workgroups
    a.nk_wg = a.kpart_sum == nullptr ? 0 : D == 256 ? a.ngroups * 2 : D == 128 ? a.ngroups : (a.ngroups + 1) / 2;
    a.nv_units = a.vmode == 0 ? (int)(a.nkv_pad / 64) : (a.vmode == 1 ? a.ngroups : 0);
    a.n_bh = B * a.H;
    const int64_t total = (int64_t)B * a.H * (a.nv_units + a.nk_wg);
    if (total == 0) return hipSuccess;
    if (total > 0x7FFFFFFF) return hipErrorInvalidValue;
    dim3 grid((unsigned)total), block(256);
    const bool has_pre = a.pre_k.gain != nullptr;
    if (D == 128 && has_pre) hipLaunchKernelGGL((prep_kernel<128, true>), grid, block, 0, st, a);
    else if (D == 128) hipLaunchKernelGGL((prep_kernel<128, false>), grid, block, 0, st, a);
    else if (D == 64 && has_pre) hipLaunchKernelGGL((prep_kernel<64, true>), grid, block, 0, st, a);
    else if (D == 64) hipLaunchKernelGGL((prep_kernel<64, false>), grid, block, 0, st, a);
    else if (D == 256 && !has_pre) hipLaunchKernelGGL((prep_kernel<256, false>), grid, block, 0, st, a);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Launch 2: one thread per (b, h, channel).
//   K: sum of the group sums in group order -> mean = fp32(sum / kept) (0 without smoothing);
//      amax = max(|kmax - mean|, |kmin - mean|) — rounding is monotone, so this IS the largest
//      |k - mean| over the kept keys; s = sqrt(amax) (1 when amax is 0 or without balancing);
//      kmul = 1/s, qmul = cmul*s.
//   V: vscale = amax/448 (1 when 0).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void stats_final_kernel(FinalArgs a) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;      // (bh, d)
    if (i >= a.total) return;
    const int64_t bh = i / a.D;
    const int d = (int)(i % a.D);
    if (a.kmean != nullptr) {
        float mean = 0.0f, s = 1.0f;
        if (a.kpart_sum != nullptr) {
            const double* p = a.kpart_sum + bh * a.ngroups * a.D + d;
            const float* q = a.kpart_mm + 2 * (bh * a.ngroups * a.D + d);
            double sum = 0.0;
            float mn = INFINITY, mx = -INFINITY;
            // loads 32 groups at a time (all independent, in flight together); sums strictly in group order
            constexpr int NB = 32;
            for (int g0 = 0; g0 < a.ngroups; g0 += NB) {
                double v[NB];
                float lo[NB], hi[NB];
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const int64_t g = g0 + j < a.ngroups ? g0 + j : a.ngroups - 1;
                    v[j] = p[g * a.D];
                    lo[j] = q[2 * g * a.D];
                    hi[j] = q[2 * g * a.D + 1];
                }
#pragma unroll
                for (int j = 0; j < NB; j++)
                    if (g0 + j < a.ngroups) { sum += v[j]; mn = fminf(mn, lo[j]); mx = fmaxf(mx, hi[j]); }
            }
            if (a.flags & 1) mean = (float)(sum / (double)a.kept);
            if (a.flags & 2) {
                const float amax = fmaxf(fabsf(mx - mean), fabsf(mn - mean));
                if (amax > 0.0f) s = sqrtf(amax);
            }
        }
        a.kmean[i] = mean;
        a.kmul[i] = 1.0f / s;
        a.qmul[i] = a.cmul * s;
    }
    if (a.vscale != nullptr) {
        const float* p = a.vpart + bh * a.ngroups * a.D + d;
        float amax = 0.0f;
        // (32 loads in flight at a time: taken one by one, each waits out a memory latency)
        constexpr int NB = 32;
        for (int g0 = 0; g0 < a.ngroups; g0 += NB) {
            float v[NB];
#pragma unroll
            for (int j = 0; j < NB; j++) v[j] = p[(int64_t)(g0 + j < a.ngroups ? g0 + j : a.ngroups - 1) * a.D];
#pragma unroll
            for (int j = 0; j < NB; j++) amax = fmaxf(amax, v[j]);
        }
        a.vscale[i] = amax > 0.0f ? amax / 448.0f : 1.0f;
    }
}

hipError_t launch_stats_final(const FinalArgs& a, hipStream_t st) {
    if (a.total <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(stats_final_kernel, dim3((unsigned)((a.total + 63) / 64)), dim3(64), 0, st, a);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Launch 3: Q blocks, K blocks and (e4m3 variant) V tiles as workgroup roles.
// ---------------------------------------------------------------------------
// Threads per workgroup (512 at 128 channels, i.e. fewer registers and more waves per SIMD, measured slower).
template <int D, bool PRE> constexpr int quant_threads() { return 256; }

template <int D, bool PRE>
__global__ __launch_bounds__(256) void quant_kernel(QuantArgs a) {
    constexpr int NT = quant_threads<D, PRE>();
    union Smem {
        float red[NT / 64];
        uint8_t tile8[64 * (D + 16)];
        uint16_t tile16[64 * D];
    };
    __shared__ __attribute__((aligned(16))) Smem sm;
    // consecutive workgroups take the same rows of consecutive heads: in [.., N, H, D] memory those
    // are neighbours, so the workgroups in flight together read whole DRAM pages between them
    const int bh = blockIdx.x % a.n_bh, r = blockIdx.x / a.n_bh;
    const int b = bh / a.H, h = bh % a.H;
    const KeyMask none{0, 0};
    if (r < a.nq_blk) {
        const float* mul = a.qmul + (int64_t)bh * D;
        const float* mean = a.kmean + (int64_t)bh * D;
#define SAGE_Q(BLK) quant_i8_block<D, BLK, false, PRE, NT>(r, h, b, a.q.p, a.q.sb, a.q.sh, a.q.sn, a.Nq, a.H, a.nq_pad, none, \
                                                       mean, mul, a.cmul, a.q8, a.qscale, a.rowdot, sm.red, a.pre_q)
        if (a.blkq == 128) SAGE_Q(128);
        else if (a.blkq == 64) SAGE_Q(64);
        else SAGE_Q(32);
#undef SAGE_Q
    } else if (r < a.nq_blk + a.nk_blk) {
        const int t = r - a.nq_blk;
        const float* mul = a.kmul + (int64_t)bh * D;
        const float* mean = a.kmean + (int64_t)bh * D;
#define SAGE_K(BLK) quant_i8_block<D, BLK, true, PRE, NT>(t, h, b, a.k.p, a.k.sb, a.k.sh, a.k.sn, a.Nkv, a.H, a.nkv_pad, a.km, \
                                                      mean, mul, 0.0f, a.k8, a.kscale, nullptr, sm.red, a.pre_k)
        if (a.blkk == 128) SAGE_K(128);
        else if (a.blkk == 64) SAGE_K(64);
        else SAGE_K(32);
#undef SAGE_K
    } else if (a.v16 != nullptr) {
        quant_v_f16_body<D>(r - a.nq_blk - a.nk_blk, h, b, a.v.p, a.v.sb, a.v.sh, a.v.sn, a.Nkv, a.H, a.nkv_pad, a.km, a.v16, sm.tile16);
    } else {
        quant_v_fp8_body<D, NT>(r - a.nq_blk - a.nk_blk, h, b, a.v.p, a.v.sb, a.v.sh, a.v.sn, a.Nkv, a.H, a.nkv_pad, a.km,
                            a.vscale, a.v8, sm.tile8);
    }
}

hipError_t launch_quant(const QuantArgs& a_in, int B, int D, hipStream_t st) {
    QuantArgs a = a_in;
    a.nq_blk = a.q8 != nullptr ? (int)(a.nq_pad / a.blkq) : 0;
    a.nk_blk = a.k8 != nullptr ? (int)(a.nkv_pad / a.blkk) : 0;
    a.nv_tile = (a.v8 != nullptr || a.v16 != nullptr) ? (int)(a.nkv_pad / 64) : 0;
    if (a.q8 != nullptr && a.nq_pad % a.blkq != 0) return hipErrorInvalidValue;
    if (a.k8 != nullptr && a.nkv_pad % a.blkk != 0) return hipErrorInvalidValue;
    a.n_bh = B * a.H;
    const int64_t total = (int64_t)B * a.H * (a.nq_blk + a.nk_blk + a.nv_tile);
    if (total <= 0 || total > 0x7FFFFFFF) return hipErrorInvalidValue;
    dim3 grid((unsigned)total);
    const bool has_pre = a.pre_q.gain != nullptr;
#define SAGE_LAUNCH_QUANT(DD, PP) hipLaunchKernelGGL((quant_kernel<DD, PP>), grid, dim3((quant_threads<DD, PP>())), 0, st, a)
    if (D == 128 && has_pre) SAGE_LAUNCH_QUANT(128, true);
    else if (D == 128) SAGE_LAUNCH_QUANT(128, false);
    else if (D == 64 && has_pre) SAGE_LAUNCH_QUANT(64, true);
    else if (D == 64) SAGE_LAUNCH_QUANT(64, false);
    else if (D == 256 && !has_pre) SAGE_LAUNCH_QUANT(256, false);
    else return hipErrorInvalidValue;
#undef SAGE_LAUNCH_QUANT
    return hipGetLastError();
}

}  // namespace sage
