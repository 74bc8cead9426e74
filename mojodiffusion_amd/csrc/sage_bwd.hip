// sage_bwd.hip — backward of scaled-dot-product attention in bf16 for gfx950.
//
// Flash-style: no N_q x N_kv matrix is ever stored.  From Q, K, V, O, dO (bf16) and the forward's
// log-sum-exp Stats (fp32) the probabilities are recomputed tile by tile,
//     P = exp(scale * Q K^T - Stats[row]),   Delta[row] = sum_d dO * O,
//     dV = P^T dO,   dS = P * (dO V^T - Delta),   dQ = scale * dS K,   dK = scale * dS^T Q,
// with v_mfma_f32_32x32x16_bf16, fp32 accumulation, P and dS rounded to bf16 as matrix operands.
//
// Two launches:
//   1. bwd_prep_kernel     Delta and Stats * log2(e) per query row (padding rows: +inf, so their
//                          probabilities vanish), and transposed copies K^T, Q^T, dO^T in tiles of
//                          64 rows whose rows sit in the slot order of the matrix instruction's
//                          operand layout (v_slot_f16); and a vector c close to the mean key.
//   2. bwd_fused_kernel    one grid of two kinds of 8-wave workgroups, the longer kind first:
//        dQ     owner = 256 query rows, loop over key tiles, as scale * (dS K - rowsum(dS) c)
//               = scale * dS (K - c)                                          (bwd_pass_body<D,0,8>)
//        dK,dV  owner = 128 keys, loop over query tiles; pairs of waves share 32 keys, one wave
//               carrying P and dV, the other dS and dK                        (bwd_dkdv_body)
//               (head dim 64: 256 keys, every wave both products — bwd_pass_body<D,1,8>)
// In both kinds a wave owns 32 rows ("x"), keeps their bf16 row blocks resident as B operands
// and walks the other side ("y") in tiles of 64 rows staged in LDS by register-bypassing copies,
// double buffered, one barrier per tile.  A 32x32 block of scores T[y,x] lands in the accumulator
// layout with the owner row as the lane's column, which is exactly the B-operand layout of the
// products that contract over y — so P and dS go from registers straight into the next matrix
// instruction, and the only transposed operands (rows = head channel, k = y) are the ones read
// from the transposed copies of launch 1.
#include "sage_internal.h"
#include <type_traits>

namespace sage {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __fp16 v2h __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr float kLog2e = 1.4426950408889634f;

// ---- LDS layouts -------------------------------------------------------------------------
// Transposed tile [D rows][64 slots] bf16: 128-byte rows, 8 chunks of 16 bytes per row; chunk
// position XORed with bits of the pair-of-rows index (same layout as the forward's V^T tile).
__device__ __forceinline__ int tr_off(int L) { return (((L >> 3) << 3) | ((L & 7) ^ ((L >> 4) & 7))) << 4; }
// Natural tile [64 rows][D] bf16: CPR chunks per row.  16 consecutive rows reading one logical
// chunk must land in 16 different 16-byte bank groups.
template <int CPR> __device__ __forceinline__ int nat_pos(int row, int c) {
    if constexpr (CPR == 16) return c ^ (row & 15);
    else return c ^ ((row >> 1) & 7);
}
template <int CPR> __device__ __forceinline__ int nat_off(int row, int c) { return (row * CPR + nat_pos<CPR>(row, c)) << 4; }

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// 16 (4) bytes per lane from global memory straight into LDS: lane l lands at base + 16*l (4*l).
__device__ __forceinline__ void dma16(const void* gbase_uniform, uint32_t goff, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base_uniform), "v"(goff), "s"(gbase_uniform)
                 : "memory");
}
__device__ __forceinline__ void dma4(const void* gbase_uniform, uint32_t goff, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(lds_base_uniform), "v"(goff), "s"(gbase_uniform)
                 : "memory");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const v2f f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2bf));       // round to nearest even
}

// inverse of v_slot_f16: which row of a 64-row tile sits at slot s
__device__ __forceinline__ int row_of_slot(int s) {
    const int g = s >> 4, r = s & 15;
    const int quad = (((r >> 2) & 1) << 1) | (r >> 3);
    return (g << 4) | (quad << 2) | (r & 3);
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// Launch 1.  Roles of one grid, per (b,h): K^T tiles | Q^T tiles | dO^T tiles | row statistics.
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void bwd_prep_kernel(BwdArgs a) {
    constexpr int CPR = D / 8;
    constexpr int LROW = D + 8;                     // LDS row stride in elements (keeps 16-byte alignment, spreads banks)
    __shared__ __attribute__((aligned(16))) uint16_t tile[64 * LROW];
    const int ntk = (int)(a.nkv_pad / 64), ntq = (int)(a.nq_pad / 64);
    const int per_bh = ntk + 3 * ntq;
    const int bh = blockIdx.x / per_bh;
    int r = blockIdx.x % per_bh;
    const int b = bh / a.H, h = bh % a.H;
    const int tid = threadIdx.x;

    if (r >= ntk + 2 * ntq) {
        // row statistics of 64 query rows: 4 threads per row
        const int row = (r - ntk - 2 * ntq) * 64 + (tid >> 2);
        const int part = tid & 3;
        float sum = 0.0f;
        if (row < a.valid_q) {
            const uint16_t* po = a.o.p + b * a.o.sb + h * a.o.sh + (int64_t)row * a.o.sn + part * (D / 4);
            const uint16_t* pg = a.dout.p + b * a.dout.sb + h * a.dout.sh + (int64_t)row * a.dout.sn + part * (D / 4);
#pragma unroll
            for (int c = 0; c < D / 32; c++) {
                const u32x4 wo = *reinterpret_cast<const u32x4*>(po + c * 8);
                const u32x4 wg = *reinterpret_cast<const u32x4*>(pg + c * 8);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    sum = fmaf(__uint_as_float(wo[e] << 16), __uint_as_float(wg[e] << 16), sum);
                    sum = fmaf(__uint_as_float(wo[e] & 0xFFFF0000u), __uint_as_float(wg[e] & 0xFFFF0000u), sum);
                }
            }
        }
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);
        if (part == 0) {
            const int64_t idx = (int64_t)bh * a.nq_pad + row;
            const bool valid = row < a.valid_q;
            a.delta[idx] = valid ? sum : 0.0f;
            a.lse2[idx] = valid ? a.stats[(int64_t)bh * a.Nq + row] * kLog2e : INFINITY;
        }
        return;
    }

    // transposed copy of one 64-row tile
    View src;
    uint16_t* dst;
    int valid, t;
    int64_t ntiles;
    const bool is_k = r < ntk;
    if (r < ntk) { src = a.k; dst = a.kT; valid = a.valid_kv; t = r; ntiles = ntk; }
    else if (r < ntk + ntq) { src = a.q; dst = a.qT; valid = a.valid_q; t = r - ntk; ntiles = ntq; }
    else { src = a.dout; dst = a.doT; valid = a.valid_q; t = r - ntk - ntq; ntiles = ntq; }
    const uint16_t* sp = src.p + b * src.sb + h * src.sh;
    // Rows of dS sum to zero in exact arithmetic, so dS K = dS (K - c) for any vector c; when O and
    // Stats come from a forward of other precision the row sum is small but not zero, and dS K
    // would multiply it by the keys' common offset.  The dQ pass therefore also sums every row of
    // dS (the rounded values the matrix instruction takes) and subtracts rowsum * c at the end,
    // with c close to the mean key: the mean of 64 keys spread evenly over the valid ones, computed
    // here once per head.  (Centring the K^T copy itself would round K - c to bf16 a second time.)
    if (is_k && t == 0) {
        float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 64 * CPR / 256; i++) {
            const int c = i * 256 + tid;
            const int smp = c / CPR, col = (c % CPR) * 8;
            const int64_t key = ((int64_t)smp * valid) >> 6;
            const u32x4 w = *reinterpret_cast<const u32x4*>(sp + key * src.sn + col);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                part[2 * e] += __uint_as_float(w[e] << 16);
                part[2 * e + 1] += __uint_as_float(w[e] & 0xFFFF0000u);
            }
        }
        // thread tid holds samples {tid / CPR + k * (256 / CPR)} of chunk tid % CPR: reduce over tid / CPR
        float* red = reinterpret_cast<float*>(tile);                 // [256 / CPR][D]
#pragma unroll
        for (int e = 0; e < 8; e++) red[(tid / CPR) * D + (tid % CPR) * 8 + e] = part[e];
        __syncthreads();
        if (tid < D) {
            float sum = 0.0f;
            for (int g = 0; g < 256 / CPR; g++) sum += red[g * D + tid];
            a.kcen[(int64_t)bh * D + tid] = sum * (1.0f / 64.0f);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 64 * CPR / 256; i++) {
        const int c = i * 256 + tid;
        const int row = c / CPR, col = (c % CPR) * 8;
        u32x4 w = {0u, 0u, 0u, 0u};
        if (t * 64 + row < valid) w = *reinterpret_cast<const u32x4*>(sp + (int64_t)(t * 64 + row) * src.sn + col);
        *reinterpret_cast<u32x4*>(&tile[row * LROW + col]) = w;
    }
    __syncthreads();
    uint16_t* out = dst + ((int64_t)bh * ntiles + t) * (int64_t)(D * 64);
#pragma unroll
    for (int i = 0; i < D * 8 / 256; i++) {
        const int c = i * 256 + tid;
        const int d = c >> 3, s0 = (c & 7) * 8;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t lo = tile[row_of_slot(s0 + 2 * e) * LROW + d];
            const uint32_t hi = tile[row_of_slot(s0 + 2 * e + 1) * LROW + d];
            w[e] = lo | (hi << 16);
        }
        *reinterpret_cast<u32x4*>(out + d * 64 + s0) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

// ---------------------------------------------------------------------------------------------
// Launch 2, the form in which one wave carries every product of its 32 owner rows: the dQ
// workgroups (PASS 0), and the dK/dV workgroups at head dim 64 (PASS 1).
// ---------------------------------------------------------------------------------------------
template <int D, int PASS>
struct PassLds {
    static constexpr int TILE_BYTES = 64 * D * 2;
    static constexpr int NTR = PASS == 0 ? 1 : 2;
    uint8_t nat[2][2][TILE_BYTES];
    uint8_t tr[2][NTR][TILE_BYTES];
    float row[2][2][64];
};

template <int D, int PASS, int NW>
__device__ __forceinline__ void bwd_pass_body(const BwdArgs& a, PassLds<D, PASS>& L, int block) {
    constexpr int XROWS = NW * 32;                  // owner rows per workgroup
    constexpr int CPR = D / 8;                      // 16-byte chunks per natural row
    constexpr int TILE_BYTES = 64 * D * 2;          // natural and transposed tiles have the same size
    constexpr int RUNS = TILE_BYTES / 1024;         // 1 KiB copies per tile
    constexpr int RPW = RUNS / NW;                  // per wave
    constexpr int KS = D / 16;                      // matrix-instruction steps over the head dim
    constexpr int DB = D / 32;                      // 32-channel output blocks
    constexpr int NTR = PASS == 0 ? 1 : 2;          // transposed operands per tile
    static_assert(RUNS % NW == 0, "tile copies must divide over the waves");

    auto& lds_nat = L.nat;
    auto& lds_tr = L.tr;
    auto& lds_row = L.row;

    const int Nx = PASS == 0 ? a.Nq : a.Nkv;
    const int valid_x = PASS == 0 ? a.valid_q : a.valid_kv;
    const int valid_y = PASS == 0 ? a.valid_kv : a.valid_q;
    const int x_tiles = (Nx + XROWS - 1) / XROWS;
    const int xt = block % x_tiles;
    const int bh = block / x_tiles;
    const int b = bh / a.H, h = bh % a.H;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const int x = xt * XROWS + wave * 32 + l32;
    // (rows past the valid length are never read: what the caller keeps there — NaNs included — must
    // not reach a valid row's gradient through a product with a zero probability)
    const int xc = min(x, max(valid_x, 1) - 1);

    // owner side: two resident row blocks (B operands: column = owner row, k = head channel)
    const View& xv1 = PASS == 0 ? a.q : a.k;
    const View& xv2 = PASS == 0 ? a.dout : a.v;
    v4i b1[KS], b2[KS];
    {
        const uint16_t* p1 = xv1.p + b * xv1.sb + h * xv1.sh + (int64_t)xc * xv1.sn + half * 8;
        const uint16_t* p2 = xv2.p + b * xv2.sb + h * xv2.sh + (int64_t)xc * xv2.sn + half * 8;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            b1[s] = *reinterpret_cast<const v4i*>(p1 + s * 16);
            b2[s] = *reinterpret_cast<const v4i*>(p2 + s * 16);
        }
    }
    float lse_x = 0.0f, delta_x = 0.0f;
    float ds_rowsum = 0.0f;                         // dQ pass: sum over the keys of this lane's dS values
    if constexpr (PASS == 0) {
        const int64_t idx = (int64_t)bh * a.nq_pad + min((int64_t)x, a.nq_pad - 1);
        lse_x = a.lse2[idx];
        delta_x = a.delta[idx];
    }
    // The plain loads above must have landed before the loop: the compiler waits for a load at the
    // first use of its result, and such a wait inside the loop would also wait for the tile copies
    // that are meant to stay in flight (they share the counter).  Using the values here puts the
    // waits here.
#pragma unroll
    for (int s = 0; s < KS; s++) asm volatile("" : "+v"(b1[s]), "+v"(b2[s]));
    asm volatile("" : "+v"(lse_x), "+v"(delta_x));
    dma_wait_all();

    // y side
    const View& yv1 = PASS == 0 ? a.k : a.q;
    const View& yv2 = PASS == 0 ? a.v : a.dout;
    const uint8_t* y1 = reinterpret_cast<const uint8_t*>(yv1.p + b * yv1.sb + h * yv1.sh);
    const uint8_t* y2 = reinterpret_cast<const uint8_t*>(yv2.p + b * yv2.sb + h * yv2.sh);
    const int64_t ny_pad = PASS == 0 ? a.nkv_pad : a.nq_pad;
    const uint8_t* t1 = reinterpret_cast<const uint8_t*>(PASS == 0 ? a.kT : a.qT) + (int64_t)bh * ny_pad * D * 2;
    const uint8_t* t2 = reinterpret_cast<const uint8_t*>(a.doT) + (int64_t)bh * ny_pad * D * 2;
    const uint8_t* rows_l = reinterpret_cast<const uint8_t*>(a.lse2 + (int64_t)bh * a.nq_pad);
    const uint8_t* rows_d = reinterpret_cast<const uint8_t*>(a.delta + (int64_t)bh * a.nq_pad);
    // owners that are all padding have nothing to compute: they only store zeros
    const int ntiles = xt * XROWS < valid_x ? (valid_y + 63) / 64 : 0;

    // per-lane pieces of the copy addresses: run i of this wave covers physical chunks
    // (i*4 + wave)*64 + lane of a tile
    int nat_row[RPW], nat_col[RPW];
    uint32_t tr_src[RPW];
#pragma unroll
    for (int i = 0; i < RPW; i++) {
        const int P = (i * NW + wave) * 64 + lane;
        const int row = P / CPR, pos = P % CPR;
        nat_row[i] = row;
        nat_col[i] = nat_pos<CPR>(row, pos) * 16;          // the XOR is its own inverse
        tr_src[i] = (uint32_t)tr_off(P);
    }
    const uint32_t nat_base = lds_addr(&lds_nat[0][0][0]), tr_base = lds_addr(&lds_tr[0][0][0]);
    const uint32_t row_base = lds_addr(&lds_row[0][0][0]);
    const uint32_t ys1 = (uint32_t)(yv1.sn * 2), ys2 = (uint32_t)(yv2.sn * 2);
    auto copy_tile = [&](int t, int stage) {
#pragma unroll
        for (int i = 0; i < RPW; i++) {
            const uint32_t row = (uint32_t)min(t * 64 + nat_row[i], valid_y - 1);      // padding repeats the last valid row
            const uint32_t dst = (uint32_t)((i * NW + wave) * 1024);
            dma16(y1, row * ys1 + nat_col[i], __builtin_amdgcn_readfirstlane(nat_base + (stage * 2 + 0) * TILE_BYTES + dst));
            dma16(y2, row * ys2 + nat_col[i], __builtin_amdgcn_readfirstlane(nat_base + (stage * 2 + 1) * TILE_BYTES + dst));
            dma16(t1 + (int64_t)t * TILE_BYTES, tr_src[i], __builtin_amdgcn_readfirstlane(tr_base + (stage * NTR + 0) * TILE_BYTES + dst));
            if constexpr (PASS == 1)
                dma16(t2 + (int64_t)t * TILE_BYTES, tr_src[i], __builtin_amdgcn_readfirstlane(tr_base + (stage * NTR + 1) * TILE_BYTES + dst));
        }
        if constexpr (PASS == 1) {
            if (wave == 0) dma4(rows_l + (int64_t)t * 256, lane * 4, __builtin_amdgcn_readfirstlane(row_base + (stage * 2 + 0) * 256));
            if (wave == 1) dma4(rows_d + (int64_t)t * 256, lane * 4, __builtin_amdgcn_readfirstlane(row_base + (stage * 2 + 1) * 256));
        }
    };

    // fragment offsets inside a tile
    int nat_frag[2][KS];                 // [32-row block][k-step]
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int s = 0; s < KS; s++) nat_frag[blk][s] = nat_off<CPR>(blk * 32 + l32, s * 2 + half);
    int tr_frag[4];                      // [k-step over the 64 slots]; 32-channel blocks are +32*128 bytes
#pragma unroll
    for (int j = 0; j < 4; j++) tr_frag[j] = tr_off(l32 * 8 + j * 2 + half);

    v16f acc1[DB], acc2[PASS == 1 ? DB : 1];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            acc1[d][i] = 0.0f;
            if constexpr (PASS == 1) acc2[d][i] = 0.0f;
        }
    const float c = a.scale * kLog2e;

    if (ntiles > 0) copy_tile(0, 0);
    for (int t = 0; t < ntiles; t++) {
        const int stage = t & 1;
        dma_wait_all();
        __syncthreads();                 // tile t is visible; every wave is done with the other stage
        if (t + 1 < ntiles) copy_tile(t + 1, stage ^ 1);
        const uint8_t* n1 = &lds_nat[stage][0][0];
        const uint8_t* n2 = &lds_nat[stage][1][0];
        const uint8_t* r1 = &lds_tr[stage][0][0];
        const uint8_t* r2 = &lds_tr[stage][NTR - 1][0];
        // Two 32-row blocks per tile, software-pipelined so that the vector work of one block is
        // issued between the matrix instructions of the other:
        //   scores(0) | scores(1) + exponentials(0) | products(0) + exponentials(1) | products(1)
        v16f tacc[2], gacc[2];
        uint32_t pp[2][8], sp[2][8];
        float lse[4], dl[4];
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
            for (int i = 0; i < 16; i++) tacc[blk][i] = 0.0f, gacc[blk][i] = 0.0f;
        // one k-step of the two score products of a block: T += Y1 . X1^T, G += Y2 . X2^T.  The
        // fragments of step ks + 1 are requested before the products of step ks are issued.
        v4i f1[2], f2[2];
        auto scores_load = [&](int blk, int ks) {
            f1[ks & 1] = *reinterpret_cast<const v4i*>(n1 + nat_frag[blk][ks]);
            f2[ks & 1] = *reinterpret_cast<const v4i*>(n2 + nat_frag[blk][ks]);
        };
        auto scores_step = [&](int blk, int ks) {
            if (ks + 1 < KS) scores_load(blk, ks + 1);
            tacc[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, f1[ks & 1]), __builtin_bit_cast(v8bf, b1[ks]), tacc[blk], 0, 0, 0);
            gacc[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, f2[ks & 1]), __builtin_bit_cast(v8bf, b2[ks]), gacc[blk], 0, 0, 0);
        };
        // elements i, i+1 of a block (i even): y rows (i>>2)*8 + half*4 + (i&3) (+1), column = owner row
        auto softmax_pair = [&](int blk, int i) {
            const int g = i >> 2;
            if ((i & 3) == 0) {
                if constexpr (PASS == 0) {
#pragma unroll
                    for (int e = 0; e < 4; e++) lse[e] = lse_x, dl[e] = delta_x;
                } else {
                    const v4f vl = *reinterpret_cast<const v4f*>(&lds_row[stage][0][blk * 32 + g * 8 + half * 4]);
                    const v4f vd = *reinterpret_cast<const v4f*>(&lds_row[stage][1][blk * 32 + g * 8 + half * 4]);
#pragma unroll
                    for (int e = 0; e < 4; e++) lse[e] = vl[e], dl[e] = vd[e];
                }
            }
            float pr[2], ds[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                float arg = fmaf(tacc[blk][i + e], c, -lse[(i & 3) + e]);
                if constexpr (PASS == 0) {
                    // keys past the valid length (only possible in the last tile)
                    if (t * 64 + blk * 32 + g * 8 + half * 4 + (i & 3) + e >= valid_y) arg = -INFINITY;
                }
                pr[e] = __builtin_amdgcn_exp2f(arg);
                ds[e] = pr[e] * (gacc[blk][i + e] - dl[(i & 3) + e]);
            }
            sp[blk][i >> 1] = pack_bf16(ds[0], ds[1]);
            // dQ pass: this lane's share of the row sum of dS, over the rounded values
            if constexpr (PASS == 0)
                ds_rowsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, sp[blk][i >> 1]),
                                                            __builtin_bit_cast(v2bf, 0x3F803F80u), ds_rowsum, false);
            if constexpr (PASS == 1) pp[blk][i >> 1] = pack_bf16(pr[0], pr[1]);
        };
        // matrix instruction m of a block's accumulation: dX1^T += Y1^T . dS  (and dX2^T += Y2^T . P)
        constexpr int ACC_M = 2 * DB * NTR;
        auto acc_step = [&](int blk, int m) {
            const int which = m / (2 * DB), j2 = (m / DB) & 1, d = m % DB;
            const int j = blk * 2 + j2;
            if (which == 0) {
                const v4i sb = {(int)sp[blk][j2 * 4], (int)sp[blk][j2 * 4 + 1], (int)sp[blk][j2 * 4 + 2], (int)sp[blk][j2 * 4 + 3]};
                const v4i fa = *reinterpret_cast<const v4i*>(r1 + tr_frag[j] + d * 32 * 128);
                acc1[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, fa), __builtin_bit_cast(v8bf, sb), acc1[d], 0, 0, 0);
            } else if constexpr (PASS == 1) {
                const v4i pb = {(int)pp[blk][j2 * 4], (int)pp[blk][j2 * 4 + 1], (int)pp[blk][j2 * 4 + 2], (int)pp[blk][j2 * 4 + 3]};
                const v4i fa = *reinterpret_cast<const v4i*>(r2 + tr_frag[j] + d * 32 * 128);
                acc2[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, fa), __builtin_bit_cast(v8bf, pb), acc2[d], 0, 0, 0);
            }
        };
        scores_load(0, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) scores_step(0, ks);
        // scores of block 1 with the exponentials of block 0: 8 pairs over KS k-steps
        scores_load(1, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            scores_step(1, ks);
#pragma unroll
            for (int q = 0; q < 8 / KS; q++) softmax_pair(0, (ks * (8 / KS) + q) * 2);
        }
        // accumulation of block 0 with the exponentials of block 1: 8 pairs over ACC_M instructions
        // (ACC_M is 4, 8 or 16; with 16 a pair goes with every second instruction)
#pragma unroll
        for (int m = 0; m < ACC_M; m++) {
            acc_step(0, m);
            if constexpr (ACC_M <= 8) {
#pragma unroll
                for (int q = 0; q < 8 / ACC_M; q++) softmax_pair(1, (m * (8 / ACC_M) + q) * 2);
            } else {
                if (m & 1) softmax_pair(1, (m >> 1) * 2);
            }
        }
#pragma unroll
        for (int m = 0; m < ACC_M; m++) acc_step(1, m);
    }

    // ---- epilogue: rows of valid owners get their gradient, padding rows zeros -----------------
    if (x < Nx) {
        const bool live = x < valid_x;
        uint16_t* o1 = (PASS == 0 ? a.dq : a.dk) + b * (PASS == 0 ? a.dq_sb : a.dk_sb) + h * (PASS == 0 ? a.dq_sh : a.dk_sh) +
                       (int64_t)x * (PASS == 0 ? a.dq_sn : a.dk_sn);
        uint16_t* o2 = PASS == 1 ? a.dv + b * a.dv_sb + h * a.dv_sh + (int64_t)x * a.dv_sn : nullptr;
        // dQ = scale * (dS K - rowsum(dS) c): the two half-waves hold different keys of the same query
        float rs = 0.0f;
        if constexpr (PASS == 0) {
            const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(ds_rowsum), __float_as_uint(ds_rowsum), false, false);
            rs = __uint_as_float(r.x) + __uint_as_float(r.y);
        }
        const float* cen = a.kcen + (int64_t)bh * D;
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int ch = d * 32 + g * 8 + half * 4;
                u32x2 w = {0u, 0u};
                if (live) {
                    float y[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) y[e] = acc1[d][g * 4 + e];
                    if constexpr (PASS == 0) {
                        const v4f c4 = *reinterpret_cast<const v4f*>(cen + ch);
#pragma unroll
                        for (int e = 0; e < 4; e++) y[e] -= rs * c4[e];
                    }
                    w.x = pack_bf16(y[0] * a.scale, y[1] * a.scale);
                    w.y = pack_bf16(y[2] * a.scale, y[3] * a.scale);
                }
                *reinterpret_cast<u32x2*>(o1 + ch) = w;
                if constexpr (PASS == 1) {
                    u32x2 u = {0u, 0u};
                    if (live) {
                        u.x = pack_bf16(acc2[d][g * 4], acc2[d][g * 4 + 1]);
                        u.y = pack_bf16(acc2[d][g * 4 + 2], acc2[d][g * 4 + 3]);
                    }
                    *reinterpret_cast<u32x2*>(o2 + ch) = u;
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Launch 2, dK/dV workgroups at head dim 128.  The single-wave form above would keep 128
// accumulator and 64 operand registers per lane and so run one wave per SIMD.  Here a PAIR of waves
// shares 32 keys:
//   the P wave keeps the keys' K rows and the dV accumulators:  T = Q K^T -> P = exp2(cT - lse) -> dV += P^T dO
//   the S wave keeps the keys' V rows and the dK accumulators:  G = dO V^T, dS = P (G - Delta)  -> dK += dS^T Q
// No product is computed twice and every fragment is read from LDS once.  P goes from the P wave
// to the S wave through LDS, in the lane layout of the accumulator, which both waves share — as
// fp16 (11 significant bits, truncated): dS is P times a difference and is itself rounded to bf16,
// and a bf16 P underneath would add a second error of the same size to every term of dK.  The S wave runs one query tile behind the P wave, so the hand-over is ordered by the
// workgroup barrier that every tile has anyway; the tiles the S wave reads (dO, Q^T, Delta) are
// copied one iteration later than the P wave's (Q, dO^T, lse), which keeps every ring at two slots.
// There is room for one hand-over slot only (160 KiB of LDS): before the P wave overwrites it, it
// checks a per-pair counter that the S wave advances as soon as it holds the previous tile's P in
// registers — at the top of the iteration, half a tile before the P wave gets there.
// ---------------------------------------------------------------------------------------------
template <int D>
struct DkDvLds {
    static constexpr int TILE_BYTES = 64 * D * 2;
    uint8_t nat[2][2][TILE_BYTES];                  // [stage][0: Q | 1: dO], natural rows
    uint8_t tr[2][2][TILE_BYTES];                   // [stage][0: Q^T | 1: dO^T]
    u32x4 p[4][2][2][64];                           // [pair][32-row block][values 0-7 | 8-15][lane], fp16 pairs
    float row[2][2][64];                            // [stage][0: lse | 1: Delta]
    int taken[4];                                   // per pair: the S wave holds P of every tile below this
};

template <int D, int ROLE>
__device__ __forceinline__ void dkdv_role(const BwdArgs& a, DkDvLds<D>& L, int bh, int xt, int wave, int lane) {
    constexpr int NW = 8;
    constexpr int CPR = D / 8;
    constexpr int TILE_BYTES = 64 * D * 2;
    constexpr int RUNS = TILE_BYTES / 1024;
    constexpr int RPW = RUNS / NW;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    static_assert(RUNS % NW == 0, "tile copies must divide over the waves");
    const int b = bh / a.H, h = bh % a.H;
    const int pair = wave & 3;
    const int l32 = lane & 31, half = lane >> 5;
    const int x = xt * 128 + pair * 32 + l32;
    const int xc = min(x, max(a.valid_kv, 1) - 1);

    // owner side: the P wave keeps K rows, the S wave V rows (B operands: column = key, k = head channel)
    const View& xv = ROLE == 0 ? a.k : a.v;
    v4i bx[KS];
    {
        const uint16_t* px = xv.p + b * xv.sb + h * xv.sh + (int64_t)xc * xv.sn + half * 8;
#pragma unroll
        for (int s = 0; s < KS; s++) bx[s] = *reinterpret_cast<const v4i*>(px + s * 16);
    }
#pragma unroll
    for (int s = 0; s < KS; s++) asm volatile("" : "+v"(bx[s]));     // the wait for these loads stays out of the loop
    dma_wait_all();

    const uint8_t* yq = reinterpret_cast<const uint8_t*>(a.q.p + b * a.q.sb + h * a.q.sh);
    const uint8_t* yg = reinterpret_cast<const uint8_t*>(a.dout.p + b * a.dout.sb + h * a.dout.sh);
    const uint8_t* tq = reinterpret_cast<const uint8_t*>(a.qT) + (int64_t)bh * a.nq_pad * D * 2;
    const uint8_t* tg = reinterpret_cast<const uint8_t*>(a.doT) + (int64_t)bh * a.nq_pad * D * 2;
    const uint8_t* rows_l = reinterpret_cast<const uint8_t*>(a.lse2 + (int64_t)bh * a.nq_pad);
    const uint8_t* rows_d = reinterpret_cast<const uint8_t*>(a.delta + (int64_t)bh * a.nq_pad);
    const int ntiles = xt * 128 < a.valid_kv ? (a.valid_q + 63) / 64 : 0;

    int nat_row[RPW], nat_col[RPW];
    uint32_t tr_src[RPW];
#pragma unroll
    for (int i = 0; i < RPW; i++) {
        const int P = (i * NW + wave) * 64 + lane;
        const int row = P / CPR, pos = P % CPR;
        nat_row[i] = row;
        nat_col[i] = nat_pos<CPR>(row, pos) * 16;
        tr_src[i] = (uint32_t)tr_off(P);
    }
    const uint32_t nat_base = lds_addr(&L.nat[0][0][0]), tr_base = lds_addr(&L.tr[0][0][0]);
    const uint32_t row_base = lds_addr(&L.row[0][0][0]);
    const uint32_t sq = (uint32_t)(a.q.sn * 2), sg = (uint32_t)(a.dout.sn * 2);
    // what the P wave reads of query tile t: Q rows, dO^T, lse
    auto copy_for_p = [&](int t, int stage) {
#pragma unroll
        for (int i = 0; i < RPW; i++) {
            const uint32_t row = (uint32_t)min(t * 64 + nat_row[i], a.valid_q - 1);
            const uint32_t dst = (uint32_t)((i * NW + wave) * 1024);
            dma16(yq, row * sq + nat_col[i], __builtin_amdgcn_readfirstlane(nat_base + (stage * 2 + 0) * TILE_BYTES + dst));
            dma16(tg + (int64_t)t * TILE_BYTES, tr_src[i], __builtin_amdgcn_readfirstlane(tr_base + (stage * 2 + 1) * TILE_BYTES + dst));
        }
        if (wave == 0) dma4(rows_l + (int64_t)t * 256, lane * 4, __builtin_amdgcn_readfirstlane(row_base + (stage * 2 + 0) * 256));
    };
    // what the S wave reads of query tile t: dO rows, Q^T, Delta
    auto copy_for_s = [&](int t, int stage) {
#pragma unroll
        for (int i = 0; i < RPW; i++) {
            const uint32_t row = (uint32_t)min(t * 64 + nat_row[i], a.valid_q - 1);
            const uint32_t dst = (uint32_t)((i * NW + wave) * 1024);
            dma16(yg, row * sg + nat_col[i], __builtin_amdgcn_readfirstlane(nat_base + (stage * 2 + 1) * TILE_BYTES + dst));
            dma16(tq + (int64_t)t * TILE_BYTES, tr_src[i], __builtin_amdgcn_readfirstlane(tr_base + (stage * 2 + 0) * TILE_BYTES + dst));
        }
        if (wave == 1) dma4(rows_d + (int64_t)t * 256, lane * 4, __builtin_amdgcn_readfirstlane(row_base + (stage * 2 + 1) * 256));
    };

    int nat_frag[2][KS];
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int s = 0; s < KS; s++) nat_frag[blk][s] = nat_off<CPR>(blk * 32 + l32, s * 2 + half);
    int tr_frag[4];
#pragma unroll
    for (int j = 0; j < 4; j++) tr_frag[j] = tr_off(l32 * 8 + j * 2 + half);

    v16f acc[DB];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[d][i] = 0.0f;
    const float c = a.scale * kLog2e;
    // (an LDS pointer by type: through a generic one the accesses become flat instructions, whose waits
    // also wait for the tile copies in flight)
    volatile __attribute__((address_space(3))) int* taken = (volatile __attribute__((address_space(3))) int*)&L.taken[pair];

    if (ntiles > 0) copy_for_p(0, 0);
    // iteration `it`: the P wave works on query tile it, the S wave on tile it - 1
    for (int it = 0; ntiles > 0 && it <= ntiles; it++) {
        const int stage = it & 1;
        dma_wait_all();
        __syncthreads();                 // this iteration's tiles and the previous one's P are visible; the other stage is free
        if (it + 1 < ntiles) copy_for_p(it + 1, stage ^ 1);
        if (it < ntiles) copy_for_s(it, stage ^ 1);
        if (ROLE == 0 ? it >= ntiles : it == 0) continue;

        const uint8_t* nt = &L.nat[stage][ROLE][0];
        const uint8_t* rt = &L.tr[stage][1 - ROLE][0];
        const float* rowv = &L.row[stage][ROLE][0];
        uint32_t hp[2][8];               // S wave: the P wave's probabilities of this tile
        if constexpr (ROLE == 1) {
#pragma unroll
            for (int blk = 0; blk < 2; blk++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const u32x4 w = L.p[pair][blk][j][lane];
#pragma unroll
                    for (int e = 0; e < 4; e++) hp[blk][j * 4 + e] = w[e];
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int blk = 0; blk < 2; blk++)
#pragma unroll
                for (int e = 0; e < 8; e++) asm volatile("" : "+v"(hp[blk][e]));
            if (lane == 0) *taken = it;
        }
        v16f sacc[2];
        uint32_t pk[2][8];               // P (P wave) or dS (S wave), packed bf16 pairs: the next product's B operand
        uint32_t ph[2][8];               // P wave: the same P as fp16 pairs, for the S wave
        float rv[4];
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[blk][i] = 0.0f;
        v4i f[2];
        auto scores_load = [&](int blk, int ks) { f[ks & 1] = *reinterpret_cast<const v4i*>(nt + nat_frag[blk][ks]); };
        auto scores_step = [&](int blk, int ks) {
            if (ks + 1 < KS) scores_load(blk, ks + 1);
            sacc[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, f[ks & 1]), __builtin_bit_cast(v8bf, bx[ks]), sacc[blk], 0, 0, 0);
        };
        // elements i, i+1 of a block (i even): query rows (i>>2)*8 + half*4 + (i&3) (+1), column = key
        auto value_pair = [&](int blk, int i) {
            const int g = i >> 2;
            if ((i & 3) == 0) {
                const v4f vr = *reinterpret_cast<const v4f*>(rowv + blk * 32 + g * 8 + half * 4);
#pragma unroll
                for (int e = 0; e < 4; e++) rv[e] = vr[e];
            }
            float y[2];
            if constexpr (ROLE == 0) {
#pragma unroll
                for (int e = 0; e < 2; e++) y[e] = __builtin_amdgcn_exp2f(fmaf(sacc[blk][i + e], c, -rv[(i & 3) + e]));
                ph[blk][i >> 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(y[0], y[1]));
            } else {
                const v2h w = __builtin_bit_cast(v2h, hp[blk][i >> 1]);
                y[0] = (float)w[0] * (sacc[blk][i] - rv[i & 3]);
                y[1] = (float)w[1] * (sacc[blk][i + 1] - rv[(i & 3) + 1]);
            }
            pk[blk][i >> 1] = pack_bf16(y[0], y[1]);
        };
        constexpr int ACC_M = 2 * DB;
        auto acc_step = [&](int blk, int m) {
            const int j2 = m / DB, d = m % DB;
            const int j = blk * 2 + j2;
            const v4i sb = {(int)pk[blk][j2 * 4], (int)pk[blk][j2 * 4 + 1], (int)pk[blk][j2 * 4 + 2], (int)pk[blk][j2 * 4 + 3]};
            const v4i fa = *reinterpret_cast<const v4i*>(rt + tr_frag[j] + d * 32 * 128);
            acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, fa), __builtin_bit_cast(v8bf, sb), acc[d], 0, 0, 0);
        };
        auto hand_over = [&](int blk) {
            if constexpr (ROLE == 0) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    L.p[pair][blk][j][lane] = u32x4{ph[blk][j * 4], ph[blk][j * 4 + 1], ph[blk][j * 4 + 2], ph[blk][j * 4 + 3]};
            }
        };
        scores_load(0, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) scores_step(0, ks);
        scores_load(1, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            scores_step(1, ks);
#pragma unroll
            for (int q = 0; q < 8 / KS; q++) value_pair(0, (ks * (8 / KS) + q) * 2);
        }
        if constexpr (ROLE == 0) {
            // the slot still holds the previous tile's P until the S wave has it in registers
            while (__builtin_amdgcn_readfirstlane(*taken) < it) __builtin_amdgcn_s_sleep(1);
            asm volatile("" ::: "memory");
        }
        hand_over(0);
#pragma unroll
        for (int m = 0; m < ACC_M; m++) {
            acc_step(0, m);
#pragma unroll
            for (int q = 0; q < 8 / ACC_M; q++) value_pair(1, (m * (8 / ACC_M) + q) * 2);
        }
        hand_over(1);
#pragma unroll
        for (int m = 0; m < ACC_M; m++) acc_step(1, m);
    }

    if (x < a.Nkv) {
        const bool live = x < a.valid_kv;
        uint16_t* o = ROLE == 0 ? a.dv + b * a.dv_sb + h * a.dv_sh + (int64_t)x * a.dv_sn
                                : a.dk + b * a.dk_sb + h * a.dk_sh + (int64_t)x * a.dk_sn;
        const float mul = ROLE == 0 ? 1.0f : a.scale;
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                u32x2 w = {0u, 0u};
                if (live) {
                    w.x = pack_bf16(acc[d][g * 4] * mul, acc[d][g * 4 + 1] * mul);
                    w.y = pack_bf16(acc[d][g * 4 + 2] * mul, acc[d][g * 4 + 3] * mul);
                }
                *reinterpret_cast<u32x2*>(o + d * 32 + g * 8 + half * 4) = w;
            }
    }
}

template <int D>
__device__ __forceinline__ void bwd_dkdv_body(const BwdArgs& a, DkDvLds<D>& L, int block) {
    const int x_tiles = (a.Nkv + 127) / 128;
    const int xt = block % x_tiles, bh = block / x_tiles;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (tid < 4) L.taken[tid] = 0;                  // ordered before the first use by the loop's first barrier
    if (wave < 4) dkdv_role<D, 0>(a, L, bh, xt, wave, lane);
    else dkdv_role<D, 1>(a, L, bh, xt, wave, lane);
}

// One grid for both: the first n_dq workgroups are the dQ pass (the longer ones first), the rest
// the dK/dV pass.  Both take a whole CU (8 waves, most of the LDS); in one grid the second
// kind starts on a CU as soon as the first kind runs out, instead of after its last workgroup.
template <int D>
__global__ __launch_bounds__(512, 2) void bwd_fused_kernel(BwdArgs a, int n_dq) {
    constexpr bool PAIRED = D > 64;                 // below, the single-wave form already fits two waves per SIMD
    using KvLds = std::conditional_t<PAIRED, DkDvLds<D>, PassLds<D, 1>>;
    constexpr size_t BYTES = sizeof(KvLds) > sizeof(PassLds<D, 0>) ? sizeof(KvLds) : sizeof(PassLds<D, 0>);
    __shared__ __attribute__((aligned(1024))) uint8_t smem[BYTES];
    const int block = (int)blockIdx.x;
    if (block < n_dq) bwd_pass_body<D, 0, 8>(a, *reinterpret_cast<PassLds<D, 0>*>(smem), block);
    else if constexpr (PAIRED) bwd_dkdv_body<D>(a, *reinterpret_cast<DkDvLds<D>*>(smem), block - n_dq);
    else bwd_pass_body<D, 1, 8>(a, *reinterpret_cast<PassLds<D, 1>*>(smem), block - n_dq);
}

template <int D>
static hipError_t launch_bwd_d(const BwdArgs& a, hipStream_t st) {
    const int64_t bh = (int64_t)a.B * a.H;
    const int64_t prep = bh * (a.nkv_pad / 64 + 3 * (a.nq_pad / 64));
    // dQ: 256 query rows per workgroup; dK, dV: 128 keys (wave pairs) or 256 keys (single-wave form)
    constexpr int KEYS_WG = D > 64 ? 128 : 256;
    const int64_t gq = bh * ((a.Nq + 255) / 256), gk = bh * ((a.Nkv + KEYS_WG - 1) / KEYS_WG);
    if (prep > 0x7FFFFFFF || gq + gk > 0x7FFFFFFF) return hipErrorInvalidValue;
    hipLaunchKernelGGL((bwd_prep_kernel<D>), dim3((unsigned)prep), dim3(256), 0, st, a);
    hipLaunchKernelGGL((bwd_fused_kernel<D>), dim3((unsigned)(gq + gk)), dim3(512), 0, st, a, (int)gq);
    return hipGetLastError();
}

hipError_t launch_bwd(const BwdArgs& a, hipStream_t st) {
    if (a.D == 128) return launch_bwd_d<128>(a, st);
    if (a.D == 64) return launch_bwd_d<64>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace sage
