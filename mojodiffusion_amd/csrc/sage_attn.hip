// sage_attn.hip — flash-style attention on quantized operands for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (batch, head); wave w owns
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
// K and V^T tiles of 64 keys are double-buffered in LDS with a 16-byte-chunk
// XOR swizzle; the next tile's global loads are issued before the current
// tile's math.  Scores are in the log2 domain (scale*log2(e) is folded into the
// Q quantizer), so the exponential is a bare v_exp_f32.
#include "sage_internal.h"

#include <hip/hip_fp16.h>

namespace sage {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Byte offset of 16-byte chunk L of a tile whose rows are grouped into 128-byte
// super-rows: chunk position inside the super-row is XORed with the super-row index.
__device__ __forceinline__ int swz(int L) { return (((L >> 3) << 3) | ((L & 7) ^ ((L >> 3) & 7))) << 4; }

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <int D, int VARIANT, bool STATS>
__global__ __launch_bounds__(256, 2) void sage_attn_kernel(
    const int8_t* __restrict__ q8, const float* __restrict__ qscale, int blkq,
    const int8_t* __restrict__ k8, const float* __restrict__ kscale, int blkk,
    const uint8_t* __restrict__ vq, const float* __restrict__ vscale,
    const float* __restrict__ qshift,
    int H, int Nq, int kv_valid, int64_t nq_pad, int64_t nkv_pad,
    uint16_t* __restrict__ o, int64_t osb, int64_t osh, int64_t osn,
    float* __restrict__ stats, int n_qtiles, int total_wg) {
    constexpr int VB = (VARIANT == 0) ? 2 : 1;          // bytes per V element
    constexpr int KSTEPS = D / 32;                      // int8 MFMA steps over the head dim
    constexpr int DB = D / 32;                          // 32-channel output blocks
    constexpr int K_BYTES = kTileKV * D;                // K tile
    constexpr int V_BYTES = D * kTileKV * VB;           // V^T tile
    constexpr int K_CH = K_BYTES / 16 / 256;            // 16-byte chunks per thread
    constexpr int V_CH = V_BYTES / 16 / 256;
    constexpr int K_CPR = D / 16;                       // chunks per K row
    constexpr int V_CPR = kTileKV * VB / 16;            // chunks per V^T row

    __shared__ __attribute__((aligned(16))) uint8_t lds_k[2][K_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t lds_v[2][V_BYTES];

    // Workgroup -> (q tile, b*h).  Hardware hands consecutive workgroup ids to the 8
    // XCDs round-robin; give each XCD a contiguous range of (head, q tile) work so the
    // workgroups sharing one head's K/V also share one L2.
    int wg = blockIdx.x;
    {
        const int per = (total_wg + 7) >> 3;
        const int xcd = wg & 7, idx = wg >> 3;
        const int full = total_wg - (per - 1) * 8;      // XCDs that own `per` items (1..8)
        wg = (xcd < full) ? xcd * per + idx : full * per + (xcd - full) * (per - 1) + idx;
    }
    const int qt = wg % n_qtiles;
    const int64_t bh = wg / n_qtiles;
    const int b = (int)(bh / H), h = (int)(bh % H);

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int l32 = lane & 31, half = lane >> 5;
    const int qrow = qt * kTileQ + wave * 32 + l32;     // this lane's query (padded index)

    // Q^T fragments: 16 bytes of the head dim per step, resident for the whole kernel.
    v4i qf[KSTEPS];
    {
        const int8_t* qp = q8 + (bh * nq_pad + qrow) * D + half * 16;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) qf[s] = *reinterpret_cast<const v4i*>(qp + s * 32);
    }
    const float sq = qscale[bh * (nq_pad / blkq) + qrow / blkq];
    const float* ksc = kscale + bh * (nkv_pad / blkk);

    const int8_t* kg = k8 + bh * nkv_pad * D;
    const uint8_t* vg = vq + bh * nkv_pad * D * VB;
    const int ntiles = (kv_valid + kTileKV - 1) / kTileKV;

    v4i kreg[K_CH], vreg[V_CH];
    auto load_tile = [&](int t) {
        const v4i* kp = reinterpret_cast<const v4i*>(kg + (int64_t)t * K_BYTES);
        const v4i* vp = reinterpret_cast<const v4i*>(vg + (int64_t)t * V_BYTES);
#pragma unroll
        for (int i = 0; i < K_CH; i++) kreg[i] = kp[i * 256 + tid];
#pragma unroll
        for (int i = 0; i < V_CH; i++) vreg[i] = vp[i * 256 + tid];
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < K_CH; i++) *reinterpret_cast<v4i*>(&lds_k[buf][swz(i * 256 + tid)]) = kreg[i];
#pragma unroll
        for (int i = 0; i < V_CH; i++) *reinterpret_cast<v4i*>(&lds_v[buf][swz(i * 256 + tid)]) = vreg[i];
    };

    v16f oacc[DB];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[d][i] = 0.0f;
    float m_run = -INFINITY;       // running row max (log2 domain)
    float l_run = 0.0f;            // this lane's share of the row sum

    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int t = 0; t < ntiles; t++) {
        const int buf = t & 1;
        if (t + 1 < ntiles) load_tile(t + 1);

        // ---- S^T = K . Q^T : two 32-key blocks ---------------------------------
        v16i sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[kb][i] = 0;
#pragma unroll
            for (int s = 0; s < KSTEPS; s++) {
                const int L = (kb * 32 + l32) * K_CPR + s * 2 + half;
                const v4i a = *reinterpret_cast<const v4i*>(&lds_k[buf][swz(L)]);
                sacc[kb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qf[s], sacc[kb], 0, 0, 0);
            }
        }

        // ---- online softmax ------------------------------------------------------
        float sf[2][16];
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const float f = sq * ksc[(t * kTileKV + kb * 32) / blkk];
#pragma unroll
            for (int i = 0; i < 16; i++) sf[kb][i] = (float)sacc[kb][i] * f;
        }
        if (t == ntiles - 1 && (kv_valid & (kTileKV - 1)) != 0) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = t * kTileKV + kb * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                    if (key >= kv_valid) sf[kb][i] = -INFINITY;
                }
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, sf[kb][i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                sf[kb][i] = __builtin_amdgcn_exp2f(sf[kb][i] - m_new);
                psum += sf[kb][i];
            }
        l_run = l_run * corr + psum;
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int d = 0; d < DB; d++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[d][i] *= corr;
        }

        // ---- O^T += V^T . P^T ----------------------------------------------------
        if (VARIANT == 0) {
#pragma unroll
            for (int j = 0; j < 4; j++) {                 // 16 key slots per step
                v8h p;
#pragma unroll
                for (int e = 0; e < 8; e++) p[e] = (_Float16)sf[j >> 1][(j & 1) * 8 + e];
#pragma unroll
                for (int d = 0; d < DB; d++) {
                    const int L = (d * 32 + l32) * V_CPR + j * 2 + half;
                    const v8h a = *reinterpret_cast<const v8h*>(&lds_v[buf][swz(L)]);
                    oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, p, oacc[d], 0, 0, 0);
                }
            }
        } else {
            // P8 = e4m3(p * 448); 32 key slots of this half-wave in 8 dwords
            v8i p;
#pragma unroll
            for (int w = 0; w < 8; w++) {
                const float* s4 = &sf[w >> 2][(w & 3) * 4];
                int pk = __builtin_amdgcn_cvt_pk_fp8_f32(s4[0] * 448.0f, s4[1] * 448.0f, 0, false);
                pk = __builtin_amdgcn_cvt_pk_fp8_f32(s4[2] * 448.0f, s4[3] * 448.0f, pk, true);
                p[w] = pk;
            }
#pragma unroll
            for (int d = 0; d < DB; d++) {
                const int L0 = (d * 32 + l32) * V_CPR + half * 2;
                const v4i a0 = *reinterpret_cast<const v4i*>(&lds_v[buf][swz(L0)]);
                const v4i a1 = *reinterpret_cast<const v4i*>(&lds_v[buf][swz(L0 + 1)]);
                const v8i a = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                oacc[d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, p, oacc[d], 0, 0, 0, 0, 0, 0);
            }
        }

        if (t + 1 < ntiles) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: normalise, bf16 round-to-nearest-even, caller's strides ---------
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / l_tot;
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
                    if (VARIANT == 1) x[e] = x[e] * vscale[bh * D + ch + e] * (1.0f / 448.0f);
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
            stats[bh * Nq + qrow] = (m_run + __builtin_amdgcn_logf(l_tot) + shift) * 0.6931471805599453f;
        }
    }
}

template <int D, int VARIANT>
static hipError_t launch_attn_dv(const AttnArgs& a, hipStream_t st) {
    const int n_qtiles = (int)(a.nq_pad / kTileQ);
    const int64_t total = (int64_t)n_qtiles * a.B * a.H;
    if (total <= 0 || total > 0x7FFFFFFF) return hipErrorInvalidValue;
    dim3 grid((unsigned)total), block(256);
    if (a.stats != nullptr)
        hipLaunchKernelGGL((sage_attn_kernel<D, VARIANT, true>), grid, block, 0, st, a.q8, a.qscale, a.blkq,
                           a.k8, a.kscale, a.blkk, (const uint8_t*)a.vq, a.vscale, a.qshift, a.H, a.Nq,
                           a.kv_valid, a.nq_pad, a.nkv_pad, a.o, a.osb, a.osh, a.osn, a.stats, n_qtiles, (int)total);
    else
        hipLaunchKernelGGL((sage_attn_kernel<D, VARIANT, false>), grid, block, 0, st, a.q8, a.qscale, a.blkq,
                           a.k8, a.kscale, a.blkk, (const uint8_t*)a.vq, a.vscale, a.qshift, a.H, a.Nq,
                           a.kv_valid, a.nq_pad, a.nkv_pad, a.o, a.osb, a.osh, a.osn, a.stats, n_qtiles, (int)total);
    return hipGetLastError();
}

hipError_t launch_attn(const AttnArgs& a, hipStream_t st) {
    if (a.D == 128) return a.variant == 0 ? launch_attn_dv<128, 0>(a, st) : launch_attn_dv<128, 1>(a, st);
    if (a.D == 64) return a.variant == 0 ? launch_attn_dv<64, 0>(a, st) : launch_attn_dv<64, 1>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace sage
