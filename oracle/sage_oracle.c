/*
 * sage_oracle.c — CPU restatement of the quantized-SDPA hot path.
 *
 * TEST INFRASTRUCTURE ONLY (see sage_oracle.h): the checker for the HIP
 * library and the timed CPU baseline.  Never linked into the product.
 *
 * Build: gcc -O3 -mavx2 -ffp-contract=off -fopenmp -shared -fPIC (see Makefile).
 * -ffp-contract=off matters: every "one fp32 operation" below must stay one
 * IEEE operation so the GPU kernels can reproduce the bits.
 */
#include "sage_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* scalar codecs                                                            */
/* ------------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float sage_oracle_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* Round-to-nearest-even to the 8-bit bf16 significand: the value
 * serenitymojo/ops/torch_bf16.mojo:27-60 computes arithmetically (nearest
 * multiple of 2^(e-7), ties to the even multiple) is what adding 0x7FFF plus
 * the keep-bit to the fp32 pattern and truncating gives. */
uint16_t sage_oracle_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN */
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float sage_oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    int exp = (h >> 10) & 0x1F;
    uint32_t man = h & 0x3FFu;
    float v;
    if (exp == 0) v = ldexpf((float)man, -24);
    else if (exp == 31) v = man ? NAN : INFINITY;
    else v = ldexpf((float)(man | 0x400u), exp - 25);
    return sign ? -v : v;
}

/* fp32 -> fp16, round-to-nearest-even, subnormals kept, finite overflow
 * saturates to +-65504 (a V value is data, an infinity would poison P*V). */
uint16_t sage_oracle_f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);          /* NaN */
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7BFFu);         /* >= 65520 (or inf) -> 65504 */
    if (a < 0x33000001u) return sign;                                /* <= 2^-25 -> 0 (tie to even) */
    int e = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7FFFFFu) | 0x800000u;                      /* 24-bit significand */
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;                   /* bits dropped */
    uint32_t keep = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) keep++;
    uint32_t out;
    if (e < -14) out = keep;                                         /* subnormal (may carry into exp=1) */
    else out = ((uint32_t)(e + 15) << 10) + (keep - 0x400u);         /* carry propagates into exp */
    return (uint16_t)(sign | out);
}

/* serenitymojo/ops/fp8.mojo:60-78 */
float sage_oracle_e4m3_to_f32(uint8_t b) {
    int sign = (b >> 7) & 1, exp = (b >> 3) & 0xF, mant = b & 7;
    float v;
    if (exp == 0) v = ldexpf((float)mant / 8.0f, -6);
    else v = ldexpf(1.0f + (float)mant / 8.0f, exp - 7);
    return sign ? -v : v;
}

/* serenitymojo/ops/fp8_quant.mojo:42-50 */
static inline int rne_nonneg(float x) {
    float fl = floorf(x);
    float frac = x - fl;
    int n = (int)fl;
    if (frac > 0.5f) n += 1;
    else if (frac == 0.5f && (n & 1)) n += 1;
    return n;
}

/* serenitymojo/ops/fp8_quant.mojo:61-93 */
uint8_t sage_oracle_f32_to_e4m3(float v) {
    uint8_t sign = 0;
    float a = v;
    if (signbit(v)) { sign = 0x80; a = -a; }
    if (a != a) return sign;            /* NaN -> +-0 */
    if (a > 448.0f) a = 448.0f;
    uint8_t byte;
    if (a < ldexpf(1.0f, -6)) {
        int m = rne_nonneg(a * 512.0f);
        byte = (m >= 8) ? 0x08 : (uint8_t)m;
    } else {
        int e = -6;
        while (e < 8 && a >= ldexpf(1.0f, e + 1)) e++;
        int m = rne_nonneg(ldexpf(a, 3 - e));
        if (m == 16) { m = 8; e++; }
        if (e > 8) byte = (uint8_t)((15 << 3) | 6);
        else byte = (uint8_t)(((e + 7) << 3) | (m - 8));
    }
    return (uint8_t)(byte | sign);
}

void sage_oracle_f32_to_bf16_n(const float* x, uint16_t* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = sage_oracle_f32_to_bf16(x[i]);
}
void sage_oracle_f32_to_f16_n(const float* x, uint16_t* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = sage_oracle_f32_to_f16(x[i]);
}
void sage_oracle_f32_to_e4m3_n(const float* x, uint8_t* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = sage_oracle_f32_to_e4m3(x[i]);
}
void sage_oracle_e4m3_to_f32_n(const uint8_t* x, float* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = sage_oracle_e4m3_to_f32(x[i]);
}

int sage_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

int64_t sage_oracle_pad(int64_t n, int64_t mult) { return (n + mult - 1) / mult * mult; }

/* ------------------------------------------------------------------------ */
/* full-precision SDPA                                                      */
/* ------------------------------------------------------------------------ */

static int bad_args(const void* q, const void* k, const void* v, const void* o,
                    int B, int H, int Nq, int Nkv, int D,
                    const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os) {
    /* same order as serenitymojo/ops/cshim/cudnn_sdpa.cpp:391-393 */
    if (!q || !k || !v || !o) return 1;
    if (B <= 0 || H <= 0 || Nq <= 0 || Nkv <= 0 || D <= 0) return 1;
    if (!qs || !ks || !vs || !os) return 1;
    return 0;
}

int sage_oracle_sdpa_f32(const float* q, const float* k, const float* v, float* o,
                         int B, int H, int Nq, int Nkv, int D, float scale,
                         const int64_t* qs, const int64_t* ks,
                         const int64_t* vs, const int64_t* os) {
    if (bad_args(q, k, v, o, B, H, Nq, Nkv, D, qs, ks, vs, os)) return -1;
    int64_t rows = (int64_t)B * H * Nq;
    int err = 0;
#pragma omp parallel
    {
        double* sc = (double*)malloc(sizeof(double) * (size_t)Nkv);
        double* acc = (double*)malloc(sizeof(double) * (size_t)D);
        if (!sc || !acc) {
#pragma omp atomic write
            err = 1;
        }
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; r++) {
            if (!sc || !acc) continue;
            int i = (int)(r % Nq);
            int h = (int)((r / Nq) % H);
            int b = (int)(r / ((int64_t)Nq * H));
            const float* qr = q + b * qs[0] + h * qs[1] + i * qs[2];
            double mx = -INFINITY;
            for (int j = 0; j < Nkv; j++) {
                const float* kr = k + b * ks[0] + h * ks[1] + j * ks[2];
                double dot = 0.0;
                for (int d = 0; d < D; d++) dot += (double)qr[d * qs[3]] * (double)kr[d * ks[3]];
                double s = dot * (double)scale;
                sc[j] = s;
                if (s > mx) mx = s;
            }
            double l = 0.0;
            for (int d = 0; d < D; d++) acc[d] = 0.0;
            for (int j = 0; j < Nkv; j++) {
                double p = exp(sc[j] - mx);
                l += p;
                const float* vr = v + b * vs[0] + h * vs[1] + j * vs[2];
                for (int d = 0; d < D; d++) acc[d] += p * (double)vr[d * vs[3]];
            }
            float* orow = o + b * os[0] + h * os[1] + i * os[2];
            for (int d = 0; d < D; d++) orow[d * os[3]] = (float)(acc[d] / l);
        }
        free(sc);
        free(acc);
    }
    return err ? -1 : 0;
}

int sage_oracle_sdpa_online_f32(const float* q, const float* k, const float* v, float* o,
                                int B, int H, int Nq, int Nkv, int D, float scale,
                                const int64_t* qs, const int64_t* ks,
                                const int64_t* vs, const int64_t* os) {
    if (bad_args(q, k, v, o, B, H, Nq, Nkv, D, qs, ks, vs, os)) return -1;
    int64_t rows = (int64_t)B * H * Nq;
    int err = 0;
#pragma omp parallel
    {
        float* acc = (float*)malloc(sizeof(float) * (size_t)D);
        if (!acc) {
#pragma omp atomic write
            err = 1;
        }
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; r++) {
            if (!acc) continue;
            int i = (int)(r % Nq);
            int h = (int)((r / Nq) % H);
            int b = (int)(r / ((int64_t)Nq * H));
            const float* qr = q + b * qs[0] + h * qs[1] + i * qs[2];
            for (int d = 0; d < D; d++) acc[d] = 0.0f;
            float m = -3.0e38f, l = 0.0f;               /* attention.mojo:61, :765-766 */
            for (int j = 0; j < Nkv; j++) {
                const float* kr = k + b * ks[0] + h * ks[1] + j * ks[2];
                const float* vr = v + b * vs[0] + h * vs[1] + j * vs[2];
                float dot = 0.0f;
                for (int d = 0; d < D; d++) dot += qr[d * qs[3]] * kr[d * ks[3]];
                float s = dot * scale;
                float m_new = m > s ? m : s;            /* :786-792 */
                float corr = expf(m - m_new);
                float p = expf(s - m_new);
                l = l * corr + p;
                for (int d = 0; d < D; d++) acc[d] = acc[d] * corr + p * vr[d * vs[3]];
                m = m_new;
            }
            float inv = 1.0f / l;
            float* orow = o + b * os[0] + h * os[1] + i * os[2];
            for (int d = 0; d < D; d++) orow[d * os[3]] = acc[d] * inv;
        }
        free(acc);
    }
    return err ? -1 : 0;
}

/* ------------------------------------------------------------------------ */
/* quantizers                                                               */
/* ------------------------------------------------------------------------ */

static int bad_quant_args(const void* x, int B, int H, int N, int D, const int64_t* st, int blk, int mult) {
    if (!x || !st) return 1;
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0) return 1;
    if (blk <= 0 || mult <= 0) return 1;
    return 0;
}

/* ---- the two ops in front of the path: RMSNorm over D, interleaved RoPE -------------- */

/* serenitymojo/ops/norm.mojo:47-79 (_rms_norm_kernel_f32): out = x * (1/sqrt(mean(x^2)+eps)) * g.
 * The reference adds the squares in the order of its 256-thread shared-memory tree; an fp32
 * sum's last bit depends on that order and nothing the reference holds pins it (its vectors
 * have 6 columns and a 1e-6 bar), so the order here is the one the GPU kernel can afford:
 * runs of 8 consecutive columns added left to right, then the run sums combined pairwise
 * (neighbours first: strides 1, 2, 4, ... runs).  Column counts that are not a multiple of 8
 * are added left to right. */
static float sumsq_blocked(const float* v, int cols) {
    int runs = cols / 8;
    if (cols % 8 == 0 && runs > 0 && runs <= 1024) {
        float part[1024];
        for (int r = 0; r < runs; r++) {
            float a = 0.0f;
            for (int e = 0; e < 8; e++) {
                float sq = v[r * 8 + e] * v[r * 8 + e];
                a = a + sq;
            }
            part[r] = a;
        }
        /* pairwise, neighbours first; an odd one out moves up unchanged */
        for (int n = runs; n > 1; n = (n + 1) / 2) {
            for (int r = 0; r + 1 < n; r += 2) part[r / 2] = part[r] + part[r + 1];
            if (n & 1) part[n / 2] = part[n - 1];
        }
        return part[0];
    }
    float a = 0.0f;
    for (int c = 0; c < cols; c++) {
        float sq = v[c] * v[c];
        a = a + sq;
    }
    return a;
}

static float rms_inv(const float* v, int cols, float eps) {
    float ss = sumsq_blocked(v, cols);
    float mean = ss / (float)cols;
    return 1.0f / sqrtf(mean + eps);           /* IEEE sqrt and divide (norm.mojo:73) */
}

int sage_oracle_rms_norm_f32(const float* x, const float* g, int64_t rows, int cols, float eps, float* out) {
    if (!x || !g || !out || rows <= 0 || cols <= 0) return -1;
    for (int64_t r = 0; r < rows; r++) {
        float inv = rms_inv(x + r * cols, cols, eps);
        for (int c = 0; c < cols; c++) {
            float t = x[r * cols + c] * inv;    /* (v * inv) * g, norm.mojo:78 */
            out[r * cols + c] = t * g[c];
        }
    }
    return 0;
}

/* serenitymojo/ops/rope.mojo:7-9, :104-122: pairs (x[2i], x[2i+1]); separate multiplies, then
 * one subtract / add (no fused multiply-add). */
int sage_oracle_rope_interleaved_f32(const float* x, const float* cs, const float* sn,
                                     int64_t rows, int D, float* out) {
    if (!x || !cs || !sn || !out || rows <= 0 || D <= 0 || (D & 1)) return -1;
    int half = D / 2;
    for (int64_t r = 0; r < rows; r++)
        for (int i = 0; i < half; i++) {
            float x0 = x[r * D + 2 * i], x1 = x[r * D + 2 * i + 1];
            float cv = cs[r * half + i], sv = sn[r * half + i];
            float a = x0 * cv, b = x1 * sv, c = x0 * sv, d = x1 * cv;
            out[r * D + 2 * i] = a - b;
            out[r * D + 2 * i + 1] = c + d;
        }
    return 0;
}

/* bf16 activations: RMSNorm with a bf16 gain, stored as bf16 (norm.mojo:81-114), then
 * interleaved RoPE with fp32 tables on that bf16 tensor, stored as bf16 (rope.mojo:104-122).
 * x is logical [B,H,N,D] through strides; tables are [rows_per_batch, D/2] with row n*H + h
 * (sampling/klein_sampler.mojo:305-307), shared by all batches when table_batch_rows == 0, else
 * batch b starts at row b*table_batch_rows; cs == NULL skips the rotation.
 * y: contiguous [B,N,H,D] bf16. */
int sage_oracle_norm_rope_bf16(const uint16_t* x, int B, int H, int N, int D, const int64_t* st,
                               const uint16_t* gain, float eps, const float* cs, const float* sn,
                               int64_t table_batch_rows, uint16_t* y) {
    if (!x || !st || !gain || !y || B <= 0 || H <= 0 || N <= 0 || D <= 0 || (D & 1) || D > 1024) return -1;
    if ((cs == NULL) != (sn == NULL)) return -1;
    int half = D / 2;
    int64_t work = (int64_t)B * N * H;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int h = (int)(w % H);
        int n = (int)((w / H) % N);
        int b = (int)(w / ((int64_t)H * N));
        float v[1024], t[1024];
        const uint16_t* src = x + b * st[0] + h * st[1] + (int64_t)n * st[2];
        for (int d = 0; d < D; d++) v[d] = sage_oracle_bf16_to_f32(src[d * st[3]]);
        float inv = rms_inv(v, D, eps);
        for (int d = 0; d < D; d++) {
            float a = v[d] * inv;
            float gq = sage_oracle_bf16_to_f32(gain[d]);
            t[d] = sage_oracle_bf16_to_f32(sage_oracle_f32_to_bf16(a * gq));
        }
        uint16_t* dst = y + (((int64_t)b * N + n) * H + h) * D;
        if (cs) {
            int64_t row = (int64_t)b * table_batch_rows + (int64_t)n * H + h;
            for (int i = 0; i < half; i++) {
                float x0 = t[2 * i], x1 = t[2 * i + 1];
                float cv = cs[row * half + i], sv = sn[row * half + i];
                float a = x0 * cv, bb = x1 * sv, c = x0 * sv, dd = x1 * cv;
                dst[2 * i] = sage_oracle_f32_to_bf16(a - bb);
                dst[2 * i + 1] = sage_oracle_f32_to_bf16(c + dd);
            }
        } else {
            for (int d = 0; d < D; d++) dst[d] = sage_oracle_f32_to_bf16(t[d]);
        }
    }
    return 0;
}

/* One block of `rows` tokens by D channels, already transformed to fp32 in
 * `tile` (row-major rows x D): scale and codes. */
static void quant_block_i8(const float* tile, int rows, int D, int8_t* dst, float* scale_out) {
    float amax = 0.0f;
    for (int i = 0; i < rows * D; i++) {
        float a = fabsf(tile[i]);
        if (a > amax) amax = a;
    }
    /* scale = amax/127, 1.0 for an all-zero block (ops/fp8_quant.mojo:117) */
    float sc = (amax > 0.0f) ? (amax / 127.0f) : 1.0f;
    *scale_out = sc;
    for (int i = 0; i < rows * D; i++) {
        float r = rintf(tile[i] / sc);          /* true divide (:138), RNE (:42-50) */
        if (r > 127.0f) r = 127.0f;
        if (r < -127.0f) r = -127.0f;
        dst[i] = (int8_t)r;
    }
}

int sage_oracle_quant_q(const uint16_t* q, int B, int H, int N, int D,
                        const int64_t* st, float scale, int blkq, int npad_mult,
                        int8_t* q8, float* qscale) {
    if (bad_quant_args(q, B, H, N, D, st, blkq, npad_mult) || !q8 || !qscale) return -1;
    const float c = (float)((double)scale * 1.4426950408889634074);   /* scale*log2(e), rounded once */
    int64_t npad = sage_oracle_pad(N, npad_mult);
    int nblk = (N + blkq - 1) / blkq;
    memset(q8, 0, (size_t)B * H * npad * D);
    int64_t work = (int64_t)B * H * nblk;
#pragma omp parallel
    {
        float* tile = (float*)malloc(sizeof(float) * (size_t)blkq * D);
#pragma omp for schedule(static)
        for (int64_t w = 0; w < work; w++) {
            int t = (int)(w % nblk);
            int h = (int)((w / nblk) % H);
            int b = (int)(w / ((int64_t)nblk * H));
            int r0 = t * blkq;
            int rows = (N - r0 < blkq) ? (N - r0) : blkq;
            for (int i = 0; i < rows; i++) {
                const uint16_t* src = q + b * st[0] + h * st[1] + (int64_t)(r0 + i) * st[2];
                for (int d = 0; d < D; d++)
                    tile[i * D + d] = sage_oracle_bf16_to_f32(src[d * st[3]]) * c;
            }
            quant_block_i8(tile, rows, D, q8 + (((int64_t)b * H + h) * npad + r0) * D,
                           qscale + ((int64_t)b * H + h) * nblk + t);
        }
        free(tile);
    }
    return 0;
}

int sage_oracle_kmean(const uint16_t* k, int B, int H, int N, int D,
                      const int64_t* st, float* kmean) {
    if (bad_quant_args(k, B, H, N, D, st, 1, 1) || !kmean) return -1;
    int64_t work = (int64_t)B * H;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int h = (int)(w % H);
        int b = (int)(w / H);
        for (int d = 0; d < D; d++) {
            /* fixed summation tree: 16-token leaves (tokens ascending), 16-leaf
             * groups (leaves ascending), groups ascending */
            double sum = 0.0;
            for (int g0 = 0; g0 < N; g0 += 256) {
                double group = 0.0;
                for (int u0 = g0; u0 < g0 + 256 && u0 < N; u0 += 16) {
                    int u1 = (u0 + 16 < N) ? u0 + 16 : N;
                    double leaf = 0.0;
                    for (int s = u0; s < u1; s++)
                        leaf += (double)sage_oracle_bf16_to_f32(k[b * st[0] + h * st[1] + (int64_t)s * st[2] + d * st[3]]);
                    group += leaf;
                }
                sum += group;
            }
            kmean[w * D + d] = (float)(sum / (double)N);
        }
    }
    return 0;
}

int sage_oracle_quant_k(const uint16_t* k, int B, int H, int N, int D,
                        const int64_t* st, const float* kmean, int blkk, int npad_mult,
                        int8_t* k8, float* kscale) {
    if (bad_quant_args(k, B, H, N, D, st, blkk, npad_mult) || !k8 || !kscale) return -1;
    int64_t npad = sage_oracle_pad(N, npad_mult);
    int nblk = (N + blkk - 1) / blkk;
    memset(k8, 0, (size_t)B * H * npad * D);
    int64_t work = (int64_t)B * H * nblk;
#pragma omp parallel
    {
        float* tile = (float*)malloc(sizeof(float) * (size_t)blkk * D);
#pragma omp for schedule(static)
        for (int64_t w = 0; w < work; w++) {
            int t = (int)(w % nblk);
            int h = (int)((w / nblk) % H);
            int b = (int)(w / ((int64_t)nblk * H));
            int r0 = t * blkk;
            int rows = (N - r0 < blkk) ? (N - r0) : blkk;
            const float* mu = kmean ? kmean + ((int64_t)b * H + h) * D : NULL;
            for (int i = 0; i < rows; i++) {
                const uint16_t* src = k + b * st[0] + h * st[1] + (int64_t)(r0 + i) * st[2];
                for (int d = 0; d < D; d++) {
                    float x = sage_oracle_bf16_to_f32(src[d * st[3]]);
                    tile[i * D + d] = mu ? (x - mu[d]) : x;
                }
            }
            quant_block_i8(tile, rows, D, k8 + (((int64_t)b * H + h) * npad + r0) * D,
                           kscale + ((int64_t)b * H + h) * nblk + t);
        }
        free(tile);
    }
    return 0;
}

int sage_oracle_quant_v_f16(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* st, int npad_mult, uint16_t* v16) {
    if (bad_quant_args(v, B, H, N, D, st, 1, npad_mult) || !v16) return -1;
    int64_t npad = sage_oracle_pad(N, npad_mult);
    memset(v16, 0, (size_t)B * H * npad * D * 2);
    int64_t work = (int64_t)B * H * N;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int s = (int)(w % N);
        int h = (int)((w / N) % H);
        int b = (int)(w / ((int64_t)N * H));
        const uint16_t* src = v + b * st[0] + h * st[1] + (int64_t)s * st[2];
        uint16_t* dst = v16 + (((int64_t)b * H + h) * npad + s) * D;
        for (int d = 0; d < D; d++) dst[d] = sage_oracle_f32_to_f16(sage_oracle_bf16_to_f32(src[d * st[3]]));
    }
    return 0;
}

int sage_oracle_quant_v_fp8(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* st, int npad_mult, uint8_t* v8, float* vscale) {
    if (bad_quant_args(v, B, H, N, D, st, 1, npad_mult) || !v8 || !vscale) return -1;
    int64_t npad = sage_oracle_pad(N, npad_mult);
    memset(v8, 0, (size_t)B * H * npad * D);
    int64_t work = (int64_t)B * H;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int h = (int)(w % H);
        int b = (int)(w / H);
        for (int d = 0; d < D; d++) {
            float amax = 0.0f;
            for (int s = 0; s < N; s++) {
                float a = fabsf(sage_oracle_bf16_to_f32(v[b * st[0] + h * st[1] + (int64_t)s * st[2] + d * st[3]]));
                if (a > amax) amax = a;
            }
            /* ops/fp8_quant.mojo:116-118 */
            vscale[w * D + d] = (amax > 0.0f) ? (amax / 448.0f) : 1.0f;
        }
        for (int s = 0; s < N; s++) {
            const uint16_t* src = v + b * st[0] + h * st[1] + (int64_t)s * st[2];
            uint8_t* dst = v8 + ((int64_t)w * npad + s) * D;
            for (int d = 0; d < D; d++)
                dst[d] = sage_oracle_f32_to_e4m3(sage_oracle_bf16_to_f32(src[d * st[3]]) / vscale[w * D + d]);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* quantized attention                                                      */
/* ------------------------------------------------------------------------ */

static inline int32_t dot_i8(const int8_t* a, const int8_t* b, int D) {
    int32_t acc = 0;
    for (int d = 0; d < D; d++) acc += (int32_t)a[d] * (int32_t)b[d];
    return acc;
}

int sage_oracle_attn(const int8_t* q8, const float* qscale, int blkq, int64_t NqPad,
                     const int8_t* k8, const float* kscale, int blkk, int64_t NkvPad,
                     const void* vq, const float* vscale, int variant,
                     int B, int H, int Nq, int Nkv, int D,
                     uint16_t* o_bf16, float* o_f32, const int64_t* os) {
    if (!q8 || !qscale || !k8 || !kscale || !vq || !os) return -1;
    if (!o_bf16 && !o_f32) return -1;
    if (B <= 0 || H <= 0 || Nq <= 0 || Nkv <= 0 || D <= 0 || blkq <= 0 || blkk <= 0) return -1;
    if (variant != 0 && variant != 1) return -1;
    if (variant == 1 && !vscale) return -1;
    int nqb = (Nq + blkq - 1) / blkq, nkb = (Nkv + blkk - 1) / blkk;
    int64_t rows = (int64_t)B * H * Nq;
    int err = 0;

    /* V decoded to fp32 once (exact for both codecs). */
    float* vf = (float*)malloc(sizeof(float) * (size_t)B * H * NkvPad * D);
    if (!vf) return -1;
    int64_t nv = (int64_t)B * H * NkvPad * D;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nv; i++)
        vf[i] = variant == 0 ? sage_oracle_f16_to_f32(((const uint16_t*)vq)[i])
                             : sage_oracle_e4m3_to_f32(((const uint8_t*)vq)[i]);

#pragma omp parallel
    {
        float* sc = (float*)malloc(sizeof(float) * (size_t)Nkv);
        float* acc = (float*)malloc(sizeof(float) * (size_t)D);
        if (!sc || !acc) {
#pragma omp atomic write
            err = 1;
        }
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; r++) {
            if (!sc || !acc) continue;
            int i = (int)(r % Nq);
            int64_t bh = r / Nq;
            int h = (int)(bh % H);
            int b = (int)(bh / H);
            const int8_t* qr = q8 + (bh * NqPad + i) * D;
            float sq = qscale[bh * nqb + i / blkq];
            float mx = -INFINITY;
            for (int j = 0; j < Nkv; j++) {
                int32_t a = dot_i8(qr, k8 + (bh * NkvPad + j) * D, D);
                float s = (float)a * (sq * kscale[bh * nkb + j / blkk]);
                sc[j] = s;
                if (s > mx) mx = s;
            }
            double l = 0.0;
            for (int d = 0; d < D; d++) acc[d] = 0.0f;
            for (int j = 0; j < Nkv; j++) {
                float p = exp2f(sc[j] - mx);
                l += (double)p;
                float pq = variant == 0
                    ? sage_oracle_f16_to_f32(sage_oracle_f32_to_f16(p))
                    : sage_oracle_e4m3_to_f32(sage_oracle_f32_to_e4m3(p * 448.0f));
                if (pq == 0.0f) continue;
                const float* vr = vf + (bh * NkvPad + j) * D;
                for (int d = 0; d < D; d++) acc[d] += pq * vr[d];
            }
            for (int d = 0; d < D; d++) {
                double o = variant == 0
                    ? (double)acc[d] / l
                    : (double)acc[d] * (double)vscale[bh * D + d] / (448.0 * l);
                int64_t off = b * os[0] + h * os[1] + (int64_t)i * os[2] + d * os[3];
                if (o_f32) o_f32[off] = (float)o;
                if (o_bf16) o_bf16[off] = sage_oracle_f32_to_bf16((float)o);
            }
        }
        free(sc);
        free(acc);
    }
    free(vf);
    return err ? -1 : 0;
}

int sage_oracle_sdpa_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                          uint16_t* o, float* o_f32,
                          int B, int H, int Nq, int Nkv, int D, float scale,
                          const int64_t* qs, const int64_t* ks,
                          const int64_t* vs, const int64_t* os,
                          int variant, int blkq, int blkk, int smooth_k) {
    if (bad_args(q, k, v, o ? (void*)o : (void*)o_f32, B, H, Nq, Nkv, D, qs, ks, vs, os)) return -1;
    if (blkq <= 0 || blkk <= 0) return -1;
    int64_t nqp = sage_oracle_pad(Nq, blkq), nkp = sage_oracle_pad(Nkv, blkk);
    int nqb = (Nq + blkq - 1) / blkq, nkb = (Nkv + blkk - 1) / blkk;
    size_t bh = (size_t)B * H;
    int8_t* q8 = (int8_t*)malloc(bh * nqp * D);
    int8_t* k8 = (int8_t*)malloc(bh * nkp * D);
    float* qsc = (float*)malloc(sizeof(float) * bh * nqb);
    float* ksc = (float*)malloc(sizeof(float) * bh * nkb);
    float* mu = (float*)malloc(sizeof(float) * bh * D);
    float* vsc = (float*)malloc(sizeof(float) * bh * D);
    void* vq = malloc(bh * nkp * D * (variant == 0 ? 2 : 1));
    int rc = -1;
    if (q8 && k8 && qsc && ksc && mu && vsc && vq) {
        rc = sage_oracle_quant_q(q, B, H, Nq, D, qs, scale, blkq, blkq, q8, qsc);
        if (!rc && smooth_k) rc = sage_oracle_kmean(k, B, H, Nkv, D, ks, mu);
        if (!rc) rc = sage_oracle_quant_k(k, B, H, Nkv, D, ks, smooth_k ? mu : NULL, blkk, blkk, k8, ksc);
        if (!rc) rc = variant == 0
            ? sage_oracle_quant_v_f16(v, B, H, Nkv, D, vs, blkk, (uint16_t*)vq)
            : sage_oracle_quant_v_fp8(v, B, H, Nkv, D, vs, blkk, (uint8_t*)vq, vsc);
        if (!rc) rc = sage_oracle_attn(q8, qsc, blkq, nqp, k8, ksc, blkk, nkp, vq, vsc, variant,
                                       B, H, Nq, Nkv, D, o, o_f32, os);
    }
    free(q8); free(k8); free(qsc); free(ksc); free(mu); free(vsc); free(vq);
    return rc;
}
