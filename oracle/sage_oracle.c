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

/* mask_lo/mask_hi: keys in [mask_lo, mask_hi) are left out (serenitymojo/ops/attention.mojo:1790-1857
 * adds -1e4 to them, which leaves exp() == 0 in fp32).  addmask: additive bias in natural-log
 * units, contiguous [B,H,Nq,Nkv] (attention.mojo:1596-1647), or NULL.  stats (optional,
 * [B,H,Nq]): natural-log log-sum-exp of the scaled, biased scores. */
int sage_oracle_sdpa_f32_ex(const float* q, const float* k, const float* v, float* o,
                            int B, int H, int Nq, int Nkv, int D, float scale,
                            const int64_t* qs, const int64_t* ks,
                            const int64_t* vs, const int64_t* os,
                            int mask_lo, int mask_hi, const float* addmask, float* stats) {
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
                if (addmask) s += (double)addmask[(((int64_t)b * H + h) * Nq + i) * (int64_t)Nkv + j];
                if (j >= mask_lo && j < mask_hi) s = -INFINITY;
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
            if (stats) stats[((int64_t)b * H + h) * Nq + i] = (float)(mx + log(l));
        }
        free(sc);
        free(acc);
    }
    return err ? -1 : 0;
}

int sage_oracle_sdpa_f32(const float* q, const float* k, const float* v, float* o,
                         int B, int H, int Nq, int Nkv, int D, float scale,
                         const int64_t* qs, const int64_t* ks,
                         const int64_t* vs, const int64_t* os) {
    return sage_oracle_sdpa_f32_ex(q, k, v, o, B, H, Nq, Nkv, D, scale, qs, ks, vs, os, 0, 0, NULL, NULL);
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

/* ---- backward of the full-precision SDPA ---------------------------------- */
/* The decomposed backward of serenitymojo/ops/attention_backward.mojo:12-19,
 *   attn = softmax(Q K^T * scale);  dV = attn^T dO;  dA = dO V^T;
 *   dS = attn * (dA - rowsum(dA * attn));  dQ = dS K * scale;  dK = dS^T Q * scale,
 * in double precision on one (b,h) at a time.  With `o` and `stats` NULL the probabilities
 * are recomputed from q and k (what torch.autograd does to ops/parity/sdpa_bwd_oracle.py:56-63);
 * with both given (the flash interface of ops/cshim/cudnn_sdpa_bwd.cpp:325-347) they are
 * attn = exp(score - stats[row]) with the caller's log-sum-exp, and rowsum(dA * attn) is taken as
 * rowsum(dO * O) — equal in exact arithmetic, and what a kernel that never holds a whole row has
 * to use.  In that form dQ = scale * dS (K - kbar) with kbar the mean of the valid keys: a row of
 * dS sums to zero when O and stats belong to these probabilities, so any constant vector may be
 * taken off the keys; when they come from a forward of other precision (the quantized one) the
 * row sum is a small non-zero number and the uncentred product would multiply it by the keys'
 * common offset.  Query rows >= real_nq and keys >= real_nkv are padding: they take no part and their
 * gradient rows are zero (cudnn_sdpa_bwd.cpp:344 real_N_q / real_N_kv). */
int sage_oracle_sdpa_bwd_f32(const float* q, const float* k, const float* v, const float* o,
                             const float* dout, const float* stats,
                             float* dq, float* dk, float* dv,
                             int B, int H, int Nq, int Nkv, int D, float scale,
                             const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                             const int64_t* dos, const int64_t* dqs, const int64_t* dks, const int64_t* dvs,
                             int real_nq, int real_nkv) {
    if (!q || !k || !v || !dout || !dq || !dk || !dv) return -1;
    if ((o == NULL) != (stats == NULL)) return -1;
    if (B <= 0 || H <= 0 || Nq <= 0 || Nkv <= 0 || D <= 0) return -1;
    if (!qs || !ks || !vs || !dos || !dqs || !dks || !dvs || (o && !os)) return -1;
    const int nq = real_nq > 0 && real_nq < Nq ? real_nq : Nq;
    const int nk = real_nkv > 0 && real_nkv < Nkv ? real_nkv : Nkv;
    double* P = (double*)malloc(sizeof(double) * (size_t)nq * (size_t)nk);
    double* dS = (double*)malloc(sizeof(double) * (size_t)nq * (size_t)nk);
    double* kbar = (double*)malloc(sizeof(double) * (size_t)D);
    if (!P || !dS || !kbar) { free(P); free(dS); free(kbar); return -1; }
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const float* qb = q + b * qs[0] + h * qs[1];
            const float* kb = k + b * ks[0] + h * ks[1];
            const float* vb = v + b * vs[0] + h * vs[1];
            const float* gb = dout + b * dos[0] + h * dos[1];
            for (int d = 0; d < D; d++) {
                double m = 0.0;
                if (stats)
                    for (int j = 0; j < nk; j++) m += (double)kb[j * ks[2] + d * ks[3]];
                kbar[d] = m / (double)nk;
            }
#pragma omp parallel for schedule(dynamic, 8)
            for (int i = 0; i < nq; i++) {
                const float* qr = qb + i * qs[2];
                const float* gr = gb + i * dos[2];
                double* Pr = P + (size_t)i * nk;
                double* Sr = dS + (size_t)i * nk;
                double mx = -INFINITY;
                for (int j = 0; j < nk; j++) {
                    const float* kr = kb + j * ks[2];
                    double dot = 0.0;
                    for (int d = 0; d < D; d++) dot += (double)qr[d * qs[3]] * (double)kr[d * ks[3]];
                    Pr[j] = dot * (double)scale;
                    if (Pr[j] > mx) mx = Pr[j];
                }
                double delta = 0.0;
                if (stats) {
                    const double lse = (double)stats[((int64_t)b * H + h) * Nq + i];
                    for (int j = 0; j < nk; j++) Pr[j] = exp(Pr[j] - lse);
                    const float* orow = o + b * os[0] + h * os[1] + i * os[2];
                    for (int d = 0; d < D; d++) delta += (double)gr[d * dos[3]] * (double)orow[d * os[3]];
                } else {
                    double l = 0.0;
                    for (int j = 0; j < nk; j++) { Pr[j] = exp(Pr[j] - mx); l += Pr[j]; }
                    for (int j = 0; j < nk; j++) Pr[j] /= l;
                }
                for (int j = 0; j < nk; j++) {
                    const float* vr = vb + j * vs[2];
                    double da = 0.0;
                    for (int d = 0; d < D; d++) da += (double)gr[d * dos[3]] * (double)vr[d * vs[3]];
                    Sr[j] = da;
                    if (!stats) delta += da * Pr[j];
                }
                for (int j = 0; j < nk; j++) Sr[j] = Pr[j] * (Sr[j] - delta);
                float* dqr = dq + b * dqs[0] + h * dqs[1] + i * dqs[2];
                for (int d = 0; d < D; d++) {
                    double a = 0.0;
                    for (int j = 0; j < nk; j++) a += Sr[j] * ((double)kb[j * ks[2] + d * ks[3]] - kbar[d]);
                    dqr[d * dqs[3]] = (float)(a * (double)scale);
                }
            }
#pragma omp parallel for schedule(dynamic, 8)
            for (int j = 0; j < nk; j++) {
                float* dkr = dk + b * dks[0] + h * dks[1] + j * dks[2];
                float* dvr = dv + b * dvs[0] + h * dvs[1] + j * dvs[2];
                for (int d = 0; d < D; d++) {
                    double ak = 0.0, av = 0.0;
                    for (int i = 0; i < nq; i++) {
                        ak += dS[(size_t)i * nk + j] * (double)qb[i * qs[2] + d * qs[3]];
                        av += P[(size_t)i * nk + j] * (double)gb[i * dos[2] + d * dos[3]];
                    }
                    dkr[d * dks[3]] = (float)(ak * (double)scale);
                    dvr[d * dvs[3]] = (float)av;
                }
            }
            for (int i = nq; i < Nq; i++)
                for (int d = 0; d < D; d++) dq[b * dqs[0] + h * dqs[1] + i * dqs[2] + d * dqs[3]] = 0.0f;
            for (int j = nk; j < Nkv; j++)
                for (int d = 0; d < D; d++) {
                    dk[b * dks[0] + h * dks[1] + j * dks[2] + d * dks[3]] = 0.0f;
                    dv[b * dvs[0] + h * dvs[1] + j * dvs[2] + d * dvs[3]] = 0.0f;
                }
        }
    free(P);
    free(dS);
    free(kbar);
    return 0;
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
 * The order in which the squares are added is the reference's own (:56-72): a block of 256
 * threads, thread t adds x[t]^2, x[t+256]^2, ... left to right into `local` (starting from 0),
 * writes it to shared[t], then the tree  shared[t] += shared[t + active]  runs for
 * active = 128, 64, ..., 1 — the far pairs first.  For D = 128 that is x[t]^2 + x[t+64]^2 first
 * (the active = 128 step adds the zeros of the idle threads), then strides 32, 16, 8, 4, 2, 1. */
static float sumsq_tree(const float* v, int cols) {
    float shared[256];
    for (int t = 0; t < 256; t++) {
        float local = 0.0f;
        for (int c = t; c < cols; c += 256) {
            float sq = v[c] * v[c];
            local = local + sq;
        }
        shared[t] = local;
    }
    for (int active = 128; active > 0; active /= 2)
        for (int t = 0; t < active; t++) shared[t] = shared[t] + shared[t + active];
    return shared[0];
}

static float rms_inv(const float* v, int cols, float eps) {
    float ss = sumsq_tree(v, cols);
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

/* serenitymojo/ops/rope.mojo:10-13, :147-165: pairs (x[i], x[i + D/2]); separate multiplies, then
 * one subtract / add. */
int sage_oracle_rope_halfsplit_f32(const float* x, const float* cs, const float* sn,
                                   int64_t rows, int D, float* out) {
    if (!x || !cs || !sn || !out || rows <= 0 || D <= 0 || (D & 1)) return -1;
    int half = D / 2;
    for (int64_t r = 0; r < rows; r++)
        for (int i = 0; i < half; i++) {
            float x0 = x[r * D + i], x1 = x[r * D + i + half];
            float cv = cs[r * half + i], sv = sn[r * half + i];
            float a = x0 * cv, b = x1 * sv, c = x1 * cv, d = x0 * sv;
            out[r * D + i] = a - b;
            out[r * D + i + half] = c + d;
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
    return sage_oracle_norm_rope_bf16_ex(x, B, H, N, D, st, gain, eps, cs, sn, table_batch_rows, 0, y);
}

/* pre_flags: bit 0 — half-split pairs (rope.mojo:10-13) instead of interleaved ones (rope.mojo:7-9),
 * the per-head RMSNorm + rope_halfsplit sequence of serenitymojo/models/anima/block.mojo:360-366;
 * bit 1 — the tables are bf16 (the kernels cast them to fp32, rope.mojo:160-163);
 * bit 2 — the RMSNorm runs over the whole row of H*D channels with a gain of H*D entries
 * (channel h*D + d), the rms_norm on [S, H*D] before the reshape of
 * serenitymojo/models/ltx2/ltx2_block.mojo:419-432. */
int sage_oracle_norm_rope_bf16_ex(const uint16_t* x, int B, int H, int N, int D, const int64_t* st,
                                  const uint16_t* gain, float eps, const void* cs, const void* sn,
                                  int64_t table_batch_rows, int pre_flags, uint16_t* y) {
    if (pre_flags & ~7) return -1;
    if (!x || !st || !gain || !y || B <= 0 || H <= 0 || N <= 0 || D <= 0 || (D & 1) || D > 1024) return -1;
    if ((cs == NULL) != (sn == NULL)) return -1;
    const int halfsplit = pre_flags & 1, tab16 = pre_flags & 2, fullrow = pre_flags & 4;
    int half = D / 2;
    /* whole-row statistic first (one value per token) */
    float* row_inv = NULL;
    if (fullrow) {
        row_inv = (float*)malloc(sizeof(float) * (size_t)B * (size_t)N);
        if (!row_inv) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < (int64_t)B * N; r++) {
            int n = (int)(r % N), b = (int)(r / N);
            float* v = (float*)malloc(sizeof(float) * (size_t)H * (size_t)D);
            for (int h = 0; h < H; h++)
                for (int d = 0; d < D; d++)
                    v[h * D + d] = sage_oracle_bf16_to_f32(x[b * st[0] + h * st[1] + (int64_t)n * st[2] + d * st[3]]);
            row_inv[r] = rms_inv(v, H * D, eps);
            free(v);
        }
    }
    int64_t work = (int64_t)B * N * H;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int h = (int)(w % H);
        int n = (int)((w / H) % N);
        int b = (int)(w / ((int64_t)H * N));
        float v[1024], t[1024];
        const uint16_t* src = x + b * st[0] + h * st[1] + (int64_t)n * st[2];
        for (int d = 0; d < D; d++) v[d] = sage_oracle_bf16_to_f32(src[d * st[3]]);
        float inv = fullrow ? row_inv[(int64_t)b * N + n] : rms_inv(v, D, eps);
        const uint16_t* gh = fullrow ? gain + (int64_t)h * D : gain;
        for (int d = 0; d < D; d++) {
            float a = v[d] * inv;
            float gq = sage_oracle_bf16_to_f32(gh[d]);
            t[d] = sage_oracle_bf16_to_f32(sage_oracle_f32_to_bf16(a * gq));
        }
        uint16_t* dst = y + (((int64_t)b * N + n) * H + h) * D;
        if (cs) {
            int64_t row = (int64_t)b * table_batch_rows + (int64_t)n * H + h;
            for (int i = 0; i < half; i++) {
                int i0 = halfsplit ? i : 2 * i, i1 = halfsplit ? i + half : 2 * i + 1;
                float x0 = t[i0], x1 = t[i1];
                float cv = tab16 ? sage_oracle_bf16_to_f32(((const uint16_t*)cs)[row * half + i]) : ((const float*)cs)[row * half + i];
                float sv = tab16 ? sage_oracle_bf16_to_f32(((const uint16_t*)sn)[row * half + i]) : ((const float*)sn)[row * half + i];
                float a = x0 * cv, bb = x1 * sv, c = x0 * sv, dd = x1 * cv;
                dst[i0] = sage_oracle_f32_to_bf16(a - bb);
                dst[i1] = sage_oracle_f32_to_bf16(c + dd);
            }
        } else {
            for (int d = 0; d < D; d++) dst[d] = sage_oracle_f32_to_bf16(t[d]);
        }
    }
    free(row_inv);
    return 0;
}

/* One block of `rows` tokens by D channels, already transformed to fp32 in
 * `tile` (row-major rows x D); keep[i] == 0 marks a masked token: it does not count for
 * the block maximum and its codes are 0.  keep == NULL: every row counts. */
static void quant_block_i8(const float* tile, const uint8_t* keep, int rows, int D, int8_t* dst, float* scale_out) {
    float amax = 0.0f;
    for (int r = 0; r < rows; r++) {
        if (keep && !keep[r]) continue;
        for (int d = 0; d < D; d++) {
            float a = fabsf(tile[r * D + d]);
            if (a > amax) amax = a;
        }
    }
    /* scale = amax/127, 1.0 for an all-zero block (ops/fp8_quant.mojo:117) */
    float sc = (amax > 0.0f) ? (amax / 127.0f) : 1.0f;
    *scale_out = sc;
    for (int r = 0; r < rows; r++)
        for (int d = 0; d < D; d++) {
            float q = 0.0f;
            if (!keep || keep[r]) {
                q = rintf(tile[r * D + d] / sc);      /* true divide (:138), RNE (:42-50) */
                if (q > 127.0f) q = 127.0f;
                if (q < -127.0f) q = -127.0f;
            }
            dst[r * D + d] = (int8_t)q;
        }
}

static inline int key_kept(int s, int N, int mask_lo, int mask_hi) {
    return s < N && !(s >= mask_lo && s < mask_hi);
}

static float c_of_scale(float scale) {
    return (float)((double)scale * 1.4426950408889634074);   /* scale*log2(e), rounded once */
}

int sage_oracle_quant_q_ch(const uint16_t* q, int B, int H, int N, int D,
                           const int64_t* st, float scale, const float* qmul, int blkq, int npad_mult,
                           int8_t* q8, float* qscale) {
    if (bad_quant_args(q, B, H, N, D, st, blkq, npad_mult) || !q8 || !qscale) return -1;
    const float c = c_of_scale(scale);
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
            const float* mul = qmul ? qmul + ((int64_t)b * H + h) * D : NULL;
            for (int i = 0; i < rows; i++) {
                const uint16_t* src = q + b * st[0] + h * st[1] + (int64_t)(r0 + i) * st[2];
                for (int d = 0; d < D; d++)
                    tile[i * D + d] = sage_oracle_bf16_to_f32(src[d * st[3]]) * (mul ? mul[d] : c);
            }
            quant_block_i8(tile, NULL, rows, D, q8 + (((int64_t)b * H + h) * npad + r0) * D,
                           qscale + ((int64_t)b * H + h) * nblk + t);
        }
        free(tile);
    }
    return 0;
}

int sage_oracle_quant_q(const uint16_t* q, int B, int H, int N, int D,
                        const int64_t* st, float scale, int blkq, int npad_mult,
                        int8_t* q8, float* qscale) {
    return sage_oracle_quant_q_ch(q, B, H, N, D, st, scale, NULL, blkq, npad_mult, q8, qscale);
}

int sage_oracle_kstats(const uint16_t* k, int B, int H, int N, int D, const int64_t* st,
                       float scale, int flags, int mask_lo, int mask_hi,
                       float* kmean, float* qmul, float* kmul) {
    if (bad_quant_args(k, B, H, N, D, st, 1, 1) || !kmean || !qmul || !kmul) return -1;
    int kept = 0;
    for (int s = 0; s < N; s++) kept += key_kept(s, N, mask_lo, mask_hi);
    if (kept == 0) return -1;
    const float c = c_of_scale(scale);
    int64_t work = (int64_t)B * H;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int h = (int)(w % H);
        int b = (int)(w / H);
        for (int d = 0; d < D; d++) {
            /* fixed summation tree: 16-token leaves (tokens ascending), 16-leaf
             * groups (leaves ascending), groups ascending; masked tokens add +0.0 */
            double sum = 0.0;
            float kmax = -INFINITY, kmin = INFINITY;
            for (int g0 = 0; g0 < N; g0 += 256) {
                double group = 0.0;
                for (int u0 = g0; u0 < g0 + 256 && u0 < N; u0 += 16) {
                    int u1 = (u0 + 16 < N) ? u0 + 16 : N;
                    double leaf = 0.0;
                    for (int s = u0; s < u1; s++) {
                        if (!key_kept(s, N, mask_lo, mask_hi)) continue;
                        float x = sage_oracle_bf16_to_f32(k[b * st[0] + h * st[1] + (int64_t)s * st[2] + d * st[3]]);
                        leaf += (double)x;
                        if (x > kmax) kmax = x;
                        if (x < kmin) kmin = x;
                    }
                    group += leaf;
                }
                sum += group;
            }
            float mean = (flags & 1) ? (float)(sum / (double)kept) : 0.0f;
            float s_d = 1.0f;
            if (flags & 2) {
                /* rounding is monotone, so the largest |k - mean| over the keys is reached at the
                 * largest or the smallest key of the channel */
                float hi = fabsf(kmax - mean), lo = fabsf(kmin - mean);
                float amax = hi > lo ? hi : lo;
                if (amax > 0.0f) s_d = sqrtf(amax);
            }
            kmean[w * D + d] = mean;
            kmul[w * D + d] = 1.0f / s_d;
            qmul[w * D + d] = c * s_d;
        }
    }
    return 0;
}

int sage_oracle_kmean(const uint16_t* k, int B, int H, int N, int D,
                      const int64_t* st, float* kmean) {
    if (bad_quant_args(k, B, H, N, D, st, 1, 1) || !kmean) return -1;
    float* tmp = (float*)malloc(sizeof(float) * 2 * (size_t)B * H * D);
    if (!tmp) return -1;
    int rc = sage_oracle_kstats(k, B, H, N, D, st, 1.0f, 1, 0, 0, kmean, tmp, tmp + (size_t)B * H * D);
    free(tmp);
    return rc;
}

int sage_oracle_quant_k_ch(const uint16_t* k, int B, int H, int N, int D,
                           const int64_t* st, const float* kmean, const float* kmul,
                           int mask_lo, int mask_hi, int blkk, int npad_mult,
                           int8_t* k8, float* kscale) {
    if (bad_quant_args(k, B, H, N, D, st, blkk, npad_mult) || !k8 || !kscale) return -1;
    int64_t npad = sage_oracle_pad(N, npad_mult);
    int nblk = (N + blkk - 1) / blkk;
    memset(k8, 0, (size_t)B * H * npad * D);
    int64_t work = (int64_t)B * H * nblk;
#pragma omp parallel
    {
        float* tile = (float*)malloc(sizeof(float) * (size_t)blkk * D);
        uint8_t* keep = (uint8_t*)malloc((size_t)blkk);
#pragma omp for schedule(static)
        for (int64_t w = 0; w < work; w++) {
            int t = (int)(w % nblk);
            int h = (int)((w / nblk) % H);
            int b = (int)(w / ((int64_t)nblk * H));
            int r0 = t * blkk;
            int rows = (N - r0 < blkk) ? (N - r0) : blkk;
            const float* mu = kmean ? kmean + ((int64_t)b * H + h) * D : NULL;
            const float* mul = kmul ? kmul + ((int64_t)b * H + h) * D : NULL;
            for (int i = 0; i < rows; i++) {
                const uint16_t* src = k + b * st[0] + h * st[1] + (int64_t)(r0 + i) * st[2];
                keep[i] = (uint8_t)key_kept(r0 + i, N, mask_lo, mask_hi);
                for (int d = 0; d < D; d++) {
                    float x = sage_oracle_bf16_to_f32(src[d * st[3]]);
                    if (mu) x = x - mu[d];
                    if (mul) x = x * mul[d];
                    tile[i * D + d] = x;
                }
            }
            quant_block_i8(tile, keep, rows, D, k8 + (((int64_t)b * H + h) * npad + r0) * D,
                           kscale + ((int64_t)b * H + h) * nblk + t);
        }
        free(tile);
        free(keep);
    }
    return 0;
}

int sage_oracle_quant_k(const uint16_t* k, int B, int H, int N, int D,
                        const int64_t* st, const float* kmean, int blkk, int npad_mult,
                        int8_t* k8, float* kscale) {
    return sage_oracle_quant_k_ch(k, B, H, N, D, st, kmean, NULL, 0, 0, blkk, npad_mult, k8, kscale);
}

int sage_oracle_quant_v_f16_masked(const uint16_t* v, int B, int H, int N, int D,
                                   const int64_t* st, int mask_lo, int mask_hi, int npad_mult, uint16_t* v16) {
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
        if (!key_kept(s, N, mask_lo, mask_hi)) continue;          /* masked rows stay 0 */
        for (int d = 0; d < D; d++) dst[d] = sage_oracle_f32_to_f16(sage_oracle_bf16_to_f32(src[d * st[3]]));
    }
    return 0;
}

int sage_oracle_quant_v_f16(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* st, int npad_mult, uint16_t* v16) {
    return sage_oracle_quant_v_f16_masked(v, B, H, N, D, st, 0, 0, npad_mult, v16);
}

int sage_oracle_quant_v_fp8_masked(const uint16_t* v, int B, int H, int N, int D,
                                   const int64_t* st, int mask_lo, int mask_hi, int npad_mult,
                                   uint8_t* v8, float* vscale) {
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
                if (!key_kept(s, N, mask_lo, mask_hi)) continue;
                float a = fabsf(sage_oracle_bf16_to_f32(v[b * st[0] + h * st[1] + (int64_t)s * st[2] + d * st[3]]));
                if (a > amax) amax = a;
            }
            /* ops/fp8_quant.mojo:116-118 */
            vscale[w * D + d] = (amax > 0.0f) ? (amax / 448.0f) : 1.0f;
        }
        for (int s = 0; s < N; s++) {
            const uint16_t* src = v + b * st[0] + h * st[1] + (int64_t)s * st[2];
            uint8_t* dst = v8 + ((int64_t)w * npad + s) * D;
            if (!key_kept(s, N, mask_lo, mask_hi)) continue;      /* masked rows stay 0 */
            for (int d = 0; d < D; d++)
                dst[d] = sage_oracle_f32_to_e4m3(sage_oracle_bf16_to_f32(src[d * st[3]]) / vscale[w * D + d]);
        }
    }
    return 0;
}

int sage_oracle_quant_v_fp8(const uint16_t* v, int B, int H, int N, int D,
                            const int64_t* st, int npad_mult, uint8_t* v8, float* vscale) {
    return sage_oracle_quant_v_fp8_masked(v, B, H, N, D, st, 0, 0, npad_mult, v8, vscale);
}

/* ------------------------------------------------------------------------ */
/* quantized attention                                                      */
/* ------------------------------------------------------------------------ */

static inline int32_t dot_i8(const int8_t* a, const int8_t* b, int D) {
    int32_t acc = 0;
    for (int d = 0; d < D; d++) acc += (int32_t)a[d] * (int32_t)b[d];
    return acc;
}

int sage_oracle_attn_ex(const int8_t* q8, const float* qscale, int blkq, int64_t NqPad,
                        const int8_t* k8, const float* kscale, int blkk, int64_t NkvPad,
                        const void* vq, const float* vscale, int variant,
                        int B, int H, int Nq, int Nkv, int D,
                        int mask_lo, int mask_hi, const float* addmask, const float* qshift,
                        uint16_t* o_bf16, float* o_f32, const int64_t* os, float* stats) {
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
                if (!key_kept(j, Nkv, mask_lo, mask_hi)) { sc[j] = -INFINITY; continue; }
                int32_t a = dot_i8(qr, k8 + (bh * NkvPad + j) * D, D);
                float s = (float)a * (sq * kscale[bh * nkb + j / blkk]);
                /* an additive mask is given in natural-log units per (b,h,i,j) */
                if (addmask) s = s + addmask[(bh * Nq + i) * (int64_t)Nkv + j] * 1.44269504088896340736f;
                sc[j] = s;
                if (s > mx) mx = s;
            }
            /* e4m3 probabilities are taken against an INTEGER reference (the row maximum rounded
             * up): moving the reference by a whole number only shifts the exponent of every
             * probability, so any kernel that keeps an integer reference within the format's
             * range rounds each probability to the same significand. */
            float mref = variant == 1 ? ceilf(mx) : mx;
            double l = 0.0;
            for (int d = 0; d < D; d++) acc[d] = 0.0f;
            for (int j = 0; j < Nkv; j++) {
                float p = exp2f(sc[j] - mref);
                float pq = variant == 0
                    ? sage_oracle_f16_to_f32(sage_oracle_f32_to_f16(p))
                    : sage_oracle_e4m3_to_f32(sage_oracle_f32_to_e4m3(p * 448.0f));
                /* The e4m3 variant normalises by the sum of the ROUNDED probabilities (the weights
                 * the product really uses): a row dominated by one key then returns that key's V
                 * exactly, whatever the rounding of its probability. */
                l += variant == 0 ? (double)p : (double)pq / 448.0;
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
            if (stats) {
                /* natural-log log-sum-exp of the scaled scores; K smoothing lowered every score of
                 * the row by qshift (log2 units) */
                double lse2 = (double)mref + log2(l) + (qshift ? (double)qshift[bh * NqPad + i] : 0.0);
                stats[bh * Nq + i] = (float)(lse2 * 0.69314718055994530942);
            }
        }
        free(sc);
        free(acc);
    }
    free(vf);
    return err ? -1 : 0;
}

int sage_oracle_attn(const int8_t* q8, const float* qscale, int blkq, int64_t NqPad,
                     const int8_t* k8, const float* kscale, int blkk, int64_t NkvPad,
                     const void* vq, const float* vscale, int variant,
                     int B, int H, int Nq, int Nkv, int D,
                     uint16_t* o_bf16, float* o_f32, const int64_t* os) {
    return sage_oracle_attn_ex(q8, qscale, blkq, NqPad, k8, kscale, blkk, NkvPad, vq, vscale, variant,
                               B, H, Nq, Nkv, D, 0, 0, NULL, NULL, o_bf16, o_f32, os, NULL);
}

/* <q*c, kmean> per query row (log2 units): what K smoothing subtracts from every score of the row. */
static void rowdot_q(const uint16_t* q, int B, int H, int N, int D, const int64_t* st, float scale,
                     const float* kmean, int64_t npad, float* out) {
    const float c = c_of_scale(scale);
    int64_t work = (int64_t)B * H * N;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; w++) {
        int i = (int)(w % N);
        int64_t bh = w / N;
        int h = (int)(bh % H), b = (int)(bh / H);
        const uint16_t* src = q + b * st[0] + h * st[1] + (int64_t)i * st[2];
        double dot = 0.0;
        for (int d = 0; d < D; d++)
            dot += (double)(sage_oracle_bf16_to_f32(src[d * st[3]]) * c) * (double)kmean[bh * D + d];
        out[bh * npad + i] = (float)dot;
    }
}

int sage_oracle_sdpa_bf16_ex(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                             uint16_t* o, float* o_f32, float* stats,
                             int B, int H, int Nq, int Nkv, int D, float scale,
                             const int64_t* qs, const int64_t* ks,
                             const int64_t* vs, const int64_t* os,
                             int variant, int blkq, int blkk, int k_flags,
                             int mask_lo, int mask_hi, const float* addmask) {
    if (bad_args(q, k, v, o ? (void*)o : (void*)o_f32, B, H, Nq, Nkv, D, qs, ks, vs, os)) return -1;
    if (blkq <= 0 || blkk <= 0) return -1;
    int64_t nqp = sage_oracle_pad(Nq, blkq), nkp = sage_oracle_pad(Nkv, blkk);
    int nqb = (Nq + blkq - 1) / blkq, nkb = (Nkv + blkk - 1) / blkk;
    size_t bh = (size_t)B * H;
    int8_t* q8 = (int8_t*)malloc(bh * nqp * D);
    int8_t* k8 = (int8_t*)malloc(bh * nkp * D);
    float* qsc = (float*)malloc(sizeof(float) * bh * nqb);
    float* ksc = (float*)malloc(sizeof(float) * bh * nkb);
    float* mu = (float*)malloc(sizeof(float) * bh * D * 3);
    float* vsc = (float*)malloc(sizeof(float) * bh * D);
    float* shift = stats ? (float*)malloc(sizeof(float) * bh * nqp) : NULL;
    void* vq = malloc(bh * nkp * D * (variant == 0 ? 2 : 1));
    int rc = -1;
    if (q8 && k8 && qsc && ksc && mu && vsc && vq && (!stats || shift)) {
        float* qmul = mu + bh * D;
        float* kmul = mu + 2 * bh * D;
        rc = sage_oracle_kstats(k, B, H, Nkv, D, ks, scale, k_flags, mask_lo, mask_hi, mu, qmul, kmul);
        if (!rc) rc = sage_oracle_quant_q_ch(q, B, H, Nq, D, qs, scale, qmul, blkq, blkq, q8, qsc);
        if (!rc) rc = sage_oracle_quant_k_ch(k, B, H, Nkv, D, ks, mu, kmul, mask_lo, mask_hi, blkk, blkk, k8, ksc);
        if (!rc) rc = variant == 0
            ? sage_oracle_quant_v_f16_masked(v, B, H, Nkv, D, vs, mask_lo, mask_hi, blkk, (uint16_t*)vq)
            : sage_oracle_quant_v_fp8_masked(v, B, H, Nkv, D, vs, mask_lo, mask_hi, blkk, (uint8_t*)vq, vsc);
        if (!rc && stats) rowdot_q(q, B, H, Nq, D, qs, scale, mu, nqp, shift);
        if (!rc) rc = sage_oracle_attn_ex(q8, qsc, blkq, nqp, k8, ksc, blkk, nkp, vq, vsc, variant,
                                          B, H, Nq, Nkv, D, mask_lo, mask_hi, addmask, shift, o, o_f32, os, stats);
    }
    free(q8); free(k8); free(qsc); free(ksc); free(mu); free(vsc); free(vq); free(shift);
    return rc;
}

int sage_oracle_sdpa_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                          uint16_t* o, float* o_f32,
                          int B, int H, int Nq, int Nkv, int D, float scale,
                          const int64_t* qs, const int64_t* ks,
                          const int64_t* vs, const int64_t* os,
                          int variant, int blkq, int blkk, int k_flags) {
    return sage_oracle_sdpa_bf16_ex(q, k, v, o, o_f32, NULL, B, H, Nq, Nkv, D, scale, qs, ks, vs, os,
                                    variant, blkq, blkk, k_flags, 0, 0, NULL);
}
