// mfma_valu_issue.hip — two measurements behind the attention kernel's design, on one MI355X:
//
//   issue   How matrix (MFMA) and vector (VALU) instructions share a SIMD's issue port:
//           (a) one wave issuing an MFMA followed by N independent VALU instructions,
//           (b) two waves on one SIMD, one issuing only MFMAs, the other only VALU work.
//           Times are shader clocks per MFMA (s_memtime).
//   clock   The shader clock under load: W workgroups of 512 threads run the kernel's
//           instruction mix (24 MFMA + ~130 VALU per wave and tile, no memory traffic) for a
//           fixed number of tiles; clock = shader cycles (s_memtime) / elapsed constant-rate
//           time (s_memrealtime, 100 MHz).  Once with the same operand registers for every
//           matrix instruction and once with operands that differ from one instruction to the
//           next (random bits), which is what real data looks like to the multipliers.
//
//   usage: mfma_valu_issue issue | clock
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

#define CHECK(x)                                                                       \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));               \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

// KIND 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_f32_32x32x16_f16; accumulators pinned to VGPRs.
template <int KIND> struct Acc { typedef v16i T; };
template <> struct Acc<1> { typedef v16f T; };

template <int KIND, typename T>
__device__ __forceinline__ void mfma(T& c, const v4i& a, const v4i& b) {
    if constexpr (KIND == 0) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// (a) one wave per SIMD: each MFMA followed by NV independent VALU instructions (VK 0: fma, 1: exp)
template <int KIND, int NV, int VK>
__global__ __launch_bounds__(256) void one_wave(int iters, float* out, unsigned long long* clk) {
    v4i a = {(int)threadIdx.x, 2, 3, 4}, b = {5, 6, 7, (int)threadIdx.x};
    typename Acc<KIND>::T c0 = {}, c1 = {}, c2 = {}, c3 = {};
    float x[8];
    for (int j = 0; j < 8; j++) x[j] = 0.001f * threadIdx.x + j;
    auto valu = [&]() {
#pragma unroll
        for (int j = 0; j < NV; j++) {
            x[j & 7] = VK == 0 ? fmaf(x[j & 7], 0.999f, 0.5f) : __builtin_amdgcn_exp2f(x[j & 7]);
            asm volatile("" : "+v"(x[j & 7]));
        }
    };
    unsigned long long t0 = __builtin_readcyclecounter();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            mfma<KIND>(c0, a, b); valu();
            mfma<KIND>(c1, a, b); valu();
            mfma<KIND>(c2, a, b); valu();
            mfma<KIND>(c3, a, b); valu();
        }
    }
    unsigned long long t1 = __builtin_readcyclecounter();
    float s = 0;
    for (int j = 0; j < 8; j++) s += x[j];
    if ((float)c0[0] + (float)c1[0] + (float)c2[0] + (float)c3[0] + s == 1.2345f) out[threadIdx.x] = 1.0f;
    if ((threadIdx.x & 63) == 0) clk[threadIdx.x >> 6] = t1 - t0;
}

// (b) two waves per SIMD: waves 0-3 issue MFMAs only, waves 4-7 VALU only (VK 0: fma, 1: exp).
// mode bit 0 enables the MFMA waves, bit 1 the VALU waves.
template <int KIND, int VK>
__global__ __launch_bounds__(512) void two_wave(int mode, int iters, float* out, unsigned long long* clk) {
    const int wave = threadIdx.x >> 6;
    unsigned long long t0 = 0, t1 = 0;
    if (wave < 4) {
        if (!(mode & 1)) return;
        v4i a = {(int)threadIdx.x, 2, 3, 4}, b = {5, 6, 7, (int)threadIdx.x};
        typename Acc<KIND>::T c0 = {}, c1 = {}, c2 = {}, c3 = {};
        t0 = __builtin_readcyclecounter();
        for (int i = 0; i < iters; i++) {
#pragma unroll
            for (int r = 0; r < 4; r++) { mfma<KIND>(c0, a, b); mfma<KIND>(c1, a, b); mfma<KIND>(c2, a, b); mfma<KIND>(c3, a, b); }
        }
        t1 = __builtin_readcyclecounter();
        if ((float)c0[0] + (float)c1[0] + (float)c2[0] + (float)c3[0] == 1.2345f) out[threadIdx.x] = 1.0f;
    } else {
        if (!(mode & 2)) return;
        float x[8];
        for (int j = 0; j < 8; j++) x[j] = 0.001f * threadIdx.x + j;
        t0 = __builtin_readcyclecounter();
        for (int i = 0; i < iters; i++) {
#pragma unroll
            for (int r = 0; r < 2; r++) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    x[j] = VK == 0 ? fmaf(x[j], 0.999f, 0.5f) : __builtin_amdgcn_exp2f(x[j]);
                    asm volatile("" : "+v"(x[j]));
                }
            }
        }
        t1 = __builtin_readcyclecounter();
        float s = 0;
        for (int j = 0; j < 8; j++) s += x[j];
        if (s == 1.2345f) out[threadIdx.x] = s;
    }
    if ((threadIdx.x & 63) == 0) clk[wave] = t1 - t0;
}

// The attention loop's instruction mix without memory traffic: per wave and "tile" 8 INT8 and
// 16 FP16 matrix instructions, 32 fma + 32 exp + 16 cvt_pk + 16 dot2 on the vector ALU.
template <bool RANDOM>
__global__ __launch_bounds__(512, 2) void mix_kernel(int tiles, float* out, unsigned long long* stamps) {
    // eight operand pairs; RANDOM: pseudo-random bytes (INT8 operands with |x| < 128, fp16
    // operands with finite exponents), rotated so that consecutive instructions differ
    v4i av[8], bv[8];
    unsigned seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int r = 0; r < 8; r++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            seed = seed * 1664525u + 1013904223u;
            av[r][e] = RANDOM ? (int)((seed >> 3) & 0x3BFF3BFFu) : (e == 0 ? (int)threadIdx.x : e + 1);
            seed = seed * 1664525u + 1013904223u;
            bv[r][e] = RANDOM ? (int)((seed >> 3) & 0x3BFF3BFFu) : (e == 3 ? (int)threadIdx.x : e + 5);
        }
    v16i s0 = {}, s1 = {};
    v16f o0 = {}, o1 = {}, o2 = {}, o3 = {};
    float l = 0.0f, f = 1e-7f, c = -0.25f;
    const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int t = 0; t < tiles; t++) {
#pragma unroll
        for (int st = 0; st < 4; st++) {
            s0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[st], bv[st], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[st + 4], bv[st + 4], s1, 0, 0, 0);
        }
        // keep the integer accumulators small (they feed exp below)
        if ((t & 7) == 7) { s0 = v16i{}; s1 = v16i{}; }
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        unsigned p[16];
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const v16i& s = u < 8 ? s0 : s1;
            const int i = (u & 7) * 2;
            const float p0 = __builtin_amdgcn_exp2f(fmaf((float)s[i], f, c));
            const float p1 = __builtin_amdgcn_exp2f(fmaf((float)s[i + 1], f, c));
            const v2h pr = {(_Float16)p0, (_Float16)p1};
            const v2h ones = {(_Float16)1.0f, (_Float16)1.0f};
            l = __builtin_amdgcn_fdot2(pr, ones, l, false);
            p[u] = __builtin_bit_cast(unsigned, pr);
            const v4i pw = {(int)p[u], (int)p[u] ^ bv[u & 7][1], (int)p[u], (int)p[u] ^ bv[u & 7][3]};
            v16f& o = (u & 3) == 0 ? o0 : (u & 3) == 1 ? o1 : (u & 3) == 2 ? o2 : o3;
            o = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, av[u & 7]), __builtin_bit_cast(v8h, pw), o, 0, 0, 0);
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
    if (o0[0] + o1[0] + o2[0] + o3[0] + l == 1.2345f) out[threadIdx.x] = l;
    if (threadIdx.x == 0) {
        stamps[blockIdx.x * 2] = t1 - t0;
        stamps[blockIdx.x * 2 + 1] = r1 - r0;
    }
}

static float* d_out;
static unsigned long long* d_clk;

template <int KIND, int NV, int VK> int run_one(const char* name) {
    unsigned long long h[8];
    const int iters = 4000;
    CHECK(hipMemset(d_clk, 0, 64));
    hipLaunchKernelGGL((one_wave<KIND, NV, VK>), dim3(1), dim3(256), 0, 0, iters, d_out, d_clk);
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(h, d_clk, 64, hipMemcpyDeviceToHost));
    std::printf("one wave   %-14s + %2d x %s : %5.1f clocks per MFMA\n", name, NV, VK ? "exp" : "fma", (double)h[0] / iters / 8);
    return 0;
}
template <int KIND> int run_one_all(const char* name) {
    return run_one<KIND, 0, 0>(name) || run_one<KIND, 2, 0>(name) || run_one<KIND, 4, 0>(name) || run_one<KIND, 6, 0>(name) ||
           run_one<KIND, 8, 0>(name) || run_one<KIND, 12, 0>(name) || run_one<KIND, 2, 1>(name) || run_one<KIND, 4, 1>(name);
}
template <int KIND, int VK> int run_two(const char* name) {
    unsigned long long h[8];
    const int iters = 4000;
    for (int mode = 1; mode <= 3; mode++) {
        CHECK(hipMemset(d_clk, 0, 64));
        hipLaunchKernelGGL((two_wave<KIND, VK>), dim3(1), dim3(512), 0, 0, mode, iters, d_out, d_clk);
        CHECK(hipDeviceSynchronize());
        CHECK(hipMemcpy(h, d_clk, 64, hipMemcpyDeviceToHost));
        std::printf("two waves  %-14s | %s : %s%s -> %5.1f clocks per MFMA, %5.2f clocks per VALU instruction\n", name,
                    VK ? "exp" : "fma", (mode & 1) ? "MFMA wave " : "", (mode & 2) ? "VALU wave" : "",
                    (double)h[0] / iters / 16, (double)h[4] / iters / 16);
    }
    return 0;
}

int main(int argc, char** argv) {
    if (argc != 2 || (std::strcmp(argv[1], "issue") && std::strcmp(argv[1], "clock"))) {
        std::fprintf(stderr, "usage: %s issue | clock\n", argv[0]);
        return 2;
    }
    CHECK(hipMalloc(&d_out, 4096));
    CHECK(hipMalloc(&d_clk, 4096 * 2 * sizeof(unsigned long long)));
    if (!std::strcmp(argv[1], "issue")) {
        if (run_one_all<0>("i8 32x32x32") || run_one_all<1>("f16 32x32x16")) return 1;
        if (run_two<0, 0>("i8 32x32x32") || run_two<0, 1>("i8 32x32x32") || run_two<1, 0>("f16 32x32x16") ||
            run_two<1, 1>("f16 32x32x16"))
            return 1;
        return 0;
    }
    const int tiles = 3000;
    std::vector<unsigned long long> h(4096 * 2);
    const int counts[] = {8, 32, 64, 128, 192, 256, 512};
    for (int random = 0; random < 2; random++)
    for (int w : counts) {
        double best_clk = 0, tile_clk = 0;
        for (int rep = 0; rep < 6; rep++) {                     // the last repetition runs on a warm chip
            if (random) hipLaunchKernelGGL(mix_kernel<true>, dim3(w), dim3(512), 0, 0, tiles, d_out, d_clk);
            else hipLaunchKernelGGL(mix_kernel<false>, dim3(w), dim3(512), 0, 0, tiles, d_out, d_clk);
            CHECK(hipDeviceSynchronize());
            CHECK(hipMemcpy(h.data(), d_clk, w * 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
            double cyc = 0, real = 0;
            for (int i = 0; i < w; i++) { cyc += (double)h[2 * i]; real += (double)h[2 * i + 1]; }
            best_clk = cyc / real * 100.0;                      // s_memrealtime counts at 100 MHz
            tile_clk = cyc / w / tiles;
        }
        std::printf("clock      %s operands, %3d workgroups x 512 threads: shader clock %6.0f MHz, %6.0f clocks per tile (2 waves per SIMD)\n",
                    random ? "varying " : "constant", w, best_clk, tile_clk);
    }
    return 0;
}
