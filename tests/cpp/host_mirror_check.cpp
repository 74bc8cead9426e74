// host_mirror_check.cpp — drives include/mi355_sage_host.hpp (the C++ statement of the serenitymojo
// attention call surface) on a GPU: inputs from the reference gate's 64-bit LCG
// (serenitymojo/ops/tests/sdpa_flash_parity.mojo:46-53, seeds 11/22/33 of :125-127), every entry
// point once, results written to a file the GPU test compares bit for bit with the Python mirror's;
// argument errors are checked here against the reference's texts.
//
// usage: host_mirror_check <output file>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <functional>

#include "mi355_sage_host.hpp"

using namespace mi355_sage_host;

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// x = (2u - 1) * amp with u = (state >> 40) / 2^24, state <- state * 6364136223846793005 + 1442695040888963407
static std::vector<uint16_t> lcg_bf16(size_t n, uint64_t seed, float amp) {
    std::vector<uint16_t> out(n);
    uint64_t state = seed;
    for (size_t i = 0; i < n; i++) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        const float u = (float)(state >> 40) / 16777216.0f;
        out[i] = f32_to_bf16((2.0f * u - 1.0f) * amp);
    }
    return out;
}

static Tensor upload(const std::vector<uint16_t>& h, std::vector<int64_t> shape) {
    Tensor t(std::move(shape), STDtype::BF16);
    if (hipMemcpy(t.unsafe_ptr(), h.data(), h.size() * 2, hipMemcpyHostToDevice) != hipSuccess) throw Error("upload failed");
    return t;
}

static FILE* g_out;
static void dump(const char* tag, const Tensor& t, const DeviceContext& ctx) {
    ctx.synchronize();
    std::vector<uint8_t> h(t.nbytes());
    if (hipMemcpy(h.data(), t.unsafe_ptr(), h.size(), hipMemcpyDeviceToHost) != hipSuccess) throw Error("download failed");
    const uint64_t n = h.size();
    char name[32] = {};
    std::strncpy(name, tag, sizeof(name) - 1);
    std::fwrite(name, 1, sizeof(name), g_out);
    std::fwrite(&n, 8, 1, g_out);
    std::fwrite(h.data(), 1, h.size(), g_out);
    std::printf("wrote %-24s %llu bytes\n", tag, (unsigned long long)n);
    std::fflush(stdout);
}

static int g_failed = 0;
static void expect_error(const char* what, const char* text, const std::function<void()>& f) {
    try {
        f();
    } catch (const Error& e) {
        if (std::strstr(e.what(), text) != nullptr) return;
        std::printf("FAIL %s: message \"%s\" does not contain \"%s\"\n", what, e.what(), text);
        g_failed++;
        return;
    }
    std::printf("FAIL %s: no error raised\n", what);
    g_failed++;
}

int main(int argc, char** argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: %s <output file>\n", argv[0]);
        return 2;
    }
    g_out = std::fopen(argv[1], "wb");
    if (!g_out) return 2;
    try {
        DeviceContext ctx;
        if (hipStreamCreate(&ctx.stream) != hipSuccess) throw Error("stream creation failed");
        const int B = 1, S = 384, Skv = 520, H = 6, Dh = 128, N_TXT = 96, REAL_TXT = 61, REAL_LEN = 300;
        const float scale = 0.08838834764831845f;       // 1/sqrt(128)
        const size_t nq = (size_t)B * S * H * Dh, nk = (size_t)B * Skv * H * Dh;
        const Tensor q = upload(lcg_bf16(nq, 11, 1.0f), {B, S, H, Dh});
        const Tensor k = upload(lcg_bf16(nq, 22, 1.0f), {B, S, H, Dh});
        const Tensor v = upload(lcg_bf16(nq, 33, 1.0f), {B, S, H, Dh});
        const Tensor g = upload(lcg_bf16(nq, 44, 1.0f), {B, S, H, Dh});
        const Tensor k2 = upload(lcg_bf16(nk, 55, 1.0f), {B, Skv, H, Dh});
        const Tensor v2 = upload(lcg_bf16(nk, 66, 1.0f), {B, Skv, H, Dh});
        const Tensor mask = upload(lcg_bf16((size_t)B * H * S * Skv, 77, 3.0f), {B, H, S, Skv});

        const SdpaFlashFwd fwd = sdpa_flash_train_fwd(q, k, v, scale, ctx);
        dump("train_fwd.o", fwd.o, ctx);
        dump("train_fwd.stats", fwd.stats, ctx);
        const SdpaFlashGrads gr = sdpa_flash_backward(fwd, g, scale, ctx);
        dump("bwd.d_q", gr.d_q, ctx);
        dump("bwd.d_k", gr.d_k, ctx);
        dump("bwd.d_v", gr.d_v, ctx);
        const SdpaFlashGrads gr2 = sdpa_flash_backward_dispatch(fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, fwd.stats, g, scale, B, S, H, Dh, ctx);
        dump("bwd_dispatch.d_k", gr2.d_k, ctx);
        const SdpaFlashFwd rect = sdpa_flash_train_fwd_rect(q, k2, v2, scale, ctx);
        dump("rect.o", rect.o, ctx);
        dump("rect.stats", rect.stats, ctx);
        const SdpaFlashFwd pad = sdpa_flash_fwd_padmask(q, k, v, REAL_LEN, scale, ctx);
        dump("padmask.o", pad.o, ctx);
        const SdpaFlashGrads gp = sdpa_flash_backward(pad, g, scale, ctx, REAL_LEN);
        dump("padmask.d_v", gp.d_v, ctx);
        dump("nomask.o", sdpa_nomask(q, k, v, scale, ctx), ctx);
        dump("nomask_fp8.o", sdpa_nomask(q, k, v, scale, ctx, PV_FP8), ctx);
        dump("tiled.o", sdpa_nomask_tiled(q, k, v, scale, ctx), ctx);
        dump("cross.o", sdpa_cross_nomask(q, k2, v2, scale, ctx), ctx);
        dump("keymask.o", sdpa_qwen_keymask(q, k, v, N_TXT, REAL_TXT, scale, ctx), ctx);
        dump("cross_masked.o", sdpa_cross_masked(q, k2, v2, mask, scale, ctx), ctx);

        // error behaviour (texts of serenitymojo/ops/attention_flash.mojo:159, ops/attention.mojo:1700-1712)
        const Tensor f32t({B, S, H, Dh}, STDtype::F32);
        expect_error("train_fwd dtype", "sdpa_flash_train_fwd: q/k/v must be BF16", [&] { sdpa_flash_train_fwd(f32t, k, v, scale, ctx); });
        expect_error("nomask dtype", "sdpa_nomask: q/k/v dtype mismatch", [&] { sdpa_nomask(q, f32t, v, scale, ctx); });
        expect_error("nomask shape", "sdpa_nomask: k/v shape does not match q [B,S,H,Dh]", [&] { sdpa_nomask(q, k2, v2, scale, ctx); });
        expect_error("padmask align", "sdpa_flash_fwd_padmask: S_BUF must be 128-aligned", [&] { sdpa_flash_fwd_padmask(k2, k2, v2, 10, scale, ctx); });
        expect_error("keymask range", "sdpa_qwen_keymask: real_txt_len out of range", [&] { sdpa_qwen_keymask(q, k, v, 10, 11, scale, ctx); });
        expect_error("keymask n_txt", "sdpa_qwen_keymask: N_TXT must be <= S", [&] { sdpa_qwen_keymask(q, k, v, S + 1, 1, scale, ctx); });
        expect_error("mask shape", "sdpa: mask must be [B,H,S,S]", [&] { sdpa(q, k, v, mask, scale, ctx); });
        expect_error("bwd shape", "sdpa_flash_backward: d_out shape does not match the forward output", [&] { sdpa_flash_backward(rect, k2, scale, ctx); });
        expect_error("dispatch bucket", "sdpa_flash_backward_dispatch: no bucket (B,S,H,Dh)=(1,385,6,128)",
                     [&] { sdpa_flash_backward_dispatch(fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, fwd.stats, g, scale, B, S + 1, H, Dh, ctx); });
        const Tensor q96 = upload(lcg_bf16((size_t)S * H * 96, 88, 1.0f), {B, S, H, 96});
        expect_error("head dim", "sdpa_nomask: shim rc=-2", [&] { sdpa_nomask(q96, q96, q96, scale, ctx); });
        ctx.synchronize();
    } catch (const std::exception& e) {
        std::printf("FAIL: %s\n", e.what());
        g_failed++;
    }
    std::fclose(g_out);
    std::printf(g_failed ? "host_mirror_check: %d failure(s)\n" : "host_mirror_check: ok\n", g_failed);
    return g_failed ? 1 : 0;
}
