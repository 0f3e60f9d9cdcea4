// Host-side sanitizer driver for the C ABI of libq8_hip: calls every entry point with null pointers, with fake (never
// dereferenced on the host) device pointers and with sizes from a grid that includes negative values, zero and INT_MAX /
// INT64_MAX-like extremes, so that AddressSanitizer and UndefinedBehaviorSanitizer see the argument validation and the
// launch-geometry arithmetic of every entry point. No GPU is needed or used: a call that passes validation fails at the
// launch with Q8_ERR_LAUNCH on a machine without a device. Built and run by tests/sanitize/run.sh.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include "../../include/q8_hip.h"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd() {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return rng_state;
}
static const int kInts[] = {-1, 0, 1, 8, 12, 16, 64, 128, 256, 384, 2048, 4096, 6144, 8192, 12288, 32768, 65535, 65536, 1 << 20, 0x7fffffff};
static const int64_t kLongs[] = {-1, 0, 1, 4, 64, 768, 6144, 12288, 1100000, (int64_t)1 << 31, (int64_t)1 << 40, INT64_MAX};
static int pick_int() { return kInts[rnd() % (sizeof(kInts) / sizeof(kInts[0]))]; }
static int64_t pick_long() { return kLongs[rnd() % (sizeof(kLongs) / sizeof(kLongs[0]))]; }
static int pick_dtype() { return (int)(rnd() % 7) - 1; }  // -1 .. 5: the valid 0 .. 4 and two invalid ones
static void* pick_ptr() {
    switch (rnd() % 4) {
        case 0: return nullptr;
        case 1: return reinterpret_cast<void*>(0x1008);  // misaligned for 16 bytes
        default: return reinterpret_cast<void*>(0x7f0000001000ull);
    }
}
static float pick_float() {
    static const float v[] = {0.f, -1.f, 1.f, 0.125f, 1e30f, 1e-30f};
    return v[rnd() % 6];
}
static long g_calls = 0, g_ok = 0;
static void note(int status) {
    ++g_calls;
    if (status == Q8_OK) ++g_ok;
    if (status > 0 || status < Q8_ERR_FLAGS) {
        std::fprintf(stderr, "status %d outside the documented range\n", status);
        std::exit(2);
    }
    const char* e = q8_last_error();
    if (e == nullptr || std::strlen(e) > 255) {
        std::fprintf(stderr, "q8_last_error text broken\n");
        std::exit(2);
    }
}
#define P pick_ptr()
#define PF static_cast<float*>(pick_ptr())
#define I pick_int()
#define L pick_long()
#define D pick_dtype()
#define F pick_float()

int main(int argc, char** argv) {
    const int rounds = argc > 1 ? std::atoi(argv[1]) : 3000;
    for (int s = -8; s <= 1; ++s) {
        if (q8_strerror(s) == nullptr) return 2;
    }
    int cu = 0, mhz = 0;
    int64_t mem = 0;
    char name[64];
    note(q8_device_info(&cu, &mhz, &mem, name));
    note(q8_device_info(nullptr, nullptr, nullptr, nullptr));
    for (int c = -2; c <= 50; ++c) {
        (void)q8_gemm_set_config(c);
        (void)q8_attn_set_config(c);
    }
    (void)q8_gemm_set_config(0);
    (void)q8_attn_set_config(0);
    for (int r = 0; r < rounds; ++r) {
        note(q8_quant_rows(P, D, P, D, PF, L, I, L, I % 8, nullptr));
        note(q8_fht(P, D, P, D, L, I, F, nullptr));
        note(q8_rmsnorm(P, D, PF, P, D, PF, L, I, F, nullptr));
        note(q8_rope(P, D, PF, PF, P, D, L, I, nullptr));
        note(q8_fma(P, D, P, D, P, D, P, D, L, I, L, L, F, nullptr));
        note(q8_adaln_rows(PF, PF, P, I, L, I, nullptr));
        note(q8_gelu(P, D, P, D, L, nullptr));
        note(q8_gelu_backward(P, D, P, D, P, D, L, nullptr));
        note(q8_rope_backward(P, D, PF, PF, P, D, L, I, nullptr));
        note(q8_rmsnorm_backward(P, D, PF, P, D, PF, P, D, L, I, nullptr));
        note(q8_fht_quant_rows(P, D, P, D, PF, L, I, F, D, I % 8, nullptr));
        note(q8_rmsnorm_quant_rows(P, D, PF, P, D, PF, PF, L, I, F, D, I % 8, nullptr));
        note(q8_norm_mod_fht_quant_rows(P, PF, I % 2, P, P, D, L, F, I % 2, F, P, D, PF, L, I, I % 8, nullptr));
        note(q8_attn_prep_qk(P, L, PF, PF, PF, P, PF, I, I, I, I, I % 9, F, D, nullptr));
        note(q8_attn_prep_qk_pair(P, L, P, L, PF, PF, PF, PF, P, PF, P, PF, I, I, I, I, I % 9, F, D, nullptr));
        note(q8_attn_prep_qkv(P, L, P, L, P, L, PF, PF, PF, PF, P, PF, P, PF, P, PF, I, I, I, I, I % 9, F, D, nullptr));
        note(q8_attn_prep_kv(P, L, P, L, PF, PF, PF, P, PF, P, PF, I, I, I, I, I % 9, F, D, nullptr));
        note(q8_attn_prep_v(P, L, P, PF, I, I, I, I, I, nullptr));
        note(q8_gemm(P, P, PF, PF, PF, P, I, I, I, I, I, D, D, I % 2, nullptr));
        note(q8_gemm_residual(P, P, PF, PF, PF, P, P, I, I, I, I, I, D, I % 2, nullptr));
        note(q8_gemm_gated_residual(P, P, PF, PF, PF, P, P, L, P, I, I, I, D, I % 2, nullptr));
        note(q8_gemm_qkv(P, P, PF, PF, PF, P, P, I, I, I, I, I, F, D, nullptr));
        note(q8_gemm_i32(static_cast<const int8_t*>(P), static_cast<const int8_t*>(P), static_cast<int32_t*>(P), I, I, I, nullptr));
        note(q8_attn_fwd(P, P, P, P, static_cast<const int32_t*>(P), PF, PF, PF, I, I, I, I, (rnd() % 4) ? 64 : I, I % 3, L, F, D, I % 32,
                         nullptr));
        (void)q8_gemm_last_kernel();
    }
    // plausible, fully valid argument sets: they pass validation and must come back with a launch error (no device) or Q8_OK
    void* const p = reinterpret_cast<void*>(0x7f0000001000ull);
    float* const pf = static_cast<float*>(p);
    note(q8_quant_rows(p, Q8_BF16, p, Q8_E4M3, pf, 12288, 2048, 2048, 0, nullptr));
    note(q8_fht(p, Q8_BF16, p, Q8_BF16, 12288, 2048, 0.02f, nullptr));
    note(q8_gemm(p, p, pf, pf, pf, p, 1, 1, 6144, 8192, 2048, Q8_E4M3, Q8_BF16, 1, nullptr));
    note(q8_gemm(p, p, pf, pf, pf, p, 1, 1, 300, 200, 144, Q8_I8, Q8_E4M3, 0, nullptr));
    note(q8_gemm_residual(p, p, pf, pf, pf, p, p, 2, 1, 6144, 2048, 2048, Q8_E4M3, 0, nullptr));
    note(q8_gemm_gated_residual(p, p, pf, pf, pf, p, p, 6144, p, 12288, 2048, 2048, Q8_I8, 0, nullptr));
    note(q8_gemm_qkv(p, p, pf, pf, pf, p, p, 12288, 6144, 2048, 4096, 6144, 0.f, Q8_E4M3, nullptr));
    note(q8_gemm_qkv(p, p, pf, pf, pf, nullptr, p, 12288, 2048, 2048, 0, 6144, 0.0442f, Q8_E4M3, nullptr));
    note(q8_attn_prep_qk_pair(p, 6144, p, 6144, nullptr, nullptr, pf, pf, p, nullptr, p, nullptr, 2, 6144, 32, 64,
                              Q8_PREP_FHT | Q8_PREP_PAIR_TABLES | Q8_PREP_SHARED_TABLES, 0.0442f, Q8_BF16, nullptr));
    note(q8_attn_fwd(p, p, p, p, nullptr, nullptr, nullptr, nullptr, 2, 32, 6144, 6144, 64, Q8_V_DS, 6144, 0.125f, Q8_BF16, 0, nullptr));
    note(q8_attn_fwd(p, p, p, p, static_cast<const int32_t*>(p), pf, pf, pf, 2, 32, 6144, 128, 64, Q8_V_SD, 64, 0.125f, Q8_E4M3, 0, nullptr));
    std::printf("abi_driver: %ld calls, %ld returned Q8_OK, no sanitizer report\n", g_calls, g_ok);
    return 0;
}
