// Pieces shared by the GEMM kernels: parameters, tile-id mapping, epilogue (dequantise + bias + GELU + store).
#pragma once
#include "q8_common.h"
#include "q8_host.h"

namespace q8 {

struct GemmParams {
    const uint8_t* A;
    const uint8_t* B;
    const float* bias;
    const float* sa;
    const float* sb;
    void* C;
    int batch_a, batch_b;
    int M, N, K;
    const void* residual = nullptr;  // bf16 [batch, M, N] added to the rounded bf16 result (persistent kernel only)
    const uint16_t* gate = nullptr;  // bf16 [ceil(M / rows_per_gate), N]: with it C = bf16(fma(bf16(result), gate, residual))
    int rows_per_gate = 0;           // a multiple of the tile height, so that a tile has one gate row
    // q8_gemm_qkv (persistent kernel only): columns n >= v_col0 (a multiple of 256, head dim 64) are not written to C but
    // cast to e4m3 (c10 cast of the bf16-rounded result) and written head-major to v_codes [rows / v_tokens, v_heads, v_tokens, 64];
    // C then has ldc = v_col0 columns per row
    uint8_t* v_codes = nullptr;
    int v_col0 = 0, v_tokens = 0, v_heads = 0;
    // != 0: the 64 columns of every head go through the 64-point Hadamard transform times this factor before the cast (the
    // queries or keys of an attention with apply_qk_hadamard, q8_kernels/functional/flash_attention.py:47-51)
    float v_fht_scale = 0.f;
};

__device__ __attribute__((aligned(16))) const uint32_t g_zero16[4] = {0, 0, 0, 0};

constexpr int Q8_OUT_I32 = 100;  // raw accumulators (int8 only)
constexpr int kGroupM = 4;

template <int IN_, int WAVES_M_, int WAVES_N_, int TM_, int TN_, int STAGES_ = 4>
struct GemmCfg {
    static constexpr int IN = IN_;
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, TM = TM_, TN = TN_;
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = NW * 64;
    static constexpr int BM = WAVES_M * TM * 16;
    static constexpr int BN = WAVES_N * TN * 16;
    static constexpr int BK = 128;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int STAGES = STAGES_;  // LDS ring of the HBM -> LDS copies
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int RG_A = BM / 8, RG_B = BN / 8;  // 1 KiB row groups per stage
    static constexpr int PER_A = RG_A / NW, PER_B = RG_B / NW;
    static_assert(RG_A % NW == 0 && RG_B % NW == 0, "row groups must divide over the waves");
    static_assert(TN % 2 == 0, "TN must be even (pairs of n tiles form one 16-byte store)");
};

// chunk swizzle of a 128-byte LDS row: (row >> 1) & 7, with bit 1 flipped for rows 4..11 of each 16
__device__ __forceinline__ int lds_swizzle(int row) { return ((row >> 1) & 7) ^ ((((row >> 2) ^ (row >> 3)) & 1) << 1); }

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
__device__ __forceinline__ void wait_vmcnt0() { __builtin_amdgcn_s_waitcnt(0x0F70 | 0); }

// column permutation inside a wave's TN*16 columns: LDS row (16 j + s) of the wave's B slab holds
// local column 32 (j/2) + 8 (s/4) + 4 (j%2) + (s%4).
__device__ __forceinline__ int bcol_of_slot(int rho) {
    const int j = rho >> 4, s = rho & 15;
    return 32 * (j >> 1) + 8 * (s >> 2) + 4 * (j & 1) + (s & 3);
}

__device__ __forceinline__ float gelu_tanh_fast(float v) {
    // 0.5 v (1 + tanh(u)) = v / (1 + exp(-2u)),  u = 0.7978845608 (v + 0.044715 v^3)
    // (csrc/gemm/fp8_matmul_bias.cu:31-35); exp2 and reciprocal on the transcendental unit.
    const float k1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
    const float k3 = k1 * 0.044715f;
    const float v2 = v * v;
    const float arg = v * fmaf(v2, k3, k1);
    const float e = __builtin_amdgcn_exp2f(arg);
    return v * __builtin_amdgcn_rcpf(1.0f + e);
}


// XCD-contiguous, grouped tile walk: workgroup ids congruent mod 8 share an XCD (and its L2); each XCD gets a
// contiguous range of tile ids, and ids walk kGroupM tile rows at a time so that concurrently resident
// workgroups reuse the same A and B panels.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    const int nb = gridDim.x, bid = blockIdx.x;
    const int xcd = bid & 7, loc = bid >> 3, per = nb >> 3, rem = nb & 7;
    const int pid = xcd * per + (xcd < rem ? xcd : rem) + loc;
    const int group_size = kGroupM * tiles_n;
    const int gid = pid / group_size, first_m = gid * kGroupM;
    const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    tile_m = first_m + (pid % group_size) % gsz;
    tile_n = (pid % group_size) / gsz;
}

// v[e] = acc[e] * (sa * sb[e]) + bias[e], optional tanh-GELU (the order of csrc/gemm/fp8_matmul_bias.cu:356-365)
template <bool GELU, typename ACC>
__device__ __forceinline__ void dequant8(const ACC (&a)[8], float sam, const float (&sbv)[8], const float (&bv)[8], float (&v)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float t = fmaf((float)a[e], sam * sbv[e], bv[e]);
        if constexpr (GELU) t = gelu_tanh_fast(t);
        v[e] = t;
    }
}

// Finish 8 consecutive columns n .. n+7 of row m: v = acc * (sa[m] * sb[n]) + bias[n] (the order of
// csrc/gemm/fp8_matmul_bias.cu:356-365), optional tanh-GELU, then one 16-byte bf16 / 8-byte e4m3 store
// (element-wise stores on the ragged right edge or when rows are not 8-aligned).
template <int OUT, bool GELU, typename ACC>
__device__ __forceinline__ void finish8(const GemmParams& p, size_t zc, float sam, int m, int n, const ACC (&a)[8],
                                        const float (&sbv)[8], const float (&bv)[8]) {
    const int N = p.N;
    const bool vec = (n + 8 <= N) && ((N & 7) == 0);
    if constexpr (OUT == Q8_OUT_I32) {
        int32_t* crow = reinterpret_cast<int32_t*>(p.C) + zc + (size_t)m * N + n;
        if (vec) {
            *reinterpret_cast<v4i*>(crow) = v4i{(int)a[0], (int)a[1], (int)a[2], (int)a[3]};
            *reinterpret_cast<v4i*>(crow + 4) = v4i{(int)a[4], (int)a[5], (int)a[6], (int)a[7]};
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (n + e < N) crow[e] = (int)a[e];
        }
    } else {
        float v[8];
        dequant8<GELU>(a, sam, sbv, bv, v);
        if constexpr (OUT == Q8_BF16) {
            uint16_t* crow = reinterpret_cast<uint16_t*>(p.C) + zc + (size_t)m * N + n;
            if (vec) {
                v4u w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = pack2_bf16(v[2 * e], v[2 * e + 1]);
                *reinterpret_cast<v4u*>(crow) = w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < N) crow[e] = (uint16_t)f32_to_bf16_bits(v[e]);
            }
        } else {
            uint8_t* crow = reinterpret_cast<uint8_t*>(p.C) + zc + (size_t)m * N + n;
            const uint32_t w0 = pack4_e4m3_sat(v[0], v[1], v[2], v[3]);
            const uint32_t w1 = pack4_e4m3_sat(v[4], v[5], v[6], v[7]);
            if (vec) {
                *reinterpret_cast<v2i*>(crow) = v2i{(int)w0, (int)w1};
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < N) crow[e] = (uint8_t)(((e < 4) ? w0 : w1) >> (8 * (e & 3)));
            }
        }
    }
}

// sb[n .. n+7] and bias[n .. n+7] (clamped at the right edge; bias may be absent)
template <int OUT>
__device__ __forceinline__ void load_col_params(const GemmParams& p, int zb, int n, float (&sbv)[8], float (&bv)[8]) {
    if constexpr (OUT != Q8_OUT_I32) {
        const float* sbp = p.sb + (size_t)zb * p.N;
        if (n + 8 <= p.N && ((p.N & 3) == 0)) {  // n is a multiple of 8: 16-byte aligned whenever N % 4 == 0
            const v4f s0 = *reinterpret_cast<const v4f*>(sbp + n), s1 = *reinterpret_cast<const v4f*>(sbp + n + 4);
            v4f b0 = {0.f, 0.f, 0.f, 0.f}, b1 = b0;
            if (p.bias) {
                b0 = *reinterpret_cast<const v4f*>(p.bias + n);
                b1 = *reinterpret_cast<const v4f*>(p.bias + n + 4);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) { sbv[e] = s0[e]; sbv[4 + e] = s1[e]; bv[e] = b0[e]; bv[4 + e] = b1[e]; }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int nn = (n + e < p.N) ? n + e : p.N - 1;
                sbv[e] = sbp[nn];
                bv[e] = p.bias ? p.bias[nn] : 0.f;
            }
        }
    }
}

}  // namespace q8
