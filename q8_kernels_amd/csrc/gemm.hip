// int8 / fp8-e4m3 GEMM for gfx950 with a fused dequantise + bias + tanh-GELU epilogue.
//
//   C[z,m,n] = epi( sum_k A[z,m,k] * B[z,n,k] ),  A and B both K-major (one byte per element).
//
// Structure of one workgroup (WAVES_M x WAVES_N waves, one BM x BN tile of C):
//   * K is walked in steps of 128 bytes. A step's A rows (BM x 128 B) and B rows (BN x 128 B) are
//     copied HBM -> LDS by `global_load_lds_dwordx4` (no VGPR staging), two LDS stages.
//   * LDS holds plain 128-byte rows whose 16-byte chunks are XOR-swizzled by ((row >> 1) & 7): the
//     16 lanes that fetch the same chunk index of 16 consecutive rows hit 16 different bank groups.
//   * A wave owns TM x TN MFMA tiles of 16x16. fp8 uses v_mfma_f32_16x16x128_f8f6f4 (one per step),
//     int8 uses two v_mfma_i32_16x16x64_i8. The B rows feed the MFMA "A" operand and the A rows the
//     "B" operand, so an accumulator lane holds four consecutive n of one m.
//   * LDS row rho of the B tile does not hold column n0 + rho but a permuted column, chosen so that
//     the two accumulators (tn = 2jj, 2jj+1) of a lane are 8 consecutive n: the epilogue then
//     writes one 16-byte bf16 store per lane and four lanes fill a 64-byte line, with no LDS staging.
//   * Rows beyond M / N are clamped on load and dropped on store; K only needs K % 16 == 0, chunks past
//     K are sourced from a 16-byte block of zeros.
//   * Workgroup ids are re-mapped so that each XCD (ids congruent mod 8 share an L2) owns a
//     contiguous range of tiles, walked in groups of GROUP_M tile rows for L2 reuse of A and B.
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
};

__device__ __attribute__((aligned(16))) const uint32_t g_zero16[4] = {0, 0, 0, 0};

constexpr int Q8_OUT_I32 = 100;  // raw accumulators (int8 only)
constexpr int kGroupM = 4;

template <int IN_, int WAVES_M_, int WAVES_N_, int TM_, int TN_>
struct GemmCfg {
    static constexpr int IN = IN_;
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, TM = TM_, TN = TN_;
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = NW * 64;
    static constexpr int BM = WAVES_M * TM * 16;
    static constexpr int BN = WAVES_N * TN * 16;
    static constexpr int BK = 128;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int RG_A = BM / 8, RG_B = BN / 8;  // 1 KiB row groups per stage
    static constexpr int PER_A = RG_A / NW, PER_B = RG_B / NW;
    static_assert(RG_A % NW == 0 && RG_B % NW == 0, "row groups must divide over the waves");
    static_assert(TN % 2 == 0, "TN must be even (pairs of n tiles form one 16-byte store)");
};

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

template <class C, int OUT, bool GELU>
__global__ __launch_bounds__(C::NT) void gemm_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    constexpr int BM = C::BM, BN = C::BN, TM = C::TM, TN = C::TN, NW = C::NW;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wave_m = wave / C::WAVES_N, wave_n = wave % C::WAVES_N;
    const int M = p.M, N = p.N, K = p.K;

    // ---- tile of this workgroup (XCD-contiguous, grouped walk)
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int pid;
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int xcd = bid & 7, loc = bid >> 3, per = nb >> 3, rem = nb & 7;
        pid = xcd * per + (xcd < rem ? xcd : rem) + loc;
    }
    const int group_size = kGroupM * tiles_n;
    const int gid = pid / group_size, first_m = gid * kGroupM;
    const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    const int tile_m = first_m + (pid % group_size) % gsz;
    const int tile_n = (pid % group_size) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int z = blockIdx.y;
    const int za = (p.batch_a == 1) ? 0 : z, zb = (p.batch_b == 1) ? 0 : z;
    const uint8_t* Ag = p.A + (size_t)za * M * K;
    const uint8_t* Bg = p.B + (size_t)zb * N * K;

    // ---- HBM -> LDS copy plan: lane (lane/8, lane%8) of row group q fills LDS row 8q + lane/8,
    //      physical chunk lane%8, from logical chunk (lane%8) ^ ((row >> 1) & 7)
    const uint8_t* src[C::PER_A + C::PER_B];
    int kchunk[C::PER_A + C::PER_B];
#pragma unroll
    for (int i = 0; i < C::PER_A + C::PER_B; ++i) {
        const bool isA = i < C::PER_A;
        const int q = isA ? (wave + i * NW) : (wave + (i - C::PER_A) * NW);
        const int rho = 8 * q + (lane >> 3);
        const int c = (lane & 7) ^ ((rho >> 1) & 7);
        kchunk[i] = c * 16;
        if (isA) {
            int m = m0 + rho;
            m = m < M ? m : M - 1;
            src[i] = Ag + (size_t)m * K + c * 16;
        } else {
            const int slab = rho / (TN * 16), within = rho % (TN * 16);
            int n = n0 + slab * (TN * 16) + bcol_of_slot(within);
            n = n < N ? n : N - 1;
            src[i] = Bg + (size_t)n * K + c * 16;
        }
    }
    auto issue_loads = [&](int stage, int k0) {
        uint8_t* base = lds + stage * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::PER_A + C::PER_B; ++i) {
            const bool isA = i < C::PER_A;
            const int q = isA ? (wave + i * NW) : (C::RG_A + wave + (i - C::PER_A) * NW);
            const uint8_t* g = (k0 + kchunk[i] < K) ? (src[i] + k0) : reinterpret_cast<const uint8_t*>(g_zero16);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                             (__attribute__((address_space(3))) void*)(base + q * 1024), 16, 0, 0);
        }
    };

    // ---- operand fetch addresses: lane (s = lane%16, gk = lane/16) reads chunks 2gk, 2gk+1 of row s
    const int s16 = lane & 15, gk = lane >> 4;
    const int pc0 = ((2 * gk) ^ ((s16 >> 1) & 7)) * 16, pc1 = pc0 ^ 16;
    const int a_row0 = wave_m * TM * 16 + s16;
    const int b_row0 = BM + wave_n * TN * 16 + s16;

    using acc_t = typename std::conditional<C::IN == Q8_I8, v4i, v4f>::type;
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    const int KT = (K + 127) / 128;
    issue_loads(0, 0);
    for (int kt = 0; kt < KT; ++kt) {
        wait_vmcnt0();
        __syncthreads();
        const uint8_t* st = lds + (kt & 1) * C::STAGE_BYTES;
        v4i a_lo[TM], a_hi[TM], b_lo[TN], b_hi[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint8_t* r = st + (b_row0 + 16 * j) * 128;
            b_lo[j] = *reinterpret_cast<const v4i*>(r + pc0);
            b_hi[j] = *reinterpret_cast<const v4i*>(r + pc1);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint8_t* r = st + (a_row0 + 16 * i) * 128;
            a_lo[i] = *reinterpret_cast<const v4i*>(r + pc0);
            a_hi[i] = *reinterpret_cast<const v4i*>(r + pc1);
        }
        if (kt + 1 < KT) issue_loads((kt + 1) & 1, (kt + 1) * 128);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (C::IN == Q8_I8) {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b_lo[j], a_lo[i], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b_hi[j], a_hi[i], acc[i][j], 0, 0, 0);
                } else {
                    const v8i bf = {b_lo[j][0], b_lo[j][1], b_lo[j][2], b_lo[j][3], b_hi[j][0], b_hi[j][1], b_hi[j][2], b_hi[j][3]};
                    const v8i af = {a_lo[i][0], a_lo[i][1], a_lo[i][2], a_lo[i][3], a_hi[i][0], a_hi[i][1], a_hi[i][2], a_hi[i][3]};
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[i][j], 0, 0, 0, 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: lane (mcol = lane%16, g = lane/16) holds, for tile (i, 2jj..2jj+1), row
    //      m = 16 i + mcol and the 8 columns 32 jj + 8 g + 0..7 of the wave's slab.
    const int g = lane >> 4;
    const int nw0 = n0 + wave_n * TN * 16;
    const size_t zc = (size_t)z * M * N;
#pragma unroll
    for (int jj = 0; jj < TN / 2; ++jj) {
        const int n = nw0 + 32 * jj + 8 * g;
        if (n >= N) continue;
        float sbv[8], bv[8];
        if constexpr (OUT != Q8_OUT_I32) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int nn = (n + e < N) ? n + e : N - 1;
                sbv[e] = p.sb[(size_t)zb * N + nn];
                bv[e] = p.bias ? p.bias[nn] : 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = m0 + wave_m * TM * 16 + 16 * i + s16;
            if (m >= M) continue;
            if constexpr (OUT == Q8_OUT_I32) {
                int32_t* crow = reinterpret_cast<int32_t*>(p.C) + zc + (size_t)m * N + n;
                if (n + 8 <= N && ((N & 7) == 0)) {
                    *reinterpret_cast<v4i*>(crow) = acc[i][2 * jj];
                    *reinterpret_cast<v4i*>(crow + 4) = acc[i][2 * jj + 1];
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (n + e < N) crow[e] = (e < 4) ? acc[i][2 * jj][e] : acc[i][2 * jj + 1][e - 4];
                }
            } else {
                const float sam = p.sa[(size_t)za * M + m];
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float a = (float)((e < 4) ? acc[i][2 * jj][e] : acc[i][2 * jj + 1][e - 4]);
                    // dequantise as acc * (sa * sb) + bias (csrc/gemm/fp8_matmul_bias.cu:356-365)
                    float t = fmaf(a, sam * sbv[e], bv[e]);
                    if constexpr (GELU) t = gelu_tanh_fast(t);
                    v[e] = t;
                }
                if constexpr (OUT == Q8_BF16) {
                    uint16_t* crow = reinterpret_cast<uint16_t*>(p.C) + zc + (size_t)m * N + n;
                    if (n + 8 <= N && ((N & 7) == 0)) {
                        v4u w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = f32_to_bf16_bits(v[2 * e]) | (f32_to_bf16_bits(v[2 * e + 1]) << 16);
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
                    if (n + 8 <= N && ((N & 7) == 0)) {
                        *reinterpret_cast<v2i*>(crow) = v2i{(int)w0, (int)w1};
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (n + e < N) crow[e] = (uint8_t)(((e < 4) ? w0 : w1) >> (8 * (e & 3)));
                    }
                }
            }
        }
    }
}

template <class C, int OUT, bool GELU>
static int launch_gemm(const GemmParams& p, hipStream_t stream) {
    const int tiles_m = (p.M + C::BM - 1) / C::BM, tiles_n = (p.N + C::BN - 1) / C::BN;
    const int batch = p.batch_a > p.batch_b ? p.batch_a : p.batch_b;
    auto kern = gemm_kernel<C, OUT, GELU>;
    static thread_local bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                C::LDS_BYTES) != hipSuccess) {
            (void)hipGetLastError();
            return fail(Q8_ERR_LAUNCH, "q8_gemm: cannot reserve %d bytes of LDS", C::LDS_BYTES);
        }
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(C::NT), C::LDS_BYTES, stream, p);
    return launch_status("q8_gemm");
}

// Tile selection: 256x256 (8 waves of 128x64) for large problems, 128x128 (4 waves of 64x64) when the
// large tile would leave most of the 256 CUs idle.
template <int IN>
using CfgBig = GemmCfg<IN, 2, 4, 8, 4>;
template <int IN>
using CfgSmall = GemmCfg<IN, 2, 2, 4, 4>;

static int g_force_cfg = 0;  // 0 = auto, 1 = big, 2 = small (test hook, see q8_gemm_set_config)

template <int IN, int OUT, bool GELU>
static int dispatch_tile(const GemmParams& p, hipStream_t stream) {
    const long big_tiles = (long)((p.M + 255) / 256) * ((p.N + 255) / 256) * (p.batch_a > p.batch_b ? p.batch_a : p.batch_b);
    const bool big = g_force_cfg == 1 || (g_force_cfg == 0 && big_tiles >= 192);
    if (big) return launch_gemm<CfgBig<IN>, OUT, GELU>(p, stream);
    return launch_gemm<CfgSmall<IN>, OUT, GELU>(p, stream);
}

static int check_gemm(const char* who, const void* A, const void* B, const void* C, int batch_a, int batch_b, int M, int N,
                      int K) {
    if (!A || !B || !C) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if (M <= 0 || N <= 0 || K <= 0 || batch_a <= 0 || batch_b <= 0)
        return fail(Q8_ERR_SHAPE, "%s: M %d N %d K %d batch %d/%d must be positive", who, M, N, K, batch_a, batch_b);
    if (batch_a != batch_b && batch_a != 1 && batch_b != 1)
        return fail(Q8_ERR_SHAPE, "%s: batch mismatch %d vs %d", who, batch_a, batch_b);
    if (K % 16 != 0) return fail(Q8_ERR_SHAPE, "%s: K = %d must be a multiple of 16", who, K);
    if (!aligned16(A) || !aligned16(B)) return fail(Q8_ERR_ALIGN, "%s: A and B must be 16-byte aligned", who);
    if ((long)((M + 127) / 128) * ((N + 127) / 128) > 0x7fffffffL || (batch_a > 65535 || batch_b > 65535))
        return fail(Q8_ERR_SHAPE, "%s: grid too large", who);
    return Q8_OK;
}

}  // namespace q8

using namespace q8;

extern "C" int q8_gemm_set_config(int cfg) {
    if (cfg < 0 || cfg > 2) return fail(Q8_ERR_FLAGS, "q8_gemm_set_config: %d", cfg);
    g_force_cfg = cfg;
    return Q8_OK;
}

extern "C" int q8_gemm(const void* A, const void* B, const float* bias, const float* sa, const float* sb, void* C,
                       int batch_a, int batch_b, int M, int N, int K, int in_dtype, int out_dtype, int fuse_gelu,
                       q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_gemm("q8_gemm", A, B, C, batch_a, batch_b, M, N, K)) return st;
    if (!sa || !sb) return fail(Q8_ERR_NULL, "q8_gemm: scales are required");
    if (in_dtype != Q8_I8 && in_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "q8_gemm: input dtype %d", in_dtype);
    if (out_dtype != Q8_BF16 && out_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "q8_gemm: output dtype %d", out_dtype);
    if (reinterpret_cast<uintptr_t>(C) % (out_dtype == Q8_BF16 ? 16 : 8))
        return fail(Q8_ERR_ALIGN, "q8_gemm: C must be 16-byte (bf16) / 8-byte (e4m3) aligned");
    GemmParams p{static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), bias, sa, sb, C, batch_a, batch_b, M, N, K};
#define Q8_GEMM_CASE(IN, OUT)                                              \
    return fuse_gelu ? dispatch_tile<IN, OUT, true>(p, stream) : dispatch_tile<IN, OUT, false>(p, stream)
    if (in_dtype == Q8_I8) {
        if (out_dtype == Q8_BF16) { Q8_GEMM_CASE(Q8_I8, Q8_BF16); } else { Q8_GEMM_CASE(Q8_I8, Q8_E4M3); }
    } else {
        if (out_dtype == Q8_BF16) { Q8_GEMM_CASE(Q8_E4M3, Q8_BF16); } else { Q8_GEMM_CASE(Q8_E4M3, Q8_E4M3); }
    }
#undef Q8_GEMM_CASE
}

extern "C" int q8_gemm_i32(const int8_t* A, const int8_t* B, int32_t* C, int M, int N, int K, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_gemm("q8_gemm_i32", A, B, C, 1, 1, M, N, K)) return st;
    if (!aligned16(C)) return fail(Q8_ERR_ALIGN, "q8_gemm_i32: C must be 16-byte aligned");
    GemmParams p{reinterpret_cast<const uint8_t*>(A), reinterpret_cast<const uint8_t*>(B), nullptr, nullptr, nullptr, C, 1, 1, M, N, K};
    return dispatch_tile<Q8_I8, Q8_OUT_I32, false>(p, stream);
}
