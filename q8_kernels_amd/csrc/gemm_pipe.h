// Software-pipelined 256x256 GEMM tile for gfx950 (the large-problem path of q8_gemm).
//
//   * 8 waves (2 along M x 4 along N), each owning 128 x 64 of the tile as 4 x 2 MFMA tiles of 32x32:
//     fp8 uses v_mfma_f32_32x32x64_f8f6f4, int8 two v_mfma_i32_32x32x32_i8 per 64-byte K half.
//   * K advances 128 bytes per stage. A stage is A 256 rows x 128 B + B 256 rows x 128 B = 64 KiB, two stages
//     in LDS, filled by global_load_lds_dwordx4 with 8 lanes per row: every request to L2 is a full 128-byte
//     line (measured 61 B/clk/CU against 28 B/clk/CU for 64-byte rows and 40 B/clk/CU through VGPRs).
//   * Two s_barriers per stage: one as soon as every wave holds the last fragments of stage k in registers
//     (buffer k & 1 is free: the copies of stage k+2 start), one after the copies of stage k+1 have landed
//     (before its first fragments are fetched). A copy has 1 to 1.5 stages of MFMA time to land.
//   * Operand fragments are double-buffered in registers over the two 64-byte K halves of a stage: the
//     ds_read_b128 of the next half are always issued before the MFMAs of the current half. LDS reads and
//     the counters are inline assembly so that exactly the waits written below are executed.
//   * LDS rows are 128 bytes = 8 chunks of 16, physical chunk = logical chunk ^ ((row >> 1) & 7); lane
//     (row % 32, half) reads chunks 4 s + 2 half and 4 s + 2 half + 1 for K half s. A ds_read_b128 is served
//     in four passes of 16 lanes, {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31} and the same + 32
//     (measured); with this swizzle each pass hits 16 different 16-byte bank groups.
//   * B rows feed the MFMA A operand, so an accumulator lane (m = lane % 32, h = lane / 32) holds 4 consecutive
//     n per register quad; LDS row (32 t + 8 w + 4 h + r) of a wave's B slab is loaded with column
//     32 t + 16 (w / 2) + 8 h + 4 (w % 2) + r so that two quads form 8 consecutive columns (one 16-byte store)
//     and the two lane halves 32 contiguous bytes.
#pragma once
#include "gemm_common.h"

namespace q8 {

constexpr int kPipeBM = 256, kPipeBN = 256, kPipeStages = 2, kPipeStageBytes = 65536;
constexpr int kPipeParamOffset = kPipeStages * kPipeStageBytes;  // sa[256], sb[256], bias[256] of the tile (fp32)
constexpr int kPipeLds = kPipeParamOffset + 3 * 256 * 4;
typedef int v16i __attribute__((ext_vector_type(16)));

template <int MT = 4>
struct PipeFragsT {
    v4i a[MT][2];  // MT m-tiles x (low, high) 16-byte halves of the lane's 32 K bytes
    v4i b[2][2];   // 2 n-tiles
};
using PipeFrags = PipeFragsT<4>;

// a0/a1 (b0/b1): byte address of the lane's low/high 16-byte chunk in row (lane % 32) of the wave's first A (B)
// tile; the following 32-row tiles are 4096 bytes apart.
template <int MT = 4>
__device__ __forceinline__ void pipe_read_frags(PipeFragsT<MT>& f, unsigned a0, unsigned a1, unsigned b0, unsigned b1) {
    f.b[0][0] = lds_read_b128<0>(b0);
    f.b[0][1] = lds_read_b128<0>(b1);
    f.a[0][0] = lds_read_b128<0>(a0);
    f.a[0][1] = lds_read_b128<0>(a1);
    f.b[1][0] = lds_read_b128<4096>(b0);
    f.b[1][1] = lds_read_b128<4096>(b1);
    f.a[1][0] = lds_read_b128<4096>(a0);
    f.a[1][1] = lds_read_b128<4096>(a1);
    f.a[2][0] = lds_read_b128<8192>(a0);
    f.a[2][1] = lds_read_b128<8192>(a1);
    if constexpr (MT == 4) {
        f.a[3][0] = lds_read_b128<12288>(a0);
        f.a[3][1] = lds_read_b128<12288>(a1);
    }
}

// The same reads in four parts, in the order in which the MFMAs of a K half need them: part 0 = B tile 0 and A tile 0
// (4 reads), part 1 = B tile 1 and A tile 1 (4), part 2 = A tile 2 (2), part 3 = A tile 3 (2, MT = 4 only).
template <int MT, int PART>
__device__ __forceinline__ void pipe_read_frags_part(PipeFragsT<MT>& f, unsigned a0, unsigned a1, unsigned b0, unsigned b1) {
    if constexpr (PART == 0) {
        f.b[0][0] = lds_read_b128<0>(b0);
        f.b[0][1] = lds_read_b128<0>(b1);
        f.a[0][0] = lds_read_b128<0>(a0);
        f.a[0][1] = lds_read_b128<0>(a1);
    } else if constexpr (PART == 1) {
        f.b[1][0] = lds_read_b128<4096>(b0);
        f.b[1][1] = lds_read_b128<4096>(b1);
        f.a[1][0] = lds_read_b128<4096>(a0);
        f.a[1][1] = lds_read_b128<4096>(a1);
    } else if constexpr (PART == 2) {
        f.a[2][0] = lds_read_b128<8192>(a0);
        f.a[2][1] = lds_read_b128<8192>(a1);
    } else if constexpr (MT == 4) {
        f.a[3][0] = lds_read_b128<12288>(a0);
        f.a[3][1] = lds_read_b128<12288>(a1);
    }
}

// Wait until every LDS read issued so far has landed; the fragments pass through the statement so that no
// MFMA consuming them can be scheduled above it.
template <int MT>
__device__ __forceinline__ void pipe_wait_frags(PipeFragsT<MT>& f) {
    static_assert(MT == 3 || MT == 4, "wave tiles of 96 or 128 rows");
    if constexpr (MT == 4) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[2][0]), "+v"(f.a[2][1]),
                       "+v"(f.a[3][0]), "+v"(f.a[3][1]), "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[1][0]), "+v"(f.b[1][1])
                     :
                     : "memory");
    } else {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[2][0]), "+v"(f.a[2][1]),
                       "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[1][0]), "+v"(f.b[1][1])
                     :
                     : "memory");
    }
}

// Compiler-level fence for the fragments: statements that consume them stay below this point, i.e. below the
// LDS reads issued before it.
template <int MT>
__device__ __forceinline__ void pipe_pin(PipeFragsT<MT>& f) {
    if constexpr (MT == 4) {
        asm volatile(""
                     : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[2][0]), "+v"(f.a[2][1]),
                       "+v"(f.a[3][0]), "+v"(f.a[3][1]), "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[1][0]), "+v"(f.b[1][1]));
    } else {
        asm volatile(""
                     : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[2][0]), "+v"(f.a[2][1]),
                       "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[1][0]), "+v"(f.b[1][1]));
    }
}

// The 2 MT (fp8) / 4 MT (int8) MFMAs of one K half. `between(j)` runs after the j-th of the 2 MT tiles with scheduling
// fences around it, so that whatever it issues (one HBM->LDS copy) stays between two MFMAs: a wave that issued
// all copies of a stage back to back would sit in the full vector-memory queue instead of feeding the matrix pipe.
template <int IN, int MT, bool ZERO = false, typename ACC, typename F>
__device__ __forceinline__ void pipe_mfma(const PipeFragsT<MT>& f, ACC (&acc)[MT][2], F between) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            // ZERO: the first products of a tile; the MFMA adds them to a constant zero instead of a cleared accumulator
            const ACC c0 = ZERO ? ACC{} : acc[i][t];
            if constexpr (IN == Q8_I8) {
                acc[i][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.b[t][0], f.a[i][0], c0, 0, 0, 0);
                acc[i][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.b[t][1], f.a[i][1], acc[i][t], 0, 0, 0);
            } else {
                const v8i bf = {f.b[t][0][0], f.b[t][0][1], f.b[t][0][2], f.b[t][0][3], f.b[t][1][0], f.b[t][1][1], f.b[t][1][2], f.b[t][1][3]};
                const v8i af = {f.a[i][0][0], f.a[i][0][1], f.a[i][0][2], f.a[i][0][3], f.a[i][1][0], f.a[i][1][1], f.a[i][1][2], f.a[i][1][3]};
                acc[i][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf, af, c0, 0, 0, 0, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            between(2 * i + t);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int IN, int OUT, bool GELU>
__global__ __launch_bounds__(512) void gemm_pipe_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    constexpr int BM = kPipeBM, BN = kPipeBN;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wave_m = wave >> 2, wave_n = wave & 3;
    const int M = p.M, N = p.N, K = p.K;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tile_m, tile_n;
    tile_of_block(tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int z = blockIdx.y;
    const int za = (p.batch_a == 1) ? 0 : z, zb = (p.batch_b == 1) ? 0 : z;
    const uint8_t* Ag = p.A + (size_t)za * M * K;
    const uint8_t* Bg = p.B + (size_t)zb * N * K;

    // ---- HBM -> LDS copy plan. A stage is 64 row groups of 1 KiB (8 rows x 128 B): groups 0..31 hold A, 32..63 B.
    //      Wave w copies groups w, w+8, w+16, w+24 of each; lane (lane/8, lane%8) fills row 8 q + lane/8,
    //      physical chunk lane%8, from logical chunk (lane%8) ^ ((row >> 1) & 7).
    const uint8_t* src[8];
    int kchunk[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q = wave + 8 * (i & 3);
        const int rho = 8 * q + (lane >> 3);
        const int c = (lane & 7) ^ ((rho >> 1) & 7);
        kchunk[i] = 16 * c;
        if (i < 4) {
            int m = m0 + rho;
            m = m < M ? m : M - 1;
            src[i] = Ag + (size_t)m * K + 16 * c;
        } else {
            const int slab = rho >> 6, t = (rho >> 5) & 1, w = (rho >> 3) & 3, hh = (rho >> 2) & 1, r = rho & 3;
            int n = n0 + 64 * slab + 32 * t + 16 * (w >> 1) + 8 * hh + 4 * (w & 1) + r;
            n = n < N ? n : N - 1;
            src[i] = Bg + (size_t)n * K + 16 * c;
        }
    }
    const int KT = (K + 127) >> 7;
    auto issue_load = [&](int stage, int i) {  // copy instruction i (0..7) of this wave for `stage`
        uint8_t* base = lds + (stage & 1) * kPipeStageBytes;
        const int k0 = stage << 7;
        const int q = (i < 4 ? 0 : 32) + wave + 8 * (i & 3);
        // stages past the end of K (and chunks past K in the last stage) read a block of zeros instead
        const uint8_t* g = (k0 + kchunk[i] < K) ? (src[i] + k0) : reinterpret_cast<const uint8_t*>(g_zero16);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                         (__attribute__((address_space(3))) void*)(base + q * 1024), 16, 0, 0);
    };
    auto issue_loads = [&](int stage) {
#pragma unroll
        for (int i = 0; i < 8; ++i) issue_load(stage, i);
    };

    // ---- operand fetch addresses: [K half s][low / high chunk], byte offsets inside a stage
    const int r32 = lane & 31, h = lane >> 5;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const unsigned a_row = lds0 + wave_m * 16384 + r32 * 128;
    const unsigned b_row = lds0 + 32768 + wave_n * 8192 + r32 * 128;
    unsigned pc[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        pc[s][0] = ((4 * s + 2 * h) ^ ((r32 >> 1) & 7)) * 16;
        pc[s][1] = pc[s][0] ^ 16;
    }
    auto read_half = [&](PipeFrags& f, int stage, int s) {
        const unsigned so = (stage & 1) * kPipeStageBytes;
        pipe_read_frags(f, a_row + so + pc[s][0], a_row + so + pc[s][1], b_row + so + pc[s][0], b_row + so + pc[s][1]);
    };

    using acc_t = typename std::conditional<IN == Q8_I8, v16i, v16f>::type;
    acc_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][t][e] = 0;

    // ---- per-row and per-column dequantization parameters of the tile: copied to LDS now (4 bytes per lane, rows
    //      and columns past the edge clamped to the last valid one), read back in the epilogue. They are the oldest
    //      outstanding copies, so every later vmcnt wait covers them.
    float* const lds_par = reinterpret_cast<float*>(lds + kPipeParamOffset);
    if constexpr (OUT != Q8_OUT_I32) {
        const int j = (wave & 3) * 64 + lane;
        if (wave < 4) {
            const int m = (m0 + j < M) ? m0 + j : M - 1;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p.sa + (size_t)za * M + m),
                                             (__attribute__((address_space(3))) void*)(lds_par + (wave & 3) * 64), 4, 0, 0);
        } else {
            const int n = (n0 + j < N) ? n0 + j : N - 1;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p.sb + (size_t)zb * N + n),
                                             (__attribute__((address_space(3))) void*)(lds_par + 256 + (wave & 3) * 64), 4, 0, 0);
        }
        if (p.bias != nullptr && wave < 4) {
            const int n = (n0 + j < N) ? n0 + j : N - 1;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p.bias + n),
                                             (__attribute__((address_space(3))) void*)(lds_par + 512 + (wave & 3) * 64), 4, 0, 0);
        }
    }

    // ---- prologue: stage 0 landed, stage 1 in flight, fragments of the first K half on their way
    PipeFrags f0, f1;
    issue_loads(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    issue_loads(1);
    read_half(f0, 0, 0);

    for (int k = 0; k < KT; ++k) {
        // f0: first K half of stage k (reads in flight); the copies of stage k+1 are in flight
        pipe_wait_frags(f0);
        read_half(f1, k, 1);
        pipe_pin(f0);
        // First half. Once the second half of stage k is in registers everywhere (barrier 1, after the 4th MFMA
        // tile), buffer k & 1 is free and the copies of stage k+2 start to trickle out, one per MFMA tile.
        pipe_mfma<IN, 4>(f0, acc, [&](int j) {
            if (j == 3) {
                pipe_wait_frags(f1);
                __builtin_amdgcn_s_barrier();
            }
            if (j >= 4) issue_load(k + 2, j - 4);
        });
        __builtin_amdgcn_sched_barrier(0);
        pipe_pin(f1);
        // Second half. After the last copy of stage k+2 is out, everything older (stage k+1) must have landed
        // (vmcnt counts in order); barrier 2 makes that true for every wave's copies, and the first half of
        // stage k+1 is fetched under the remaining MFMA tiles. A copy has between 1 and 1.5 stages of MFMA
        // time to land.
        pipe_mfma<IN, 4>(f1, acc, [&](int j) {
            if (j < 4) issue_load(k + 2, 4 + j);
            if (j == 4) {
                asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                read_half(f0, k + 1, 0);
            }
        });
        __builtin_amdgcn_sched_barrier(0);
    }
    // drain: the look-ahead loads and fragment reads past the last stage target LDS / registers that nobody uses
    // (f0 is an operand of a wait so that its registers stay reserved until the last reads have landed)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    pipe_wait_frags(f0);

    // ---- epilogue: lane (mcol = lane % 32, h) holds for tile (i, t) and register quad w the 4 columns
    //      32 t + 16 (w / 2) + 8 h + 4 (w % 2) + 0..3 of the wave's 64-column slab, row 32 i + mcol.
    const size_t zc = (size_t)z * M * N;
    const int nw0 = n0 + wave_n * 64;
    // Interior tiles with bf16 output go through LDS: every wave lays its 128 x 64 results out as 128 rows of 128
    // bytes (16-byte chunks swizzled by (row >> 1) & 7, conflict-free both ways) and then writes 8 full rows of 128
    // contiguous bytes per instruction, i.e. whole cache lines instead of 32-byte pieces.
    const bool staged = (OUT == Q8_BF16) && (m0 + BM <= M) && (n0 + BN <= N) && ((N & 7) == 0);
    uint8_t* stage_out = lds + wave * 16384;
    if (staged) __builtin_amdgcn_s_barrier();  // every wave has finished reading the operand stages
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int wp = 0; wp < 2; ++wp) {
            const int n = nw0 + 32 * t + 16 * wp + 8 * h;
            if (n >= N) continue;
            float sbv[8], bv[8];
            if constexpr (OUT != Q8_OUT_I32) {
                const int nl = n - n0;  // multiple of 8: two 16-byte LDS reads each
                const v4f s0 = *reinterpret_cast<const v4f*>(lds_par + 256 + nl), s1 = *reinterpret_cast<const v4f*>(lds_par + 260 + nl);
                v4f b0 = {0.f, 0.f, 0.f, 0.f}, b1 = b0;
                if (p.bias != nullptr) {
                    b0 = *reinterpret_cast<const v4f*>(lds_par + 512 + nl);
                    b1 = *reinterpret_cast<const v4f*>(lds_par + 516 + nl);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) { sbv[e] = s0[e]; sbv[4 + e] = s1[e]; bv[e] = b0[e]; bv[4 + e] = b1[e]; }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + wave_m * 128 + 32 * i + r32;
                if (m >= M) continue;
                const float sam = (OUT == Q8_OUT_I32) ? 0.f : lds_par[wave_m * 128 + 32 * i + r32];
                using elem_t = typename std::conditional<IN == Q8_I8, int, float>::type;
                elem_t a8[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) a8[e] = acc[i][t][8 * wp + e];
                if constexpr (OUT == Q8_BF16) {
                    if (staged) {
                        float v[8];
                        dequant8<GELU>(a8, sam, sbv, bv, v);
                        const int row = 32 * i + r32, chunk = (4 * t + 2 * wp + h) ^ ((row >> 1) & 7);
                        *reinterpret_cast<v4u*>(stage_out + row * 128 + chunk * 16) =
                            v4u{pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]), pack2_bf16(v[4], v[5]), pack2_bf16(v[6], v[7])};
                        continue;
                    }
                }
                finish8<OUT, GELU>(p, zc, sam, m, n, a8, sbv, bv);
            }
        }
    }
    if constexpr (OUT == Q8_BF16) {
        if (staged) {
            uint16_t* cbase = reinterpret_cast<uint16_t*>(p.C) + zc + (size_t)(m0 + wave_m * 128) * N + nw0;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int row = 8 * j + (lane >> 3), chunk = (lane & 7) ^ ((row >> 1) & 7);
                const v4u w = *reinterpret_cast<const v4u*>(stage_out + row * 128 + chunk * 16);
                *reinterpret_cast<v4u*>(cbase + (size_t)row * N + (lane & 7) * 8) = w;
            }
        }
    }
}

}  // namespace q8
