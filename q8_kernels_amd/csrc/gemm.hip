// int8 / fp8-e4m3 GEMM for gfx950 with a fused dequantise + bias + tanh-GELU epilogue.
//
//   C[z,m,n] = epi( sum_k A[z,m,k] * B[z,n,k] ),  A and B both K-major (one byte per element).
//
// Structure of one workgroup (WAVES_M x WAVES_N waves, one BM x BN tile of C):
//   * K is walked in steps of 128 bytes. A step's A rows (BM x 128 B) and B rows (BN x 128 B) are
//     copied HBM -> LDS by `global_load_lds_dwordx4` (no VGPR staging), four LDS stages, copies three steps ahead.
//   * LDS holds plain 128-byte rows whose 16-byte chunks are XOR-swizzled by lds_swizzle(row). A
//     ds_read_b128 is served in four passes of 16 lanes, and the lanes of one pass are NOT consecutive:
//     measured on gfx950 they are {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the same
//     + 32. With operand lane = (row % 16, k-chunk pair lane / 16) a pass therefore touches all 16 rows,
//     rows {0-3, 12-15} at one chunk pair and rows {4-11} at the neighbouring one; the swizzle makes
//     those 16 accesses fall into the 16 different 16-byte bank groups (256 B/clk, no conflicts).
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
#include "gemm_common.h"
#include "gemm_persist.h"

namespace q8 {

template <class C, int OUT, bool GELU>
__global__ __launch_bounds__(C::NT) void gemm_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    constexpr int BM = C::BM, BN = C::BN, TM = C::TM, TN = C::TN, NW = C::NW;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wave_m = wave / C::WAVES_N, wave_n = wave % C::WAVES_N;
    const int M = p.M, N = p.N, K = p.K;

    // ---- tile of this workgroup
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tile_m, tile_n;
    tile_of_block(tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int z = blockIdx.y;
    const int za = (p.batch_a == 1) ? 0 : z, zb = (p.batch_b == 1) ? 0 : z;
    const uint8_t* Ag = p.A + (size_t)za * M * K;
    const uint8_t* Bg = p.B + (size_t)zb * N * K;

    // ---- HBM -> LDS copy plan: lane (lane/8, lane%8) of row group q fills LDS row 8q + lane/8,
    //      physical chunk lane%8, from logical chunk (lane%8) ^ lds_swizzle(row)
    const uint8_t* src[C::PER_A + C::PER_B];
    int kchunk[C::PER_A + C::PER_B];
#pragma unroll
    for (int i = 0; i < C::PER_A + C::PER_B; ++i) {
        const bool isA = i < C::PER_A;
        const int q = isA ? (wave + i * NW) : (wave + (i - C::PER_A) * NW);
        const int rho = 8 * q + (lane >> 3);
        const int c = (lane & 7) ^ lds_swizzle(rho);
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
    auto issue_loads = [&](int stage, int k0) {  // (k0 may lie past K: the whole step then comes from the block of zeros)
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
    const int pc0 = ((2 * gk) ^ lds_swizzle(s16)) * 16, pc1 = pc0 ^ 16;
    const int a_row0 = wave_m * TM * 16 + s16;
    const int b_row0 = BM + wave_n * TN * 16 + s16;

    using acc_t = typename std::conditional<C::IN == Q8_I8, v4i, v4f>::type;
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    // C::STAGES LDS stages and two sets of operand registers. In step kt the wave multiplies the operands of step kt, which
    // it requested from LDS during step kt - 1, while the operands of step kt + 1 travel from LDS to the other register set
    // and the copies of steps kt + 2 .. kt + STAGES - 1 travel from HBM to LDS. Every wave issues the same number of copies
    // per step - past the end of K from a block of zeros - so "all but the (STAGES - 3) PER youngest copies" is exactly
    // "step kt + 1 has landed". One barrier per step: it publishes step kt + 1 and says that everyone holds the operands
    // of step kt - 1 (waited for before that step's multiplications), whose buffer the copies of step kt + STAGES - 1
    // overwrite.
    constexpr int PER = C::PER_A + C::PER_B, STAGES = C::STAGES;
    static_assert(STAGES >= 4 && (STAGES - 3) * PER <= 63, "vmcnt holds 6 bits");
    const int KT = (K + 127) / 128;
    const unsigned lds0 = lds_addr(lds);
    struct Frags { v4i a_lo[TM], a_hi[TM], b_lo[TN], b_hi[TN]; };
    auto read_frags = [&](Frags& f, int stage) {
        const unsigned st = lds0 + stage * C::STAGE_BYTES;
        const unsigned br = st + b_row0 * 128, ar = st + a_row0 * 128;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            f.b_lo[j] = lds_read_b128<0>(br + 2048 * j + pc0);
            f.b_hi[j] = lds_read_b128<0>(br + 2048 * j + pc1);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            f.a_lo[i] = lds_read_b128<0>(ar + 2048 * i + pc0);
            f.a_hi[i] = lds_read_b128<0>(ar + 2048 * i + pc1);
        }
    };
    auto wait_frags = [&](Frags& f) {  // every LDS read issued so far has landed; the registers of `f` pass through the wait
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(f.a_lo[i]), "+v"(f.a_hi[i]));
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(f.b_lo[j]), "+v"(f.b_hi[j]));
    };
    auto multiply = [&](const Frags& f) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (C::IN == Q8_I8) {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f.b_lo[j], f.a_lo[i], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f.b_hi[j], f.a_hi[i], acc[i][j], 0, 0, 0);
                } else {
                    const v8i bf = {f.b_lo[j][0], f.b_lo[j][1], f.b_lo[j][2], f.b_lo[j][3], f.b_hi[j][0], f.b_hi[j][1], f.b_hi[j][2], f.b_hi[j][3]};
                    const v8i af = {f.a_lo[i][0], f.a_lo[i][1], f.a_lo[i][2], f.a_lo[i][3], f.a_hi[i][0], f.a_hi[i][1], f.a_hi[i][2], f.a_hi[i][3]};
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[i][j], 0, 0, 0, 0, 0, 0);
                }
            }
        }
    };
    // one step: `cur` holds (in flight) the operands of step kt, `nxt` receives those of step kt + 1
    auto step = [&](int kt, Frags& cur, Frags& nxt) {
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"((STAGES - 3) * PER) : "memory");
        __builtin_amdgcn_s_barrier();
        issue_loads((kt + STAGES - 1) % STAGES, (kt + STAGES - 1) * 128);
        wait_frags(cur);
        read_frags(nxt, (kt + 1) % STAGES);
        __builtin_amdgcn_sched_barrier(0);
        multiply(cur);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int s = 0; s < STAGES - 2; ++s) issue_loads(s, s * 128);
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((STAGES - 3) * PER) : "memory");
    __builtin_amdgcn_s_barrier();
    issue_loads(STAGES - 2, (STAGES - 2) * 128);
    Frags f0, f1;
    read_frags(f0, 0);
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        step(kt, f0, f1);
        step(kt + 1, f1, f0);
    }
    if (kt < KT) step(kt, f0, f1);
    // (the operand reads of the step past the last one target registers that nobody uses)
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f0.a_lo[0]), "+v"(f1.a_lo[0]) : : "memory");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the look-ahead copies past the last step

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
        load_col_params<OUT>(p, zb, n, sbv, bv);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = m0 + wave_m * TM * 16 + 16 * i + s16;
            if (m >= M) continue;
            const float sam = (OUT == Q8_OUT_I32) ? 0.f : p.sa[(size_t)za * M + m];
            using elem_t = typename std::conditional<C::IN == Q8_I8, int, float>::type;
            const elem_t a8[8] = {acc[i][2 * jj][0], acc[i][2 * jj][1], acc[i][2 * jj][2], acc[i][2 * jj][3],
                                  acc[i][2 * jj + 1][0], acc[i][2 * jj + 1][1], acc[i][2 * jj + 1][2], acc[i][2 * jj + 1][3]};
            finish8<OUT, GELU>(p, zc, sam, m, n, a8, sbv, bv);
        }
    }
}

// which kernel the last q8_gemm* call of this thread launched (q8_gemm_last_kernel)
static thread_local int g_last_kernel = 0;

// A kernel's dynamic LDS limit is a per-device attribute: it is set once per (thread, kernel, device). `done_dev` is
// the caller's thread-local record of the device it was last set on.
static int reserve_lds(const void* kern, int bytes, int& done_dev) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return fail(Q8_ERR_LAUNCH, "q8_gemm: no current device");
    }
    if (done_dev == dev) return Q8_OK;
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return fail(Q8_ERR_LAUNCH, "q8_gemm: cannot reserve %d bytes of LDS", bytes);
    }
    done_dev = dev;
    return Q8_OK;
}

template <class C, int OUT, bool GELU>
static int launch_gemm(const GemmParams& p, hipStream_t stream) {
    g_last_kernel = C::BM == 64 ? Q8_GEMM_KERNEL_TILE64 : Q8_GEMM_KERNEL_TILE128;
    const int tiles_m = (p.M + C::BM - 1) / C::BM, tiles_n = (p.N + C::BN - 1) / C::BN;
    const int batch = p.batch_a > p.batch_b ? p.batch_a : p.batch_b;
    if ((long)tiles_m * tiles_n > 0x7fffffffL) return fail(Q8_ERR_SHAPE, "q8_gemm: grid too large");
    auto kern = gemm_kernel<C, OUT, GELU>;
    static thread_local int lds_dev = -1;
    if (int st = reserve_lds(reinterpret_cast<const void*>(kern), C::LDS_BYTES, lds_dev)) return st;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(C::NT), C::LDS_BYTES, stream, p);
    return launch_status("q8_gemm");
}

// Tile selection: pipelined 256x256 tiles (gemm_pipe.h / gemm_persist.h) for large problems, this file's 128x128 or 64x64
// tiles when the large tile would leave most of the 256 CUs idle.
// Two shapes (measured on 2048-deep problems; a K step costs about in proportion to the tile's bytes, so what counts is
// how many CUs the tiles reach): 8 waves (2 x 4, wave tiles of 64 x 32) on 128x128 tiles, and 4 waves (2 x 2, wave tiles
// of 32 x 32) on 64x64 tiles, two workgroups per CU, for problems with at most 512 such tiles - 256 x 4096 x 2048: 8.5 us
// against 12.5 us, 2048 x 2048 x 2048: 19.2 us against 14.6 us.
template <int IN>
using CfgSmall = GemmCfg<IN, 2, 4, 4, 2>;
template <int IN>
using CfgSmall64 = GemmCfg<IN, 2, 2, 2, 2>;

// per-thread override (q8_gemm_set_config): 0 = auto, 1 = pipelined 256x256 (one tile per workgroup), 2 = 128x128,
// 3 = 64x64, 4 = persistent pipelined 256x256 where eligible
static thread_local int g_force_cfg = 0;

template <int IN, int OUT, bool GELU>
static int launch_pipe(const GemmParams& p, hipStream_t stream) {
    const int tiles_m = (p.M + kPipeBM - 1) / kPipeBM, tiles_n = (p.N + kPipeBN - 1) / kPipeBN;
    const int batch = p.batch_a > p.batch_b ? p.batch_a : p.batch_b;
    auto kern = gemm_pipe_kernel<IN, OUT, GELU>;
    g_last_kernel = Q8_GEMM_KERNEL_PIPE256;
    static thread_local int lds_dev = -1;
    if (int st = reserve_lds(reinterpret_cast<const void*>(kern), kPipeLds, lds_dev)) return st;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(512), kPipeLds, stream, p);
    return launch_status("q8_gemm");
}

// One workgroup per CU walking over the tiles (gemm_persist.h); bf16 or e4m3 output, N % 8 == 0, K a multiple of 128 above 256.
// The tile height is 256 or 192 rows, whichever gives the shorter schedule: work per CU = rounds x tile height, with
// 20 % charged to the smaller tile (measured: a 192-row round takes 0.90 of a 256-row round, not 0.75: it moves 17 %
// more operand bytes per flop and pays the same epilogue and barrier overheads).
static int persist_cus() {
    static thread_local int cus = 0, cus_dev = -1;  // of the device the count was read on
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 256;
    }
    if (cus_dev != dev) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            n = 256;
        }
        cus = n >= 8 ? (n / 8) * 8 : 8;  // a multiple of the 8 XCDs keeps every workgroup's tiles on one XCD
        cus_dev = dev;
    }
    return cus;
}

template <int IN, bool GELU, int MT, bool RES, bool E4M3OUT, int VSPLIT = 0>
static int launch_persist_mt(const GemmParams& p, hipStream_t stream) {
    constexpr int BM = 64 * MT;
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + kPipeBN - 1) / kPipeBN;
    const int batch = p.batch_a > p.batch_b ? p.batch_a : p.batch_b;
    const long total = (long)tiles_m * tiles_n * batch;
    if (total > 0x7fffffffL) return fail(Q8_ERR_SHAPE, "q8_gemm: too many tiles");
    auto kern = gemm_persist_kernel<IN, GELU, MT, RES, E4M3OUT, VSPLIT>;
    g_last_kernel = (MT == 4 ? Q8_GEMM_KERNEL_PERSIST256 : Q8_GEMM_KERNEL_PERSIST192) | (RES ? Q8_GEMM_KERNEL_RESIDUAL : 0);
    static thread_local int lds_dev = -1;
    if (int st = reserve_lds(reinterpret_cast<const void*>(kern), kPersistLds, lds_dev)) return st;
    const int cus = persist_cus();
    const int grid = total < cus ? (int)total : cus;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), kPersistLds, stream, p, tiles_m, tiles_n, (int)total);
    return launch_status("q8_gemm");
}

static thread_local int g_persist_mt = 0;  // 0 = choose, 3 / 4 = forced tile height 192 / 256 (tuning, per thread)

template <int IN, bool GELU, bool E4M3OUT = false>
static int launch_persist(const GemmParams& p, hipStream_t stream) {
    const long batch = p.batch_a > p.batch_b ? p.batch_a : p.batch_b;
    const long tn = (p.N + kPipeBN - 1) / kPipeBN, cus = persist_cus();
    // (with a residual the 256-row kernel is 256 registers short by a dozen: it spills copy offsets around its epilogue
    //  and runs 10-15 % slower than its tile count says, measured; the 192-row kernel does not)
    //  (the same holds for the Hadamard form of the head-major epilogue)
    const double cost256 = (!E4M3OUT && (p.residual != nullptr || (p.v_codes != nullptr && p.v_fht_scale != 0.f))) ? 1.25 : 1.0;
    auto cost = [&](int bm) {
        const long tiles = (long)((p.M + bm - 1) / bm) * tn * batch;
        return (double)((tiles + cus - 1) / cus) * bm * (bm == 256 ? cost256 : 1.2);
    };
    const bool small = g_persist_mt == 3 || (g_persist_mt == 0 && cost(192) < cost(256));
    if constexpr (!E4M3OUT && !GELU) {
        if (p.v_codes != nullptr && p.v_fht_scale != 0.f)
            return small ? launch_persist_mt<IN, false, 3, false, false, 2>(p, stream) : launch_persist_mt<IN, false, 4, false, false, 2>(p, stream);
        if (p.v_codes != nullptr)
            return small ? launch_persist_mt<IN, false, 3, false, false, 1>(p, stream) : launch_persist_mt<IN, false, 4, false, false, 1>(p, stream);
    }
    if constexpr (!E4M3OUT) {
        if (p.residual != nullptr)
            return small ? launch_persist_mt<IN, GELU, 3, true, false>(p, stream) : launch_persist_mt<IN, GELU, 4, true, false>(p, stream);
    }
    return small ? launch_persist_mt<IN, GELU, 3, false, E4M3OUT>(p, stream) : launch_persist_mt<IN, GELU, 4, false, E4M3OUT>(p, stream);
}

// shapes the persistent kernel takes (bf16 or e4m3 output)
static bool persist_eligible(const GemmParams& p) {
    return (p.N % 8) == 0 && p.K > 256 && (p.K % 128) == 0 && (uint64_t)p.M * p.K < (1ull << 32) && (uint64_t)p.N * p.K < (1ull << 32);
}

template <int IN, int OUT, bool GELU>
static int dispatch_tile(const GemmParams& p, hipStream_t stream) {
    const long big_tiles = (long)((p.M + 255) / 256) * ((p.N + 255) / 256) * (p.batch_a > p.batch_b ? p.batch_a : p.batch_b);
    const bool big = g_force_cfg == 1 || g_force_cfg == 4 || (g_force_cfg == 0 && big_tiles >= 192);
    if constexpr (OUT == Q8_BF16 || OUT == Q8_E4M3) {
        if (big && g_force_cfg != 1 && persist_eligible(p)) return launch_persist<IN, GELU, OUT == Q8_E4M3>(p, stream);
    }
    if (big) return launch_pipe<IN, OUT, GELU>(p, stream);
    const long tiles64 = (long)((p.M + 63) / 64) * ((p.N + 63) / 64) * (p.batch_a > p.batch_b ? p.batch_a : p.batch_b);
    if (g_force_cfg == 3 || (g_force_cfg == 0 && tiles64 <= 512)) return launch_gemm<CfgSmall64<IN>, OUT, GELU>(p, stream);
    return launch_gemm<CfgSmall<IN>, OUT, GELU>(p, stream);
}

// An output without rows or columns (no tokens): nothing to compute or to write. Negative sizes, K <= 0 and bad batch
// counts are still errors (check_gemm).
static bool gemm_output_is_empty(int batch_a, int batch_b, int M, int N, int K) {
    return (M == 0 || N == 0) && M >= 0 && N >= 0 && K > 0 && batch_a > 0 && batch_b > 0;
}

static int check_gemm(const char* who, const void* A, const void* B, const void* C, int batch_a, int batch_b, int M, int N,
                      int K) {
    if (!A || !B || !C) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if (M <= 0 || N <= 0 || K <= 0 || batch_a <= 0 || batch_b <= 0)
        return fail(Q8_ERR_SHAPE, "%s: M %d N %d K %d batch %d/%d must be positive", who, M, N, K, batch_a, batch_b);
    // (2^30 keeps every rounded-up tile count of the launch geometry inside int)
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return fail(Q8_ERR_SHAPE, "%s: M %d N %d K %d too large", who, M, N, K);
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

extern "C" int q8_gemm_last_kernel(void) { return g_last_kernel; }

extern "C" int q8_gemm_set_config(int cfg) {
    if (cfg == 43 || cfg == 44 || cfg == 40) { g_persist_mt = cfg - 40; return Q8_OK; }  // tuning: persistent tile height
    if (cfg < 0 || cfg > 4) return fail(Q8_ERR_FLAGS, "q8_gemm_set_config: %d", cfg);
    g_force_cfg = cfg;
    return Q8_OK;
}

extern "C" int q8_gemm(const void* A, const void* B, const float* bias, const float* sa, const float* sb, void* C,
                       int batch_a, int batch_b, int M, int N, int K, int in_dtype, int out_dtype, int fuse_gelu,
                       q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (gemm_output_is_empty(batch_a, batch_b, M, N, K)) return Q8_OK;
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

extern "C" int q8_gemm_residual(const void* A, const void* B, const float* bias, const float* sa, const float* sb,
                                const void* residual, void* C, int batch_a, int batch_b, int M, int N, int K, int in_dtype,
                                int fuse_gelu, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (gemm_output_is_empty(batch_a, batch_b, M, N, K)) return Q8_OK;
    if (int st = check_gemm("q8_gemm_residual", A, B, C, batch_a, batch_b, M, N, K)) return st;
    if (!sa || !sb || !residual) return fail(Q8_ERR_NULL, "q8_gemm_residual: scales and residual are required");
    if (in_dtype != Q8_I8 && in_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "q8_gemm_residual: input dtype %d", in_dtype);
    if ((reinterpret_cast<uintptr_t>(C) % 16) || (reinterpret_cast<uintptr_t>(residual) % 16))
        return fail(Q8_ERR_ALIGN, "q8_gemm_residual: C and residual must be 16-byte aligned");
    GemmParams p{static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), bias, sa, sb, C, batch_a, batch_b, M, N, K};
    p.residual = residual;
    if (!persist_eligible(p))
        return fail(Q8_ERR_SHAPE, "q8_gemm_residual: needs N %% 8 == 0 and K a multiple of 128 above 256 (N %d K %d)", N, K);
    if (in_dtype == Q8_I8) return fuse_gelu ? launch_persist<Q8_I8, true>(p, stream) : launch_persist<Q8_I8, false>(p, stream);
    return fuse_gelu ? launch_persist<Q8_E4M3, true>(p, stream) : launch_persist<Q8_E4M3, false>(p, stream);
}

extern "C" int q8_gemm_qkv(const void* A, const void* B, const float* bias, const float* sa, const float* sb, void* C, void* v_codes,
                           int M, int N, int K, int v_col0, int tokens, float v_fht_scale, int in_dtype, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "q8_gemm_qkv";
    if (gemm_output_is_empty(1, 1, M, N, K)) return Q8_OK;
    // (v_col0 == 0: a V projection of its own, every column goes to v_codes and C is not used)
    if (int st = check_gemm(who, A, B, v_col0 == 0 ? v_codes : C, 1, 1, M, N, K)) return st;
    if (!sa || !sb || !v_codes) return fail(Q8_ERR_NULL, "%s: scales and v_codes are required", who);
    if (in_dtype != Q8_I8 && in_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "%s: input dtype %d", who, in_dtype);
    if ((reinterpret_cast<uintptr_t>(C) % 16) || (reinterpret_cast<uintptr_t>(v_codes) % 16))
        return fail(Q8_ERR_ALIGN, "%s: C and v_codes must be 16-byte aligned", who);
    // whole 256-column tiles on either side of the split, whole heads of 64 in the V part, whole batch elements in M
    if (v_col0 < 0 || v_col0 >= N || v_col0 % 256 != 0 || (N - v_col0) % 64 != 0)
        return fail(Q8_ERR_SHAPE, "%s: v_col0 = %d must be a multiple of 256 below N = %d with N - v_col0 a multiple of 64", who, v_col0, N);
    if (tokens <= 0 || M % tokens != 0) return fail(Q8_ERR_SHAPE, "%s: M = %d must be a multiple of tokens = %d", who, M, tokens);
    if (!(v_fht_scale >= 0.f) || v_fht_scale > 3.0e38f) return fail(Q8_ERR_SHAPE, "%s: v_fht_scale = %g must be finite and not negative", who, (double)v_fht_scale);
    GemmParams p{static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), bias, sa, sb, C, 1, 1, M, N, K};
    p.v_codes = static_cast<uint8_t*>(v_codes);
    p.v_fht_scale = v_fht_scale;
    p.v_col0 = v_col0;
    p.v_tokens = tokens;
    p.v_heads = (N - v_col0) / 64;
    if (!persist_eligible(p))
        return fail(Q8_ERR_SHAPE, "%s: needs N %% 8 == 0 and K a multiple of 128 above 256 (N %d K %d)", who, N, K);
    return in_dtype == Q8_I8 ? launch_persist<Q8_I8, false>(p, stream) : launch_persist<Q8_E4M3, false>(p, stream);
}

extern "C" int q8_gemm_gated_residual(const void* A, const void* B, const float* bias, const float* sa, const float* sb,
                                      const void* residual, const void* gate, int64_t rows_per_gate, void* C, int M, int N, int K,
                                      int in_dtype, int fuse_gelu, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "q8_gemm_gated_residual";
    if (gemm_output_is_empty(1, 1, M, N, K)) return Q8_OK;
    if (int st = check_gemm(who, A, B, C, 1, 1, M, N, K)) return st;
    if (!sa || !sb || !residual || !gate) return fail(Q8_ERR_NULL, "%s: scales, residual and gate are required", who);
    if (in_dtype != Q8_I8 && in_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "%s: input dtype %d", who, in_dtype);
    if ((reinterpret_cast<uintptr_t>(C) % 16) || (reinterpret_cast<uintptr_t>(residual) % 16) || (reinterpret_cast<uintptr_t>(gate) % 16))
        return fail(Q8_ERR_ALIGN, "%s: C, residual and gate must be 16-byte aligned", who);
    // a tile (192 or 256 rows) must lie inside one group of rows that share a gate row
    if (rows_per_gate <= 0 || rows_per_gate % 768 != 0 || rows_per_gate > 0x7fffffffLL)
        return fail(Q8_ERR_SHAPE, "%s: rows_per_gate = %lld must be a positive multiple of 768", who, (long long)rows_per_gate);
    GemmParams p{static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(B), bias, sa, sb, C, 1, 1, M, N, K};
    p.residual = residual;
    p.gate = static_cast<const uint16_t*>(gate);
    p.rows_per_gate = (int)rows_per_gate;
    if (!persist_eligible(p))
        return fail(Q8_ERR_SHAPE, "%s: needs N %% 8 == 0 and K a multiple of 128 above 256 (N %d K %d)", who, N, K);
    if (in_dtype == Q8_I8) return fuse_gelu ? launch_persist<Q8_I8, true>(p, stream) : launch_persist<Q8_I8, false>(p, stream);
    return fuse_gelu ? launch_persist<Q8_E4M3, true>(p, stream) : launch_persist<Q8_E4M3, false>(p, stream);
}

extern "C" int q8_gemm_i32(const int8_t* A, const int8_t* B, int32_t* C, int M, int N, int K, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (gemm_output_is_empty(1, 1, M, N, K)) return Q8_OK;
    if (int st = check_gemm("q8_gemm_i32", A, B, C, 1, 1, M, N, K)) return st;
    if (!aligned16(C)) return fail(Q8_ERR_ALIGN, "q8_gemm_i32: C must be 16-byte aligned");
    GemmParams p{reinterpret_cast<const uint8_t*>(A), reinterpret_cast<const uint8_t*>(B), nullptr, nullptr, nullptr, C, 1, 1, M, N, K};
    return dispatch_tile<Q8_I8, Q8_OUT_I32, false>(p, stream);
}
