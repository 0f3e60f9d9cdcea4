// Persistent form of the pipelined 256x256 GEMM tile (gemm_pipe.h): one workgroup per CU walks over several output
// tiles and the HBM->LDS copy pipeline runs straight across the tile boundaries.
//
//   * The tile is 256 x 256, or 192 x 256 (3 instead of 4 MFMA tiles per wave along M) when that spreads the work more
//     evenly over the CUs.
//   * Work item v (tile id + tiles * batch index) is handled by workgroup v % gridDim.x, which runs on XCD v % 8;
//     the tile walk is the XCD-contiguous grouped walk of tile_of_block, so the L2 reuse is the same.
//   * The compute side counts K stages globally (g); the copy side runs two stages ahead of it (gl = g + 2) with its
//     own (item, k) position and source pointers. While the last two stages of a tile are multiplied, the first two
//     stages of the next tile are already on their way, and they land while the epilogue of the finished tile runs.
//   * The epilogue therefore may not touch the two stage buffers: every wave stages its results through 2 KiB of its
//     own (16 rows x 128 B per round, two rounds per 32-row MFMA tile, chunks swizzled by (row >> 1) & 7) and writes
//     8 complete 128-byte lines per store instruction. (With GELU fused and no residual the lanes store their chunks
//     directly instead, see the epilogue.) All LDS traffic of the epilogue is inline assembly with its own
//     lgkmcnt waits; the stores are never waited for, they drain under the next tile's MFMAs.
//   * sa / sb / bias of a tile are copied to LDS (double-buffered) when the copy side enters the tile.
//   * Every wave issues the same number of copy instructions per stage (8, and 2 more in a stage where the copy
//     side moves to the next tile; past the last tile the copies read a block of zeros), so the in-order vmcnt
//     waits are exact.
#pragma once
#include "gemm_pipe.h"

namespace q8 {

constexpr int kPersistParBytes = 3 * 256 * 4 + 256 * 2;                      // sa[256], sb[256], bias[256] fp32, gate[256] bf16
constexpr int kPersistParOffset = kPipeStages * kPipeStageBytes;            // 2 x parameters of a tile
constexpr int kPersistStageOutOffset = kPersistParOffset + 2 * kPersistParBytes;   // 8 waves x 2 KiB
constexpr int kPersistLds = kPersistStageOutOffset + 8 * 2048;

__device__ __forceinline__ void lds_write_b128(unsigned addr, v4u v) {
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ float lds_read_b32(unsigned addr) {
    float r;
    asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}

// tile of work item `pid_in` out of `nb` = tiles_m * tiles_n (same walk as tile_of_block)
__device__ __forceinline__ void tile_of_id(int bid, int nb, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    const int xcd = bid & 7, loc = bid >> 3, per = nb >> 3, rem = nb & 7;
    const int pid = xcd * per + (xcd < rem ? xcd : rem) + loc;
    const int group_size = kGroupM * tiles_n;
    const int gid = pid / group_size, first_m = gid * kGroupM;
    const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    tile_m = first_m + (pid % group_size) % gsz;
    tile_n = (pid % group_size) / gsz;
}

// Requirements checked by the host: K % 128 == 0 and K > 256 (at least 3 whole stages per tile), N % 8 == 0,
// M * K and N * K below 2^32 (32-bit source offsets).
// E4M3OUT: the output is e4m3 (saturating cast, the reference's default output type, csrc/gemm/q8_gemm_api.cpp:82-87) instead
// of bf16: the lanes store their codes straight from the MFMA layout, 16 bytes each after a swap between the two lanes of
// a row (no residual form).
// MT = 32-row MFMA tiles per wave along M: the tile is 64 MT x 256, i.e. 256 x 256 (MT = 4) or 192 x 256 (MT = 3, for
// problems whose 256-row tiles do not divide evenly over the CUs).
// RES: C = bf16(bf16(result) + residual), the residual connection around a projection (two roundings, as the separate
// element-wise addition of the two bf16 tensors gives); with p.gate (uniform) C = bf16(fma(bf16(result), gate, residual)),
// the gated residual of an AdaLN block (blocks/ltx_transformer_block.py:44,57 in the reference), one gate row per
// rows_per_gate rows: what the fused multiply-add kernel gives on the rounded projection.
// VSPLIT (bf16 output, no residual): the tiles from column p.v_col0 on hold the V projection of a fused QKV layer; their
// results are rounded to bf16 like the others, then cast to e4m3 (the c10 cast of q8_kernels/functional/flash_attention.py:
// 38-45) and written token-major per head, [B, H, S, 64], the Q8_V_SD operand of the attention kernel: what the attention
// prologue otherwise produces from the bf16 projection. C holds the other columns only (p.v_col0 per row).
// VSPLIT == 2: the bf16-rounded results of a head (a wave's 64-column slab) go through the 64-point Hadamard transform
// times p.v_fht_scale before the cast: the Q or K operand of an attention with apply_qk_hadamard
// (q8_kernels/functional/flash_attention.py:47-51) straight from the projection.
template <int IN, bool GELU, int MT, bool RES, bool E4M3OUT = false, int VSPLIT = 0>
__global__ __launch_bounds__(512) void gemm_persist_kernel(const GemmParams p, int tiles_m, int tiles_n, int total) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    static_assert(!(RES && E4M3OUT), "the residual epilogue writes bf16");
    static_assert(VSPLIT == 0 || (!RES && !E4M3OUT), "the V split belongs to the plain bf16 epilogue");
    constexpr int BM = 64 * MT, BN = kPipeBN;
    constexpr int NCOPY = MT + 4;  // copy instructions per wave and stage: MT row groups of A, 4 of B
    const int tid = threadIdx.x, lane = tid & 63;
    // The wave index is read back as a scalar: everything derived from it then lives in scalar registers. With it in
    // a vector register the 256-row variants spill tile-change and epilogue state, and every reload of a spilled value
    // costs a wait for ALL outstanding copies (scratch loads share the in-order counter of the copy pipeline).
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2, wave_n = wave & 3;
    const int M = p.M, N = p.N, K = p.K;
    const int tiles = tiles_m * tiles_n;
    const int KT = (K + 127) >> 7;
    const int G = gridDim.x;
    const int count = (total - (int)blockIdx.x + G - 1) / G;  // >= 1: the grid never exceeds `total`

    struct Item { int m0, n0, z, za, zb; };
    auto item_of = [&](int idx) {
        const int v = blockIdx.x + idx * G;
        const int z = v / tiles;
        int tm, tn;
        tile_of_id(v - z * tiles, tiles, tiles_m, tiles_n, tm, tn);
        return Item{tm * BM, tn * BN, z, (p.batch_a == 1) ? 0 : z, (p.batch_b == 1) ? 0 : z};
    };

    // ---- copy side ------------------------------------------------------------------------------------------
    // A stage is 8 MT + 32 row groups of 1 KiB (8 rows x 128 B): the first 8 MT hold A, the others B. Wave w copies
    // groups w, w+8, ... of each; lane (lane/8, lane%8) fills row 8 q + lane/8, physical chunk lane%8, from logical
    // chunk (lane%8) ^ ((row >> 1) & 7).
    // (the swizzle term is the same for the 8 row groups of a wave: their rows differ by multiples of 64).
    // Sources are a uniform base per operand plus a 32-bit byte offset per lane and row group.
    uint32_t off[NCOPY];
    const uint8_t* baseA;
    const uint8_t* baseB;
    const uint32_t kchunk = 16 * ((lane & 7) ^ ((4 * wave + (lane >> 4)) & 7));
    bool copy_live = true;  // the copy side still points at a real tile
    auto set_src = [&](const Item& it) {
        baseA = p.A + (size_t)it.za * M * K;
        baseB = p.B + (size_t)it.zb * N * K;
#pragma unroll
        for (int i = 0; i < NCOPY; ++i) {
            const int rho = 8 * (wave + 8 * (i < MT ? i : i - MT)) + (lane >> 3);
            if (i < MT) {
                int m = it.m0 + rho;
                m = m < M ? m : M - 1;
                off[i] = (uint32_t)m * (uint32_t)K + kchunk;
            } else {
                const int slab = rho >> 6, t = (rho >> 5) & 1, w = (rho >> 3) & 3, hh = (rho >> 2) & 1, r = rho & 3;
                int n = it.n0 + 64 * slab + 32 * t + 16 * (w >> 1) + 8 * hh + 4 * (w & 1) + r;
                n = n < N ? n : N - 1;
                off[i] = (uint32_t)n * (uint32_t)K + kchunk;
            }
        }
    };
    auto set_src_zeros = [&]() {  // past the last tile: every lane reads the same 16 zero bytes
        baseA = baseB = reinterpret_cast<const uint8_t*>(g_zero16);
#pragma unroll
        for (int i = 0; i < NCOPY; ++i) off[i] = 0;
    };
    // two 4-byte-per-lane copies per wave: waves 0-3 bring sa and bias, waves 4-7 sb and the tile's gate row (256 bf16 =
    // 128 dwords: waves 4 / 6 the first 64, waves 5 / 7 the others; without a gate sb a second time, to keep the count equal)
    auto copy_params = [&](const Item& it, int buf, bool live) {
        float* par = reinterpret_cast<float*>(lds + kPersistParOffset + buf * kPersistParBytes);
        const int j = (wave & 3) * 64 + lane;
        const float* g0;
        const float* g1;
        float* d0;
        float* d1;
        if (wave < 4) {
            const int m = (it.m0 + j < M) ? it.m0 + j : M - 1;  // (rows past the tile's BM are copied but never read)
            const int n = (it.n0 + j < N) ? it.n0 + j : N - 1;
            g0 = p.sa + (size_t)it.za * M + m;
            g1 = (p.bias != nullptr) ? p.bias + n : reinterpret_cast<const float*>(g_zero16);
            d0 = par + (wave & 3) * 64;
            d1 = par + 512 + (wave & 3) * 64;
        } else {
            const int n = (it.n0 + j < N) ? it.n0 + j : N - 1;
            g0 = g1 = p.sb + (size_t)it.zb * N + n;
            d0 = d1 = par + 256 + (wave & 3) * 64;
            if constexpr (RES) {
                if (p.gate != nullptr) {
                    const int jj = (wave & 1) * 64 + lane;  // columns 2 jj, 2 jj + 1 of the tile (N is even)
                    const int n2 = (it.n0 + 2 * jj + 1 < N) ? it.n0 + 2 * jj : N - 2;
                    g1 = reinterpret_cast<const float*>(p.gate + (size_t)(it.m0 / p.rows_per_gate) * N + n2);
                    d1 = par + 768 + (wave & 1) * 64;
                }
            }
        }
        if (!live) g0 = g1 = reinterpret_cast<const float*>(g_zero16);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g0,
                                         (__attribute__((address_space(3))) void*)d0, 4, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g1,
                                         (__attribute__((address_space(3))) void*)d1, 4, 0, 0);
    };
    int l_item = 0, l_k = 0, gl = 0;  // copy side: item, stage inside the item, global stage count
    Item nxt{};                       // the tile the copy side moved to last: the compute side's next one
    auto issue_copy = [&](int i) {    // copy instruction i (0 .. NCOPY-1) of the copy side's current stage
        uint8_t* base = lds + (gl & 1) * kPipeStageBytes;
        const uint32_t k0 = copy_live ? (uint32_t)l_k << 7 : 0u;
        const int q = (i < MT ? 8 * i : 8 * MT + 8 * (i - MT)) + wave;
        const uint8_t* g = (i < MT ? baseA : baseB) + k0 + off[i];
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                         (__attribute__((address_space(3))) void*)(base + q * 1024), 16, 0, 0);
    };
    // after the 8th copy of a stage; returns true when the copy side moved to the next tile (2 more copies issued)
    auto advance_copy = [&]() {
        ++gl;
        if (++l_k < KT) return false;
        l_k = 0;
        ++l_item;
        copy_live = l_item < count;
        const Item it = item_of(copy_live ? l_item : 0);
        nxt = it;
        if (copy_live) set_src(it);
        else set_src_zeros();
        copy_params(it, l_item & 1, copy_live);
        return true;
    };

    // ---- operand fetch addresses: [K half s][low / high chunk], byte offsets inside a stage
    const unsigned lds0 = lds_addr(lds);
    const unsigned a_row = lds0 + wave_m * (MT * 4096) + (lane & 31) * 128;
    const unsigned b_row = lds0 + BM * 128 + wave_n * 8192 + (lane & 31) * 128;
    unsigned pc[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        pc[s][0] = ((4 * s + 2 * (lane >> 5)) ^ (((lane & 31) >> 1) & 7)) * 16;
        pc[s][1] = pc[s][0] ^ 16;
    }
    auto read_half = [&](PipeFragsT<MT>& f, int stage, int s) {
        const unsigned so = (stage & 1) * kPipeStageBytes;
        pipe_read_frags<MT>(f, a_row + so + pc[s][0], a_row + so + pc[s][1], b_row + so + pc[s][0], b_row + so + pc[s][1]);
    };
    auto read_part = [&](PipeFragsT<MT>& f, int stage, int s, auto part) {  // one of the four parts of read_half
        const unsigned so = (stage & 1) * kPipeStageBytes;
        pipe_read_frags_part<MT, decltype(part)::value>(f, a_row + so + pc[s][0], a_row + so + pc[s][1], b_row + so + pc[s][0], b_row + so + pc[s][1]);
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    using P3 = std::integral_constant<int, 3>;

    using acc_t = typename std::conditional<IN == Q8_I8, v16i, v16f>::type;
    acc_t acc[MT][2];

    // ---- prologue: stage 0 landed, stage 1 in flight, fragments of the first K half on their way
    Item cur = item_of(0);
    set_src(cur);
    copy_params(cur, 0, true);
#pragma unroll
    for (int i = 0; i < NCOPY; ++i) issue_copy(i);
    advance_copy();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < NCOPY; ++i) issue_copy(i);
    advance_copy();
    PipeFragsT<MT> f0, f1;
    read_half(f0, 0, 0);

    int g = 0;  // compute side: global stage count
    for (int item = 0; item < count; ++item) {
        // One K stage. FIRST (the first stage of a tile, peeled off the loop below) starts the accumulators from a
        // constant zero in its first K half instead of clearing them beforehand.
        auto stage = [&](auto first_tag, const bool last) {
            constexpr bool FIRST = decltype(first_tag)::value;
            // f0: first K half of stage g (reads in flight); the copies of stage g+1 are in flight
            pipe_wait_frags(f0);
            pipe_pin(f0);
            // First half. The operand reads of the second half go out a part after each of the first MFMAs, not as one
            // burst: a wave that issues a dozen LDS reads back to back keeps the matrix pipe waiting, and its partner on
            // the SIMD does the same at the same time. Once the second half of stage g is in registers everywhere
            // (barrier 1), buffer g & 1 is free and the copies of stage g+2 start to trickle out, one per MFMA tile.
            pipe_mfma<IN, MT, FIRST>(f0, acc, [&](int j) {
                if (j == 0) read_part(f1, g, 1, P0{});
                if (j == 1) {
                    read_part(f1, g, 1, P1{});
                    if constexpr (MT == 3) read_part(f1, g, 1, P2{});
                }
                if (MT == 4 && j == 2) {
                    read_part(f1, g, 1, P2{});
                    read_part(f1, g, 1, P3{});
                }
                if (j == MT - 1) {
                    pipe_wait_frags(f1);
                    __builtin_amdgcn_s_barrier();
                }
                if (j >= MT) issue_copy(j - MT);
            });
            __builtin_amdgcn_sched_barrier(0);
            pipe_pin(f1);
            // Second half. After the last copy of stage g+2 everything older (stage g+1, and the stores of the
            // previous epilogue) must have completed; barrier 2 makes that true for every wave's copies, then the
            // first half of stage g+1 is fetched under the remaining MFMA tiles (after the epilogue at a tile's end).
            bool moved = false;
            pipe_mfma<IN, MT>(f1, acc, [&](int j) {
                if (j < 4) issue_copy(MT + j);
                if (j == 3) moved = advance_copy();
                if (j == 4) {
                    if (moved) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NCOPY + 2) : "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NCOPY) : "memory");
                    __builtin_amdgcn_s_barrier();
                    // the fragment registers are free for the epilogue after the last stage of a tile; the reads of the
                    // next stage's first half are spread over the remaining MFMA slots like those above
                    if (!last) {
                        read_part(f0, g + 1, 0, P0{});
                        if constexpr (MT == 3) read_part(f0, g + 1, 0, P1{});
                    }
                }
                if (!last && j == 5) {
                    if constexpr (MT == 4) read_part(f0, g + 1, 0, P1{});
                    else read_part(f0, g + 1, 0, P2{});
                }
                if (!last && MT == 4 && j == 6) {
                    read_part(f0, g + 1, 0, P2{});
                    read_part(f0, g + 1, 0, P3{});
                }
            });
            __builtin_amdgcn_sched_barrier(0);
            ++g;
        };
        stage(std::true_type{}, false);  // K > 256: never the last stage
        for (int k = 1; k < KT; ++k) stage(std::false_type{}, k == KT - 1);

        // ---- epilogue of tile `item`: lane (r32, h) holds for MFMA tile (i, t) and register octet wp the 8 columns
        //      32 t + 16 wp + 8 h .. + 7 of the wave's 64-column slab, row 32 i + r32.
        // (the lane id passes through an empty asm so that none of the address arithmetic below is hoisted out of
        //  the tile loop, where it would take registers away from the main loop)
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const int r32 = lane_e & 31, h = lane_e >> 5;
        const unsigned stage_out = lds0 + kPersistStageOutOffset + wave * 2048;
        const unsigned par = lds0 + kPersistParOffset + (item & 1) * kPersistParBytes;
        const size_t zc = (size_t)cur.z * M * N;
        const int mw0 = cur.m0 + wave_m * (32 * MT), nw0 = cur.n0 + wave_n * 64;
        v4i sbq[2][2][2], bq[2][2][2];  // [t][wp][low / high 4 columns]
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int wp = 0; wp < 2; ++wp) {
                const unsigned o = (wave_n * 64 + 32 * t + 16 * wp + 8 * h) * 4;
                sbq[t][wp][0] = lds_read_b128<1024>(par + o);
                sbq[t][wp][1] = lds_read_b128<1024 + 16>(par + o);
                bq[t][wp][0] = lds_read_b128<2048>(par + o);
                bq[t][wp][1] = lds_read_b128<2048 + 16>(par + o);
            }
        float sam[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) sam[i] = lds_read_b32(par + (wave_m * (32 * MT) + 32 * (i < MT ? i : 0) + r32) * 4);
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(sam[0]), "+v"(sam[1]), "+v"(sam[2]), "+v"(sam[3]), "+v"(sbq[0][0][0]), "+v"(sbq[0][0][1]),
                       "+v"(sbq[0][1][0]), "+v"(sbq[0][1][1]), "+v"(sbq[1][0][0]), "+v"(sbq[1][0][1]), "+v"(sbq[1][1][0]),
                       "+v"(sbq[1][1][1]), "+v"(bq[0][0][0]), "+v"(bq[0][0][1]), "+v"(bq[0][1][0]), "+v"(bq[0][1][1]),
                       "+v"(bq[1][0][0]), "+v"(bq[1][0][1]), "+v"(bq[1][1][0]), "+v"(bq[1][1][1])
                     :
                     : "memory");
        const bool rows16 = (N & 15) == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;  // e4m3 output: rows start 16-byte aligned
        (void)rows16;
        const int ldc = VSPLIT != 0 ? p.v_col0 : N;  // columns per row of C
        const bool vtile = VSPLIT != 0 && cur.n0 >= p.v_col0;  // uniform: this tile holds V columns
        (void)vtile;
        uint16_t* const cbase = reinterpret_cast<uint16_t*>(p.C) + (VSPLIT != 0 ? (size_t)cur.z * M * ldc : zc);
        const uint16_t* const rbase = reinterpret_cast<const uint16_t*>(p.residual) + zc;
        v4i gq = v4i{0, 0, 0, 0};  // the gate of the 8 columns this lane stores (RES with p.gate)
        if constexpr (RES) {
            if (p.gate != nullptr) {
                gq = lds_read_b128<3072>(par + (wave_n * 64 + (lane_e & 7) * 8) * 2);
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(gq) : : "memory");
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            // the residual rows this lane will store in the four rounds of this MFMA tile: fetched now, used after the
            // arithmetic below
            v4u res[2][2];
            if constexpr (RES) {
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int m = mw0 + 32 * i + 16 * half + 8 * j + (lane_e >> 3);
                        const int n = nw0 + (lane_e & 7) * 8;
                        res[half][j] = (m < M && n < N) ? *reinterpret_cast<const v4u*>(rbase + (size_t)m * N + n) : v4u{0u, 0u, 0u, 0u};
                    }
            }
            // the lane's 4 chunks of row 32 i + r32: chunk c = 4 t + 2 wp + h
            v4u outc[2][2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                uint32_t e8[2][2];  // e4m3 output: [wp][low / high 4 codes]
                (void)e8;
#pragma unroll
                for (int wp = 0; wp < 2; ++wp) {
                    float v[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float sbv = __int_as_float(sbq[t][wp][e >> 2][e & 3]);
                        const float bv = __int_as_float(bq[t][wp][e >> 2][e & 3]);
                        float x = fmaf((float)acc[i][t][8 * wp + e], sam[i] * sbv, bv);
                        if constexpr (GELU) x = gelu_tanh_fast(x);
                        v[e] = x;
                    }
                    if constexpr (E4M3OUT) {
                        // 8 codes of row 32 i + r32, columns 32 t + 16 wp + 8 h .. + 7 of the slab
                        e8[wp][0] = pack4_e4m3_sat(v[0], v[1], v[2], v[3]);
                        e8[wp][1] = pack4_e4m3_sat(v[4], v[5], v[6], v[7]);
                    } else {
                        outc[t][wp] = v4u{pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]), pack2_bf16(v[4], v[5]), pack2_bf16(v[6], v[7])};
                    }
                }
                if constexpr (VSPLIT == 1) {
                    if (vtile) {
                        // the wave's 64-column slab is one head: codes of the bf16-rounded results, the two lanes of a row
                        // swap a chunk as below and store 16 bytes each of the (token, head) row
#pragma unroll
                        for (int wp = 0; wp < 2; ++wp) {
                            float f[8];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                f[2 * e] = __uint_as_float(outc[t][wp][e] << 16);
                                f[2 * e + 1] = __uint_as_float(outc[t][wp][e] & 0xffff0000u);
                            }
                            e8[wp][0] = pack4_e4m3_c10(f[0], f[1], f[2], f[3]);
                            e8[wp][1] = pack4_e4m3_c10(f[4], f[5], f[6], f[7]);
                        }
                        const auto s0 = __builtin_amdgcn_permlane32_swap(e8[0][0], e8[1][0], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(e8[0][1], e8[1][1], false, false);
                        const int m = mw0 + 32 * i + r32, n = nw0 + 32 * t + 16 * h;
                        if (m < M && n < N) {
                            const int bb = m / p.v_tokens, ss = m - bb * p.v_tokens, head = (nw0 - p.v_col0) >> 6;
                            uint8_t* dst = p.v_codes + (((size_t)cur.z * (M / p.v_tokens) + bb) * p.v_heads + head) * (size_t)p.v_tokens * 64 +
                                           (size_t)ss * 64 + 32 * t + 16 * h;
                            *reinterpret_cast<v4u*>(dst) = v4u{s0[0], s1[0], s0[1], s1[1]};
                        }
                    }
                }
                if constexpr (E4M3OUT) {
                    // the two lanes of a row exchange one 8-byte chunk each (v_permlane32_swap: the upper half of the first
                    // operand against the lower half of the second): lane half 0 then holds columns 32 t .. + 15, lane
                    // half 1 columns 32 t + 16 .. + 31, 16 bytes per lane and 32 contiguous bytes per row and instruction
                    // (only when every row starts on a 16-byte boundary, N % 16 == 0 and C aligned - uniform; otherwise each
                    //  lane stores its two 8-byte chunks where they are)
                    const int m = mw0 + 32 * i + r32;
                    uint8_t* const row = reinterpret_cast<uint8_t*>(p.C) + zc + (size_t)m * N;
                    if (rows16) {
                        const auto s0 = __builtin_amdgcn_permlane32_swap(e8[0][0], e8[1][0], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(e8[0][1], e8[1][1], false, false);
                        const int n = nw0 + 32 * t + 16 * h;
                        if (m < M && n < N) *reinterpret_cast<v4u*>(row + n) = v4u{s0[0], s1[0], s0[1], s1[1]};
                    } else {
#pragma unroll
                        for (int wp = 0; wp < 2; ++wp) {
                            const int n = nw0 + 32 * t + 16 * wp + 8 * h;
                            if (m < M && n < N) *reinterpret_cast<v2i*>(row + n) = v2i{(int)e8[wp][0], (int)e8[wp][1]};
                        }
                    }
                }
            }
            if constexpr (VSPLIT == 2) {
                if (vtile) {
                    // Column c = 32 t + 16 wp + 8 h + e of the head: the butterflies run over the bits of c from the lowest
                    // up, as the row kernels' transform does (registers e, the lane half h, registers wp and t), every
                    // stage the plain (a + b, a - b), so signed zeros come out as there too.
                    float x[2][2][8];
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int wp = 0; wp < 2; ++wp) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                x[t][wp][2 * e] = __uint_as_float(outc[t][wp][e] << 16);
                                x[t][wp][2 * e + 1] = __uint_as_float(outc[t][wp][e] & 0xffff0000u);
                            }
#pragma unroll
                            for (int sft = 1; sft < 8; sft <<= 1)
#pragma unroll
                                for (int e = 0; e < 8; ++e)
                                    if ((e & sft) == 0) {
                                        const float a = x[t][wp][e], b = x[t][wp][e + sft];
                                        x[t][wp][e] = a + b;
                                        x[t][wp][e + sft] = a - b;
                                    }
                            // lane halves: after the swap of two copies every lane holds the lower half's value (a) and
                            // the upper half's (b); the lower half keeps a + b, the upper a - b
                            const float sgn = h ? -1.0f : 1.0f;
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x[t][wp][e]), __float_as_uint(x[t][wp][e]), false, false);
                                x[t][wp][e] = __builtin_fmaf(__uint_as_float(r[1]), sgn, __uint_as_float(r[0]));
                            }
                        }
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float a = x[t][0][e], b = x[t][1][e];
                            x[t][0][e] = a + b;
                            x[t][1][e] = a - b;
                        }
                    const int m = mw0 + 32 * i + r32;
                    const int bb = m / p.v_tokens, ss = m - bb * p.v_tokens, head = (nw0 - p.v_col0) >> 6;
                    uint8_t* const dst = p.v_codes + (((size_t)cur.z * (M / p.v_tokens) + bb) * p.v_heads + head) * (size_t)p.v_tokens * 64 +
                                         (size_t)ss * 64 + 16 * h;
                    uint32_t e8[2][2][2];
#pragma unroll
                    for (int wp = 0; wp < 2; ++wp) {
                        float y[2][8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float a = x[0][wp][e], b = x[1][wp][e];
                            y[0][e] = (a + b) * p.v_fht_scale;
                            y[1][e] = (a - b) * p.v_fht_scale;
                        }
#pragma unroll
                        for (int t = 0; t < 2; ++t) {
                            e8[t][wp][0] = pack4_e4m3_c10(y[t][0], y[t][1], y[t][2], y[t][3]);
                            e8[t][wp][1] = pack4_e4m3_c10(y[t][4], y[t][5], y[t][6], y[t][7]);
                        }
                    }
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const auto s0 = __builtin_amdgcn_permlane32_swap(e8[t][0][0], e8[t][1][0], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(e8[t][0][1], e8[t][1][1], false, false);
                        if (m < M && nw0 + 32 * t + 16 * h < N) *reinterpret_cast<v4u*>(dst + 32 * t) = v4u{s0[0], s1[0], s0[1], s1[1]};
                    }
                }
            }
            if constexpr (VSPLIT != 0) {
                if (vtile) continue;
            }
            if constexpr (E4M3OUT) {
                continue;
            } else if constexpr (GELU && !RES) {
                // With GELU the epilogue is bound by its arithmetic, and the round trips through the staging buffer
                // below only add latency to it: the lane's four 16-byte chunks of row 32 i + r32 go straight to
                // memory, 32 contiguous bytes per row and instruction (the four instructions complete the row's
                // 128-byte line within a few hundred cycles, so the L2 merges them). Measured 2.5-3.3 % faster per
                // launch than the staged form on the GELU shapes and 1-4 % slower without GELU, where the stores
                // are what the epilogue waits for and whole lines per instruction pay off.
                const int m = mw0 + 32 * i + r32;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int wp = 0; wp < 2; ++wp) {
                        const int n = nw0 + 32 * t + 16 * wp + 8 * h;
                        if (m < M && n < N) *reinterpret_cast<v4u*>(cbase + (size_t)m * ldc + n) = outc[t][wp];
                    }
            } else {
            // rows 16 half .. 16 half + 15 of the MFMA tile: their lanes write, then all lanes read 16 full rows. The
            // two rounds use the same 2 KiB and are issued back to back without a wait in between: a wave's LDS
            // instructions execute in order, so the reads of a round see its writes and the writes of the second
            // round come after the reads of the first. Only the stores wait, for the data they send.
            v4i w[2][2];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if ((r32 >> 4) == half) {
                    const int row = r32 & 15;
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int wp = 0; wp < 2; ++wp)
                            lds_write_b128(stage_out + row * 128 + (((4 * t + 2 * wp + h) ^ ((row >> 1) & 7)) * 16), outc[t][wp]);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int row = 8 * j + (lane_e >> 3);
                    w[half][j] = lds_read_b128<0>(stage_out + row * 128 + (((lane_e & 7) ^ ((row >> 1) & 7)) * 16));
                }
            }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if (half == 0) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(w[0][0]), "+v"(w[0][1]) : : "memory");
                else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(w[1][0]), "+v"(w[1][1]) : : "memory");
                if constexpr (RES) {
                    if (p.gate != nullptr) {
#pragma unroll
                        for (int j = 0; j < 2; ++j)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint32_t a = (uint32_t)w[half][j][e], r = res[half][j][e], gg = (uint32_t)gq[e];
                                w[half][j][e] = (int)pack2_bf16(
                                    __builtin_fmaf(__uint_as_float(a << 16), __uint_as_float(gg << 16), __uint_as_float(r << 16)),
                                    __builtin_fmaf(__uint_as_float(a & 0xffff0000u), __uint_as_float(gg & 0xffff0000u),
                                                   __uint_as_float(r & 0xffff0000u)));
                            }
                    } else {
#pragma unroll
                        for (int j = 0; j < 2; ++j)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint32_t a = (uint32_t)w[half][j][e], r = res[half][j][e];
                                w[half][j][e] = (int)pack2_bf16(__uint_as_float(a << 16) + __uint_as_float(r << 16),
                                                                __uint_as_float(a & 0xffff0000u) + __uint_as_float(r & 0xffff0000u));
                            }
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int m = mw0 + 32 * i + 16 * half + 8 * j + (lane_e >> 3);
                    const int n = nw0 + (lane_e & 7) * 8;
                    if (m < M && n < N) *reinterpret_cast<v4i*>(cbase + (size_t)m * ldc + n) = w[half][j];
                }
            }
            }
        }
        cur = nxt;  // the copy side entered tile item + 1 two stages before this tile's last one (K > 256: and no further tile yet)
        read_half(f0, g, 0);  // first fragments of the next tile (its first two stages landed before barrier 2 above)
    }
    // drain: the look-ahead copies and fragment reads past the last stage target LDS / registers that nobody uses
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    pipe_wait_frags(f0);
}

}  // namespace q8
