// Shared pieces of the row kernels: the thread-to-element mapping, reductions over the threads of a row, the
// Hadamard butterfly stages, the quantizer's code/scale arithmetic and the dispatch on the padded row length.
//
// Row mapping: a row of `dim` elements is padded to N = 8 * LANES * CH (a power of two). LANES consecutive
// threads own a row, thread t of the row holds the elements (c * LANES + t) * 8 + 0..7 for c = 0..CH-1, i.e.
// one 128-bit bf16 load per chunk; t is the thread's index in the row, or in the kernels that run a Hadamard
// transform a permutation of it inside groups of 16 lanes (row_thread). A block is 256 threads = 256 / LANES rows.
// Element-index bits therefore map, low to high, to (register index, thread, chunk), which is also the order in
// which the Hadamard butterflies run, so that every output is produced by the same sequence of fp32 additions as
// the ascending-stride butterfly network of the reference
// (csrc/fast_hadamard/fast_hadamard_transform_cuda.cu:84-108).
//
// fp contraction is off in every file that includes this header: products and sums round separately, like
// the element-wise fp32 arithmetic they are checked against.
#pragma once
#include "q8_common.h"
#include "q8_host.h"

#pragma clang fp contract(off)

namespace q8 {


constexpr int kBlock = 256;

// ---- reductions over the LANES threads of a row (LANES <= 256) -------------------------------

// v[r], r < RPT: one value per row this thread works on; red: RPT * 4 floats of LDS
template <int LANES, bool IS_MAX, int RPT>
__device__ __forceinline__ void row_reduce(float (&v)[RPT], float* red) {
    constexpr int WL = LANES < 64 ? LANES : 64;
#pragma unroll
    for (int r = 0; r < RPT; ++r) v[r] = IS_MAX ? group_max<WL>(v[r]) : group_sum<WL>(v[r]);
    if constexpr (LANES > 64) {
        constexpr int WPR = LANES / 64;  // waves per row
        const int wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) {
#pragma unroll
            for (int r = 0; r < RPT; ++r) red[r * 4 + wave] = v[r];
        }
        __syncthreads();
        const int w0 = (wave / WPR) * WPR;
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            float x = red[r * 4 + w0];
#pragma unroll
            for (int i = 1; i < WPR; ++i) x = IS_MAX ? fmaxf(x, red[r * 4 + w0 + i]) : (x + red[r * 4 + w0 + i]);
            v[r] = x;
        }
        __syncthreads();
    }
}

// ---- token-wise quantizer -----------------------------------------------------------------------

// Rows per thread group: several rows are loaded before the first reduction so that more bytes are in flight
// per thread (one 16-byte load per thread does not cover the HBM latency at 2048 threads per CU).
template <int LANES, int CH>
struct RowsPerThread { static constexpr int value = (CH == 1) ? 4 : (CH == 2 ? 2 : 1); };

// ---- loading a row ----------------------------------------------------------------------------------

// v[c] = the 8 elements (c * LANES + t) * 8 + 0..7 of the row at xr as fp32, zeros beyond dim or when the row does
// not exist. `full` (uniform over the block: every row of the block exists and dim == 8 * LANES * CH) selects a
// branch-free path on which all CH loads of a thread are issued back to back; the guarded path waits for each
// load inside its own branch. NZ: also returns whether this thread read anything but zeros (of either sign).
template <int IN, int LANES, int CH, bool NZ = false>
__device__ __forceinline__ bool load_row(const void* xr, int t, bool row_ok, int dim, bool full, float (&v)[CH][8]) {
    unsigned raw_or = 0;
    auto ld = [&](int e, float (&o)[8]) {
        if constexpr (NZ) load8<IN>(xr, e, o, raw_or); else load8<IN>(xr, e, o);
    };
    if (full) {
#pragma unroll
        for (int c = 0; c < CH; ++c) ld((c * LANES + t) * 8, v[c]);
    } else {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int e = (c * LANES + t) * 8;
            if (row_ok && e < dim) {
                ld(e, v[c]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
            }
        }
    }
    if constexpr (NZ) return (raw_or & sign_clear_mask<IN>()) != 0;
    else return true;
}

// ---- Hadamard butterfly stages ------------------------------------------------------------------
//
// A butterfly stage over lane bit k replaces x by x + x[partner] in the thread whose element bit is clear and by
// x[partner] - x in the thread whose bit is set. Here every such stage is ONE fused multiply-add per value,
//     x <- x + s * x[partner],   s = +1 (bit clear) or -1 (bit set), a per-thread constant,
// which is the exact sum (one rounding, like the addition) in the first kind of thread and the exact NEGATIVE of
// the wanted difference in the second. The sign is not repaired stage by stage: negation commutes with every
// later addition and rounding, so a thread simply carries all of its values with the sign
// (-1)^popcount(thread bits processed), and the multiplication by the transform's scale that ends every
// transform here takes that sign along (fht_row's last step). The only trace is the sign of exact zeros, which
// that last step fixes to +0. The sequential network returns a zero other than +0 only when every input of the
// transform is a zero (x + y = -0 needs x = y = -0 and x - y = -0 needs x = -0, y = +0, so a -0 has only zeros
// beneath it): rows of zeros are detected before the transform and take the plain form of every stage
// (fht_*_exact: partner + (own with its sign flipped where the bit is set), the reference's own additions), so
// the signs of their zeros are the reference's too.
//
// The partner value arrives through the DPP operand of the multiply-add for thread bits 0..3 and through the
// LDS crossbar (ds_swizzle / ds_bpermute, no LDS memory) for bits 4 and 5. DPP has no "lane ^ 4" or "lane ^ 8"
// pattern but it has mirrors: row_half_mirror pairs lane l with l ^ 7 and row_mirror with l ^ 15. The threads of
// a row therefore own the 16-byte chunks of 16 lanes in a permuted order (row_thread): chunk bits
// (e0, e1, e2, e3) = (l0 ^ l2, l1 ^ l2, l2 ^ l3, l3) of lane bits l0..l3, under which flipping l0 flips e0 only,
// l1 -> e1, half mirror -> e2 only and full mirror -> e3 only. 16 lanes still read and write the same 256
// contiguous bytes; reductions over the lanes of a row pair the same elements as without the permutation.

// position of this thread among the LANES threads of its row (the "t" of the row mapping)
template <int LANES>
__device__ __forceinline__ int row_thread() {
    const int l = threadIdx.x, p = l & 15;
    const int e = p ^ (((p >> 2) & 1) * 3) ^ (((p >> 3) & 1) << 2);
    return ((l & ~15) | e) & (LANES - 1);
}

// +1.0f or -1.0f: the factor s of the stage over thread bit `bit`
__device__ __forceinline__ float fht_stage_sign(int t, int bit) {
    return __uint_as_float(0x3f800000u | ((unsigned)((t >> bit) & 1) << 31));
}

#define Q8_FHT_DPP8(CTRL)                                                                                        \
    asm volatile("s_nop 1\n" /* 2 wait states between a VALU write of a VGPR and a DPP read of it */             \
                 "v_fmac_f32_dpp %0, %0, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %1, %1, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %2, %2, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %3, %3, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %4, %4, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %5, %5, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %6, %6, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 "v_fmac_f32_dpp %7, %7, %8 " CTRL " row_mask:0xf bank_mask:0xf\n"                               \
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]) \
                 : "v"(s))

// one stage over thread bit log2(MASK) for the 8 values of a chunk; s = fht_stage_sign of that bit
template <int MASK>
__device__ __forceinline__ void fht_lane_stage(float (&v)[8], float s) {
    if constexpr (MASK == 1) {
        Q8_FHT_DPP8("quad_perm:[1,0,3,2]");
    } else if constexpr (MASK == 2) {
        Q8_FHT_DPP8("quad_perm:[2,3,0,1]");
    } else if constexpr (MASK == 4) {
        Q8_FHT_DPP8("row_half_mirror");
    } else if constexpr (MASK == 8) {
        Q8_FHT_DPP8("row_mirror");
    } else {
        static_assert(MASK == 16 || MASK == 32, "fht_lane_stage: mask must be 1..32");
        int p[8];
        if constexpr (MASK == 16) {
#pragma unroll
            for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_ds_swizzle(__float_as_int(v[i]), 0x401F);  // lane ^ 16
        } else {
            const int peer = (int)((threadIdx.x & 63) ^ 32) * 4;
#pragma unroll
            for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_ds_bpermute(peer, __float_as_int(v[i]));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(__int_as_float(p[i]), s, v[i]);
    }
}

// the register stages (element bits 0..2) of one chunk
__device__ __forceinline__ void fht_chunk_stages(float (&v)[8]) {
#pragma unroll
    for (int s = 1; s < 8; s <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((i & s) == 0) {
                const float a = v[i], b = v[i + s];
                v[i] = a + b;
                v[i + s] = a - b;
            }
        }
    }
}

// whether any of the values is not a zero (of either sign)
template <int NV>
__device__ __forceinline__ bool any_nonzero(const float (&v)[NV]) {
    unsigned acc = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) acc |= __float_as_uint(v[i]);
    return (acc & 0x7fffffffu) != 0;
}

// nz: whether this thread holds a non-zero value. True when some group of LANES threads handled by this wave
// (LANES <= 64; a group of inactive lanes counts) or some wave of this block (LANES > 64, with one barrier: every
// thread of the block must call it, and the answer is uniform over the block) holds only zeros.
template <int LANES>
__device__ __forceinline__ bool fht_zero_group(bool nz) {
    unsigned long long m = __ballot(nz);
    if constexpr (LANES > 64) {
        __shared__ int wave_zero[kBlock / 64];
        if ((threadIdx.x & 63) == 0) wave_zero[threadIdx.x >> 6] = (m == 0);
        __syncthreads();
        const v4i z = *reinterpret_cast<const v4i*>(wave_zero);
        return ((z[0] | z[1]) | (z[2] | z[3])) != 0;
    } else if constexpr (LANES == 64) {
        return m == 0;
    } else {
#pragma unroll
        for (int s = 1; s < LANES; s <<= 1) m |= m >> s;  // bit g * LANES = "group g has a non-zero"
        constexpr unsigned long long low = LANES == 1 ? ~0ull : LANES == 2 ? 0x5555555555555555ull
                                         : LANES == 4 ? 0x1111111111111111ull : LANES == 8 ? 0x0101010101010101ull
                                         : LANES == 16 ? 0x0001000100010001ull : 0x0000000100000001ull;
        return (~m & low) != 0;
    }
}

// plain form of the stage over thread bit BIT: y = x[partner] + (bit set ? -x : x)
template <int BIT>
__device__ __forceinline__ void fht_lane_stage_exact(float (&v)[8], int t) {
    constexpr int pm = BIT == 0 ? 1 : BIT == 1 ? 2 : BIT == 2 ? 7 : BIT == 3 ? 15 : BIT == 4 ? 16 : 32;
    const int peer = (int)((threadIdx.x & 63) ^ pm) * 4;
    const unsigned m = (unsigned)((t >> BIT) & 1) << 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float p = __int_as_float(__builtin_amdgcn_ds_bpermute(peer, __float_as_int(v[i])));
        v[i] = p + __uint_as_float(__float_as_uint(v[i]) ^ m);
    }
}

// D-point transform of the 8 * LH elements of a head held by LH threads (t = row_thread), times scale
template <int LH>
__device__ __forceinline__ void fht_head(float (&v)[8], int t, float scale) {
    const bool zeros = fht_zero_group<LH>(any_nonzero(v));
    fht_chunk_stages(v);
    if (zeros) {
        if constexpr (LH > 1) fht_lane_stage_exact<0>(v, t);
        if constexpr (LH > 2) fht_lane_stage_exact<1>(v, t);
        if constexpr (LH > 4) fht_lane_stage_exact<2>(v, t);
        if constexpr (LH > 8) fht_lane_stage_exact<3>(v, t);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] *= scale;
    } else {
        if constexpr (LH > 1) fht_lane_stage<1>(v, fht_stage_sign(t, 0));
        if constexpr (LH > 2) fht_lane_stage<2>(v, fht_stage_sign(t, 1));
        if constexpr (LH > 4) fht_lane_stage<4>(v, fht_stage_sign(t, 2));
        if constexpr (LH > 8) fht_lane_stage<8>(v, fht_stage_sign(t, 3));
        const float ss = (__builtin_popcount(t & (LH - 1)) & 1) ? -scale : scale;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(v[i], ss, 0.f);
    }
}

// the chunk stages (element bits above the thread bits)
template <int CH>
__device__ __forceinline__ void fht_upper_stages(float (&v)[CH][8]) {
#pragma unroll
    for (int s = 1; s < CH; s <<= 1) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            if ((c & s) == 0) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float a = v[c][i], b = v[c + s][i];
                    v[c][i] = a + b;
                    v[c + s][i] = a - b;
                }
            }
        }
    }
}

// exchange buffer of the wave stages: two halves used by alternate chunks, each [2][kBlock] 16-byte slots
__device__ __forceinline__ v4f* fht_exchange_buffer() {
    __shared__ v4f xch[2 * 2 * kBlock];
    return xch;
}

// the stages over the wave bits of the thread index (LANES = 128, 256): one exchange through LDS per chunk, both
// stages evaluated from the 2 or 4 wave values. One barrier per chunk: chunk c + 1 writes the other half of the
// buffer, and the half of chunk c is written again only behind the barrier of chunk c + 1, which no wave passes
// before every wave has read chunk c. FMA: the one-instruction form with the carried sign.
template <int LANES, int CH, bool FMA>
__device__ __forceinline__ void fht_wave_stages(float (&v)[CH][8], int t) {
    v4f* const xch = fht_exchange_buffer();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const float s6 = fht_stage_sign(t, 6), s7 = fht_stage_sign(t, 7);
    // y = b + (a with the sign of s): a + b or b - a
    auto stage = [](float a, float s, float b) {
        if constexpr (FMA) return __builtin_fmaf(b, s, a);  // a + s b
        else return b + __uint_as_float(__float_as_uint(a) ^ (__float_as_uint(s) & 0x80000000u));
    };
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        v4f* const x0 = xch + (c & 1) * 2 * kBlock;
        v4f* const x1 = x0 + kBlock;
        x0[threadIdx.x] = v4f{v[c][0], v[c][1], v[c][2], v[c][3]};
        x1[threadIdx.x] = v4f{v[c][4], v[c][5], v[c][6], v[c][7]};
        __syncthreads();
        auto peer = [&](int w, float (&o)[8]) {
            const v4f a = x0[w * 64 + lane], b = x1[w * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
        };
        float p1[8];
        peer(wave ^ 1, p1);
        if constexpr (LANES == 128) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = stage(v[c][i], s6, p1[i]);
        } else {
            float p2[8], p3[8];
            peer(wave ^ 2, p2);
            peer(wave ^ 3, p3);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float ya = stage(v[c][i], s6, p1[i]);  // this wave's value after the first stage
                const float yb = stage(p2[i], s6, p3[i]);    // wave ^ 2's
                v[c][i] = stage(ya, s7, yb);
            }
        }
    }
    __syncthreads();  // the buffer may be written again by a later call
}

// All butterfly stages of one row held in registers as v[CH][8] (thread t = row_thread<LANES>() of the row,
// element index (c * LANES + t) * 8 + i): registers, lanes, waves, chunks, in this order, then the
// multiplication by `scale`. zeros = fht_zero_group<LANES>(...) of the values in v: selects the plain stage forms.
// Contains barriers when LANES > 64: every thread of the block must call it.
template <int LANES, int CH>
__device__ __forceinline__ void fht_row(float (&v)[CH][8], int t, float scale, bool zeros) {
#pragma unroll
    for (int c = 0; c < CH; ++c) fht_chunk_stages(v[c]);
    if (zeros) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            if constexpr (LANES > 1) fht_lane_stage_exact<0>(v[c], t);
            if constexpr (LANES > 2) fht_lane_stage_exact<1>(v[c], t);
            if constexpr (LANES > 4) fht_lane_stage_exact<2>(v[c], t);
            if constexpr (LANES > 8) fht_lane_stage_exact<3>(v[c], t);
            if constexpr (LANES > 16) fht_lane_stage_exact<4>(v[c], t);
            if constexpr (LANES > 32) fht_lane_stage_exact<5>(v[c], t);
        }
        if constexpr (LANES > 64) fht_wave_stages<LANES, CH, false>(v, t);
        fht_upper_stages<CH>(v);
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] *= scale;
        return;
    }
    const float s0 = fht_stage_sign(t, 0), s1 = fht_stage_sign(t, 1), s2 = fht_stage_sign(t, 2),
                s3 = fht_stage_sign(t, 3), s4 = fht_stage_sign(t, 4), s5 = fht_stage_sign(t, 5);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if constexpr (LANES > 1) fht_lane_stage<1>(v[c], s0);
        if constexpr (LANES > 2) fht_lane_stage<2>(v[c], s1);
        if constexpr (LANES > 4) fht_lane_stage<4>(v[c], s2);
        if constexpr (LANES > 8) fht_lane_stage<8>(v[c], s3);
    }
    // the two stages through the LDS crossbar, all chunks of a stage together so that many exchanges are in flight
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if constexpr (LANES > 16) fht_lane_stage<16>(v[c], s4);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if constexpr (LANES > 32) fht_lane_stage<32>(v[c], s5);
    }
    if constexpr (LANES > 64) fht_wave_stages<LANES, CH, true>(v, t);
    fht_upper_stages<CH>(v);
    // scale, the carried sign, and +0 for exact zeros (a product of -0 plus +0 is +0)
    const float ss = (__builtin_popcount(t) & 1) ? -scale : scale;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) v[c][i] = __builtin_fmaf(v[c][i], ss, 0.f);
}

// ---- 8-element chunks with a run-time element type (uniform switch) ------------------------------------

__device__ __forceinline__ void load8_any(const void* p, int dt, int64_t e, float (&v)[8]) {
    switch (dt) {
        case Q8_BF16: load8<Q8_BF16>(p, e, v); break;
        case Q8_F32: load8<Q8_F32>(p, e, v); break;
        default: load8<Q8_E4M3>(p, e, v); break;
    }
}
__device__ __forceinline__ void store8_any(void* p, int dt, int64_t e, const float (&v)[8]) {
    if (dt == Q8_BF16) store8<Q8_BF16>(p, e, v); else store8<Q8_E4M3>(p, e, v);
}

// ---- quantizer arithmetic -------------------------------------------------------------------------

// value an intermediate tensor of dtype MID would hold (round trip through its storage format)
template <int MID>
__device__ __forceinline__ float round_mid(float x) {
    if constexpr (MID == Q8_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
    else return x;
}
// the same for 8 values at once: four hardware pair conversions and their unpacking (bf16), or the c10 e4m3 cast
// and its decoding
template <int MID>
__device__ __forceinline__ void round_mid8(float (&v)[8]) {
    if constexpr (MID == Q8_E4M3) {
        const int w0 = (int)pack4_e4m3_c10(v[0], v[1], v[2], v[3]), w1 = (int)pack4_e4m3_c10(v[4], v[5], v[6], v[7]);
        v[0] = e4m3_to_f32<0>(w0); v[1] = e4m3_to_f32<1>(w0); v[2] = e4m3_to_f32<2>(w0); v[3] = e4m3_to_f32<3>(w0);
        v[4] = e4m3_to_f32<0>(w1); v[5] = e4m3_to_f32<1>(w1); v[6] = e4m3_to_f32<2>(w1); v[7] = e4m3_to_f32<3>(w1);
    } else if constexpr (MID == Q8_BF16) {
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const uint32_t u = pack2_bf16(v[i], v[i + 1]);
            v[i] = __uint_as_float(u << 16);
            v[i + 1] = __uint_as_float(u & 0xffff0000u);
        }
    }
}

// reference order: r = QMAX / absmax, code = x * r, stored scale = 1 / r
// (csrc/quantizer/tokenwise_quant_cuda.cu:135-147), in IEEE fp32; a row of zeros gets codes 0 and scale 0.
template <int OUT>
__device__ __forceinline__ float quant_ratio(float amax) {
    constexpr float QMAX = (OUT == Q8_I8) ? 127.f : 448.f;
    return (amax > 0.f) ? QMAX / amax : 0.f;
}
template <int OUT>
__device__ __forceinline__ float quant_scale(float amax, float ratio, int flags) {
    constexpr float QMAX = (OUT == Q8_I8) ? 127.f : 448.f;
    if (!(amax > 0.f)) return 0.f;
    return (flags & Q8_QUANT_SCALE_DIV) ? amax / QMAX : 1.0f / ratio;
}
// 8 codes of one chunk
template <int OUT>
__device__ __forceinline__ v2i quant_codes8(const float (&v)[8], float ratio, int flags) {
    v2i w;
    if constexpr (OUT == Q8_I8) {
        // |q| <= 127 (1 + 2^-23). Round half away from zero = truncate(q + copysign(0.5 - 2^-25, q)) for every
        // fp32 |q| < 2^22 (the sum rounds up to the next integer exactly for the ties and for nothing below them);
        // round half even = v_rndne. Two saturating 32->16 packs and one byte permute gather the 4 codes of a word.
        int qi[8];
        if (flags & Q8_QUANT_RNE) {  // uniform
#pragma unroll
            for (int i = 0; i < 8; ++i) qi[i] = (int)rintf(v[i] * ratio);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float q = v[i] * ratio;
                const float half = __uint_as_float(0x3effffffu | (__float_as_uint(q) & 0x80000000u));
                qi[i] = (int)(q + half);  // the conversion truncates
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            typedef short v2s __attribute__((ext_vector_type(2)));
            const v2s p0 = __builtin_amdgcn_cvt_pk_i16(qi[4 * j], qi[4 * j + 1]);
            const v2s p1 = __builtin_amdgcn_cvt_pk_i16(qi[4 * j + 2], qi[4 * j + 3]);
            uint32_t u0, u1;
            __builtin_memcpy(&u0, &p0, 4);
            __builtin_memcpy(&u1, &p1, 4);
            w[j] = (int)__builtin_amdgcn_perm(u1, u0, 0x06040200u);  // bytes 0 and 2 of u0, then of u1
        }
    } else {
        // |x * r| <= 448 (1 + 2^-23): never reaches the NaN range of the c10 cast
        uint32_t p0 = cvt_pk_e4m3(v[0] * ratio, v[1] * ratio, 0u, false);
        p0 = cvt_pk_e4m3(v[2] * ratio, v[3] * ratio, p0, true);
        uint32_t p1 = cvt_pk_e4m3(v[4] * ratio, v[5] * ratio, 0u, false);
        p1 = cvt_pk_e4m3(v[6] * ratio, v[7] * ratio, p1, true);
        w[0] = (int)p0;
        w[1] = (int)p1;
    }
    return w;
}

// the codes of a row to out (the row's first byte); full: as in load_row, no guards
template <int OUT, int LANES, int CH>
__device__ __forceinline__ void store_codes_row(uint8_t* out, int t, int dim, bool full, const float (&v)[CH][8],
                                                float ratio, int flags) {
    if (full) {
#pragma unroll
        for (int c = 0; c < CH; ++c)
            *reinterpret_cast<v2i*>(out + (c * LANES + t) * 8) = quant_codes8<OUT>(v[c], ratio, flags);
    } else {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int e = (c * LANES + t) * 8;
            if (e < dim) *reinterpret_cast<v2i*>(out + e) = quant_codes8<OUT>(v[c], ratio, flags);
        }
    }
}

// ---- dispatch ------------------------------------------------------------------------------------

// N = padded row length (power of two, 8..32768). Up to N = 4096 a row stays inside one wave (reductions and
// butterflies need neither LDS nor barriers, and CH independent 16-byte loads per thread are in flight);
// longer rows spread over 2 or 4 waves.
#define Q8_ROW_SHAPE_SWITCH(N, ...)                                                       \
    switch (N) {                                                                          \
        case 8:     { constexpr int LANES = 1,   CH = 1;  __VA_ARGS__; } break;           \
        case 16:    { constexpr int LANES = 2,   CH = 1;  __VA_ARGS__; } break;           \
        case 32:    { constexpr int LANES = 4,   CH = 1;  __VA_ARGS__; } break;           \
        case 64:    { constexpr int LANES = 8,   CH = 1;  __VA_ARGS__; } break;           \
        case 128:   { constexpr int LANES = 16,  CH = 1;  __VA_ARGS__; } break;           \
        case 256:   { constexpr int LANES = 32,  CH = 1;  __VA_ARGS__; } break;           \
        case 512:   { constexpr int LANES = 64,  CH = 1;  __VA_ARGS__; } break;           \
        case 1024:  { constexpr int LANES = 64,  CH = 2;  __VA_ARGS__; } break;           \
        case 2048:  { constexpr int LANES = 64,  CH = 4;  __VA_ARGS__; } break;           \
        case 4096:  { constexpr int LANES = 64,  CH = 8;  __VA_ARGS__; } break;           \
        case 8192:  { constexpr int LANES = 128, CH = 8;  __VA_ARGS__; } break;           \
        case 16384: { constexpr int LANES = 256, CH = 8;  __VA_ARGS__; } break;           \
        case 32768: { constexpr int LANES = 256, CH = 16; __VA_ARGS__; } break;           \
        default: return fail(Q8_ERR_SHAPE, "row length %d not supported", (int)(N));      \
    }

inline int pow2_ceil(int d) {
    int n = 8;
    while (n < d) n <<= 1;
    return n;
}

inline int check_rows(const char* who, int64_t rows, int dim) {
    // (2^40 rows bound every rows * dim product and every rounded-up row count far below the range of int64)
    if (rows < 0 || rows > ((int64_t)1 << 40)) return fail(Q8_ERR_SHAPE, "%s: rows = %lld", who, (long long)rows);
    if (dim <= 0 || dim % 8 != 0 || dim > 32768)
        return fail(Q8_ERR_SHAPE, "%s: dim = %d must be a multiple of 8 in [8, 32768]", who, dim);
    return Q8_OK;
}

}  // namespace q8
