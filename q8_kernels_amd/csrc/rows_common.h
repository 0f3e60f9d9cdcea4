// Shared pieces of the row kernels: the thread-to-element mapping, reductions over the threads of a row, the
// Hadamard butterfly stages, the quantizer's code/scale arithmetic and the dispatch on the padded row length.
//
// Row mapping: a row of `dim` elements is padded to N = 8 * LANES * CH (a power of two). LANES consecutive
// threads own a row, thread t of the row holds the elements (c * LANES + t) * 8 + 0..7 for c = 0..CH-1, i.e.
// one 128-bit bf16 load per chunk. A block is 256 threads = 256 / LANES rows. Element-index bits therefore
// map, low to high, to (register index, lane, wave, chunk), which is also the order in which the Hadamard
// butterflies run, so that every output is produced by the same sequence of fp32 additions as the
// ascending-stride butterfly network of the reference
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

// ---- Hadamard butterfly stages ------------------------------------------------------------------

// One butterfly stage across lanes l and l ^ MASK: y[l] = x[l] + x[l ^ MASK] in the lane with the bit clear,
// x[l ^ MASK] - x[l] in the lane with the bit set (the same two roundings as the sequential butterfly).
//
// MASK 1, 2: the own value gets its sign flipped where the bit is set (one xor), then one add whose first
//            operand comes through a DPP quad permutation.
// MASK 4, 8: the lanes with the bit clear and the lanes with the bit set are whole DPP banks, so an add and a
//            subtract with complementary bank masks do the stage in two instructions.
// MASK 16, 32: two registers a, b at a time: a lane-half swap brings (a[l], a[l ^ MASK]) of the lower halves
//            and (b[l], b[l ^ MASK]) of the upper halves into the same lanes, sum and difference are formed
//            there, and a second swap puts them back. Four instructions per two values, no selects.
template <int MASK>
__device__ __forceinline__ void fht_lane_stage(float (&v)[8], unsigned sign_if_set) {
    if constexpr (MASK == 1 || MASK == 2) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float own = __uint_as_float(__float_as_uint(v[i]) ^ sign_if_set);
            const int o = __builtin_amdgcn_mov_dpp(__float_as_int(v[i]), MASK == 1 ? 0xB1 : 0x4E, 0xf, 0xf, true);
            v[i] = __int_as_float(o) + own;
        }
    } else if constexpr (MASK == 4) {
        float y[8];
        // 2 wait states between a VALU write of a VGPR and a DPP read of it
        asm volatile(
            "s_nop 1\n"
            "v_add_f32_dpp %0, %8, %8 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %1, %9, %9 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %2, %10, %10 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %3, %11, %11 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %4, %12, %12 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %5, %13, %13 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %6, %14, %14 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_add_f32_dpp %7, %15, %15 row_shl:4 row_mask:0xf bank_mask:0x5\n"
            "v_sub_f32_dpp %0, %8, %8 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %1, %9, %9 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %2, %10, %10 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %3, %11, %11 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %4, %12, %12 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %5, %13, %13 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %6, %14, %14 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            "v_sub_f32_dpp %7, %15, %15 row_shr:4 row_mask:0xf bank_mask:0xa\n"
            : "=&v"(y[0]), "=&v"(y[1]), "=&v"(y[2]), "=&v"(y[3]), "=&v"(y[4]), "=&v"(y[5]), "=&v"(y[6]), "=&v"(y[7])
            : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = y[i];
    } else if constexpr (MASK == 8) {
        float y[8];
        asm volatile(
            "s_nop 1\n"
            "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %4, %12, %12 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %5, %13, %13 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %6, %14, %14 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_add_f32_dpp %7, %15, %15 row_ror:8 row_mask:0xf bank_mask:0x3\n"
            "v_sub_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %4, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %5, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %6, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            "v_sub_f32_dpp %7, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n"
            : "=&v"(y[0]), "=&v"(y[1]), "=&v"(y[2]), "=&v"(y[3]), "=&v"(y[4]), "=&v"(y[5]), "=&v"(y[6]), "=&v"(y[7])
            : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = y[i];
    } else {
        static_assert(MASK == 16 || MASK == 32, "fht_lane_stage: mask must be 1..32");
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const unsigned a = __float_as_uint(v[i]), b = __float_as_uint(v[i + 1]);
            // r[0] = a in the lanes with the bit clear, b[l ^ MASK] in the others; r[1] = a[l ^ MASK] | b
            const auto r = (MASK == 16) ? __builtin_amdgcn_permlane16_swap(a, b, false, false)
                                        : __builtin_amdgcn_permlane32_swap(a, b, false, false);
            const float lo = __uint_as_float(r[0]), hi = __uint_as_float(r[1]);
            const float sum = lo + hi, dif = lo - hi;
            const auto w = (MASK == 16)
                               ? __builtin_amdgcn_permlane16_swap(__float_as_uint(sum), __float_as_uint(dif), false, false)
                               : __builtin_amdgcn_permlane32_swap(__float_as_uint(sum), __float_as_uint(dif), false, false);
            v[i] = __uint_as_float(w[0]);
            v[i + 1] = __uint_as_float(w[1]);
        }
    }
}


// All butterfly stages of one row held in registers as v[CH][8] (thread t of the row, element index
// (c * LANES + t) * 8 + i): registers, lanes, waves (one exchange through LDS), chunks, in this order.
template <int LANES, int CH>
__device__ __forceinline__ void fht_row(float (&v)[CH][8], int t) {
    // element bits 0..2: inside the 8 registers of a chunk
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
        for (int s = 1; s < 8; s <<= 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if ((i & s) == 0) {
                    const float a = v[c][i], b = v[c][i + s];
                    v[c][i] = a + b;
                    v[c][i + s] = a - b;
                }
            }
        }
    }
    // lane bits
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if constexpr (LANES > 1) fht_lane_stage<1>(v[c], (unsigned)(t & 1) << 31);
        if constexpr (LANES > 2) fht_lane_stage<2>(v[c], (unsigned)(t & 2) << 30);
        if constexpr (LANES > 4) fht_lane_stage<4>(v[c], 0u);
        if constexpr (LANES > 8) fht_lane_stage<8>(v[c], 0u);
        if constexpr (LANES > 16) fht_lane_stage<16>(v[c], 0u);
        if constexpr (LANES > 32) fht_lane_stage<32>(v[c], 0u);
    }
    // wave bits: one exchange through LDS per chunk, both stages evaluated from the 2 or 4 wave values
    if constexpr (LANES > 64) {
        __shared__ v4f xch[2][kBlock];
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
        const unsigned m1 = (unsigned)(wave & 1) << 31, m2 = (unsigned)(wave & 2) << 30;
        auto flip = [](float x, unsigned m) { return __uint_as_float(__float_as_uint(x) ^ m); };
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            xch[0][threadIdx.x] = v4f{v[c][0], v[c][1], v[c][2], v[c][3]};
            xch[1][threadIdx.x] = v4f{v[c][4], v[c][5], v[c][6], v[c][7]};
            __syncthreads();
            auto peer = [&](int w, float (&o)[8]) {
                const v4f a = xch[0][w * 64 + lane], b = xch[1][w * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
            };
            float p1[8];
            peer(wave ^ 1, p1);
            if constexpr (LANES == 128) {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[c][i] = p1[i] + flip(v[c][i], m1);
            } else {
                float p2[8], p3[8];
                peer(wave ^ 2, p2);
                peer(wave ^ 3, p3);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float ya = p1[i] + flip(v[c][i], m1);
                    const float yb = p3[i] + flip(p2[i], m1);
                    v[c][i] = yb + flip(ya, m2);
                }
            }
            __syncthreads();
        }
    }
    // chunk bits
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
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float q = v[i] * ratio;
            if (flags & Q8_QUANT_RNE) {
                qi[i] = (int)rintf(q);
            } else {
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
    if (rows < 0) return fail(Q8_ERR_SHAPE, "%s: rows = %lld", who, (long long)rows);
    if (dim <= 0 || dim % 8 != 0 || dim > 32768)
        return fail(Q8_ERR_SHAPE, "%s: dim = %d must be a multiple of 8 in [8, 32768]", who, dim);
    return Q8_OK;
}

}  // namespace q8
