// Shared device helpers for the gfx950 kernels: element conversions with the exact rounding
// rules of the reference's stores, wave64 cross-lane exchanges, 128-bit row loads and stores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/q8_hip.h"

namespace q8 {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------- conversions

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16, round to nearest even, NaN -> 0x7fc0: the c10::BFloat16 constructor used by every
// `out_vals_store[i] = out_vals[i]` in the reference (e.g. csrc/ops/rms_norm_cuda.cu:60-66).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return ((u & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : r;
}

// Two fp32 -> packed bf16 pair with the hardware converter (v_cvt_pk_bf16_f32, round to nearest even).
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// e4m3fn -> fp32 of byte `SEL` of a packed word (v_cvt_f32_fp8, OCP format on gfx950).
template <int SEL>
__device__ __forceinline__ float e4m3_to_f32(uint32_t packed) {
    return __builtin_amdgcn_cvt_f32_fp8((int)packed, SEL);
}

// a register with unspecified contents (no instruction): the `old` operand of a conversion whose other half is written next
// (used where the instruction count is the bound, the attention tile loop; elsewhere the fence of the volatile statement
//  costs the scheduler more than the move it saves)
__device__ __forceinline__ uint32_t any_u32() {
    uint32_t u;
    asm volatile("" : "=v"(u));
    return u;
}

// Two fp32 -> two e4m3fn codes in the low or high half of a word, hardware RNE.
__device__ __forceinline__ uint32_t cvt_pk_e4m3(float a, float b, uint32_t old, bool hi) {
    return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}

// c10::Float8_e4m3fn(float) semantics: RNE, |v| > 464 (and NaN) -> 0x7f with the sign bit kept.
// This is the cast of the reference's quantizer / FHT / RMSNorm / RoPE stores
// (e.g. csrc/fast_hadamard/fast_hadamard_transform_common.h:146-161).
__device__ __forceinline__ uint32_t e4m3_overflow_fix(uint32_t code, float v) {
    uint32_t u = __float_as_uint(v);
    return ((u & 0x7fffffffu) > 0x43e80000u) ? (0x7fu | ((u >> 24) & 0x80u)) : code;
}

__device__ __forceinline__ uint32_t pack4_e4m3_c10(float a, float b, float c, float d) {
    uint32_t p = cvt_pk_e4m3(a, b, 0u, false);
    p = cvt_pk_e4m3(c, d, p, true);
    // Up to |v| = 464 the hardware conversion IS the c10 cast; only larger magnitudes and NaN need the code patched in.
    // One maximum of the four magnitudes and two unordered comparisons say whether any value of any lane is such a one,
    // and only then the wave runs the per-byte repair below (same codes either way).
    const float m = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(a), __builtin_fabsf(b)), __builtin_fmaxf(__builtin_fabsf(c), __builtin_fabsf(d)));
    const bool rare = !(m <= 464.f) || __builtin_isunordered(a, b) || __builtin_isunordered(c, d);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(rare) == 0, 1)) return p;
    uint32_t b0 = e4m3_overflow_fix(p & 0xffu, a);
    uint32_t b1 = e4m3_overflow_fix((p >> 8) & 0xffu, b);
    uint32_t b2 = e4m3_overflow_fix((p >> 16) & 0xffu, c);
    uint32_t b3 = e4m3_overflow_fix((p >> 24) & 0xffu, d);
    return b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
}

// Saturating-finite cast (__NV_SATFINITE of the reference's GEMM epilogue and attention stores,
// csrc/gemm/fp8_matmul_bias.cu:42-52): clamp to +-448, NaN stays NaN.
__device__ __forceinline__ float clamp448(float v) {
    v = (v > 448.f) ? 448.f : v;
    v = (v < -448.f) ? -448.f : v;
    return v;
}
__device__ __forceinline__ uint32_t pack4_e4m3_sat(float a, float b, float c, float d) {
    // One v_med3_f32 per value clamps everything that is not NaN (a NaN would come out as -448); two unordered
    // comparisons say whether any of the four values of any lane is NaN, and only then the wave takes the form that
    // keeps NaN (compare-and-select clamps, 0x7f patched over the code). Same codes as that form for every input.
    const bool any_nan = __builtin_isunordered(a, b) || __builtin_isunordered(c, d);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(any_nan) != 0, 0)) {
        uint32_t p = cvt_pk_e4m3(clamp448(a), clamp448(b), 0u, false);
        p = cvt_pk_e4m3(clamp448(c), clamp448(d), p, true);
        uint32_t m = 0u;
        m |= (a != a) ? 0x0000007fu : 0u;
        m |= (b != b) ? 0x00007f00u : 0u;
        m |= (c != c) ? 0x007f0000u : 0u;
        m |= (d != d) ? 0x7f000000u : 0u;
        return p | m;
    }
    uint32_t p = cvt_pk_e4m3(__builtin_amdgcn_fmed3f(a, -448.f, 448.f), __builtin_amdgcn_fmed3f(b, -448.f, 448.f), 0u, false);
    return cvt_pk_e4m3(__builtin_amdgcn_fmed3f(c, -448.f, 448.f), __builtin_amdgcn_fmed3f(d, -448.f, 448.f), p, true);
}

// ---------------------------------------------------------------- cross-lane exchange (wave64)

// Value held by lane (lane ^ MASK), MASK a power of two below 64. DPP / permlane only: no LDS traffic.
template <int MASK>
__device__ __forceinline__ float lane_xor(float x) {
    int xi = __float_as_int(x);
    if constexpr (MASK == 1) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
    } else if constexpr (MASK == 2) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
    } else if constexpr (MASK == 4) {
        int t = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xf, 0xf, true);                 // row_half_mirror: i^7
        return __int_as_float(__builtin_amdgcn_mov_dpp(t, 0x1B, 0xf, 0xf, true));    // quad_perm [3,2,1,0]: ^3
    } else if constexpr (MASK == 8) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0x128, 0xf, 0xf, true));  // row_ror:8
    } else if constexpr (MASK == 16) {
        auto r = __builtin_amdgcn_permlane16_swap((unsigned)xi, (unsigned)xi, false, false);
        return __int_as_float((int)((threadIdx.x & 16) ? r[0] : r[1]));
    } else {
        static_assert(MASK == 32, "lane_xor: mask must be 1..32");
        auto r = __builtin_amdgcn_permlane32_swap((unsigned)xi, (unsigned)xi, false, false);
        return __int_as_float((int)((threadIdx.x & 32) ? r[0] : r[1]));
    }
}

// IEEE-754 maximum (NaN-propagating; v_maximum3_f32 on gfx950). Unlike fmaxf it needs no canonicalization of operands the
// compiler cannot prove free of signalling NaNs (MFMA results, lane swaps): one instruction per two new values.
__device__ __forceinline__ float max_ieee(float a, float b) { return __builtin_elementwise_maximum(a, b); }
// max of a value over the two lanes l, l ^ 32: v_permlane32_swap of two copies leaves (low half, low half) in one and
// (high half, high half) in the other, so every lane holds both values and no select is needed
__device__ __forceinline__ float half_pair_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return max_ieee(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
template <int LANES>
__device__ __forceinline__ float group_max(float v) {
    if constexpr (LANES > 1) v = fmaxf(v, lane_xor<1>(v));
    if constexpr (LANES > 2) v = fmaxf(v, lane_xor<2>(v));
    if constexpr (LANES > 4) v = fmaxf(v, lane_xor<4>(v));
    if constexpr (LANES > 8) v = fmaxf(v, lane_xor<8>(v));
    if constexpr (LANES > 16) v = fmaxf(v, lane_xor<16>(v));
    if constexpr (LANES > 32) v = fmaxf(v, lane_xor<32>(v));
    return v;
}
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LANES > 1) v += lane_xor<1>(v);
    if constexpr (LANES > 2) v += lane_xor<2>(v);
    if constexpr (LANES > 4) v += lane_xor<4>(v);
    if constexpr (LANES > 8) v += lane_xor<8>(v);
    if constexpr (LANES > 16) v += lane_xor<16>(v);
    if constexpr (LANES > 32) v += lane_xor<32>(v);
    return v;
}

// ---------------------------------------------------------------- LDS access with explicit waits

// ds_read_b128 as inline assembly: invisible to the compiler's wait-count insertion, which would otherwise put
// a full s_waitcnt vmcnt(0) in front of every LDS read that follows a global_load_lds. The caller must execute
// an s_waitcnt lgkmcnt that names the result as an operand (lds_wait) before using it.
template <int OFFSET>
__device__ __forceinline__ v4i lds_read_b128(unsigned addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET) : "memory");
    return r;
}

// LDS byte address of a pointer into __shared__ memory
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// ---------------------------------------------------------------- 8-element row chunks

// Load 8 consecutive elements of `DT` starting at element index `e` of row pointer `p` into fp32.
template <int DT>
__device__ __forceinline__ void load8(const void* p, int64_t e, float (&v)[8]) {
    if constexpr (DT == Q8_BF16) {
        v4u w = *reinterpret_cast<const v4u*>(reinterpret_cast<const uint16_t*>(p) + e);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    } else if constexpr (DT == Q8_F16) {
        v4u w = *reinterpret_cast<const v4u*>(reinterpret_cast<const uint16_t*>(p) + e);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = f16_bits_to_f32(w[i] & 0xffffu);
            v[2 * i + 1] = f16_bits_to_f32(w[i] >> 16);
        }
    } else if constexpr (DT == Q8_F32) {
        const v4f* q = reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(p) + e);
        v4f a = q[0], b = q[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
    } else {
        static_assert(DT == Q8_E4M3, "load8: unsupported element type");
        v2i w = *reinterpret_cast<const v2i*>(reinterpret_cast<const uint8_t*>(p) + e);
        v[0] = e4m3_to_f32<0>(w[0]); v[1] = e4m3_to_f32<1>(w[0]);
        v[2] = e4m3_to_f32<2>(w[0]); v[3] = e4m3_to_f32<3>(w[0]);
        v[4] = e4m3_to_f32<0>(w[1]); v[5] = e4m3_to_f32<1>(w[1]);
        v[6] = e4m3_to_f32<2>(w[1]); v[7] = e4m3_to_f32<3>(w[1]);
    }
}

// The same, and the OR of the raw words read is accumulated into raw_or (BF16, E4M3): all of the 8 elements are
// zeros of either sign exactly when (raw_or & sign_clear_mask<DT>()) == 0.
template <int DT>
__device__ __forceinline__ void load8(const void* p, int64_t e, float (&v)[8], unsigned& raw_or) {
    if constexpr (DT == Q8_BF16) {
        v4u w = *reinterpret_cast<const v4u*>(reinterpret_cast<const uint16_t*>(p) + e);
        raw_or |= (w[0] | w[1]) | (w[2] | w[3]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    } else {
        static_assert(DT == Q8_E4M3, "load8 with raw_or: unsupported element type");
        v2i w = *reinterpret_cast<const v2i*>(reinterpret_cast<const uint8_t*>(p) + e);
        raw_or |= (unsigned)(w[0] | w[1]);
        v[0] = e4m3_to_f32<0>(w[0]); v[1] = e4m3_to_f32<1>(w[0]);
        v[2] = e4m3_to_f32<2>(w[0]); v[3] = e4m3_to_f32<3>(w[0]);
        v[4] = e4m3_to_f32<0>(w[1]); v[5] = e4m3_to_f32<1>(w[1]);
        v[6] = e4m3_to_f32<2>(w[1]); v[7] = e4m3_to_f32<3>(w[1]);
    }
}
template <int DT>
__device__ __forceinline__ constexpr unsigned sign_clear_mask() { return DT == Q8_BF16 ? 0x7fff7fffu : 0x7f7f7f7fu; }

// Store 8 fp32 values as `DT` (BF16: RNE; E4M3: c10 cast) at element index `e`.
template <int DT>
__device__ __forceinline__ void store8(void* p, int64_t e, const float (&v)[8]) {
    if constexpr (DT == Q8_BF16) {
        v4u w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack2_bf16(v[2 * i], v[2 * i + 1]);
        *reinterpret_cast<v4u*>(reinterpret_cast<uint16_t*>(p) + e) = w;
    } else {
        static_assert(DT == Q8_E4M3, "store8: unsupported element type");
        v2i w;
        w[0] = (int)pack4_e4m3_c10(v[0], v[1], v[2], v[3]);
        w[1] = (int)pack4_e4m3_c10(v[4], v[5], v[6], v[7]);
        *reinterpret_cast<v2i*>(reinterpret_cast<uint8_t*>(p) + e) = w;
    }
}

}  // namespace q8
