// Memory-bound row kernels for gfx950: token-wise absmax quantizer, fast Walsh-Hadamard transform,
// RMSNorm and RoPE.
//
// Row mapping shared by the three reducing kernels: a row of `dim` elements is padded to
// N = 8 * LANES * CH (a power of two). LANES consecutive threads own a row, thread t of the row holds
// the elements (c * LANES + t) * 8 + 0..7 for c = 0..CH-1, i.e. one 128-bit bf16 load per chunk.
// A block is 256 threads = 256 / LANES rows. Element-index bits therefore map, low to high, to
// (register index, lane, wave, chunk), which is also the order in which the Hadamard butterflies
// run, so that every output is produced by the same sequence of fp32 additions as the ascending-stride
// butterfly network of the reference (csrc/fast_hadamard/fast_hadamard_transform_cuda.cu:84-108).
//
// fp contraction is off in this file: products and sums round separately, like the element-wise fp32
// arithmetic they are checked against.
#include "q8_common.h"
#include "q8_host.h"

#pragma clang fp contract(off)

namespace q8 {

constexpr int kBlock = 256;

// ---- reductions over the LANES threads of a row (LANES <= 256) -------------------------------

template <int LANES, bool IS_MAX>
__device__ __forceinline__ float row_reduce(float v, float* red) {
    constexpr int WL = LANES < 64 ? LANES : 64;
    v = IS_MAX ? group_max<WL>(v) : group_sum<WL>(v);
    if constexpr (LANES > 64) {
        constexpr int WPR = LANES / 64;  // waves per row
        const int wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) red[wave] = v;
        __syncthreads();
        const int w0 = (wave / WPR) * WPR;
        float r = red[w0];
#pragma unroll
        for (int i = 1; i < WPR; ++i) r = IS_MAX ? fmaxf(r, red[w0 + i]) : (r + red[w0 + i]);
        __syncthreads();
        v = r;
    }
    return v;
}

// ---- token-wise quantizer -----------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void quant_rows_kernel(const void* __restrict__ x, void* __restrict__ codes,
                                                            float* __restrict__ scales, int64_t rows, int dim,
                                                            int64_t x_row_stride, int flags) {
    constexpr int RPB = kBlock / LANES;
    __shared__ float red[4];
    const int t = threadIdx.x % LANES;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * x_row_stride * (IN == Q8_F32 ? 4 : (IN == Q8_E4M3 ? 1 : 2));

    float v[CH][8];
    float amax = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (row_ok && e < dim) {
            load8<IN>(xr, e, v[c]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[c][i]));
    }
    amax = row_reduce<LANES, true>(amax, red);

    constexpr float QMAX = (OUT == Q8_I8) ? 127.f : 448.f;
    // reference order: r = QMAX / absmax, code = x * r, stored scale = 1 / r
    // (csrc/quantizer/tokenwise_quant_cuda.cu:135-147), in IEEE fp32.
    const float r = (amax > 0.f) ? QMAX / amax : 0.f;
    if (row_ok && t == 0) {
        float s = 0.f;
        if (amax > 0.f) s = (flags & Q8_QUANT_SCALE_DIV) ? amax / QMAX : 1.0f / r;
        scales[row] = s;
    }
    if (!row_ok) return;
    uint8_t* out = reinterpret_cast<uint8_t*>(codes) + row * (int64_t)dim;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;
        v2i w;
        if constexpr (OUT == Q8_I8) {
            uint32_t b[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float q = v[c][i] * r;
                const float qr = (flags & Q8_QUANT_RNE) ? rintf(q) : roundf(q);
                b[i] = (uint32_t)(int)qr & 0xffu;
            }
            w[0] = (int)(b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24));
            w[1] = (int)(b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
        } else {
            // |x * r| <= 448 (1 + 2^-23): never reaches the NaN range of the c10 cast
            uint32_t p0 = cvt_pk_e4m3(v[c][0] * r, v[c][1] * r, 0u, false);
            p0 = cvt_pk_e4m3(v[c][2] * r, v[c][3] * r, p0, true);
            uint32_t p1 = cvt_pk_e4m3(v[c][4] * r, v[c][5] * r, 0u, false);
            p1 = cvt_pk_e4m3(v[c][6] * r, v[c][7] * r, p1, true);
            w[0] = (int)p0;
            w[1] = (int)p1;
        }
        *reinterpret_cast<v2i*>(out + e) = w;
    }
}

// ---- fast Walsh-Hadamard transform --------------------------------------------------------------

template <int MASK>
__device__ __forceinline__ void fht_lane_stage(float (&v)[8], int lane_bit_set) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float o = lane_xor<MASK>(v[i]);
        v[i] = lane_bit_set ? (o - v[i]) : (v[i] + o);
    }
}

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void fht_kernel(const void* __restrict__ x, void* __restrict__ y, int64_t rows,
                                                     int dim, float scale) {
    constexpr int RPB = kBlock / LANES;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    constexpr int OUT_B = (OUT == Q8_E4M3) ? 1 : 2;
    const int t = threadIdx.x % LANES;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * IN_B;

    float v[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (row_ok && e < dim) {
            load8<IN>(xr, e, v[c]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
        }
    }

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
        if constexpr (LANES > 1) fht_lane_stage<1>(v[c], t & 1);
        if constexpr (LANES > 2) fht_lane_stage<2>(v[c], t & 2);
        if constexpr (LANES > 4) fht_lane_stage<4>(v[c], t & 4);
        if constexpr (LANES > 8) fht_lane_stage<8>(v[c], t & 8);
        if constexpr (LANES > 16) fht_lane_stage<16>(v[c], t & 16);
        if constexpr (LANES > 32) fht_lane_stage<32>(v[c], t & 32);
    }
    // wave bits: one exchange through LDS per chunk, both stages evaluated from the 2 or 4 wave values
    if constexpr (LANES > 64) {
        __shared__ v4f xch[2][kBlock];
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
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
                for (int i = 0; i < 8; ++i) v[c][i] = (wave & 1) ? (p1[i] - v[c][i]) : (v[c][i] + p1[i]);
            } else {
                float p2[8], p3[8];
                peer(wave ^ 2, p2);
                peer(wave ^ 3, p3);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float ya = (wave & 1) ? (p1[i] - v[c][i]) : (v[c][i] + p1[i]);
                    const float yb = (wave & 1) ? (p3[i] - p2[i]) : (p2[i] + p3[i]);
                    v[c][i] = (wave & 2) ? (yb - ya) : (ya + yb);
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

    if (!row_ok) return;
    char* yr = reinterpret_cast<char*>(y) + row * (int64_t)dim * OUT_B;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[c][i] *= scale;
        store8<OUT>(yr, e, v[c]);
    }
}

// ---- RMSNorm ---------------------------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void rmsnorm_kernel(const void* __restrict__ x, const float* __restrict__ w,
                                                         void* __restrict__ y, float* __restrict__ rstd_out,
                                                         int64_t rows, int dim, float eps) {
    constexpr int RPB = kBlock / LANES;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    constexpr int OUT_B = (OUT == Q8_E4M3) ? 1 : 2;
    __shared__ float red[4];
    const int t = threadIdx.x % LANES;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * IN_B;

    float v[CH][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (row_ok && e < dim) {
            load8<IN>(xr, e, v[c]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += v[c][i] * v[c][i];
    }
    ss = row_reduce<LANES, false>(ss, red);
    // rstd = rsqrt(mean(x^2)) with no epsilon in the reference (csrc/ops/rms_norm_cuda.cu:127-156)
    const float rstd = 1.0f / sqrtf(ss * (1.0f / (float)dim) + eps);
    if (!row_ok) return;
    if (rstd_out != nullptr && t == 0) rstd_out[row] = rstd;
    char* yr = reinterpret_cast<char*>(y) + row * (int64_t)dim * OUT_B;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;
        if (w != nullptr) {
            float wv[8];
            load8<Q8_F32>(w, e, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = (v[c][i] * rstd) * wv[i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = v[c][i] * rstd;
        }
        store8<OUT>(yr, e, v[c]);
    }
}

// ---- RoPE ------------------------------------------------------------------------------------------

template <int IN, int OUT>
__global__ __launch_bounds__(kBlock) void rope_kernel(const void* __restrict__ x, const float* __restrict__ cs,
                                                      const float* __restrict__ sn, void* __restrict__ y,
                                                      int64_t nchunks) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    const int64_t e = idx * 8;
    float xv[8], c[8], s[8], o[8];
    load8<IN>(x, e, xv);
    load8<Q8_F32>(cs, e, c);
    load8<Q8_F32>(sn, e, s);
    // interleaved pairs, per-element tables (csrc/ops/rope_cuda.cu:99-103)
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
        o[i] = xv[i] * c[i] - xv[i + 1] * s[i];
        o[i + 1] = xv[i + 1] * c[i + 1] + xv[i] * s[i + 1];
    }
    store8<OUT>(y, e, o);
}

// ---- dispatch ------------------------------------------------------------------------------------

// N = padded row length (power of two, 8..32768): LANES = min(N / 8, 256), CH = N / (8 * LANES).
#define Q8_ROW_SHAPE_SWITCH(N, ...)                                                       \
    switch (N) {                                                                          \
        case 8:     { constexpr int LANES = 1,   CH = 1;  __VA_ARGS__; } break;           \
        case 16:    { constexpr int LANES = 2,   CH = 1;  __VA_ARGS__; } break;           \
        case 32:    { constexpr int LANES = 4,   CH = 1;  __VA_ARGS__; } break;           \
        case 64:    { constexpr int LANES = 8,   CH = 1;  __VA_ARGS__; } break;           \
        case 128:   { constexpr int LANES = 16,  CH = 1;  __VA_ARGS__; } break;           \
        case 256:   { constexpr int LANES = 32,  CH = 1;  __VA_ARGS__; } break;           \
        case 512:   { constexpr int LANES = 64,  CH = 1;  __VA_ARGS__; } break;           \
        case 1024:  { constexpr int LANES = 128, CH = 1;  __VA_ARGS__; } break;           \
        case 2048:  { constexpr int LANES = 256, CH = 1;  __VA_ARGS__; } break;           \
        case 4096:  { constexpr int LANES = 256, CH = 2;  __VA_ARGS__; } break;           \
        case 8192:  { constexpr int LANES = 256, CH = 4;  __VA_ARGS__; } break;           \
        case 16384: { constexpr int LANES = 256, CH = 8;  __VA_ARGS__; } break;           \
        case 32768: { constexpr int LANES = 256, CH = 16; __VA_ARGS__; } break;           \
        default: return fail(Q8_ERR_SHAPE, "row length %d not supported", (int)(N));      \
    }

static int pow2_ceil(int d) {
    int n = 8;
    while (n < d) n <<= 1;
    return n;
}

static int check_rows(const char* who, int64_t rows, int dim) {
    if (rows < 0) return fail(Q8_ERR_SHAPE, "%s: rows = %lld", who, (long long)rows);
    if (dim <= 0 || dim % 8 != 0 || dim > 32768)
        return fail(Q8_ERR_SHAPE, "%s: dim = %d must be a multiple of 8 in [8, 32768]", who, dim);
    return Q8_OK;
}

}  // namespace q8

using namespace q8;

extern "C" int q8_quant_rows(const void* x, int x_dtype, void* codes, int code_dtype, float* scales, int64_t rows,
                             int dim, int64_t x_row_stride, int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_quant_rows", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (!x || !codes || !scales) return fail(Q8_ERR_NULL, "q8_quant_rows: null pointer");
    if (flags & ~(Q8_QUANT_RNE | Q8_QUANT_SCALE_DIV)) return fail(Q8_ERR_FLAGS, "q8_quant_rows: flags 0x%x", flags);
    if (code_dtype != Q8_I8 && code_dtype != Q8_E4M3)
        return fail(Q8_ERR_DTYPE, "q8_quant_rows: code dtype %d (want I8 or E4M3)", code_dtype);
    const int esz = elem_size(x_dtype);
    if (esz == 0 || x_dtype == Q8_I8) return fail(Q8_ERR_DTYPE, "q8_quant_rows: input dtype %d", x_dtype);
    if (x_row_stride < dim) return fail(Q8_ERR_SHAPE, "q8_quant_rows: row stride %lld < dim %d", (long long)x_row_stride, dim);
    const int need = (x_dtype == Q8_E4M3) ? 8 : 16;
    if ((reinterpret_cast<uintptr_t>(x) % need) || ((x_row_stride * esz) % need) || (reinterpret_cast<uintptr_t>(codes) % 8) ||
        (reinterpret_cast<uintptr_t>(scales) % 4))
        return fail(Q8_ERR_ALIGN, "q8_quant_rows: x rows must be %d-byte aligned, codes 8-byte aligned", need);
    const int N = pow2_ceil(dim);
#define LAUNCH_Q(IN, OUT)                                                                              \
    Q8_ROW_SHAPE_SWITCH(N, {                                                                           \
        const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);                         \
        hipLaunchKernelGGL((quant_rows_kernel<LANES, CH, IN, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, \
                           codes, scales, rows, dim, x_row_stride, flags);                             \
    })
#define LAUNCH_Q_IN(OUT)                                         \
    switch (x_dtype) {                                           \
        case Q8_BF16: LAUNCH_Q(Q8_BF16, OUT); break;             \
        case Q8_F16: LAUNCH_Q(Q8_F16, OUT); break;               \
        case Q8_F32: LAUNCH_Q(Q8_F32, OUT); break;               \
        default: LAUNCH_Q(Q8_E4M3, OUT); break;                  \
    }
    if (code_dtype == Q8_I8) { LAUNCH_Q_IN(Q8_I8) } else { LAUNCH_Q_IN(Q8_E4M3) }
#undef LAUNCH_Q_IN
#undef LAUNCH_Q
    return launch_status("q8_quant_rows");
}

#define Q8_IO_SWITCH(XD, YD, ...)                                                                  \
    if (XD == Q8_BF16 && YD == Q8_BF16) { constexpr int IN = Q8_BF16, OUT = Q8_BF16; __VA_ARGS__; } \
    else if (XD == Q8_BF16 && YD == Q8_E4M3) { constexpr int IN = Q8_BF16, OUT = Q8_E4M3; __VA_ARGS__; } \
    else if (XD == Q8_E4M3 && YD == Q8_BF16) { constexpr int IN = Q8_E4M3, OUT = Q8_BF16; __VA_ARGS__; } \
    else { constexpr int IN = Q8_E4M3, OUT = Q8_E4M3; __VA_ARGS__; }

static int check_io(const char* who, const void* x, int xd, const void* y, int yd) {
    if (!x || !y) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if ((xd != Q8_BF16 && xd != Q8_E4M3) || (yd != Q8_BF16 && yd != Q8_E4M3))
        return fail(Q8_ERR_DTYPE, "%s: dtypes (%d -> %d) must be BF16 or E4M3", who, xd, yd);
    if ((reinterpret_cast<uintptr_t>(x) % (xd == Q8_BF16 ? 16 : 8)) || (reinterpret_cast<uintptr_t>(y) % (yd == Q8_BF16 ? 16 : 8)))
        return fail(Q8_ERR_ALIGN, "%s: x / y must be 16-byte (bf16) or 8-byte (e4m3) aligned", who);
    return Q8_OK;
}

extern "C" int q8_fht(const void* x, int x_dtype, void* y, int y_dtype, int64_t rows, int dim, float scale,
                      q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_fht", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_io("q8_fht", x, x_dtype, y, y_dtype)) return st;
    const int N = pow2_ceil(dim);
    Q8_IO_SWITCH(x_dtype, y_dtype, {
        Q8_ROW_SHAPE_SWITCH(N, {
            const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);
            hipLaunchKernelGGL((fht_kernel<LANES, CH, IN, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, y, rows,
                               dim, scale);
        })
    })
    return launch_status("q8_fht");
}

extern "C" int q8_rmsnorm(const void* x, int x_dtype, const float* w, void* y, int y_dtype, float* rstd, int64_t rows,
                          int dim, float eps, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_rmsnorm", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_io("q8_rmsnorm", x, x_dtype, y, y_dtype)) return st;
    if (w && !aligned16(w)) return fail(Q8_ERR_ALIGN, "q8_rmsnorm: weights must be 16-byte aligned");
    const int N = pow2_ceil(dim);
    Q8_IO_SWITCH(x_dtype, y_dtype, {
        Q8_ROW_SHAPE_SWITCH(N, {
            const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);
            hipLaunchKernelGGL((rmsnorm_kernel<LANES, CH, IN, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, w, y,
                               rstd, rows, dim, eps);
        })
    })
    return launch_status("q8_rmsnorm");
}

extern "C" int q8_rope(const void* x, int x_dtype, const float* cos_t, const float* sin_t, void* y, int y_dtype,
                       int64_t rows, int dim, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || dim <= 0 || dim % 8 != 0) return fail(Q8_ERR_SHAPE, "q8_rope: rows %lld dim %d (dim %% 8 == 0)", (long long)rows, dim);
    if (rows == 0) return Q8_OK;
    if (int st = check_io("q8_rope", x, x_dtype, y, y_dtype)) return st;
    if (!cos_t || !sin_t) return fail(Q8_ERR_NULL, "q8_rope: null table");
    if (!aligned16(cos_t) || !aligned16(sin_t)) return fail(Q8_ERR_ALIGN, "q8_rope: tables must be 16-byte aligned");
    const int64_t nchunks = rows * (int64_t)dim / 8;
    const int64_t grid = (nchunks + kBlock - 1) / kBlock;
    if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_rope: too many elements");
    Q8_IO_SWITCH(x_dtype, y_dtype, {
        hipLaunchKernelGGL((rope_kernel<IN, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, cos_t, sin_t, y, nchunks);
    })
    return launch_status("q8_rope");
}
