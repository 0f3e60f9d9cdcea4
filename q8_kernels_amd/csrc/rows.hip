// Memory-bound row kernels for gfx950: token-wise absmax quantizer, fast Walsh-Hadamard transform,
// RMSNorm and RoPE. The thread-to-element mapping and the shared arithmetic are in rows_common.h.
#include "rows_common.h"

namespace q8 {

// ---- token-wise quantizer -----------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void quant_rows_kernel(const void* __restrict__ x, void* __restrict__ codes,
                                                            float* __restrict__ scales, int64_t rows, int dim,
                                                            int64_t x_row_stride, int flags) {
    constexpr int RPB = kBlock / LANES, RPT = RowsPerThread<LANES, CH>::value;
    constexpr int ESZ = (IN == Q8_F32 ? 4 : (IN == Q8_E4M3 ? 1 : 2));
    __shared__ float red[RPT * 4];
    const int t = threadIdx.x % LANES;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPT * RPB <= rows;
    int64_t row[RPT];
    bool row_ok[RPT];
    float v[RPT][CH][8];
    float amax[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        row[r] = ((int64_t)blockIdx.x * RPT + r) * RPB + threadIdx.x / LANES;
        row_ok[r] = row[r] < rows;
        const char* xr = reinterpret_cast<const char*>(x) + row[r] * x_row_stride * ESZ;
        load_row<IN, LANES, CH>(xr, t, row_ok[r], dim, full, v[r]);
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        amax[r] = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) amax[r] = fmaxf(amax[r], fabsf(v[r][c][i]));
    }
    row_reduce<LANES, true, RPT>(amax, red);

#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        if (!row_ok[r]) continue;
        const float ratio = quant_ratio<OUT>(amax[r]);
        if (t == 0) scales[row[r]] = quant_scale<OUT>(amax[r], ratio, flags);
        uint8_t* out = reinterpret_cast<uint8_t*>(codes) + row[r] * (int64_t)dim;
        store_codes_row<OUT, LANES, CH>(out, t, dim, full, v[r], ratio, flags);
    }
}

// ---- fast Walsh-Hadamard transform --------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void fht_kernel(const void* __restrict__ x, void* __restrict__ y, int64_t rows,
                                                     int dim, float scale) {
    constexpr int RPB = kBlock / LANES;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    constexpr int OUT_B = (OUT == Q8_E4M3) ? 1 : 2;
    const int t = row_thread<LANES>();
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPB <= rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * IN_B;

    float v[CH][8];
    const bool nz = load_row<IN, LANES, CH, true>(xr, t, row_ok, dim, full, v);
    fht_row<LANES, CH>(v, t, scale, fht_zero_group<LANES>(nz));

    if (!row_ok) return;
    char* yr = reinterpret_cast<char*>(y) + row * (int64_t)dim * OUT_B;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;
        store8<OUT>(yr, e, v[c]);
    }
}

// ---- RMSNorm ---------------------------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT>
__global__ __launch_bounds__(kBlock) void rmsnorm_kernel(const void* __restrict__ x, const float* __restrict__ w,
                                                         void* __restrict__ y, float* __restrict__ rstd_out,
                                                         int64_t rows, int dim, float eps) {
    constexpr int RPB = kBlock / LANES, RPT = RowsPerThread<LANES, CH>::value;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    constexpr int OUT_B = (OUT == Q8_E4M3) ? 1 : 2;
    __shared__ float red[RPT * 4];
    const int t = threadIdx.x % LANES;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPT * RPB <= rows;
    int64_t row[RPT];
    bool row_ok[RPT];
    float v[RPT][CH][8];
    float ss[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        row[r] = ((int64_t)blockIdx.x * RPT + r) * RPB + threadIdx.x / LANES;
        row_ok[r] = row[r] < rows;
        const char* xr = reinterpret_cast<const char*>(x) + row[r] * (int64_t)dim * IN_B;
        load_row<IN, LANES, CH>(xr, t, row_ok[r], dim, full, v[r]);
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        ss[r] = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) ss[r] += v[r][c][i] * v[r][c][i];
    }
    row_reduce<LANES, false, RPT>(ss, red);
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        if (!row_ok[r]) continue;
        // rstd = rsqrt(mean(x^2)) with no epsilon in the reference (csrc/ops/rms_norm_cuda.cu:127-156)
        const float rstd = 1.0f / sqrtf(ss[r] * (1.0f / (float)dim) + eps);
        if (rstd_out != nullptr && t == 0) rstd_out[row[r]] = rstd;
        char* yr = reinterpret_cast<char*>(y) + row[r] * (int64_t)dim * OUT_B;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int e = (c * LANES + t) * 8;
            if (e >= dim) continue;
            if (w != nullptr) {
                float wv[8];
                load8<Q8_F32>(w, e, wv);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[r][c][i] = (v[r][c][i] * rstd) * wv[i];
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[r][c][i] = v[r][c][i] * rstd;
            }
            store8<OUT>(yr, e, v[r][c]);
        }
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
    if (x_row_stride < dim || x_row_stride > ((int64_t)1 << 40))
        return fail(Q8_ERR_SHAPE, "q8_quant_rows: row stride %lld (dim %d)", (long long)x_row_stride, dim);
    const int need = (x_dtype == Q8_E4M3) ? 8 : 16;
    if ((reinterpret_cast<uintptr_t>(x) % need) || ((x_row_stride * esz) % need) || (reinterpret_cast<uintptr_t>(codes) % 8) ||
        (reinterpret_cast<uintptr_t>(scales) % 4))
        return fail(Q8_ERR_ALIGN, "q8_quant_rows: x rows must be %d-byte aligned, codes 8-byte aligned", need);
    const int N = pow2_ceil(dim);
#define LAUNCH_Q(IN, OUT)                                                                              \
    Q8_ROW_SHAPE_SWITCH(N, {                                                                           \
        constexpr int RB = (kBlock / LANES) * RowsPerThread<LANES, CH>::value;                         \
        const int64_t grid = (rows + RB - 1) / RB;                                                     \
        if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_quant_rows: too many rows for one launch"); \
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
            if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_fht: too many rows for one launch");
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
            constexpr int RB = (kBlock / LANES) * RowsPerThread<LANES, CH>::value;
            const int64_t grid = (rows + RB - 1) / RB;
            if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_rmsnorm: too many rows for one launch");
            hipLaunchKernelGGL((rmsnorm_kernel<LANES, CH, IN, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, w, y,
                               rstd, rows, dim, eps);
        })
    })
    return launch_status("q8_rmsnorm");
}

extern "C" int q8_rope(const void* x, int x_dtype, const float* cos_t, const float* sin_t, void* y, int y_dtype,
                       int64_t rows, int dim, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || rows > ((int64_t)1 << 40) || dim <= 0 || dim % 8 != 0)
        return fail(Q8_ERR_SHAPE, "q8_rope: rows %lld dim %d (dim %% 8 == 0)", (long long)rows, dim);
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
