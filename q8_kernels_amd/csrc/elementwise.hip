// Element-wise and row-reduction helpers around the 8-bit layers: the AdaLN multiply-add, tanh-GELU forward
// and backward, the transposed rotation of RoPE's backward and the RMSNorm backward. All are HBM-bound: every
// thread moves 8 consecutive elements per operand with one vector load / store each; element types are uniform
// run-time switches (the type pairs of the reference and any other mix of bf16 / e4m3 / fp32 where noted).
#include "rows_common.h"

namespace q8 {

// s = 0.5 (1 + tanh(t)) = 1 / (1 + exp(-2 t)) and 1 - s, both without cancellation in either tail:
// with u = exp(-2 |t|) <= 1, (s, 1 - s) = (1, u) / (1 + u) for t >= 0 and (u, 1) / (1 + u) for t < 0.
__device__ __forceinline__ void half_one_plus_tanh(float t, float& s, float& one_minus_s) {
    const float u = __builtin_amdgcn_exp2f(-2.885390081777927f * fabsf(t));  // exp(-2 |t|)
    const float r = __builtin_amdgcn_rcpf(1.0f + u);
    const float big = r, small = u * r;
    s = (t >= 0.f) ? big : small;
    one_minus_s = (t >= 0.f) ? small : big;
}

constexpr float kGeluK = 0.7978845608028654f, kGeluC = 0.044715f;

// ---- out = x * (y + scale_add) + z, y and z broadcast over groups of rows ---------------------------------

__global__ __launch_bounds__(kBlock) void fma_kernel(const void* __restrict__ x, int xd, const void* __restrict__ y, int yd,
                                                     const void* __restrict__ z, int zd, void* __restrict__ out, int od,
                                                     int64_t nchunks, int chunks_per_row, int64_t y_every,
                                                     int64_t z_every, float scale_add) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    const int64_t row = idx / chunks_per_row;
    const int64_t col = (idx - row * chunks_per_row) * 8;
    const int64_t dim = (int64_t)chunks_per_row * 8;
    float xv[8], yv[8], zv[8], o[8];
    load8_any(x, xd, idx * 8, xv);
    load8_any(y, yd, (row / y_every) * dim + col, yv);
    load8_any(z, zd, (row / z_every) * dim + col, zv);
    // one rounding for the product and the sum, as the contraction of the reference's
    // x * (y + scale_add) + z (csrc/ops/fma_cuda.cu:94) gives
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = __builtin_fmaf(xv[i], yv[i] + scale_add, zv[i]);
    store8_any(out, od, idx * 8, o);
}

// ---- tanh-GELU ------------------------------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void gelu_kernel(const void* __restrict__ x, int xd, void* __restrict__ out, int od,
                                                      int64_t nchunks) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    float v[8], o[8];
    load8_any(x, xd, idx * 8, v);
    // 0.5 x (1 + tanh(k (x + c x^3)))  (csrc/ops/gelu_forward_cuda.cu:12-16), with 0.5 (1 + tanh) formed directly
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float s, q;
        half_one_plus_tanh(kGeluK * (v[i] + kGeluC * v[i] * v[i] * v[i]), s, q);
        o[i] = v[i] * s;
    }
    store8_any(out, od, idx * 8, o);
}

__global__ __launch_bounds__(kBlock) void gelu_backward_kernel(const void* __restrict__ x, int xd,
                                                               const void* __restrict__ g, int gd, void* __restrict__ out,
                                                               int od, int64_t nchunks) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    float v[8], gv[8], o[8];
    load8_any(x, xd, idx * 8, v);
    load8_any(g, gd, idx * 8, gv);
    // grad * (0.5 (1 + phi) + 0.5 x (1 - phi^2) k (1 + 3 c x^2)), phi = tanh(tau)  (csrc/ops/gelu_backward_cuda.cu:94-100)
    // with s = 0.5 (1 + phi): 1 - phi^2 = 4 s (1 - s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float s, q;
        half_one_plus_tanh(kGeluK * (v[i] + kGeluC * v[i] * v[i] * v[i]), s, q);
        const float dtau = kGeluK * (1.0f + kGeluC * 3.0f * v[i] * v[i]);
        o[i] = gv[i] * (s + 2.0f * v[i] * (s * q) * dtau);
    }
    store8_any(out, od, idx * 8, o);
}

// ---- RoPE backward: the transposed rotation ------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void rope_backward_kernel(const void* __restrict__ g, int gd,
                                                               const float* __restrict__ cs, const float* __restrict__ sn,
                                                               void* __restrict__ out, int od, int64_t nchunks) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    const int64_t e = idx * 8;
    float gv[8], c[8], s[8], o[8];
    load8_any(g, gd, e, gv);
    load8<Q8_F32>(cs, e, c);
    load8<Q8_F32>(sn, e, s);
    // csrc/ops/rope_backward_cuda.cu:106-107
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
        o[i] = gv[i] * c[i] + gv[i + 1] * s[i + 1];
        o[i + 1] = -gv[i] * s[i] + gv[i + 1] * c[i + 1];
    }
    store8_any(out, od, e, o);
}

// ---- RMSNorm backward --------------------------------------------------------------------------------------
//
// dx = rstd / dim * (dim * g * w - y / w * sum_j(g_j * y_j)), y the normalised (and weighted) forward output
// (csrc/ops/rms_norm_backward_cuda.cu:140-160). Row mapping of rows_common.h.
template <int LANES, int CH>
__global__ __launch_bounds__(kBlock) void rmsnorm_backward_kernel(const void* __restrict__ y, int yd,
                                                                  const float* __restrict__ rstd,
                                                                  const void* __restrict__ g, int gd,
                                                                  const float* __restrict__ w, void* __restrict__ out,
                                                                  int od, int64_t rows, int dim) {
    constexpr int RPB = kBlock / LANES;
    __shared__ float red[4];
    const int t = threadIdx.x % LANES;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    float yv[CH][8], gv[CH][8], wv[CH][8];
    float dot[1] = {0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (row_ok && e < dim) {
            load8_any(y, yd, row * (int64_t)dim + e, yv[c]);
            load8_any(g, gd, row * (int64_t)dim + e, gv[c]);
            if (w != nullptr) {
                load8<Q8_F32>(w, e, wv[c]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) wv[c][i] = 1.0f;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) { yv[c][i] = 0.f; gv[c][i] = 0.f; wv[c][i] = 1.0f; }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) dot[0] += gv[c][i] * yv[c][i];
    }
    row_reduce<LANES, false, 1>(dot, red);
    if (!row_ok) return;
    const float r = rstd[row], fdim = (float)dim;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = r / fdim * (fdim * gv[c][i] * wv[c][i] - yv[c][i] / wv[c][i] * dot[0]);
        store8_any(out, od, row * (int64_t)dim + e, o);
    }
}

}  // namespace q8

using namespace q8;

static bool is_8or16(int dt) { return dt == Q8_BF16 || dt == Q8_E4M3; }
static bool is_operand(int dt) { return dt == Q8_BF16 || dt == Q8_E4M3 || dt == Q8_F32; }
static bool aligned_for(const void* p, int dt) { return (reinterpret_cast<uintptr_t>(p) % (dt == Q8_E4M3 ? 8 : 16)) == 0; }

// The modulation rows of an AdaLN block (q8_kernels/blocks/ltx_transformer_block.py:30-36): rows[p, r, :] =
// bf16(table[p, :] + timestep[r, p * dim .. (p + 1) * dim)), the fp32 sum rounded once, row-major per parameter p so that
// each of the `params` modulation tensors is contiguous. One 8-element chunk per thread.
__global__ __launch_bounds__(kBlock) void adaln_rows_kernel(const float* __restrict__ table, const float* __restrict__ timestep,
                                                            uint16_t* __restrict__ rows, int params, int64_t tokens, int chunks_per_row,
                                                            int64_t nchunks) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nchunks) return;
    const int c = (int)(idx % chunks_per_row);
    const int64_t pr = idx / chunks_per_row, p = pr / tokens, r = pr - p * tokens;
    float a[8], b[8];
    load8<Q8_F32>(table, (p * chunks_per_row + c) * 8, a);
    load8<Q8_F32>(timestep, ((r * params + p) * chunks_per_row + c) * 8, b);
    v4u o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack2_bf16(a[2 * i] + b[2 * i], a[2 * i + 1] + b[2 * i + 1]);
    *reinterpret_cast<v4u*>(rows + idx * 8) = o;
}

static int grid_for(const char* who, int64_t nchunks, unsigned* grid) {
    const int64_t g = (nchunks + kBlock - 1) / kBlock;
    if (g > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "%s: too many elements", who);
    *grid = (unsigned)g;
    return Q8_OK;
}

extern "C" int q8_fma(const void* x, int x_dtype, const void* y, int y_dtype, const void* z, int z_dtype, void* out,
                      int out_dtype, int64_t rows, int dim, int64_t y_rows_every, int64_t z_rows_every, float scale_add,
                      q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || rows > ((int64_t)1 << 40) || dim <= 0 || dim % 8 != 0)
        return fail(Q8_ERR_SHAPE, "q8_fma: rows %lld dim %d (dim %% 8 == 0)", (long long)rows, dim);
    if (rows == 0) return Q8_OK;  // (with no rows the broadcast periods mean nothing; a caller with zero tokens passes 0)
    if (y_rows_every <= 0 || z_rows_every <= 0) return fail(Q8_ERR_SHAPE, "q8_fma: broadcast periods must be positive");
    if (!x || !y || !z || !out) return fail(Q8_ERR_NULL, "q8_fma: null pointer");
    if (!is_8or16(x_dtype) || !is_8or16(out_dtype) || !is_operand(y_dtype) || !is_operand(z_dtype))
        return fail(Q8_ERR_DTYPE, "q8_fma: dtypes x %d y %d z %d out %d", x_dtype, y_dtype, z_dtype, out_dtype);
    if (!aligned_for(x, x_dtype) || !aligned_for(y, y_dtype) || !aligned_for(z, z_dtype) || !aligned_for(out, out_dtype))
        return fail(Q8_ERR_ALIGN, "q8_fma: operands must be 16-byte (8-byte for e4m3) aligned");
    unsigned grid;
    const int64_t nchunks = rows * (int64_t)(dim / 8);
    if (int st = grid_for("q8_fma", nchunks, &grid)) return st;
    hipLaunchKernelGGL(fma_kernel, dim3(grid), dim3(kBlock), 0, stream, x, x_dtype, y, y_dtype, z, z_dtype, out, out_dtype,
                       nchunks, dim / 8, y_rows_every, z_rows_every, scale_add);
    return launch_status("q8_fma");
}

static int check_ew(const char* who, const void* x, int xd, const void* out, int od, int64_t n) {
    if (n < 0 || n % 8 != 0) return fail(Q8_ERR_SHAPE, "%s: element count %lld must be a multiple of 8", who, (long long)n);
    if (n == 0) return Q8_OK;
    if (!x || !out) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if (!is_8or16(xd) || !is_8or16(od)) return fail(Q8_ERR_DTYPE, "%s: dtypes (%d -> %d) must be BF16 or E4M3", who, xd, od);
    if (!aligned_for(x, xd) || !aligned_for(out, od)) return fail(Q8_ERR_ALIGN, "%s: operands must be 16-byte (8-byte for e4m3) aligned", who);
    return Q8_OK;
}

extern "C" int q8_adaln_rows(const float* table, const float* timestep, void* rows, int params, int64_t tokens, int dim,
                             q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (params <= 0 || params > 64 || tokens < 0 || tokens > ((int64_t)1 << 32) || dim <= 0 || dim % 8 != 0)
        return fail(Q8_ERR_SHAPE, "q8_adaln_rows: params %d tokens %lld dim %d (dim %% 8 == 0)", params, (long long)tokens, dim);
    if (tokens == 0) return Q8_OK;
    if (!table || !timestep || !rows) return fail(Q8_ERR_NULL, "q8_adaln_rows: null pointer");
    if (!aligned16(table) || !aligned16(timestep) || !aligned16(rows))
        return fail(Q8_ERR_ALIGN, "q8_adaln_rows: table, timestep and rows must be 16-byte aligned");
    unsigned grid;
    const int64_t nchunks = (int64_t)params * tokens * (dim / 8);
    if (int st = grid_for("q8_adaln_rows", nchunks, &grid)) return st;
    hipLaunchKernelGGL(adaln_rows_kernel, dim3(grid), dim3(kBlock), 0, stream, table, timestep, static_cast<uint16_t*>(rows), params,
                       tokens, dim / 8, nchunks);
    return launch_status("q8_adaln_rows");
}

extern "C" int q8_gelu(const void* x, int x_dtype, void* out, int out_dtype, int64_t n, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_ew("q8_gelu", x, x_dtype, out, out_dtype, n)) return st;
    if (n == 0) return Q8_OK;
    unsigned grid;
    if (int st = grid_for("q8_gelu", n / 8, &grid)) return st;
    hipLaunchKernelGGL(gelu_kernel, dim3(grid), dim3(kBlock), 0, stream, x, x_dtype, out, out_dtype, n / 8);
    return launch_status("q8_gelu");
}

extern "C" int q8_gelu_backward(const void* x, int x_dtype, const void* grad, int grad_dtype, void* out, int out_dtype,
                                int64_t n, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_ew("q8_gelu_backward", x, x_dtype, out, out_dtype, n)) return st;
    if (n == 0) return Q8_OK;
    if (!grad) return fail(Q8_ERR_NULL, "q8_gelu_backward: null pointer");
    if (!is_8or16(grad_dtype)) return fail(Q8_ERR_DTYPE, "q8_gelu_backward: grad dtype %d", grad_dtype);
    if (!aligned_for(grad, grad_dtype)) return fail(Q8_ERR_ALIGN, "q8_gelu_backward: grad must be 16-byte (8-byte for e4m3) aligned");
    unsigned grid;
    if (int st = grid_for("q8_gelu_backward", n / 8, &grid)) return st;
    hipLaunchKernelGGL(gelu_backward_kernel, dim3(grid), dim3(kBlock), 0, stream, x, x_dtype, grad, grad_dtype, out, out_dtype,
                       n / 8);
    return launch_status("q8_gelu_backward");
}

extern "C" int q8_rope_backward(const void* grad, int grad_dtype, const float* cos_t, const float* sin_t, void* out,
                                int out_dtype, int64_t rows, int dim, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || rows > ((int64_t)1 << 40) || dim <= 0 || dim % 8 != 0)
        return fail(Q8_ERR_SHAPE, "q8_rope_backward: rows %lld dim %d (dim %% 8 == 0)", (long long)rows, dim);
    if (int st = check_ew("q8_rope_backward", grad, grad_dtype, out, out_dtype, rows * (int64_t)dim)) return st;
    if (rows == 0) return Q8_OK;
    if (!cos_t || !sin_t) return fail(Q8_ERR_NULL, "q8_rope_backward: null table");
    if (!aligned16(cos_t) || !aligned16(sin_t)) return fail(Q8_ERR_ALIGN, "q8_rope_backward: tables must be 16-byte aligned");
    unsigned grid;
    const int64_t nchunks = rows * (int64_t)dim / 8;
    if (int st = grid_for("q8_rope_backward", nchunks, &grid)) return st;
    hipLaunchKernelGGL(rope_backward_kernel, dim3(grid), dim3(kBlock), 0, stream, grad, grad_dtype, cos_t, sin_t, out, out_dtype,
                       nchunks);
    return launch_status("q8_rope_backward");
}

extern "C" int q8_rmsnorm_backward(const void* y, int y_dtype, const float* rstd, const void* grad, int grad_dtype,
                                   const float* w, void* out, int out_dtype, int64_t rows, int dim, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_rmsnorm_backward", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_ew("q8_rmsnorm_backward", y, y_dtype, out, out_dtype, rows * (int64_t)dim)) return st;
    if (!rstd || !grad) return fail(Q8_ERR_NULL, "q8_rmsnorm_backward: null pointer");
    if (!is_8or16(grad_dtype)) return fail(Q8_ERR_DTYPE, "q8_rmsnorm_backward: grad dtype %d", grad_dtype);
    if (!aligned_for(grad, grad_dtype) || (w && !aligned16(w)) || (reinterpret_cast<uintptr_t>(rstd) % 4))
        return fail(Q8_ERR_ALIGN, "q8_rmsnorm_backward: grad / weights must be 16-byte aligned");
    const int N = pow2_ceil(dim);
    Q8_ROW_SHAPE_SWITCH(N, {
        const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);
        if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_rmsnorm_backward: too many rows for one launch");
        hipLaunchKernelGGL((rmsnorm_backward_kernel<LANES, CH>), dim3((unsigned)grid), dim3(kBlock), 0, stream, y, y_dtype, rstd,
                           grad, grad_dtype, w, out, out_dtype, rows, dim);
    })
    return launch_status("q8_rmsnorm_backward");
}
