// FP8 FlashAttention-2 forward for gfx950, head dim 64, non-causal, optional per-batch KV length.
//
// One workgroup = 4 waves = 4 x 64 query rows of one (batch, head); KV is walked forward in tiles of
// 64 keys that all four waves share through LDS (two stages, filled by global_load_lds_dwordx4).
//
// Everything is computed transposed so that no operand ever passes through LDS or a cross-lane
// shuffle between the two matrix products:
//   S^T = K Q^T   v_mfma_f32_32x32x64_f8f6f4, A = 32 K rows x 64 d (LDS), B = Q^T (registers).
//                 An accumulator lane (q = lane%32, h = lane/32) then holds 16 keys of ONE query.
//   O^T = V^T P^T A = 32 d rows x 64 keys of V^T (LDS), B = P^T: the 2 x 16 probabilities of a lane,
//                 cast to e4m3, ARE the 32-byte B operand of that lane. For this the K rows are
//                 placed in LDS in the order in which the S^T accumulator rows come out, such that
//                 lane half h owns keys 32h .. 32h+31 of the tile in operand byte order.
// Softmax runs in the log2 domain in fp32: p = exp2(s * c - m + 8), c = softmax_scale * log2(e); the row
// sum accumulates the unrounded p while e4m3_sat(p) multiplies V (csrc/flash_attention/
// flash_attention_cuda.cu:197-221,437). The factor 2^8 cancels in O / l; it places the row maximum at 256 so
// that probabilities down to 2^-14 of the maximum stay in the normal range of e4m3 (with the reference's p <= 1
// everything below 2^-10 is flushed to zero, which biases long, flat rows). Q8_ATTN_P_UNIT_RANGE restores p <= 1. Tiles that lie entirely beyond the valid KV length are
// skipped, the partial tile is masked with -inf (the reference walks backwards and needs -1e6 instead,
// flash_attention_cuda_mask.cu:244).
#include "q8_common.h"
#include "q8_host.h"

namespace q8 {

struct AttnParams {
    const uint8_t* q;
    const uint8_t* k;
    const uint8_t* v;
    void* o;
    const int32_t* kv_len;
    const float* sq;
    const float* sk;
    const float* sv;
    int B, H, M, N;
    int64_t v_row_stride;  // V^T row stride in bytes-elements (>= N, multiple of 16)
    float scale_log2;      // softmax_scale * log2(e)
    float p_shift;         // probabilities are formed as 2^(x - max + p_shift)
    int flags;
};

__device__ __attribute__((aligned(16))) const uint32_t g_attn_zero16[4] = {0, 0, 0, 0};

constexpr int kQT = 2;          // 32-query tiles per wave
constexpr int kWaves = 4;
constexpr int kBlockQ = kWaves * kQT * 32;  // 256 queries per workgroup
constexpr int kKV = 64;         // keys per tile
constexpr int kStage = 8192;    // K tile 4 KiB + V^T tile 4 KiB

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int OUT, bool SCALED>
__global__ __launch_bounds__(kWaves * 64) void attn_fwd_kernel(const AttnParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * kStage];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int ql = lane & 31, h = lane >> 5;
    const int bh = blockIdx.y, b = bh / p.H;
    const int M = p.M, N = p.N;
    int valid = N;
    if (p.kv_len) {
        const int len = p.kv_len[b];
        valid = len < N ? (len < 0 ? 0 : len) : N;
    }
    const uint8_t* Qg = p.q + (size_t)bh * M * 64;
    const uint8_t* Kg = p.k + (size_t)bh * N * 64;
    const uint8_t* Vg = p.v + (size_t)bh * 64 * p.v_row_stride;
    const int q0 = blockIdx.x * kBlockQ + wave * (kQT * 32);

    // Q^T operand: lane (q, h) holds bytes 32h .. 32h+31 of query row q
    v8i qf[kQT];
    float sqc[kQT];
#pragma unroll
    for (int t = 0; t < kQT; ++t) {
        int row = q0 + 32 * t + ql;
        row = row < M ? row : M - 1;
        const v4i* src = reinterpret_cast<const v4i*>(Qg + (size_t)row * 64 + 32 * h);
        const v4i a = src[0], c = src[1];
        qf[t] = v8i{a[0], a[1], a[2], a[3], c[0], c[1], c[2], c[3]};
        sqc[t] = SCALED ? p.sq[(size_t)bh * M + row] * p.scale_log2 : p.scale_log2;
    }

    // copy plan: wave w fills LDS rows 16w .. 16w+15 of both tiles (64-byte rows, 4 chunks of 16 bytes,
    // physical chunk = logical chunk ^ ((row >> 2) & 3)).
    const int crow = 16 * wave + (lane >> 2);
    const int cchunk = (lane & 3) ^ ((crow >> 2) & 3);
    int k_src_row;  // key index inside the tile held by LDS row `crow`
    {
        const int t = crow >> 5, i = crow & 31;
        k_src_row = 32 * ((i >> 2) & 1) + 16 * t + 4 * (i >> 3) + (i & 3);
    }
    auto issue_loads = [&](int stage, int kv0) {
        uint8_t* base = lds + stage * kStage;
        int kr = kv0 + k_src_row;
        kr = kr < N ? kr : N - 1;
        const uint8_t* ks = Kg + (size_t)kr * 64 + cchunk * 16;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ks,
                                         (__attribute__((address_space(3))) void*)(base + wave * 1024), 16, 0, 0);
        const int col = kv0 + cchunk * 16;
        const uint8_t* vs = (col < p.v_row_stride) ? (Vg + (size_t)crow * p.v_row_stride + col)
                                                   : reinterpret_cast<const uint8_t*>(g_attn_zero16);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vs,
                                         (__attribute__((address_space(3))) void*)(base + 4096 + wave * 1024), 16, 0, 0);
    };

    // operand fetch: lane (i = lane%32, h) reads chunks 2h, 2h+1 of row (32 t + i)
    const int frow = ql * 64;
    const int fpc0 = ((2 * h) ^ ((ql >> 2) & 3)) * 16, fpc1 = fpc0 ^ 16;

    v16f o_acc[kQT][2];
#pragma unroll
    for (int t = 0; t < kQT; ++t)
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int e = 0; e < 16; ++e) o_acc[t][d][e] = 0.f;
    float m_run[kQT], l_run[kQT];
#pragma unroll
    for (int t = 0; t < kQT; ++t) { m_run[t] = -INFINITY; l_run[t] = 0.f; }

    const int n_tiles = (valid + kKV - 1) / kKV;

    // per-token V scales enter P before its e4m3 cast as sv[j] / max_j sv[j] (<= 1, so the product stays in the
    // normal range of e4m3); the common factor max_j sv[j] is applied to O at the end.
    float sv_ref = 1.f, sv_inv = 1.f;
    if constexpr (SCALED) {
        __shared__ float red[kWaves];
        float mx = 0.f;
        for (int j = tid; j < valid; j += kWaves * 64) mx = fmaxf(mx, p.sv[(size_t)bh * N + j]);
        mx = group_max<64>(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        sv_ref = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        sv_inv = sv_ref > 0.f ? 1.0f / sv_ref : 0.f;
    }

    if (n_tiles > 0) issue_loads(0, 0);
    for (int it = 0; it < n_tiles; ++it) {
        const int kv0 = it * kKV;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        const uint8_t* st = lds + (it & 1) * kStage;
        v8i kf[2], vf[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint8_t* r = st + t * 2048 + frow;
            const v4i a = *reinterpret_cast<const v4i*>(r + fpc0), c = *reinterpret_cast<const v4i*>(r + fpc1);
            kf[t] = v8i{a[0], a[1], a[2], a[3], c[0], c[1], c[2], c[3]};
            const uint8_t* rv = st + 4096 + t * 2048 + frow;
            const v4i av = *reinterpret_cast<const v4i*>(rv + fpc0), cv = *reinterpret_cast<const v4i*>(rv + fpc1);
            vf[t] = v8i{av[0], av[1], av[2], av[3], cv[0], cv[1], cv[2], cv[3]};
        }
        if (it + 1 < n_tiles) issue_loads((it + 1) & 1, kv0 + kKV);

        // per-key scales of this lane's 32 keys (key = kv0 + 32h + 16t + e)
        float skv[SCALED ? 32 : 1], svv[SCALED ? 32 : 1];
        if constexpr (SCALED) {
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                int key = kv0 + 32 * h + e;
                key = key < N ? key : N - 1;
                skv[e] = p.sk[(size_t)bh * N + key];
                svv[e] = p.sv[(size_t)bh * N + key] * sv_inv;
            }
        }
        const bool partial = kv0 + kKV > valid;

#pragma unroll
        for (int qt = 0; qt < kQT; ++qt) {
            v16f s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                v16f z;
#pragma unroll
                for (int e = 0; e < 16; ++e) z[e] = 0.f;
                s[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[t], qf[qt], z, 0, 0, 0, 0, 0, 0);
            }
            float x[32];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float val = s[t][e];
                    if constexpr (SCALED) val *= skv[16 * t + e];
                    x[16 * t + e] = val * sqc[qt];
                }
            if (partial) {
#pragma unroll
                for (int e = 0; e < 32; ++e)
                    if (kv0 + 32 * h + e >= valid) x[e] = -INFINITY;
            }
            float mx = x[0];
#pragma unroll
            for (int e = 1; e < 32; ++e) mx = fmaxf(mx, x[e]);
            mx = fmaxf(mx, lane_xor<32>(mx));
            const float m_new = fmaxf(m_run[qt], mx);
            const float alpha = fast_exp2(m_run[qt] - m_new);
            m_run[qt] = m_new;
            const float m_sub = m_new - p.p_shift;
            float psum = 0.f;
            float pr[32];
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                const float pe = fast_exp2(x[e] - m_sub);
                psum += pe;
                pr[e] = SCALED ? pe * svv[e] : pe;
            }
            v8i pf;
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                uint32_t u = cvt_pk_e4m3(clamp448(pr[4 * w]), clamp448(pr[4 * w + 1]), 0u, false);
                u = cvt_pk_e4m3(clamp448(pr[4 * w + 2]), clamp448(pr[4 * w + 3]), u, true);
                pf[w] = (int)u;
            }
            if (p.flags & Q8_ATTN_SUM_ROUNDED_P) {
                psum = 0.f;
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    psum += e4m3_to_f32<0>(pf[w]) + e4m3_to_f32<1>(pf[w]) + e4m3_to_f32<2>(pf[w]) + e4m3_to_f32<3>(pf[w]);
                }
            }
            l_run[qt] = l_run[qt] * alpha + psum;
#pragma unroll
            for (int d = 0; d < 2; ++d) {
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[qt][d][e] *= alpha;
                o_acc[qt][d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[d], pf, o_acc[qt][d], 0, 0, 0, 0, 0, 0);
            }
        }
    }

    // ---- finalize: O^T lane (q, h), tile d, register e holds dim 32 d + 8 (e/4) + 4 h + (e%4)
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        const int row = q0 + 32 * qt + ql;
        float l = l_run[qt] + lane_xor<32>(l_run[qt]);
        const float inv = ((l == 0.f || l != l) ? 1.f : 1.f / l) * sv_ref;
        if (row >= M) continue;
#pragma unroll
        for (int d = 0; d < 2; ++d) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int dim = 32 * d + 8 * w + 4 * h;
                const float a0 = o_acc[qt][d][4 * w] * inv, a1 = o_acc[qt][d][4 * w + 1] * inv;
                const float a2 = o_acc[qt][d][4 * w + 2] * inv, a3 = o_acc[qt][d][4 * w + 3] * inv;
                if constexpr (OUT == Q8_BF16) {
                    uint16_t* dst = reinterpret_cast<uint16_t*>(p.o) + ((size_t)bh * M + row) * 64 + dim;
                    v2i wv;
                    wv[0] = (int)(f32_to_bf16_bits(a0) | (f32_to_bf16_bits(a1) << 16));
                    wv[1] = (int)(f32_to_bf16_bits(a2) | (f32_to_bf16_bits(a3) << 16));
                    *reinterpret_cast<v2i*>(dst) = wv;
                } else {
                    uint8_t* dst = reinterpret_cast<uint8_t*>(p.o) + ((size_t)bh * M + row) * 64 + dim;
                    *reinterpret_cast<uint32_t*>(dst) = pack4_e4m3_sat(a0, a1, a2, a3);
                }
            }
        }
    }
}

}  // namespace q8

using namespace q8;

extern "C" int q8_attn_fwd(const void* q, const void* k, const void* v, void* o, const int32_t* kv_len, const float* sq,
                           const float* sk, const float* sv, int B, int H, int M, int N, int D, int v_layout,
                           int64_t v_row_stride, float softmax_scale, int out_dtype, int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!q || !k || !v || !o) return fail(Q8_ERR_NULL, "q8_attn_fwd: null pointer");
    if (D != 64) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: head dim %d (only 64 is supported)", D);
    if (B <= 0 || H <= 0 || M <= 0 || N <= 0) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: B %d H %d M %d N %d", B, H, M, N);
    if ((long)B * H > 65535) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: B*H = %ld exceeds 65535", (long)B * H);
    if (out_dtype != Q8_BF16 && out_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "q8_attn_fwd: output dtype %d", out_dtype);
    if (flags & ~(Q8_ATTN_SUM_ROUNDED_P | Q8_ATTN_P_UNIT_RANGE)) return fail(Q8_ERR_FLAGS, "q8_attn_fwd: flags 0x%x", flags);
    if (v_layout != Q8_V_DS) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: V layout %d (only Q8_V_DS [B,H,64,Nv] is implemented)", v_layout);
    if (v_row_stride < N || v_row_stride % 16 != 0)
        return fail(Q8_ERR_SHAPE, "q8_attn_fwd: V row stride %lld must be >= N and a multiple of 16", (long long)v_row_stride);
    const bool scaled = sq || sk || sv;
    if (scaled && !(sq && sk && sv)) return fail(Q8_ERR_NULL, "q8_attn_fwd: sq, sk, sv must be given together");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (reinterpret_cast<uintptr_t>(o) % 8))
        return fail(Q8_ERR_ALIGN, "q8_attn_fwd: q, k, v must be 16-byte and o 8-byte aligned");
    AttnParams p{static_cast<const uint8_t*>(q), static_cast<const uint8_t*>(k), static_cast<const uint8_t*>(v), o, kv_len, sq, sk, sv,
                 B, H, M, N, v_row_stride, softmax_scale * 1.44269504088896340736f,
                 (flags & Q8_ATTN_P_UNIT_RANGE) ? 0.f : 8.f, flags};
    const dim3 grid((unsigned)((M + kBlockQ - 1) / kBlockQ), (unsigned)(B * H));
    const dim3 block(kWaves * 64);
    if (out_dtype == Q8_BF16) {
        if (scaled) hipLaunchKernelGGL((attn_fwd_kernel<Q8_BF16, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((attn_fwd_kernel<Q8_BF16, false>), grid, block, 0, stream, p);
    } else {
        if (scaled) hipLaunchKernelGGL((attn_fwd_kernel<Q8_E4M3, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((attn_fwd_kernel<Q8_E4M3, false>), grid, block, 0, stream, p);
    }
    return launch_status("q8_attn_fwd");
}
