// Row kernels that fuse what the reference runs as separate launches with a 16-bit tensor in HBM between them:
//   FHT -> token-wise quantizer            (the Q8Linear prologue, q8_kernels/functional/linear.py:30-31)
//   RMSNorm -> token-wise quantizer        (norm followed by an 8-bit linear, q8_kernels/modules/attention.py:67-77)
//   qk-RMSNorm -> RoPE -> head split -> FHT -> e4m3   (q8_kernels/modules/attention.py:67-87 and the Q / K side of
//                                             q8_kernels/functional/flash_attention.py:47-55)
//   head split -> e4m3 -> transpose        (the V side, flash_attention.py:38-45)
// Every intermediate value is rounded to the dtype the unfused sequence would have stored (template MID), so the
// results are the same bits as the separate kernels give.
#include "rows_common.h"

namespace q8 {

// ---- FHT -> quantizer ------------------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT, int MID>
__global__ __launch_bounds__(kBlock) void fht_quant_kernel(const void* __restrict__ x, void* __restrict__ codes,
                                                           float* __restrict__ scales, int64_t rows, int dim,
                                                           float fht_scale, int flags) {
    constexpr int RPB = kBlock / LANES;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    __shared__ float red[4];
    const int t = row_thread<LANES>();
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPB <= rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * IN_B;

    float v[CH][8];
    const bool nz = load_row<IN, LANES, CH, true>(xr, t, row_ok, dim, full, v);
    fht_row<LANES, CH>(v, t, fht_scale, fht_zero_group<LANES>(nz));

    float amax[1] = {0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        round_mid8<MID>(v[c]);
        if (e < dim) {  // outputs beyond dim are dropped
#pragma unroll
            for (int i = 0; i < 8; ++i) amax[0] = fmaxf(amax[0], fabsf(v[c][i]));
        }
    }
    row_reduce<LANES, true, 1>(amax, red);
    if (!row_ok) return;
    const float ratio = quant_ratio<OUT>(amax[0]);
    if (t == 0) scales[row] = quant_scale<OUT>(amax[0], ratio, flags);
    uint8_t* out = reinterpret_cast<uint8_t*>(codes) + row * (int64_t)dim;
    store_codes_row<OUT, LANES, CH>(out, t, dim, full, v, ratio, flags);
}

// ---- RMSNorm -> quantizer ----------------------------------------------------------------------------

template <int LANES, int CH, int IN, int OUT, int MID>
__global__ __launch_bounds__(kBlock) void rmsnorm_quant_kernel(const void* __restrict__ x, const float* __restrict__ w,
                                                               void* __restrict__ codes, float* __restrict__ scales,
                                                               float* __restrict__ rstd_out, int64_t rows, int dim,
                                                               float eps, int flags) {
    constexpr int RPB = kBlock / LANES;
    constexpr int IN_B = (IN == Q8_E4M3) ? 1 : 2;
    __shared__ float red[4];
    const int t = threadIdx.x % LANES;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPB <= rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * IN_B;

    float v[CH][8];
    load_row<IN, LANES, CH>(xr, t, row_ok, dim, full, v);
    float ss[1] = {0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) ss[0] += v[c][i] * v[c][i];
    row_reduce<LANES, false, 1>(ss, red);
    const float rstd = 1.0f / sqrtf(ss[0] * (1.0f / (float)dim) + eps);

    float amax[1] = {0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e >= dim) continue;  // the padding stays zero
        if (w != nullptr) {
            float wv[8];
            load8<Q8_F32>(w, e, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = (v[c][i] * rstd) * wv[i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = v[c][i] * rstd;
        }
        round_mid8<MID>(v[c]);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax[0] = fmaxf(amax[0], fabsf(v[c][i]));
    }
    row_reduce<LANES, true, 1>(amax, red);
    if (!row_ok) return;
    const float ratio = quant_ratio<OUT>(amax[0]);
    if (t == 0) {
        scales[row] = quant_scale<OUT>(amax[0], ratio, flags);
        if (rstd_out != nullptr) rstd_out[row] = rstd;
    }
    uint8_t* out = reinterpret_cast<uint8_t*>(codes) + row * (int64_t)dim;
    store_codes_row<OUT, LANES, CH>(out, t, dim, full, v, ratio, flags);
}

// ---- RMSNorm -> AdaLN modulation -> FHT -> quantizer ---------------------------------------------------------
//
// The prologue of an int8 projection behind a modulated norm (q8_kernels/blocks/ltx_transformer_block.py:38-40 followed
// by q8_kernels/functional/linear.py:30-31): y1 = bf16(rmsnorm(x) w), y2 = bf16(y1 (mod_scale + scale_add) + mod_shift)
// (one fused multiply-add, as q8_fma), y3 = bf16(FHT(y2) fht_scale), codes = quant(y3). Each step is optional
// (w, mod_scale / mod_shift NULL, apply_fht 0) and rounds where the separate kernels store a bfloat16 tensor.
template <int LANES, int CH, int OUT>
__global__ __launch_bounds__(kBlock) void norm_mod_fht_quant_kernel(const void* __restrict__ x, const float* __restrict__ w,
                                                                    int apply_norm, const void* __restrict__ ms,
                                                                    const void* __restrict__ mt, int mod_dtype,
                                                                    int64_t rows_per_mod, float scale_add, int apply_fht,
                                                                    float fht_scale, void* __restrict__ codes,
                                                                    float* __restrict__ scales, int64_t rows, int dim,
                                                                    int flags) {
    constexpr int RPB = kBlock / LANES;
    __shared__ float red[4];
    const int t = row_thread<LANES>();
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LANES;
    const bool row_ok = row < rows;
    const bool full = dim == 8 * LANES * CH && ((int64_t)blockIdx.x + 1) * RPB <= rows;
    const char* xr = reinterpret_cast<const char*>(x) + row * (int64_t)dim * 2;

    float v[CH][8];
    load_row<Q8_BF16, LANES, CH>(xr, t, row_ok, dim, full, v);
    // Norm weights and bfloat16 modulation rows are requested with the row, the latter as raw words (up to 4 chunks per
    // thread): asked for chunk by chunk where they are used, every chunk waits for trips to the cache of its own.
    constexpr bool EARLY = CH <= 4;
    constexpr int EC = EARLY ? CH : 1;
    float wv[EC][8];
    v4u rs[EC], rt[EC];
    const bool early_w = EARLY && apply_norm && w != nullptr;
    const bool early_mod = EARLY && ms != nullptr && mod_dtype == Q8_BF16;
    const int64_t mrow = row_ok ? row / rows_per_mod : 0;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const int e = (c * LANES + t) * 8;
        if (full || e < dim) {
            if (early_w) load8<Q8_F32>(w, e, wv[c]);
            if (early_mod) {
                rs[c] = *reinterpret_cast<const v4u*>(reinterpret_cast<const uint16_t*>(ms) + mrow * dim + e);
                rt[c] = *reinterpret_cast<const v4u*>(reinterpret_cast<const uint16_t*>(mt) + mrow * dim + e);
            }
        }
    }
    if (apply_norm) {
        float ss[1] = {0.f};
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) ss[0] += v[c][i] * v[c][i];
        row_reduce<LANES, false, 1>(ss, red);
        const float rstd = 1.0f / sqrtf(ss[0] * (1.0f / (float)dim));
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int e = (c * LANES + t) * 8;
            if (e >= dim) continue;
            if (w != nullptr) {
                if (!early_w) load8<Q8_F32>(w, e, wv[EARLY ? c : 0]);
                const float (&wc)[8] = wv[EARLY ? c : 0];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[c][i] = (v[c][i] * rstd) * wc[i];
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[c][i] = v[c][i] * rstd;
            }
            round_mid8<Q8_BF16>(v[c]);
        }
    }
    if (ms != nullptr) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int e = (c * LANES + t) * 8;
            if (e >= dim) continue;
            float sv[8], tv[8];
            if (early_mod) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sv[2 * i] = __uint_as_float(rs[EARLY ? c : 0][i] << 16);
                    sv[2 * i + 1] = __uint_as_float(rs[EARLY ? c : 0][i] & 0xffff0000u);
                    tv[2 * i] = __uint_as_float(rt[EARLY ? c : 0][i] << 16);
                    tv[2 * i + 1] = __uint_as_float(rt[EARLY ? c : 0][i] & 0xffff0000u);
                }
            } else {
                load8_any(ms, mod_dtype, mrow * dim + e, sv);
                load8_any(mt, mod_dtype, mrow * dim + e, tv);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = __builtin_fmaf(v[c][i], sv[i] + scale_add, tv[i]);
            round_mid8<Q8_BF16>(v[c]);
        }
    }
    if (apply_fht) {
        const bool nz = any_nonzero(reinterpret_cast<const float (&)[CH * 8]>(v));
        fht_row<LANES, CH>(v, t, fht_scale, fht_zero_group<LANES>(nz));
#pragma unroll
        for (int c = 0; c < CH; ++c) round_mid8<Q8_BF16>(v[c]);
    }
    float amax[1] = {0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int e = (c * LANES + t) * 8;
        if (e < dim) {
#pragma unroll
            for (int i = 0; i < 8; ++i) amax[0] = fmaxf(amax[0], fabsf(v[c][i]));
        }
    }
    row_reduce<LANES, true, 1>(amax, red);
    if (!row_ok) return;
    const float ratio = quant_ratio<OUT>(amax[0]);
    if (t == 0) scales[row] = quant_scale<OUT>(amax[0], ratio, flags);
    uint8_t* out = reinterpret_cast<uint8_t*>(codes) + row * (int64_t)dim;
    store_codes_row<OUT, LANES, CH>(out, t, dim, full, v, ratio, flags);
}

// ---- attention prologue for Q and K ---------------------------------------------------------------------
//
// LANES threads per token: the row of H * D = 8 * LANES * CH elements (H heads of D = 8 * LH) uses the row mapping,
// so a head is one group of LH consecutive lanes of one chunk and the D-point Hadamard transform is the register
// stages plus log2(LH) lane stages. Codes go to the head-major layout [B, H, S, D] the attention kernel reads.
// The options are uniform branches: cs != NULL rotates, scales != NULL quantizes per (token, head).
// PAIR: a second tensor (K next to Q of a self-attention) goes through the same steps with the same tables, which are
// then read once: they are 8 of the 11 bytes per element that one tensor moves. xv != NULL (uniform): the V projection
// of the same tokens is cast to e4m3 on the way (per (token, head) absmax scales when scales_v != NULL) and written
// token-major per head, [B, H, S, D], the layout the attention kernel reads with Q8_V_SD
// (the cast of q8_kernels/functional/flash_attention.py:38-45 without its transposed copy).
template <int LANES, int CH, int LH, bool PAIR>
__global__ __launch_bounds__(kBlock) void attn_prep_qk_kernel(const uint16_t* __restrict__ x, int64_t x_row_stride,
                                                              const uint16_t* __restrict__ x2, int64_t x2_row_stride,
                                                              const float* __restrict__ nw, const float* __restrict__ nw2,
                                                              const float* __restrict__ cs, const float* __restrict__ sn,
                                                              uint8_t* __restrict__ codes, float* __restrict__ scales,
                                                              uint8_t* __restrict__ codes2, float* __restrict__ scales2,
                                                              const uint16_t* __restrict__ xv, int64_t xv_row_stride,
                                                              uint8_t* __restrict__ codes_v, float* __restrict__ scales_v,
                                                              int64_t tokens, int S, int flags, float scale,
                                                              int mid_bf16) {
    static_assert(LH <= LANES, "a head may not span tokens");
    constexpr int DIM = LANES * CH * 8, D = LH * 8, H = DIM / D, NT = PAIR ? 2 : 1;
    const int t = row_thread<LANES>();
    const int64_t tok = (int64_t)blockIdx.x * (kBlock / LANES) + threadIdx.x / LANES;
    if (tok >= tokens) return;  // no barrier below; the lane exchanges stay inside a head, i.e. inside a token
    const int64_t b = tok / S, s = tok - b * S;
    auto mid8 = [&](float (&f)[8]) { if (mid_bf16) round_mid8<Q8_BF16>(f); };

    float v[NT][CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        load8<Q8_BF16>(x + tok * x_row_stride, (c * LANES + t) * 8, v[0][c]);
        if constexpr (PAIR) load8<Q8_BF16>(x2 + tok * x2_row_stride, (c * LANES + t) * 8, v[NT - 1][c]);
    }
    // qk-RMSNorm over the whole row (all heads) with fp32 weights, no epsilon: the sum runs in the order of
    // rmsnorm_kernel (chunks, registers, lanes), so the result is the same bits (csrc/ops/rms_norm_cuda.cu:127-156)
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const float* w = n == 0 ? nw : nw2;
        if (w == nullptr) continue;
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += v[n][c][i] * v[n][c][i];
        ss = group_sum<LANES>(ss);
        const float rstd = 1.0f / sqrtf(ss * (1.0f / (float)DIM));
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float wv[8];
            load8<Q8_F32>(w, (c * LANES + t) * 8, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[n][c][i] = (v[n][c][i] * rstd) * wv[i];
            mid8(v[n][c]);
        }
    }
    if (cs != nullptr) {
        // interleaved pairs (csrc/ops/rope_cuda.cu:99-103). The tables hold one entry per element, [rows, DIM], or with
        // Q8_PREP_PAIR_TABLES one per rotated pair, [rows, DIM / 2] (tables built by repeating every frequency twice,
        // q8_kernels/models/LTXVideo.py:95-148, carry each value twice); rows = the tokens, or with
        // Q8_PREP_SHARED_TABLES the S positions of one batch element, which then serve every batch element.
        const int64_t trow = (flags & Q8_PREP_SHARED_TABLES) ? s : tok;
        auto rotate = [&](int c, const float (&cv)[8], const float (&sv)[8]) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    o[i] = v[n][c][i] * cv[i] - v[n][c][i + 1] * sv[i];
                    o[i + 1] = v[n][c][i + 1] * cv[i + 1] + v[n][c][i] * sv[i + 1];
                }
                mid8(o);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[n][c][i] = o[i];
            }
        };
        if (flags & Q8_PREP_PAIR_TABLES) {
            v4f hc[CH], hs[CH];  // requested together: half the bytes, and one trip to memory for all chunks
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int64_t e = trow * (DIM / 2) + (c * LANES + t) * 4;
                hc[c] = *reinterpret_cast<const v4f*>(cs + e);
                hs[c] = *reinterpret_cast<const v4f*>(sn + e);
            }
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                float cv[8], sv[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) { cv[i] = hc[c][i >> 1]; sv[i] = hs[c][i >> 1]; }
                rotate(c, cv, sv);
            }
        } else {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int64_t e = trow * DIM + (c * LANES + t) * 8;
                float cv[8], sv[8];
                load8<Q8_F32>(cs, e, cv);
                load8<Q8_F32>(sn, e, sv);
                rotate(c, cv, sv);
            }
        }
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        uint8_t* const cout = n == 0 ? codes : codes2;
        float* const sout = n == 0 ? scales : scales2;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            if (flags & Q8_PREP_FHT) {
                fht_head<LH>(v[n][c], t, scale);
            }
            const int h = (c * LANES + t) / LH;
            const int64_t orow = (b * H + h) * S + s;
            v2i w;
            if (sout != nullptr) {
                float amax = 0.f;
                mid8(v[n][c]);
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[n][c][i]));
                amax = group_max<LH>(amax);
                const float ratio = quant_ratio<Q8_E4M3>(amax);
                if ((t % LH) == 0) sout[orow] = quant_scale<Q8_E4M3>(amax, ratio, 0);
                w = quant_codes8<Q8_E4M3>(v[n][c], ratio, 0);
            } else {
                w[0] = (int)pack4_e4m3_c10(v[n][c][0], v[n][c][1], v[n][c][2], v[n][c][3]);
                w[1] = (int)pack4_e4m3_c10(v[n][c][4], v[n][c][5], v[n][c][6], v[n][c][7]);
            }
            *reinterpret_cast<v2i*>(cout + orow * D + (t % LH) * 8) = w;
        }
    }
    if (xv != nullptr) {
        float vv[CH][8];
#pragma unroll
        for (int c = 0; c < CH; ++c) load8<Q8_BF16>(xv + tok * xv_row_stride, (c * LANES + t) * 8, vv[c]);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int h = (c * LANES + t) / LH;
            const int64_t orow = (b * H + h) * S + s;
            v2i w;
            if (scales_v != nullptr) {
                float amax = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(vv[c][i]));
                amax = group_max<LH>(amax);
                const float ratio = quant_ratio<Q8_E4M3>(amax);
                if ((t % LH) == 0) scales_v[orow] = quant_scale<Q8_E4M3>(amax, ratio, 0);
                w = quant_codes8<Q8_E4M3>(vv[c], ratio, 0);
            } else {
                w[0] = (int)pack4_e4m3_c10(vv[c][0], vv[c][1], vv[c][2], vv[c][3]);
                w[1] = (int)pack4_e4m3_c10(vv[c][4], vv[c][5], vv[c][6], vv[c][7]);
            }
            *reinterpret_cast<v2i*>(codes_v + orow * D + (t % LH) * 8) = w;
        }
    }
}

// ---- attention prologue for V ---------------------------------------------------------------------------
//
// x [B, S, H * 64] (token-major, bf16) -> e4m3 codes [B, H, 64, S_pad] (channel-major per head, the layout of the
// attention kernel's V operand), columns S..S_pad-1 zero. One block transposes 64 tokens x 64 channels of one head
// through LDS. SCALED: one absmax scale per (token, head), written to scales [B, H, S].
template <bool SCALED>
__global__ __launch_bounds__(kBlock) void attn_prep_v_kernel(const uint16_t* __restrict__ x, int64_t x_row_stride,
                                                             uint8_t* __restrict__ codes, float* __restrict__ scales,
                                                             int S, int S_pad, int H) {
    __shared__ uint32_t tile[64][17];  // [token][channel / 4], one pad word per row
    const int b = blockIdx.z, h = blockIdx.y, s0 = blockIdx.x * 64;
    {
        const int tok = threadIdx.x >> 2, part = threadIdx.x & 3;  // 16 channels per thread
        const int s = s0 + tok;
        float v[2][8];
        if (s < S) {
            const uint16_t* xr = x + ((int64_t)b * S + s) * x_row_stride + h * 64 + part * 16;
            load8<Q8_BF16>(xr, 0, v[0]);
            load8<Q8_BF16>(xr, 8, v[1]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[0][i] = v[1][i] = 0.f;
        }
        uint32_t w[4];
        if constexpr (SCALED) {
            float amax = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fmaxf(fabsf(v[0][i]), fabsf(v[1][i])));
            amax = group_max<4>(amax);
            const float ratio = quant_ratio<Q8_E4M3>(amax);
            if (part == 0 && s < S) scales[((int64_t)b * H + h) * S + s] = quant_scale<Q8_E4M3>(amax, ratio, 0);
            const v2i c0 = quant_codes8<Q8_E4M3>(v[0], ratio, 0), c1 = quant_codes8<Q8_E4M3>(v[1], ratio, 0);
            w[0] = (uint32_t)c0[0]; w[1] = (uint32_t)c0[1]; w[2] = (uint32_t)c1[0]; w[3] = (uint32_t)c1[1];
        } else {
            w[0] = pack4_e4m3_c10(v[0][0], v[0][1], v[0][2], v[0][3]);
            w[1] = pack4_e4m3_c10(v[0][4], v[0][5], v[0][6], v[0][7]);
            w[2] = pack4_e4m3_c10(v[1][0], v[1][1], v[1][2], v[1][3]);
            w[3] = pack4_e4m3_c10(v[1][4], v[1][5], v[1][6], v[1][7]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) tile[tok][part * 4 + i] = w[i];
    }
    __syncthreads();
    {
        const int d = threadIdx.x >> 2, part = threadIdx.x & 3;  // channel d, tokens part * 16 .. + 15
        if (s0 + part * 16 >= S_pad) return;
        const uint8_t* tb = reinterpret_cast<const uint8_t*>(&tile[0][0]);
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t acc = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) acc |= (uint32_t)tb[(part * 16 + i * 4 + j) * 68 + d] << (8 * j);
            w[i] = acc;
        }
        uint8_t* out = codes + (((int64_t)b * H + h) * 64 + d) * S_pad + s0 + part * 16;
        *reinterpret_cast<v4u*>(out) = v4u{w[0], w[1], w[2], w[3]};
    }
}

}  // namespace q8

using namespace q8;

static int check_quant_args(const char* who, const void* x, int x_dtype, const void* codes, int code_dtype,
                            const float* scales, int mid_dtype, int flags) {
    if (!x || !codes || !scales) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if (flags & ~(Q8_QUANT_RNE | Q8_QUANT_SCALE_DIV)) return fail(Q8_ERR_FLAGS, "%s: flags 0x%x", who, flags);
    if (code_dtype != Q8_I8 && code_dtype != Q8_E4M3)
        return fail(Q8_ERR_DTYPE, "%s: code dtype %d (want I8 or E4M3)", who, code_dtype);
    if (x_dtype != Q8_BF16 && x_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "%s: input dtype %d (want BF16 or E4M3)", who, x_dtype);
    if (mid_dtype != Q8_BF16 && mid_dtype != Q8_F32 && !(mid_dtype == Q8_E4M3 && x_dtype == Q8_E4M3))
        return fail(Q8_ERR_DTYPE, "%s: intermediate dtype %d (want BF16 or F32, or E4M3 for an E4M3 input)", who, mid_dtype);
    if ((reinterpret_cast<uintptr_t>(x) % (x_dtype == Q8_BF16 ? 16 : 8)) || (reinterpret_cast<uintptr_t>(codes) % 8) ||
        (reinterpret_cast<uintptr_t>(scales) % 4))
        return fail(Q8_ERR_ALIGN, "%s: x must be 16-byte (bf16) or 8-byte (e4m3) aligned, codes 8-byte aligned", who);
    return Q8_OK;
}

#define Q8_FUSED_SWITCH(XD, CD, MD, ...)                                                              \
    if (XD == Q8_BF16 && CD == Q8_I8 && MD == Q8_BF16) { constexpr int IN = Q8_BF16, OUT = Q8_I8, MID = Q8_BF16; __VA_ARGS__; } \
    else if (XD == Q8_BF16 && CD == Q8_E4M3 && MD == Q8_BF16) { constexpr int IN = Q8_BF16, OUT = Q8_E4M3, MID = Q8_BF16; __VA_ARGS__; } \
    else if (XD == Q8_BF16 && CD == Q8_I8) { constexpr int IN = Q8_BF16, OUT = Q8_I8, MID = Q8_F32; __VA_ARGS__; } \
    else if (XD == Q8_BF16) { constexpr int IN = Q8_BF16, OUT = Q8_E4M3, MID = Q8_F32; __VA_ARGS__; } \
    else if (CD == Q8_I8 && MD == Q8_E4M3) { constexpr int IN = Q8_E4M3, OUT = Q8_I8, MID = Q8_E4M3; __VA_ARGS__; } \
    else if (CD == Q8_E4M3 && MD == Q8_E4M3) { constexpr int IN = Q8_E4M3, OUT = Q8_E4M3, MID = Q8_E4M3; __VA_ARGS__; } \
    else if (CD == Q8_I8 && MD == Q8_BF16) { constexpr int IN = Q8_E4M3, OUT = Q8_I8, MID = Q8_BF16; __VA_ARGS__; } \
    else if (CD == Q8_E4M3 && MD == Q8_BF16) { constexpr int IN = Q8_E4M3, OUT = Q8_E4M3, MID = Q8_BF16; __VA_ARGS__; } \
    else if (CD == Q8_I8) { constexpr int IN = Q8_E4M3, OUT = Q8_I8, MID = Q8_F32; __VA_ARGS__; } \
    else { constexpr int IN = Q8_E4M3, OUT = Q8_E4M3, MID = Q8_F32; __VA_ARGS__; }

extern "C" int q8_fht_quant_rows(const void* x, int x_dtype, void* codes, int code_dtype, float* scales, int64_t rows,
                                 int dim, float fht_scale, int mid_dtype, int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_fht_quant_rows", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_quant_args("q8_fht_quant_rows", x, x_dtype, codes, code_dtype, scales, mid_dtype, flags)) return st;
    const int N = pow2_ceil(dim);
    Q8_FUSED_SWITCH(x_dtype, code_dtype, mid_dtype, {
        Q8_ROW_SHAPE_SWITCH(N, {
            const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);
            if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_fht_quant_rows: too many rows for one launch");
            hipLaunchKernelGGL((fht_quant_kernel<LANES, CH, IN, OUT, MID>), dim3((unsigned)grid), dim3(kBlock), 0, stream,
                               x, codes, scales, rows, dim, fht_scale, flags);
        })
    })
    return launch_status("q8_fht_quant_rows");
}

extern "C" int q8_rmsnorm_quant_rows(const void* x, int x_dtype, const float* w, void* codes, int code_dtype,
                                     float* scales, float* rstd, int64_t rows, int dim, float eps, int mid_dtype,
                                     int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int st = check_rows("q8_rmsnorm_quant_rows", rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_quant_args("q8_rmsnorm_quant_rows", x, x_dtype, codes, code_dtype, scales, mid_dtype, flags)) return st;
    if (w && !aligned16(w)) return fail(Q8_ERR_ALIGN, "q8_rmsnorm_quant_rows: weights must be 16-byte aligned");
    const int N = pow2_ceil(dim);
    Q8_FUSED_SWITCH(x_dtype, code_dtype, mid_dtype, {
        Q8_ROW_SHAPE_SWITCH(N, {
            const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);
            if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_rmsnorm_quant_rows: too many rows for one launch");
            hipLaunchKernelGGL((rmsnorm_quant_kernel<LANES, CH, IN, OUT, MID>), dim3((unsigned)grid), dim3(kBlock), 0,
                               stream, x, w, codes, scales, rstd, rows, dim, eps, flags);
        })
    })
    return launch_status("q8_rmsnorm_quant_rows");
}

extern "C" int q8_norm_mod_fht_quant_rows(const void* x, const float* norm_w, int apply_norm, const void* mod_scale,
                                          const void* mod_shift, int mod_dtype, int64_t rows_per_mod, float scale_add,
                                          int apply_fht, float fht_scale, void* codes, int code_dtype, float* scales,
                                          int64_t rows, int dim, int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "q8_norm_mod_fht_quant_rows";
    if (int st = check_rows(who, rows, dim)) return st;
    if (rows == 0) return Q8_OK;
    if (int st = check_quant_args(who, x, Q8_BF16, codes, code_dtype, scales, Q8_BF16, flags)) return st;
    if (norm_w && !aligned16(norm_w)) return fail(Q8_ERR_ALIGN, "%s: weights must be 16-byte aligned", who);
    if ((mod_scale == nullptr) != (mod_shift == nullptr)) return fail(Q8_ERR_NULL, "%s: scale and shift come together", who);
    if (mod_scale) {
        if (mod_dtype != Q8_BF16 && mod_dtype != Q8_F32) return fail(Q8_ERR_DTYPE, "%s: modulation dtype %d (want BF16 or F32)", who, mod_dtype);
        if (rows_per_mod <= 0) return fail(Q8_ERR_SHAPE, "%s: rows_per_mod must be positive", who);
        if (!aligned16(mod_scale) || !aligned16(mod_shift)) return fail(Q8_ERR_ALIGN, "%s: modulation rows must be 16-byte aligned", who);
    }
    const int N = pow2_ceil(dim);
    const int64_t rpm = mod_scale ? rows_per_mod : 1;
#define NMQ_LAUNCH(OUT)                                                                                                  \
    Q8_ROW_SHAPE_SWITCH(N, {                                                                                             \
        const int64_t grid = (rows + (kBlock / LANES) - 1) / (kBlock / LANES);                                           \
        if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "q8_norm_mod_fht_quant_rows: too many rows for one launch"); \
        hipLaunchKernelGGL((norm_mod_fht_quant_kernel<LANES, CH, OUT>), dim3((unsigned)grid), dim3(kBlock), 0, stream, x, \
                           norm_w, apply_norm, mod_scale, mod_shift, mod_dtype, rpm, scale_add, apply_fht, fht_scale,    \
                           codes, scales, rows, dim, flags);                                                             \
    })
    if (code_dtype == Q8_I8) { NMQ_LAUNCH(Q8_I8) } else { NMQ_LAUNCH(Q8_E4M3) }
#undef NMQ_LAUNCH
    return launch_status(who);
}

static int attn_prep_qk_impl(const char* who, const void* x, int64_t x_row_stride, const void* x2, int64_t x2_row_stride,
                             const float* norm_w, const float* norm_w2, const float* cos_t, const float* sin_t, void* codes, float* scales, void* codes2,
                             float* scales2, const void* xv, int64_t xv_row_stride, void* codes_v, float* scales_v, int B, int S,
                             int H, int D, int flags, float scale, int mid_dtype, hipStream_t stream) {
    const bool pair = x2 != nullptr;
    if (B < 0 || S < 0 || H <= 0) return fail(Q8_ERR_SHAPE, "%s: B %d S %d H %d", who, B, S, H);
    if (D != 64 && D != 128) return fail(Q8_ERR_SHAPE, "%s: head dim %d (want 64 or 128)", who, D);
    const int64_t dim = (int64_t)H * D;
    const bool small = dim == 64 || dim == 128 || dim == 256;
    if (!small && (dim % 512 != 0 || dim > 4096))
        return fail(Q8_ERR_SHAPE, "%s: H * D = %lld must be 64, 128, 256 or a multiple of 512 up to 4096", who, (long long)dim);
    if ((int64_t)B * S == 0) return Q8_OK;
    if (!x || !codes || (pair && !codes2)) return fail(Q8_ERR_NULL, "%s: null pointer", who);
    if ((cos_t == nullptr) != (sin_t == nullptr)) return fail(Q8_ERR_NULL, "%s: cos and sin come together", who);
    if (flags & ~(Q8_PREP_FHT | Q8_PREP_PAIR_TABLES | Q8_PREP_SHARED_TABLES)) return fail(Q8_ERR_FLAGS, "%s: unknown flag bits 0x%x", who, flags);
    if (!cos_t && (flags & (Q8_PREP_PAIR_TABLES | Q8_PREP_SHARED_TABLES)))
        return fail(Q8_ERR_FLAGS, "%s: table flags 0x%x without tables", who, flags);
    if (pair && ((scales == nullptr) != (scales2 == nullptr))) return fail(Q8_ERR_NULL, "%s: both scale outputs or none", who);
    if (x_row_stride < dim || x_row_stride % 8 != 0 || (pair && (x2_row_stride < dim || x2_row_stride % 8 != 0)))
        return fail(Q8_ERR_SHAPE, "%s: row stride %lld / %lld", who, (long long)x_row_stride, (long long)x2_row_stride);
    if ((norm_w && !aligned16(norm_w)) || (norm_w2 && !aligned16(norm_w2)))
        return fail(Q8_ERR_ALIGN, "%s: norm weights must be 16-byte aligned", who);
    if (!aligned16(x) || (pair && !aligned16(x2)) || (cos_t && (!aligned16(cos_t) || !aligned16(sin_t))) ||
        (reinterpret_cast<uintptr_t>(codes) % 8) || (pair && (reinterpret_cast<uintptr_t>(codes2) % 8)))
        return fail(Q8_ERR_ALIGN, "%s: x and tables must be 16-byte aligned, codes 8-byte aligned", who);
    if (mid_dtype != Q8_BF16 && mid_dtype != Q8_F32) return fail(Q8_ERR_DTYPE, "%s: intermediate dtype %d", who, mid_dtype);
    if (xv) {
        if (!codes_v) return fail(Q8_ERR_NULL, "%s: null pointer", who);
        if (xv_row_stride < dim || xv_row_stride % 8 != 0) return fail(Q8_ERR_SHAPE, "%s: V row stride %lld", who, (long long)xv_row_stride);
        if (!aligned16(xv) || (reinterpret_cast<uintptr_t>(codes_v) % 8))
            return fail(Q8_ERR_ALIGN, "%s: V must be 16-byte aligned, its codes 8-byte aligned", who);
        if ((scales_v == nullptr) != (scales == nullptr)) return fail(Q8_ERR_NULL, "%s: all scale outputs or none", who);
    }
    const int64_t tokens = (int64_t)B * S;
    const int lanes = small ? (int)(dim / 8) : 64;
    const int64_t grid = (tokens + (kBlock / lanes) - 1) / (kBlock / lanes);
    if (grid > 0x7fffffffLL) return fail(Q8_ERR_SHAPE, "%s: too many tokens", who);
#define PREP_ARGS                                                                                                        \
    static_cast<const uint16_t*>(x), x_row_stride, static_cast<const uint16_t*>(x2), x2_row_stride, norm_w, norm_w2,     \
        cos_t, sin_t,                                                                                                    \
        static_cast<uint8_t*>(codes), scales, static_cast<uint8_t*>(codes2), scales2,                                    \
        static_cast<const uint16_t*>(xv), xv_row_stride, static_cast<uint8_t*>(codes_v), scales_v, tokens, S, flags, \
        scale, mid_dtype == Q8_BF16 ? 1 : 0
#define PREP_LAUNCH(LANES, CH, LH)                                                                                       \
    if (pair) hipLaunchKernelGGL((attn_prep_qk_kernel<LANES, CH, LH, true>), dim3((unsigned)grid), dim3(kBlock), 0, stream, PREP_ARGS); \
    else hipLaunchKernelGGL((attn_prep_qk_kernel<LANES, CH, LH, false>), dim3((unsigned)grid), dim3(kBlock), 0, stream, PREP_ARGS)
#define PREP_D(LANES, CH) \
    if (D == 64) { PREP_LAUNCH(LANES, CH, 8); } else { PREP_LAUNCH(LANES, CH, 16); }
    switch (dim) {
        case 64: PREP_LAUNCH(8, 1, 8); break;
        case 128: PREP_D(16, 1); break;
        case 256: PREP_D(32, 1); break;
        case 512: PREP_D(64, 1); break;
        case 1024: PREP_D(64, 2); break;
        case 1536: PREP_D(64, 3); break;
        case 2048: PREP_D(64, 4); break;
        case 2560: PREP_D(64, 5); break;
        case 3072: PREP_D(64, 6); break;
        case 3584: PREP_D(64, 7); break;
        default: PREP_D(64, 8); break;
    }
#undef PREP_D
#undef PREP_LAUNCH
#undef PREP_ARGS
    return launch_status(who);
}

extern "C" int q8_attn_prep_qk(const void* x, int64_t x_row_stride, const float* norm_w, const float* cos_t,
                               const float* sin_t, void* codes, float* scales, int B, int S, int H, int D, int flags,
                               float scale, int mid_dtype, q8_stream_t stream_) {
    return attn_prep_qk_impl("q8_attn_prep_qk", x, x_row_stride, nullptr, 0, norm_w, nullptr, cos_t, sin_t, codes, scales, nullptr,
                             nullptr, nullptr, 0, nullptr, nullptr, B, S, H, D, flags, scale, mid_dtype,
                             static_cast<hipStream_t>(stream_));
}

extern "C" int q8_attn_prep_qk_pair(const void* xq, int64_t xq_row_stride, const void* xk, int64_t xk_row_stride,
                                    const float* norm_wq, const float* norm_wk, const float* cos_t, const float* sin_t,
                                    void* codes_q, float* scales_q, void* codes_k, float* scales_k, int B, int S, int H,
                                    int D, int flags, float scale, int mid_dtype, q8_stream_t stream_) {
    if (!xk) return fail(Q8_ERR_NULL, "q8_attn_prep_qk_pair: null pointer");
    return attn_prep_qk_impl("q8_attn_prep_qk_pair", xq, xq_row_stride, xk, xk_row_stride, norm_wq, norm_wk, cos_t, sin_t, codes_q, scales_q,
                             codes_k, scales_k, nullptr, 0, nullptr, nullptr, B, S, H, D, flags, scale, mid_dtype,
                             static_cast<hipStream_t>(stream_));
}

extern "C" int q8_attn_prep_qkv(const void* xq, int64_t xq_row_stride, const void* xk, int64_t xk_row_stride, const void* xv,
                                int64_t xv_row_stride, const float* norm_wq, const float* norm_wk, const float* cos_t,
                                const float* sin_t, void* codes_q, float* scales_q, void* codes_k, float* scales_k,
                                void* codes_v, float* scales_v, int B, int S, int H, int D, int flags, float scale,
                                int mid_dtype, q8_stream_t stream_) {
    if (!xk || !xv) return fail(Q8_ERR_NULL, "q8_attn_prep_qkv: null pointer");
    return attn_prep_qk_impl("q8_attn_prep_qkv", xq, xq_row_stride, xk, xk_row_stride, norm_wq, norm_wk, cos_t, sin_t, codes_q, scales_q,
                             codes_k, scales_k, xv, xv_row_stride, codes_v, scales_v, B, S, H, D, flags, scale, mid_dtype,
                             static_cast<hipStream_t>(stream_));
}

extern "C" int q8_attn_prep_kv(const void* xk, int64_t xk_row_stride, const void* xv, int64_t xv_row_stride, const float* norm_wk,
                               const float* cos_t, const float* sin_t, void* codes_k, float* scales_k, void* codes_v,
                               float* scales_v, int B, int S, int H, int D, int flags, float scale, int mid_dtype,
                               q8_stream_t stream_) {
    if (!xv) return fail(Q8_ERR_NULL, "q8_attn_prep_kv: null pointer");
    return attn_prep_qk_impl("q8_attn_prep_kv", xk, xk_row_stride, nullptr, 0, norm_wk, nullptr, cos_t, sin_t, codes_k, scales_k, nullptr,
                             nullptr, xv, xv_row_stride, codes_v, scales_v, B, S, H, D, flags, scale, mid_dtype,
                             static_cast<hipStream_t>(stream_));
}

extern "C" int q8_attn_prep_v(const void* x, int64_t x_row_stride, void* codes, float* scales, int B, int S, int H, int D,
                              int S_pad, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (B < 0 || S < 0 || H <= 0 || H > 65535 || B > 65535) return fail(Q8_ERR_SHAPE, "q8_attn_prep_v: B %d S %d H %d", B, S, H);
    if (D != 64) return fail(Q8_ERR_SHAPE, "q8_attn_prep_v: head dim %d (want 64)", D);
    if (S_pad < S || S_pad % 16 != 0 || S_pad > (1 << 30))
        return fail(Q8_ERR_SHAPE, "q8_attn_prep_v: S_pad %d must be a multiple of 16 >= S %d (at most 2^30)", S_pad, S);
    if (B == 0 || S_pad == 0) return Q8_OK;
    if (!x || !codes) return fail(Q8_ERR_NULL, "q8_attn_prep_v: null pointer");
    if (x_row_stride < (int64_t)H * D || x_row_stride % 8 != 0) return fail(Q8_ERR_SHAPE, "q8_attn_prep_v: row stride %lld", (long long)x_row_stride);
    if (!aligned16(x) || !aligned16(codes)) return fail(Q8_ERR_ALIGN, "q8_attn_prep_v: x and codes must be 16-byte aligned");
    const dim3 grid((unsigned)((S_pad + 63) / 64), (unsigned)H, (unsigned)B);
    if (scales)
        hipLaunchKernelGGL((attn_prep_v_kernel<true>), grid, dim3(kBlock), 0, stream, static_cast<const uint16_t*>(x),
                           x_row_stride, static_cast<uint8_t*>(codes), scales, S, S_pad, H);
    else
        hipLaunchKernelGGL((attn_prep_v_kernel<false>), grid, dim3(kBlock), 0, stream, static_cast<const uint16_t*>(x),
                           x_row_stride, static_cast<uint8_t*>(codes), scales, S, S_pad, H);
    return launch_status("q8_attn_prep_v");
}
