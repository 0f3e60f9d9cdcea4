// FP8 FlashAttention-2 forward for gfx950, head dim 64, non-causal, optional per-batch KV length.
//
// One workgroup = 8 waves x 32 query rows of one (batch, head) with unit scales, 4 waves x 32 with per-token scales (whose
// register need allows three such workgroups on a CU but only one of 8 waves); 4 x 64 is instantiated as well. KV is
// walked forward in tiles of 64 keys that all waves share through a four-stage LDS ring filled by
// global_load_lds_dwordx4. Key / value sequences of at most 128 tokens take attn_short_kernel instead.
// V arrives either channel-major per head (V^T [B,H,64,Nv], Q8_V_DS) or token-major like K ([B,H,N,64], Q8_V_SD); the
// token-major tile is turned while it is read from LDS (ds_read_b64_tr_b8), so no transposed copy of V exists in HBM.
//
// Everything is computed transposed so that no operand ever passes through LDS or a cross-lane
// shuffle between the two matrix products:
//   S^T = K Q^T   v_mfma_f32_32x32x64_f8f6f4, A = 32 K rows x 64 d (LDS), B = Q^T (registers).
//                 An accumulator lane (q = lane%32, h = lane/32) then holds 16 keys of ONE query.
//   O^T = V^T P^T A = 32 d rows x 64 keys of V^T (LDS), B = P^T: the 2 x 16 probabilities of a lane,
//                 cast to e4m3, ARE the 32-byte B operand of that lane. For this the K rows are
//                 placed in LDS in the order in which the S^T accumulator rows come out, such that
//                 lane half h owns keys 32h .. 32h+31 of the tile in operand byte order.
// Softmax runs in the log2 domain in fp32: p = exp2(s * c - m + 8), c = softmax_scale * log2(e), m the running row
// maximum; the row sum accumulates the unrounded p while e4m3_sat(p) multiplies V (csrc/flash_attention/
// flash_attention_cuda.cu:197-221,437). The factor 2^8 cancels in O / l; it places the row maximum at 256 so
// that probabilities down to 2^-14 of the maximum stay in the normal range of e4m3 (with the reference's p <= 1
// everything below 2^-10 is flushed to zero, which biases long, flat rows). Q8_ATTN_P_UNIT_RANGE restores p <= 1.
// Q8_ATTN_LAZY_MAX lets m trail the running maximum: it is raised only when the running maximum exceeds it by more than
// 3 (p = exp2(s * c - m + 5) <= 2^8 still), so the rescaling of O and l by 2^(m_old - m_new), which otherwise runs in every
// tile that raises the maximum of one of the wave's 32 rows, is paid in the first tiles and hardly ever after. The same
// error bound holds, but the largest weight of a row is no longer a power of two, i.e. no longer exact: on sharply
// peaked rows the mean error grows by about two thirds, which is why it is not the default.
// Tiles that lie entirely beyond the valid KV length are
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
    int64_t v_row_stride;  // V^T row stride in elements (>= N, multiple of 16); unused for token-major V
    float scale_log2;      // softmax_scale * log2(e)
    float p_shift;         // probabilities are formed as 2^(x - m + p_shift), m = the row's reference maximum
    float m_slack;         // m is raised to the running maximum once that exceeds it by more than m_slack (0: m is the running maximum)
    int flags;
};

__device__ __attribute__((aligned(16))) const uint32_t g_attn_zero16[4] = {0, 0, 0, 0};

constexpr int kKV = 64;         // keys per tile
constexpr int kStage = 8192;    // K tile 4 KiB + V^T tile 4 KiB
constexpr int kStages = 4;      // LDS ring: one tile being read, up to three in flight
constexpr float kMaxSlack = 3.f;  // Q8_ATTN_LAZY_MAX: log2 units by which a row's running maximum may exceed its reference maximum

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ds_read_b64_tr_b8: the 16 lanes of a group name an 8 x 16 byte matrix M (lane 2 r + c points at M[r][8 c .. 8 c + 7]) and
// lane i of the group receives its column i, M[0..7][i]. Like lds_read_b128 the read is invisible to the compiler's
// wait-count insertion: an s_waitcnt lgkmcnt that names the result must follow.
template <int OFFSET>
__device__ __forceinline__ v2i lds_read_tr_b64(unsigned addr) {
    v2i r;
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET) : "memory");
    return r;
}

// Output stage shared by the attention kernels. The O^T accumulators of a 32-query tile: lane (q, h), tile d, register e
// holds dim 32 d + 8 (e / 4) + 4 h + (e % 4) of query q, i.e. the two lanes of a query hold alternate groups of 4 dims.
// One v_permlane32_swap per packed word hands every lane 8 consecutive dims (lane half 0 those of the even groups of 8,
// lane half 1 the odd ones), so a lane stores 16 bytes of bf16 (8 bytes of e4m3) and the two lanes of a query 32 (16)
// contiguous bytes per instruction: half as many, twice as large write requests as storing the groups of 4 directly
// (e4m3: a second exchange, 16 bytes per lane as well).
template <int OUT>
__device__ __forceinline__ void store_o_tile(void* o, size_t row_off, int h, const v16f (&o_acc)[2], float inv, bool live) {
#pragma unroll
    for (int d = 0; d < 2; ++d) {
        uint32_t c8[2][2];  // e4m3: [wp] the 8 codes of dims 32 d + 16 wp + 8 h .. + 7
#pragma unroll
        for (int wp = 0; wp < 2; ++wp) {  // the pair of 8-dim groups 2 wp, 2 wp + 1 of this 32-dim tile
            float a[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = o_acc[d][8 * wp + e] * inv;
            // before: a[0..3] = dims 16 wp + 4 h + 0..3, a[4..7] = dims 16 wp + 8 + 4 h + 0..3 (relative to 32 d)
            const int dim = 32 * d + 16 * wp + 8 * h;  // after: 8 consecutive dims from here
            if constexpr (OUT == Q8_BF16) {
                const auto s0 = __builtin_amdgcn_permlane32_swap(pack2_bf16(a[0], a[1]), pack2_bf16(a[4], a[5]), false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(pack2_bf16(a[2], a[3]), pack2_bf16(a[6], a[7]), false, false);
                if (live) *reinterpret_cast<v4u*>(reinterpret_cast<uint16_t*>(o) + row_off + dim) = v4u{s0[0], s1[0], s0[1], s1[1]};
            } else {
                const auto s0 = __builtin_amdgcn_permlane32_swap(pack4_e4m3_sat(a[0], a[1], a[2], a[3]),
                                                                 pack4_e4m3_sat(a[4], a[5], a[6], a[7]), false, false);
                c8[wp][0] = s0[0];
                c8[wp][1] = s0[1];
            }
        }
        if constexpr (OUT != Q8_BF16) {
            // a second exchange of the same kind between the two 8-byte chunks: lane half 0 ends up with dims 32 d .. + 15,
            // lane half 1 with dims 32 d + 16 .. + 31, so every lane stores 16 bytes and the two lanes of a query 32
            const auto t0 = __builtin_amdgcn_permlane32_swap(c8[0][0], c8[1][0], false, false);
            const auto t1 = __builtin_amdgcn_permlane32_swap(c8[0][1], c8[1][1], false, false);
            if (live) *reinterpret_cast<v4u*>(reinterpret_cast<uint8_t*>(o) + row_off + 32 * d + 16 * h) = v4u{t0[0], t1[0], t0[1], t1[1]};
        }
    }
}

// kQT = 32-query tiles per wave, kWaves = waves per workgroup (4 or 8); a workgroup covers kWaves * kQT * 32 queries.
// VTOK: V is token-major ([B,H,N,64]).
// MSUM (Q8_ATTN_SUM_ROUNDED_P; unit scales, kQT = 1): the row sum is taken over the e4m3-rounded probabilities, by the
// matrix pipe: one v_mfma_f32_16x16x128_f8f6f4 per tile multiplies the P^T operand by a 16 x 128 matrix of ones and zeros.
// In that instruction lane l of an operand holds 32 of the 128 reduction indices (block g = l / 16) of row or column
// l % 16, and result register 0 of lane l is D[4 (l / 16)][l % 16]. P^T, laid out for the 32 x 32 product, puts query
// (l % 32), key half (l / 32) into lane l: column n of the 16 x 128 view meets query n in blocks 0 and 2 and query n + 16
// in blocks 1 and 3. With rows 0, 8 = ones on blocks {0, 2} and rows 4, 12 = ones on blocks {1, 3}, register 0 of EVERY
// lane receives the complete row sum (both key halves) of that lane's own query: no cross-lane step, and the 32
// additions per tile of the vector ALU are gone.
template <int OUT, bool SCALED, int kQT, int kWaves, bool VTOK = false, bool MSUM = false>
__global__ __launch_bounds__(kWaves * 64, (SCALED && kWaves == 4 && kQT == 1) ? 3 : (!SCALED && kWaves == 8 && kQT == 1) ? 4 : 1) void attn_fwd_kernel(const AttnParams p) {
    static_assert(!MSUM || (!SCALED && kQT == 1), "the matrix-pipe row sum is built for unit scales and one query tile per wave");
    constexpr int kBlockQ = kWaves * kQT * 32;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kStages * kStage];
    __shared__ __attribute__((aligned(256))) float lds_sc[SCALED ? kStages * 128 : 4];  // per stage: sk[64], sv[64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: what is derived from it stays off the VALU
    const int ql = lane & 31, h = lane >> 5;
    // Workgroups are handed to the 8 XCDs (each with an L2 of its own) round-robin in launch order. With the query blocks of
    // a (batch, head) next to each other in that order every L2 would see the keys and values of every (batch, head) in
    // flight (about 21 x 0.8 MB at S = 6144); instead the launch order is re-read so that all query blocks of a
    // (batch, head) run on one XCD, which then walks through its share of the (batch, head) pairs one after the other.
    int bx = blockIdx.x, bh = blockIdx.y;
    if ((gridDim.y & 7) == 0) {
        const int nx = gridDim.x, lin = bh * nx + bx, slot = lin >> 3;
        bh = (lin & 7) * (gridDim.y >> 3) + slot / nx;
        bx = slot - (slot / nx) * nx;
    }
    const int b = bh / p.H;
    const int M = p.M, N = p.N;
    int valid = N;
    if (p.kv_len) {
        const int len = p.kv_len[b];
        valid = len < N ? (len < 0 ? 0 : len) : N;
    }
    const uint8_t* Qg = p.q + (size_t)bh * M * 64;
    const uint8_t* Kg = p.k + (size_t)bh * N * 64;
    const uint8_t* Vg = p.v + (size_t)bh * 64 * (VTOK ? (size_t)N : (size_t)p.v_row_stride);
    const int q0 = bx * kBlockQ + wave * (kQT * 32);
    // output row r of this (batch, head): element offset o_base + r * o_rs
    const bool o_tok = (p.flags & Q8_ATTN_O_TOKEN_MAJOR) != 0;
    const size_t o_base = o_tok ? ((size_t)b * M * p.H + (size_t)(bh - b * p.H)) * 64 : (size_t)bh * M * 64;
    const size_t o_rs = o_tok ? (size_t)p.H * 64 : 64;

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
        // an all-zero query row has scale 0: kept strictly positive, so that a masked key's -inf times it stays -inf
        // instead of becoming NaN (the row then weighs its valid keys uniformly, as zero logits do)
        sqc[t] = SCALED ? fmaxf(p.sq[(size_t)bh * M + row] * p.scale_log2, 1.17549435e-38f) : p.scale_log2;
    }

    // copy plan: wave w fills LDS rows 16w .. 16w+15 of both tiles (64-byte rows, 4 chunks of 16 bytes,
    // physical chunk = logical chunk ^ ((row >> 2) & 3)).
    // (with 8 waves, waves 0..3 copy the K tile and waves 4..7 the V^T tile; with 4 waves every wave copies both)
    const int cw = wave & 3;
    const bool copy_k = (kWaves == 4) || wave < 4, copy_v = (kWaves == 4) || wave >= 4;
    const int crow = 16 * cw + (lane >> 2);
    const int cchunk = (lane & 3) ^ ((crow >> 2) & 3);
    // token-major V tile: LDS row = key of the tile, physical chunk = logical chunk ^ (2 * ((row >> 2) & 1)), which keeps
    // the 8 rows x 16 bytes that a 16-lane group of the transposing read touches on distinct banks
    const int vchunk = (lane & 3) ^ (((crow >> 2) & 1) << 1);
    int k_src_row;  // key index inside the tile held by LDS row `crow`
    {
        const int t = crow >> 5, i = crow & 31;
        k_src_row = 32 * ((i >> 2) & 1) + 16 * t + 4 * (i >> 3) + (i & 3);
    }
    // Every wave issues exactly one (4 waves: two) copy per tile, also for tiles past the end (from a block of
    // zeros into a free stage), so that "s_waitcnt vmcnt(n)" always means "all but the n youngest tiles".
    // A tile that lies wholly inside the sequence (all but the last one) takes its source addresses from a uniform base,
    // advanced on the scalar unit, plus a per-lane byte offset that never changes; only the last tile clamps its rows.
    const uint32_t k_off = (uint32_t)k_src_row * 64u + (uint32_t)cchunk * 16u;
    const bool v_off32 = VTOK || (uint64_t)p.v_row_stride * 64u < (1ull << 32);  // the per-lane V offset fits 32 bits
    const uint32_t v_off = VTOK ? (uint32_t)crow * 64u + (uint32_t)vchunk * 16u
                                : (uint32_t)crow * (uint32_t)p.v_row_stride + (uint32_t)cchunk * 16u;
    auto issue_loads = [&](int tile, bool real) {
        uint8_t* base = lds + (tile & (kStages - 1)) * kStage;
        const int kv0 = tile * kKV;
        const bool inside = real && kv0 + kKV <= N && v_off32 && (VTOK || (int64_t)kv0 + kKV <= p.v_row_stride);  // uniform
        const uint8_t* zero = reinterpret_cast<const uint8_t*>(g_attn_zero16);
        if (copy_k) {
            const uint8_t* ks;
            if (inside) {
                ks = (Kg + (size_t)kv0 * 64) + k_off;
            } else {
                int kr = kv0 + k_src_row;
                kr = kr < N ? kr : N - 1;
                ks = real ? Kg + (size_t)kr * 64 + cchunk * 16 : zero;
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ks,
                                             (__attribute__((address_space(3))) void*)(base + cw * 1024), 16, 0, 0);
        }
        if (copy_v) {
            const uint8_t* vs;
            if (inside) {
                vs = (VTOK ? Vg + (size_t)kv0 * 64 : Vg + kv0) + v_off;
            } else if constexpr (VTOK) {
                int vr = kv0 + crow;
                vr = vr < N ? vr : N - 1;  // rows past the end repeat the last key; their probabilities are zero
                vs = real ? Vg + (size_t)vr * 64 + vchunk * 16 : zero;
            } else {
                const int col = kv0 + cchunk * 16;
                vs = (real && col < p.v_row_stride) ? (Vg + (size_t)crow * p.v_row_stride + col) : zero;
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vs,
                                             (__attribute__((address_space(3))) void*)(base + 4096 + cw * 1024), 16, 0, 0);
        }
        if constexpr (SCALED) {
            if (wave == 0) {  // the 64 key scales and value scales of the tile, one dword per lane
                const float* zf = reinterpret_cast<const float*>(g_attn_zero16);
                float* dst = lds_sc + (tile & (kStages - 1)) * 128;
                const float *ksrc, *vsrc;
                if (inside) {  // uniform base of the tile + the lane's dword
                    const uint32_t lane4 = (uint32_t)lane * 4u;
                    ksrc = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(p.sk + (size_t)bh * N + kv0) + lane4);
                    vsrc = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(p.sv + (size_t)bh * N + kv0) + lane4);
                } else {
                    int key = kv0 + lane;
                    key = key < N ? key : N - 1;
                    ksrc = real ? p.sk + (size_t)bh * N + key : zf;
                    vsrc = real ? p.sv + (size_t)bh * N + key : zf;
                }
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ksrc,
                                                 (__attribute__((address_space(3))) void*)dst, 4, 0, 0);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vsrc,
                                                 (__attribute__((address_space(3))) void*)(dst + 64), 4, 0, 0);
            }
        }
    };

    // operand fetch: lane (i = lane%32, h) reads chunks 2h, 2h+1 of row (32 t + i)
    const unsigned fbase = lds_addr(lds) + ql * 64;
    const unsigned fpc0 = ((2 * h) ^ ((ql >> 2) & 3)) * 16, fpc1 = fpc0 ^ 16;
    // token-major V: the 16-lane group (a = (lane / 16) % 2, h) turns, per read, keys 32 h + 8 j .. + 7 x channels
    // 32 d + 16 a .. + 15; lane l of the group points at key row l / 2, half l % 2 of the 16 channel bytes
    unsigned vtb[2];
    {
        const int l16 = lane & 15, a = (lane >> 4) & 1, f = ((l16 >> 3) & 1) << 1;  // f: swizzle of row l16 / 2 (+ multiples of 8)
        const unsigned row_off = (unsigned)(32 * h + (l16 >> 1)) * 64 + (l16 & 1) * 8;
        vtb[0] = lds_addr(lds) + 4096 + row_off + ((0 + a) ^ f) * 16;
        vtb[1] = lds_addr(lds) + 4096 + row_off + ((2 + a) ^ f) * 16;
    }

    v16f o_acc[kQT][2];
#pragma unroll
    for (int t = 0; t < kQT; ++t)
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int e = 0; e < 16; ++e) o_acc[t][d][e] = 0.f;
    float m_run[kQT], l_run[kQT];
    float m_thr[kQT], m_sub[kQT];  // m_run + m_slack (the threshold of the next move), m_run - exp_bias: kept beside m_run, they change with it
#pragma unroll
    for (int t = 0; t < kQT; ++t) { m_run[t] = m_thr[t] = m_sub[t] = -INFINITY; l_run[t] = 0.f; }
    v4f l_acc = {0.f, 0.f, 0.f, 0.f};  // MSUM: [0] = row sum of this lane's query
    v8i ones;                          // MSUM: this lane's 32 bytes of the ones-and-zeros matrix (e4m3 1.0 = 0x38)
    {
        const int mrow = lane & 15, blk = lane >> 4;
        const int on = ((mrow & 3) == 0 && ((mrow >> 2) & 1) == (blk & 1)) ? 0x38383838 : 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) ones[w] = on;
    }
    (void)l_acc; (void)ones;

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
        sv_ref = red[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) sv_ref = fmaxf(sv_ref, red[w]);
        sv_inv = sv_ref > 0.f ? 1.0f / sv_ref : 1.f;
    }
    // 2^p_shift / max_j sv_j, as an exponent: p' = 2^(x - m + p_shift) / svmax, P = e4m3(p' sv_j) <= 2^p_shift, l' = sum p';
    // the factor svmax then comes out of O / l' by itself.
    const float exp_bias = p.p_shift + (SCALED ? __builtin_log2f(sv_inv) : 0.f);
    (void)sv_ref;

    if (n_tiles > 0) {
        issue_loads(0, true);
        issue_loads(1, 1 < n_tiles);
        issue_loads(2, 2 < n_tiles);
    }
    for (int it = 0; it < n_tiles; ++it) {
        const int kv0 = it * kKV;
        // tile `it` has landed (the two younger tiles may still be in flight) - for every wave after the barrier,
        // which also says that all waves are done reading tile it-1, whose stage the next copy overwrites
        {
            const int per_tile = (kWaves == 4 ? 2 : 1) + ((SCALED && wave == 0) ? 2 : 0);  // copies this wave issues per tile
            if (per_tile == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
            else if (per_tile == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else if (per_tile == 3) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();
        issue_loads(it + 3, it + 3 < n_tiles);
        const unsigned st = fbase + (it & (kStages - 1)) * kStage;
        const unsigned so = (it & (kStages - 1)) * kStage;
        const unsigned sc = lds_addr(lds_sc) + (it & (kStages - 1)) * 512 + 128 * h;
        (void)so; (void)sc;
        // The LDS reads of a tile. Unit scales: K and V operands together, one wait. Per-token scales: K and the 32 key
        // scales of this lane first (the logits wait for the K operand only, the scales arrive under the two MFMAs); the
        // value scales and the V operand are requested once the logits have been scaled and arrive under the exponentials.
        v4i kl[2], kh[2], vl[2], vh[2], rk[SCALED ? 8 : 1], rv[SCALED ? 8 : 1];
        v2i vr[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            kl[t] = t ? lds_read_b128<2048>(st + fpc0) : lds_read_b128<0>(st + fpc0);
            kh[t] = t ? lds_read_b128<2048>(st + fpc1) : lds_read_b128<0>(st + fpc1);
        }
        auto read_v = [&]() __attribute__((always_inline)) {
            if constexpr (VTOK) {
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    vr[d][0] = lds_read_tr_b64<0>(so + vtb[d]);
                    vr[d][1] = lds_read_tr_b64<512>(so + vtb[d]);
                    vr[d][2] = lds_read_tr_b64<1024>(so + vtb[d]);
                    vr[d][3] = lds_read_tr_b64<1536>(so + vtb[d]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    vl[t] = t ? lds_read_b128<4096 + 2048>(st + fpc0) : lds_read_b128<4096>(st + fpc0);
                    vh[t] = t ? lds_read_b128<4096 + 2048>(st + fpc1) : lds_read_b128<4096>(st + fpc1);
                }
            }
        };
        // s_waitcnt lgkmcnt(0) that names the V operand registers, then the operand in MFMA form
        v8i kf[2], vf[2];
        auto wait_v = [&]() __attribute__((always_inline)) {
            if constexpr (VTOK) {
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(vr[0][0]), "+v"(vr[0][1]), "+v"(vr[0][2]), "+v"(vr[0][3]), "+v"(vr[1][0]), "+v"(vr[1][1]),
                               "+v"(vr[1][2]), "+v"(vr[1][3])
                             :
                             : "memory");
#pragma unroll
                for (int d = 0; d < 2; ++d)
                    vf[d] = v8i{vr[d][0][0], vr[d][0][1], vr[d][1][0], vr[d][1][1], vr[d][2][0], vr[d][2][1], vr[d][3][0], vr[d][3][1]};
            } else {
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vl[0]), "+v"(vh[0]), "+v"(vl[1]), "+v"(vh[1]) : : "memory");
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    vf[t] = v8i{vl[t][0], vl[t][1], vl[t][2], vl[t][3], vh[t][0], vh[t][1], vh[t][2], vh[t][3]};
            }
        };
        if constexpr (SCALED) {
            rk[0] = lds_read_b128<0>(sc); rk[1] = lds_read_b128<16>(sc); rk[2] = lds_read_b128<32>(sc); rk[3] = lds_read_b128<48>(sc);
            rk[4] = lds_read_b128<64>(sc); rk[5] = lds_read_b128<80>(sc); rk[6] = lds_read_b128<96>(sc); rk[7] = lds_read_b128<112>(sc);
            // LDS reads return in order: at most the 8 scale reads outstanding = the K operand is there
            asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(kl[0]), "+v"(kh[0]), "+v"(kl[1]), "+v"(kh[1]) : : "memory");
        } else {
            read_v();
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kl[0]), "+v"(kh[0]), "+v"(kl[1]), "+v"(kh[1]) : : "memory");
            wait_v();
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
            kf[t] = v8i{kl[t][0], kl[t][1], kl[t][2], kl[t][3], kh[t][0], kh[t][1], kh[t][2], kh[t][3]};

        // per-key scales of this lane's 32 keys (key = kv0 + 32h + e): broadcast reads from the stage's scale rows
        float skv[SCALED ? 32 : 1], svv[SCALED ? 32 : 1];
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
            if constexpr (SCALED) {
                if (qt == 0) {
                    asm volatile("s_waitcnt lgkmcnt(0)"
                                 : "+v"(rk[0]), "+v"(rk[1]), "+v"(rk[2]), "+v"(rk[3]), "+v"(rk[4]), "+v"(rk[5]), "+v"(rk[6]), "+v"(rk[7])
                                 :
                                 : "memory");
#pragma unroll
                    for (int e = 0; e < 32; ++e) skv[e] = __int_as_float(rk[e >> 2][e & 3]);
                }
            }
            // logits in units of log2: x = s * c (c > 0); the maximum is taken on the raw accumulators
            float x[32];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) x[16 * t + e] = SCALED ? s[t][e] * skv[16 * t + e] : s[t][e];
            if constexpr (SCALED) {
                if (qt == 0) {
                    // the scaled logits exist (with one query tile per wave the key scales and the K operand are dead now):
                    // the value scales and the V operand are requested and arrive under the exponentials
                    asm volatile("" : "+v"(x[15]), "+v"(x[31]));
                    rv[0] = lds_read_b128<256>(sc); rv[1] = lds_read_b128<272>(sc); rv[2] = lds_read_b128<288>(sc); rv[3] = lds_read_b128<304>(sc);
                    rv[4] = lds_read_b128<320>(sc); rv[5] = lds_read_b128<336>(sc); rv[6] = lds_read_b128<352>(sc); rv[7] = lds_read_b128<368>(sc);
                    read_v();
                }
            }
            if (partial) {
#pragma unroll
                for (int e = 0; e < 32; ++e)
                    if (kv0 + 32 * h + e >= valid) x[e] = -INFINITY;
            }
            float mx = max_ieee(x[0], x[1]);
#pragma unroll
            for (int e = 2; e < 32; e += 2) mx = max_ieee(max_ieee(mx, x[e]), x[e + 1]);
            mx = half_pair_max(mx);
            const float c = sqc[qt];
            // The reference maximum m of a row moves (and O, l are rescaled) only when the tile's maximum exceeds it by
            // more than m_slack (0 unless Q8_ATTN_LAZY_MAX: the running maximum), so p <= 2^(p_shift + m_slack). Each
            // row decides for itself (its result does not depend on the rows it shares a wave with); the wave skips
            // the multiplications when no row moves.
            const float mxc = mx * c;
            const bool grow = mxc > (MSUM ? m_run[qt] + p.m_slack : m_thr[qt]);  // (MSUM is short of registers: it recomputes the two)
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
                const float alpha = grow ? fast_exp2(m_run[qt] - mxc) : 1.f;
                m_run[qt] = grow ? mxc : m_run[qt];
                if constexpr (!MSUM) {
                    m_thr[qt] = m_run[qt] + p.m_slack;
                    m_sub[qt] = m_run[qt] - exp_bias;
                }
                if constexpr (MSUM) l_acc[0] *= alpha; else l_run[qt] *= alpha;
#pragma unroll
                for (int d = 0; d < 2; ++d)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o_acc[qt][d][e] *= alpha;
            }
            const float ms = MSUM ? m_run[qt] - exp_bias : m_sub[qt];
            float psum = 0.f;
            float pr[32];
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                pr[e] = fast_exp2(fmaf(x[e], c, -ms));   // <= 2^(p_shift + m_slack) = 2^8 or 1: inside the e4m3 range
                if constexpr (!MSUM) psum = e ? psum + pr[e] : pr[0];
            }
            if constexpr (SCALED) {
                if (qt == 0) {
                    asm volatile("s_waitcnt lgkmcnt(0)"
                                 : "+v"(rv[0]), "+v"(rv[1]), "+v"(rv[2]), "+v"(rv[3]), "+v"(rv[4]), "+v"(rv[5]), "+v"(rv[6]), "+v"(rv[7])
                                 :
                                 : "memory");
                    wait_v();
#pragma unroll
                    for (int e = 0; e < 32; ++e) svv[e] = __int_as_float(rv[e >> 2][e & 3]);
                }
#pragma unroll
                for (int e = 0; e < 32; ++e) pr[e] *= svv[e];
            }
            v8i pf;
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                uint32_t u = cvt_pk_e4m3(pr[4 * w], pr[4 * w + 1], any_u32(), false);
                u = cvt_pk_e4m3(pr[4 * w + 2], pr[4 * w + 3], u, true);
                pf[w] = (int)u;
            }
            if constexpr (MSUM) l_acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf, l_acc, 0, 0, 0, 0, 0, 0);
            else l_run[qt] += psum;
#pragma unroll
            for (int d = 0; d < 2; ++d)
                o_acc[qt][d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[d], pf, o_acc[qt][d], 0, 0, 0, 0, 0, 0);
        }
    }

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // look-ahead copies of the last tiles

    // ---- finalize: O^T lane (q, h), tile d, register e holds dim 32 d + 8 (e/4) + 4 h + (e%4)
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        const int row = q0 + 32 * qt + ql;
        const float l = MSUM ? l_acc[0] : l_run[qt] + lane_xor<32>(l_run[qt]);
        const float inv = (l == 0.f || l != l) ? 1.f : 1.f / l;
        store_o_tile<OUT>(p.o, o_base + (size_t)row * o_rs, h, o_acc[qt], inv, row < M);
    }
}

// One 32-query tile of attn_short_kernel against NB key blocks that lie in LDS at `st` (lane's row address; `so` the same
// without the lane's row: base of the transposing V reads).
// SCALED: `c` = sq[query] * scale_log2 of this lane's query, `bias` the exponent bias (p_shift + m_slack + log2(1 / max sv)),
// `sc` the LDS address of this lane half's 32 key scales of block 0 (value scales 512 bytes further, block 1 256 bytes
// further): the per-token scales enter as in attn_fwd_kernel.
template <int OUT, bool VTOK, bool SCALED, int NB>
__device__ __forceinline__ void short_tile(const AttnParams& p, const v8i& qf, unsigned st, unsigned so, unsigned fpc0, unsigned fpc1,
                                           const unsigned (&vtb)[2], int valid, uint32_t keep, int h, size_t row_off, bool live,
                                           float c, float bias, unsigned sc) {
    v4i kl[NB][2], kh[NB][2];
#pragma unroll
    for (int kb = 0; kb < NB; ++kb)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            kl[kb][t] = t ? lds_read_b128<2048>(st + kb * kStage + fpc0) : lds_read_b128<0>(st + kb * kStage + fpc0);
            kh[kb][t] = t ? lds_read_b128<2048>(st + kb * kStage + fpc1) : lds_read_b128<0>(st + kb * kStage + fpc1);
        }
    if constexpr (NB == 2)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(kl[0][0]), "+v"(kh[0][0]), "+v"(kl[0][1]), "+v"(kh[0][1]), "+v"(kl[NB - 1][0]), "+v"(kh[NB - 1][0]),
                       "+v"(kl[NB - 1][1]), "+v"(kh[NB - 1][1])
                     :
                     : "memory");
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kl[0][0]), "+v"(kh[0][0]), "+v"(kl[0][1]), "+v"(kh[0][1]) : : "memory");
    float x[NB][32];
#pragma unroll
    for (int kb = 0; kb < NB; ++kb)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const v8i kf = v8i{kl[kb][t][0], kl[kb][t][1], kl[kb][t][2], kl[kb][t][3], kh[kb][t][0], kh[kb][t][1], kh[kb][t][2], kh[kb][t][3]};
            v16f z;
#pragma unroll
            for (int e = 0; e < 16; ++e) z[e] = 0.f;
            const v16f s = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf, qf, z, 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 16; ++e) x[kb][16 * t + e] = s[e];
        }
    if constexpr (SCALED) {
        // the key scales of this lane's 32 keys per block (broadcast reads) multiply the raw logits
#pragma unroll
        for (int kb = 0; kb < NB; ++kb) {
            v4i rk[8];
            rk[0] = lds_read_b128<0>(sc + kb * 256); rk[1] = lds_read_b128<16>(sc + kb * 256);
            rk[2] = lds_read_b128<32>(sc + kb * 256); rk[3] = lds_read_b128<48>(sc + kb * 256);
            rk[4] = lds_read_b128<64>(sc + kb * 256); rk[5] = lds_read_b128<80>(sc + kb * 256);
            rk[6] = lds_read_b128<96>(sc + kb * 256); rk[7] = lds_read_b128<112>(sc + kb * 256);
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(rk[0]), "+v"(rk[1]), "+v"(rk[2]), "+v"(rk[3]), "+v"(rk[4]), "+v"(rk[5]), "+v"(rk[6]), "+v"(rk[7])
                         :
                         : "memory");
#pragma unroll
            for (int e = 0; e < 32; ++e) x[kb][e] *= __int_as_float(rk[e >> 2][e & 3]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // Masking in the last block that holds valid keys (the only one that can be partial): bit e of `keep` says that this
    // lane's key e of that block is valid; a sign-extending bit-field extract and a bit select per logit, no comparison
    // (32 independent comparisons would each hold a pair of scalar registers).
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NB; ++kb) {
        if (kb == NB - 1 && 64 * NB > valid) {
            // (the mask passes through an empty asm: the 64 words derived from it would otherwise be computed once,
            //  outside the tile loop, and held in registers)
            asm volatile("" : "+v"(keep));
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)keep, e, 1);  // all ones: keep
                x[kb][e] = __uint_as_float((__float_as_uint(x[kb][e]) & m) | (0xff800000u & ~m));
            }
        }
#pragma unroll
        for (int e = 0; e < 32; e += 2) mx = max_ieee(max_ieee(mx, x[kb][e]), x[kb][e + 1]);
    }
    mx = half_pair_max(mx);
    const float m_sub = mx * c - bias;  // the final maximum is known: the slack of Q8_ATTN_LAZY_MAX is head room not needed
    float psum = 0.f, psum_rounded = 0.f;
    v16f o_acc[2];
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[d][e] = 0.f;
#pragma unroll
    for (int kb = 0; kb < NB; ++kb) {
        // (scheduling fence: the second block's exponentials and reads stay behind the first block's products, which keeps
        //  the live registers at one block's worth)
        __builtin_amdgcn_sched_barrier(0);
        // the V operand of this block is requested now and arrives under the block's exponentials
        v4i vl[2], vh[2];
        v2i vr[2][4];
        (void)vl; (void)vh; (void)vr;
        if constexpr (VTOK) {
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                vr[d][0] = lds_read_tr_b64<0>(so + kb * kStage + vtb[d]);
                vr[d][1] = lds_read_tr_b64<512>(so + kb * kStage + vtb[d]);
                vr[d][2] = lds_read_tr_b64<1024>(so + kb * kStage + vtb[d]);
                vr[d][3] = lds_read_tr_b64<1536>(so + kb * kStage + vtb[d]);
            }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                vl[t] = t ? lds_read_b128<4096 + 2048>(st + kb * kStage + fpc0) : lds_read_b128<4096>(st + kb * kStage + fpc0);
                vh[t] = t ? lds_read_b128<4096 + 2048>(st + kb * kStage + fpc1) : lds_read_b128<4096>(st + kb * kStage + fpc1);
            }
        }
        v4i rv[SCALED ? 8 : 1];
        if constexpr (SCALED) {
            rv[0] = lds_read_b128<512>(sc + kb * 256); rv[1] = lds_read_b128<528>(sc + kb * 256);
            rv[2] = lds_read_b128<544>(sc + kb * 256); rv[3] = lds_read_b128<560>(sc + kb * 256);
            rv[4] = lds_read_b128<576>(sc + kb * 256); rv[5] = lds_read_b128<592>(sc + kb * 256);
            rv[6] = lds_read_b128<608>(sc + kb * 256); rv[7] = lds_read_b128<624>(sc + kb * 256);
        }
        v8i pf;
        float pr[32];
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            pr[e] = fast_exp2(fmaf(x[kb][e], c, -m_sub));
            psum += pr[e];
        }
        if constexpr (SCALED) {
            // (the V operand reads were issued before these: in-order return, so this wait covers them as well)
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(rv[0]), "+v"(rv[1]), "+v"(rv[2]), "+v"(rv[3]), "+v"(rv[4]), "+v"(rv[5]), "+v"(rv[6]), "+v"(rv[7])
                         :
                         : "memory");
#pragma unroll
            for (int e = 0; e < 32; ++e) pr[e] *= __int_as_float(rv[e >> 2][e & 3]);
        }
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            uint32_t u = cvt_pk_e4m3(pr[4 * w], pr[4 * w + 1], any_u32(), false);
            u = cvt_pk_e4m3(pr[4 * w + 2], pr[4 * w + 3], u, true);
            pf[w] = (int)u;
        }
        if (p.flags & Q8_ATTN_SUM_ROUNDED_P) {
#pragma unroll
            for (int w = 0; w < 8; ++w)
                psum_rounded += e4m3_to_f32<0>(pf[w]) + e4m3_to_f32<1>(pf[w]) + e4m3_to_f32<2>(pf[w]) + e4m3_to_f32<3>(pf[w]);
        }
        // (the probabilities pass through the wait as well: the exponentials stay above it, under the reads' latency)
        if constexpr (VTOK) {
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(vr[0][0]), "+v"(vr[0][1]), "+v"(vr[0][2]), "+v"(vr[0][3]), "+v"(vr[1][0]), "+v"(vr[1][1]),
                           "+v"(vr[1][2]), "+v"(vr[1][3]), "+v"(pf)
                         :
                         : "memory");
        } else {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vl[0]), "+v"(vh[0]), "+v"(vl[1]), "+v"(vh[1]), "+v"(pf) : : "memory");
        }
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            v8i vf;
            if constexpr (VTOK)
                vf = v8i{vr[d][0][0], vr[d][0][1], vr[d][1][0], vr[d][1][1], vr[d][2][0], vr[d][2][1], vr[d][3][0], vr[d][3][1]};
            else
                vf = v8i{vl[d][0], vl[d][1], vl[d][2], vl[d][3], vh[d][0], vh[d][1], vh[d][2], vh[d][3]};
            o_acc[d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf, o_acc[d], 0, 0, 0, 0, 0, 0);
        }
    }
    // ---- O^T lane (q, h), tile d, register e holds dim 32 d + 8 (e/4) + 4 h + (e%4)
    if (p.flags & Q8_ATTN_SUM_ROUNDED_P) psum = psum_rounded;
    const float l = psum + lane_xor<32>(psum);
    const float inv = (l == 0.f || l != l) ? 1.f : 1.f / l;
    store_o_tile<OUT>(p.o, row_off, h, o_acc, inv, live);
}

// Short key / value sequences (N <= 128: cross-attention to a text prompt, csrc/flash_attention/
// flash_attention_cuda_mask.cu:254-535 in the reference). The whole K and V of a (batch, head) are 16 KiB: they are copied
// to LDS once, in the tile layouts of attn_fwd_kernel (two 64-key blocks), and every wave of the workgroup walks over
// several 32-query tiles with them, so a tile costs one 2 KiB read of Q (requested one tile ahead), 16 operand reads from
// LDS and one store of O. All keys of a query are present at once: no running maximum, the probabilities are rounded
// against the final maximum like the oracle's. Operand layouts, masking, P rounding and the output stage are those of
// attn_fwd_kernel; a 64-key block beyond the valid length is skipped. A workgroup (4 waves, three per CU) belongs to one
// head and takes its share of the queries of EVERY batch in turn - the valid lengths differ per batch, and with a
// workgroup per (batch, head) the launch would last as long as its longest batch - and while it works on one batch the
// K / V of the next one are already on their way into the other half of the LDS buffer.
template <int OUT, bool VTOK, bool SCALED>
__global__ __launch_bounds__(256, (SCALED || VTOK) ? 2 : 3) void attn_short_kernel(const AttnParams p, int tiles_per_wave) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * 2 * kStage];  // [batch parity][key block]: K tile, V tile
    __shared__ __attribute__((aligned(256))) float lds_sc[SCALED ? 2 * 256 : 4];  // [batch parity]: sk[128], sv[128]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int M = p.M, N = p.N, head = blockIdx.y;
    const bool o_tok = (p.flags & Q8_ATTN_O_TOKEN_MAJOR) != 0;
    const size_t o_rs = o_tok ? (size_t)p.H * 64 : 64;
    const int q_tiles = (M + 31) >> 5;
    const int tile0 = blockIdx.x * (4 * tiles_per_wave) + wave;  // this wave's tiles: tile0 + 4 it

    auto valid_of = [&](int b) {
        if (!p.kv_len) return N;
        const int len = p.kv_len[b];
        return len < N ? (len < 0 ? 0 : len) : N;
    };
    // copy plan of attn_fwd_kernel with 4 waves: wave w fills LDS rows 16 w .. 16 w + 15 of the K tile and of the V tile of
    // both key blocks, 4 copies per wave and batch (blocks without valid keys are filled from a block of zeros, so that
    // every wave always issues the same number of copies)
    const int crow = 16 * wave + (lane >> 2);
    const int cchunk = (lane & 3) ^ ((crow >> 2) & 3);
    const int vchunk = (lane & 3) ^ (((crow >> 2) & 1) << 1);
    int k_src_row;
    {
        const int t = crow >> 5, i = crow & 31;
        k_src_row = 32 * ((i >> 2) & 1) + 16 * t + 4 * (i >> 3) + (i & 3);
    }
    auto issue_copies = [&](int b) {
        const int bh = b * p.H + head;
        const uint8_t* Kg = p.k + (size_t)bh * N * 64;
        const uint8_t* Vg = p.v + (size_t)bh * 64 * (VTOK ? (size_t)N : (size_t)p.v_row_stride);
        const int n_blocks = (valid_of(b) + 63) >> 6;
        const uint8_t* zero = reinterpret_cast<const uint8_t*>(g_attn_zero16);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            uint8_t* base = lds + ((b & 1) * 2 + kb) * kStage;
            const bool real = kb < n_blocks;
            int kr = 64 * kb + k_src_row;
            kr = kr < N ? kr : N - 1;
            const uint8_t* ks = real ? Kg + (size_t)kr * 64 + cchunk * 16 : zero;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ks,
                                             (__attribute__((address_space(3))) void*)(base + wave * 1024), 16, 0, 0);
            const uint8_t* vs;
            if constexpr (VTOK) {
                int vr = 64 * kb + crow;
                vr = vr < N ? vr : N - 1;  // rows past the end repeat the last key; their probabilities are zero
                vs = real ? Vg + (size_t)vr * 64 + vchunk * 16 : zero;
            } else {
                const int col = 64 * kb + cchunk * 16;
                vs = (real && col < p.v_row_stride) ? (Vg + (size_t)crow * p.v_row_stride + col) : zero;
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vs,
                                             (__attribute__((address_space(3))) void*)(base + 4096 + wave * 1024), 16, 0, 0);
        }
        if constexpr (SCALED) {
            if (wave < 2) {  // wave kb copies the 64 key scales and the 64 value scales of block kb, one dword per lane
                int key = 64 * wave + lane;
                key = key < N ? key : N - 1;
                const bool real = wave < n_blocks;
                const float* zf = reinterpret_cast<const float*>(g_attn_zero16);
                float* dst = lds_sc + (b & 1) * 256 + 64 * wave;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(real ? p.sk + (size_t)bh * N + key : zf),
                                                 (__attribute__((address_space(3))) void*)dst, 4, 0, 0);
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(real ? p.sv + (size_t)bh * N + key : zf),
                                                 (__attribute__((address_space(3))) void*)(dst + 128), 4, 0, 0);
            }
        }
    };
    // operand fetch addresses inside a key block (as in attn_fwd_kernel)
    const unsigned fbase = lds_addr(lds) + ql * 64;
    const unsigned fpc0 = ((2 * h) ^ ((ql >> 2) & 3)) * 16, fpc1 = fpc0 ^ 16;
    unsigned vtb[2];
    {
        const int l16 = lane & 15, a = (lane >> 4) & 1, f = ((l16 >> 3) & 1) << 1;
        const unsigned row_off = (unsigned)(32 * h + (l16 >> 1)) * 64 + (l16 & 1) * 8;
        vtb[0] = lds_addr(lds) + 4096 + row_off + ((0 + a) ^ f) * 16;
        vtb[1] = lds_addr(lds) + 4096 + row_off + ((2 + a) ^ f) * 16;
    }
    auto load_q = [&](int b, int tile) {  // Q^T operand: lane (q, h) holds bytes 32 h .. 32 h + 31 of query row q
        int row = 32 * tile + ql;
        row = row < M ? row : M - 1;
        const v4i* src = reinterpret_cast<const v4i*>(p.q + ((size_t)(b * p.H + head) * M + row) * 64 + 32 * h);
        const v4i a = src[0], c = src[1];
        return v8i{a[0], a[1], a[2], a[3], c[0], c[1], c[2], c[3]};
    };
    // per-token scales: c of a tile's query, kept strictly positive like in attn_fwd_kernel (a masked key's -inf stays -inf)
    auto load_c = [&](int b, int tile) {
        if constexpr (!SCALED) return p.scale_log2;
        int row = 32 * tile + ql;
        row = row < M ? row : M - 1;
        return fmaxf(p.sq[(size_t)(b * p.H + head) * M + row] * p.scale_log2, 1.17549435e-38f);
    };
    issue_copies(0);
    v8i qf = load_q(0, tile0 < q_tiles ? tile0 : 0);
    float cq = load_c(0, tile0 < q_tiles ? tile0 : 0);
    for (int b = 0; b < p.B; ++b) {
        // the copies of batch b (issued one batch ago) have landed - for every wave after the barrier, which also says that
        // all waves are done with batch b - 1, whose half of the buffer the next copies overwrite
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        if (b + 1 < p.B) issue_copies(b + 1);
        const int bh = b * p.H + head;
        const size_t o_base = o_tok ? ((size_t)b * M * p.H + (size_t)head) * 64 : (size_t)bh * M * 64;
        const int valid = valid_of(b);
        const int n_blocks = (valid + 63) >> 6;  // 64-key blocks that hold valid keys: 0, 1 or 2
        const unsigned buf = (b & 1) * 2 * kStage;
        // per-token V scales enter P as sv[j] / max_j sv[j] (maximum over the valid keys), the factor 1 / max as an exponent bias
        float bias = p.p_shift + p.m_slack;
        if constexpr (SCALED) {
            const float* sv = lds_sc + (b & 1) * 256 + 128;
            float mxv = fmaxf(lane < valid ? sv[lane] : 0.f, lane + 64 < valid ? sv[lane + 64] : 0.f);
            mxv = group_max<64>(mxv);
            bias += __builtin_log2f(mxv > 0.f ? 1.0f / mxv : 1.f);
        }
        const unsigned sc = lds_addr(lds_sc) + (b & 1) * 1024 + 128 * h;
        // valid keys among this lane's 32 of the last block with valid keys (keys 64 (n_blocks - 1) + 32 h + e), as a bit mask
        uint32_t keep = 0xffffffffu;
        {
            const int lim = valid - 64 * (n_blocks - 1) - 32 * h;
            keep = lim >= 32 ? 0xffffffffu : (lim <= 0 ? 0u : ((1u << lim) - 1u));
        }
        for (int it = 0; it < tiles_per_wave; ++it) {
            const int tile = tile0 + 4 * it;
            // the Q operand of this wave's next tile (of the next batch after the last one of this batch)
            const bool last_it = it + 1 == tiles_per_wave;
            const int nb = last_it ? (b + 1 < p.B ? b + 1 : b) : b;
            const int nt = last_it ? tile0 : tile + 4;
            const v8i qn = load_q(nb, nt < q_tiles ? nt : 0);
            const float cn = load_c(nb, nt < q_tiles ? nt : 0);
            if (tile < q_tiles) {
                const size_t row_off = o_base + (size_t)(32 * tile + ql) * o_rs;
                const bool live = 32 * tile + ql < M;
                // straight-line code per number of key blocks (uniform per batch)
                if (n_blocks == 2) short_tile<OUT, VTOK, SCALED, 2>(p, qf, fbase + buf, buf, fpc0, fpc1, vtb, valid, keep, h, row_off, live, cq, bias, sc);
                else if (n_blocks == 1) short_tile<OUT, VTOK, SCALED, 1>(p, qf, fbase + buf, buf, fpc0, fpc1, vtb, valid, keep, h, row_off, live, cq, bias, sc);
                else {  // no valid key at all: the output is zero
                    v16f o_acc[2];
#pragma unroll
                    for (int d = 0; d < 2; ++d)
#pragma unroll
                        for (int e = 0; e < 16; ++e) o_acc[d][e] = 0.f;
                    store_o_tile<OUT>(p.o, row_off, h, o_acc, 1.f, live);
                }
            }
            qf = qn;
            cq = cn;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace q8

using namespace q8;

// per thread: 0 = default (unit scales: 8 waves x 32 queries; per-token scales: 4 waves x 32 queries), 1 = 4 waves x 64
// queries, 2 = 4 waves x 32 queries, 3 = the default shape of the mode, 4 = 8 waves x 32 queries; 1 .. 4 all select the general
// kernel, also for N <= 128, which under 0 takes the short-sequence kernel
static thread_local int g_attn_cfg = 0;

extern "C" int q8_attn_set_config(int cfg) {
    if (cfg < 0 || cfg > 4) return fail(Q8_ERR_FLAGS, "q8_attn_set_config: %d", cfg);
    g_attn_cfg = cfg;
    return Q8_OK;
}

extern "C" int q8_attn_fwd(const void* q, const void* k, const void* v, void* o, const int32_t* kv_len, const float* sq,
                           const float* sk, const float* sv, int B, int H, int M, int N, int D, int v_layout,
                           int64_t v_row_stride, float softmax_scale, int out_dtype, int flags, q8_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (D != 64) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: head dim %d (only 64 is supported)", D);
    if (B < 0 || H <= 0 || M < 0 || N <= 0 || M > (1 << 30) || N > (1 << 30)) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: B %d H %d M %d N %d", B, H, M, N);
    if (B == 0 || M == 0) return Q8_OK;  // no queries: nothing to compute or to write
    if (!q || !k || !v || !o) return fail(Q8_ERR_NULL, "q8_attn_fwd: null pointer");
    if ((long)B * H > 65535) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: B*H = %ld exceeds 65535", (long)B * H);
    if (out_dtype != Q8_BF16 && out_dtype != Q8_E4M3) return fail(Q8_ERR_DTYPE, "q8_attn_fwd: output dtype %d", out_dtype);
    if (flags & ~(Q8_ATTN_SUM_ROUNDED_P | Q8_ATTN_P_UNIT_RANGE | Q8_ATTN_O_TOKEN_MAJOR | Q8_ATTN_LAZY_MAX)) return fail(Q8_ERR_FLAGS, "q8_attn_fwd: flags 0x%x", flags);
    if (v_layout != Q8_V_DS && v_layout != Q8_V_SD) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: V layout %d", v_layout);
    const bool vtok = v_layout == Q8_V_SD;
    if (!vtok && (v_row_stride < N || v_row_stride % 16 != 0))
        return fail(Q8_ERR_SHAPE, "q8_attn_fwd: V row stride %lld must be >= N and a multiple of 16", (long long)v_row_stride);
    const bool scaled = sq || sk || sv;
    if (scaled && !(sq && sk && sv)) return fail(Q8_ERR_NULL, "q8_attn_fwd: sq, sk, sv must be given together");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return fail(Q8_ERR_ALIGN, "q8_attn_fwd: q, k, v and o must be 16-byte aligned");
    if ((flags & Q8_ATTN_LAZY_MAX) && (flags & Q8_ATTN_P_UNIT_RANGE))
        return fail(Q8_ERR_FLAGS, "q8_attn_fwd: Q8_ATTN_LAZY_MAX needs the head room of the default probability range (not P_UNIT_RANGE)");
    if ((flags & Q8_ATTN_SUM_ROUNDED_P) && scaled)
        return fail(Q8_ERR_FLAGS, "q8_attn_fwd: Q8_ATTN_SUM_ROUNDED_P is defined for unit scales only (with per-token scales P carries V's scales)");
    const float slack = (flags & Q8_ATTN_LAZY_MAX) ? kMaxSlack : 0.f;
    AttnParams p{static_cast<const uint8_t*>(q), static_cast<const uint8_t*>(k), static_cast<const uint8_t*>(v), o, kv_len, sq, sk, sv,
                 B, H, M, N, v_row_stride, softmax_scale * 1.44269504088896340736f,
                 (flags & Q8_ATTN_P_UNIT_RANGE) ? 0.f : 8.f - slack, slack, flags};
    if (!(softmax_scale > 0.f)) return fail(Q8_ERR_SHAPE, "q8_attn_fwd: softmax_scale must be positive");
    const int cfg = g_attn_cfg;
    if (vtok && cfg == 1)
        return fail(Q8_ERR_FLAGS, "q8_attn_fwd: the 4 waves x 64 queries tuning shape reads V^T only (Q8_V_DS)");
    const bool msum = (flags & Q8_ATTN_SUM_ROUNDED_P) != 0;
    if (msum && cfg == 1)
        return fail(Q8_ERR_FLAGS, "q8_attn_fwd: the 4 waves x 64 queries tuning shape has no Q8_ATTN_SUM_ROUNDED_P form");
    if (N <= 128 && cfg == 0) {  // (a shape override always means the general kernel in that shape)
        // K and V stay in LDS; enough workgroups of 4 waves to fill every CU once (three per CU with unit scales and V^T,
        // whose code fits 168 registers, two otherwise), each wave walking over several query tiles of every batch
        const long q_tiles = (M + 31) / 32;
        const long wave_slots = (scaled || vtok) ? 2048 : 3072;
        long tpw = (q_tiles * H + wave_slots - 1) / wave_slots;
        tpw = tpw < 1 ? 1 : (tpw > 16 ? 16 : tpw);
        const unsigned gx = (unsigned)((q_tiles + 4 * tpw - 1) / (4 * tpw));
#define Q8_ATTN_SHORT_L(OUTT, VT, SC) \
    hipLaunchKernelGGL((attn_short_kernel<OUTT, VT, SC>), dim3(gx, (unsigned)H), dim3(256), 0, stream, p, (int)tpw)
#define Q8_ATTN_SHORT(OUTT)                                                                              \
    if (vtok) { if (scaled) Q8_ATTN_SHORT_L(OUTT, true, true); else Q8_ATTN_SHORT_L(OUTT, true, false); }  \
    else { if (scaled) Q8_ATTN_SHORT_L(OUTT, false, true); else Q8_ATTN_SHORT_L(OUTT, false, false); }
        if (out_dtype == Q8_BF16) { Q8_ATTN_SHORT(Q8_BF16) } else { Q8_ATTN_SHORT(Q8_E4M3) }
#undef Q8_ATTN_SHORT_L
#undef Q8_ATTN_SHORT
        return launch_status("q8_attn_fwd");
    }
    // Shapes: with unit scales 8 waves x 32 queries fit 128 registers (two workgroups = 4 waves per SIMD) and share a K / V
    // tile among 256 queries. With per-token scales a wave also holds the 64 scales of a tile and needs about 150 registers:
    // 4 waves x 32 queries then place three workgroups on a CU (3 waves per SIMD) where the 8-wave shape places one.
    const int waves = (cfg == 1 || cfg == 2) ? 4 : (cfg == 4 ? 8 : (scaled ? 4 : 8));
    const int qtiles = cfg == 1 ? 2 : 1;
#define Q8_ATTN_LAUNCH(OUTT, SC, QT, WV, VT, MS)                                                                           \
    hipLaunchKernelGGL((attn_fwd_kernel<OUTT, SC, QT, WV, VT, MS>), dim3((unsigned)((M + WV * QT * 32 - 1) / (WV * QT * 32)), \
                                                                          (unsigned)(B * H)), dim3(WV * 64), 0, stream, p)
#define Q8_ATTN_VT(OUTT, SC, WV, MS) \
    if (vtok) Q8_ATTN_LAUNCH(OUTT, SC, 1, WV, true, MS); else Q8_ATTN_LAUNCH(OUTT, SC, 1, WV, false, MS)
#define Q8_ATTN_CFG(OUTT, SC)                                     \
    if (qtiles == 2) Q8_ATTN_LAUNCH(OUTT, SC, 2, 4, false, false); \
    else if (waves == 4) { Q8_ATTN_VT(OUTT, SC, 4, false); }       \
    else { Q8_ATTN_VT(OUTT, SC, 8, false); }
#define Q8_ATTN_MSUM(OUTT) \
    if (waves == 4) { Q8_ATTN_VT(OUTT, false, 4, true); } else { Q8_ATTN_VT(OUTT, false, 8, true); }
    if (out_dtype == Q8_BF16) {
        if (msum) { Q8_ATTN_MSUM(Q8_BF16) } else if (scaled) { Q8_ATTN_CFG(Q8_BF16, true) } else { Q8_ATTN_CFG(Q8_BF16, false) }
    } else {
        if (msum) { Q8_ATTN_MSUM(Q8_E4M3) } else if (scaled) { Q8_ATTN_CFG(Q8_E4M3, true) } else { Q8_ATTN_CFG(Q8_E4M3, false) }
    }
#undef Q8_ATTN_MSUM
#undef Q8_ATTN_CFG
#undef Q8_ATTN_VT
#undef Q8_ATTN_LAUNCH
    return launch_status("q8_attn_fwd");
}
