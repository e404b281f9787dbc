// Attention core for float32 tensors (the reference's default `precision`): forward, delta, dK/dV, dQ.
//
// Exact fp32 semantics of core/nn/attention/attention.py:108-213 with an fp32 tensor dtype: scores, softmax,
// probabilities and both products in fp32 (probs.to(value.dtype) is the identity), on the fp32 matrix pipe
// (v_mfma_f32_32x32x2_f32, 157 TFLOP/s class, a sixteenth of the bf16 rate).  This is the completeness path for
// `precision: float32` models, not a tuned one: one wavefront per workgroup, 32 x 32 score tiles, every operand
// tile staged once in LDS with rows padded by one float (conflict-free for both the row-operand and the
// column-gather access), no software pipelining.  Same masks, GQA index math, layouts, lse and workspace contract
// as the 16-bit kernels; no dropout and no fused rotary (rotate with mi_rotary / mi_rotary_complex first).
//
// v_mfma_f32_32x32x2_f32 operands, lane = 32 g + l32:  A: row l32, k = g;  B: column l32, k = g;
// C / D: column l32, rows 8 (r / 4) + 4 g + r % 4 for r = 0..15.  A C tile is reused as the B operand of the next
// product one register at a time: register r contributes the two contraction indices 8 (r / 4) + r % 4 (lanes of
// g = 0) and 4 more (g = 1), and the A operand gathers exactly those two rows.
#include "attn_common.h"

namespace {

constexpr float kLog2eF = 1.4426950408889634f;

__device__ __forceinline__ f32x16_t mfma_f32(float a, float b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// row index inside a 32-row tile that accumulator register r stands for in lane half g
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

struct F32Params {
    const float* q; const float* k; const float* v; float* o; float* lse;
    const float* d_o; float* dq; float* dk; float* dv; float* delta;
    AttnParams m;     // masks, sizes, strides (the pointer members of m are not used)
};

// 32 rows x D floats, rows first_row .. first_row + 31 of `base` (row stride `st`, rows past last_row repeat it),
// into an LDS tile with LD = D + 1 floats per row; one wavefront, 128-bit global reads.
template <int D>
__device__ __forceinline__ void stage_tile(float* tile, const float* base, int64_t st, int first_row, int last_row, int lane) {
    constexpr int LD = D + 1, VPR = D / 4;
#pragma unroll
    for (int j = 0; j < 32 * VPR / 64; ++j) {
        const int idx = j * 64 + lane;
        const int row = idx / VPR, c4 = idx % VPR;
        int src_row = first_row + row;
        src_row = src_row < last_row ? src_row : last_row;
        src_row = src_row < 0 ? 0 : src_row;
        const f32x4_t x = *reinterpret_cast<const f32x4_t*>(base + (int64_t)src_row * st + 4 * c4);
        float* d = tile + row * LD + 4 * c4;
        d[0] = x[0]; d[1] = x[1]; d[2] = x[2]; d[3] = x[3];
    }
}

// C (+)= A B^T over the head dimension: A rows from tile_a (row l32), B rows from tile_b (row l32)
template <int D>
__device__ __forceinline__ f32x16_t rows_product(const float* tile_a, const float* tile_b, int l32, int g) {
    constexpr int LD = D + 1;
    f32x16_t c;
#pragma unroll
    for (int r = 0; r < 16; ++r) c[r] = 0.f;
    const float* ar = tile_a + l32 * LD + g;
    const float* br = tile_b + l32 * LD + g;
#pragma unroll 8
    for (int ks = 0; ks < D / 2; ++ks) c = mfma_f32(ar[2 * ks], br[2 * ks], c);
    return c;
}

// acc[dt] += gather(tile)^T x : contraction over the 32 rows of `tile`, x = a C tile used register by register
template <int D>
__device__ __forceinline__ void cols_product(f32x16_t (&acc)[D / 32], const float* tile, const f32x16_t& x, int l32, int g) {
    constexpr int LD = D + 1;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt] = mfma_f32(tile[acc_row(r, g) * LD + 32 * dt + l32], x[r], acc[dt]);
}

// lane (token, g): acc[dt][r] is feature 32 dt + 8 (r / 4) + 4 g + r % 4 of the token's row
template <int D>
__device__ __forceinline__ void store_rows(float* row, const f32x16_t (&acc)[D / 32], float scale, int g) {
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            f32x4_t x;
#pragma unroll
            for (int c = 0; c < 4; ++c) x[c] = acc[dt][4 * a + c] * scale;
            *reinterpret_cast<f32x4_t*>(row + 32 * dt + 8 * a + 4 * g) = x;
        }
}

__device__ __forceinline__ void wave_min_max(int& lo, int& hi) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off, 64));
        hi = max(hi, __shfl_xor(hi, off, 64));
    }
}

// ---- forward: a wavefront owns 32 queries of one head; S^T = K Q^T (lane = query), O^T += V^T P^T -----------------
template <int D>
__global__ __launch_bounds__(64) void attn_f32_fwd_kernel(const F32Params fp) {
    constexpr int LD = D + 1, DT = D / 32;
    __shared__ float q_s[32 * LD], k_s[32 * LD], v_s[32 * LD];
    const AttnParams& p = fp.m;
    const int lane = threadIdx.x, l32 = lane & 31, g = lane >> 5;
    const int head = blockIdx.x % p.nq, qb = blockIdx.x / p.nq;
    const int kvh = head / p.n_rep;
    const int tq = qb * 32 + l32;
    int klo, khi;
    key_range(p, tq, klo, khi);
    int wmin = khi > klo ? klo : 0x7fffffff, wmax = khi > klo ? khi : 0;
    wave_min_max(wmin, wmax);
    if (wmax <= wmin) { wmin = 0; wmax = 0; }
    const int kt0 = wmin & ~31;
    const int n_tiles = (wmax - kt0 + 31) / 32;

    stage_tile<D>(q_s, fp.q + (int64_t)head * p.q_sh, p.q_st, qb * 32, p.total_q - 1, lane);
    f32x16_t o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;
    const float c2 = p.scale_log2;
    for (int t = 0; t < n_tiles; ++t) {
        const int kt = kt0 + 32 * t;
        __syncthreads();                  // the previous tile's readers are done
        stage_tile<D>(k_s, fp.k + (int64_t)kvh * p.k_sh, p.k_st, kt, p.total_k - 1, lane);
        stage_tile<D>(v_s, fp.v + (int64_t)kvh * p.v_sh, p.v_st, kt, p.total_k - 1, lane);
        __syncthreads();
        f32x16_t s = rows_product<D>(k_s, q_s, l32, g);        // rows = keys, column = this lane's query
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kt + acc_row(r, g);
            if (key < klo || key >= khi) s[r] = -INFINITY;
            mx = fmaxf(mx, s[r]);
        }
        mx = pair_max(mx);
        const float m_new = fmaxf(m_i, mx * c2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_i - m_new);
        m_i = m_new;
        float rs = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] = fast_exp2(s[r] * c2 - m_use);
            rs += s[r];
        }
        l_i = l_i * alpha + rs;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
        cols_product<D>(o_acc, v_s, s, l32, g);
    }
    const float l_tot = pair_sum(l_i);
    if (tq < p.total_q) {
        store_rows<D>(fp.o + (int64_t)tq * p.o_st + (int64_t)head * p.o_sh, o_acc, l_tot > 0.f ? 1.0f / l_tot : 0.f, g);
        if (g == 0 && fp.lse != nullptr)
            fp.lse[(int64_t)head * p.total_q + tq] = l_tot > 0.f ? (m_i + __log2f(l_tot)) * 0.6931471805599453f : INFINITY;
    }
}

// ---- delta[h][t] = sum_d dO[t][h][d] O[t][h][d] -----------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_f32_delta_kernel(const F32Params fp) {
    constexpr int LPR = D / 4;            // lanes per (token, head) row: 8, 16, 24 or 32
    constexpr int RPB = 256 / 32;         // rows per block: 32 lanes are reserved per row whatever D
    const AttnParams& p = fp.m;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / 32;
    const int c = threadIdx.x % 32;
    const int64_t n_rows = (int64_t)p.total_q * p.nq;
    float acc = 0.f;
    const bool ok = row < n_rows && c < LPR;
    const int64_t t = row < n_rows ? row / p.nq : 0;
    const int h = row < n_rows ? (int)(row % p.nq) : 0;
    if (ok) {
        const f32x4_t a = *reinterpret_cast<const f32x4_t*>(fp.o + t * p.o_st + (int64_t)h * p.o_sh + 4 * c);
        const f32x4_t b = *reinterpret_cast<const f32x4_t*>(fp.d_o + t * p.o_st + (int64_t)h * p.o_sh + 4 * c);
        acc = a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
    acc = group_sum<32>(acc);
    if (row < n_rows && c == 0) fp.delta[(int64_t)h * p.total_q + t] = acc;
}

// ---- dK / dV: a wavefront owns 32 keys of one KV head (K, V rows resident in LDS), loops over the group's query
// heads and over 32-query tiles: S = Q K^T, dP = dO V^T (lane = key), dV^T += dO^T P, dK^T += Q^T dS ----------------
template <int D>
__global__ __launch_bounds__(64) void attn_f32_dkdv_kernel(const F32Params fp) {
    constexpr int LD = D + 1, DT = D / 32;
    __shared__ float k_s[32 * LD], v_s[32 * LD], q_s[32 * LD], do_s[32 * LD];
    __shared__ float lse_s[32], delta_s[32];
    const AttnParams& p = fp.m;
    const int lane = threadIdx.x, l32 = lane & 31, g = lane >> 5;
    const int kvh = blockIdx.x % p.nkv, kb = blockIdx.x / p.nkv;
    const int key = kb * 32 + l32;
    int qlo, qhi;
    query_range(p, key, qlo, qhi);
    int wmin = qhi > qlo ? qlo : 0x7fffffff, wmax = qhi > qlo ? qhi : 0;
    wave_min_max(wmin, wmax);
    if (wmax <= wmin) { wmin = 0; wmax = 0; }
    const int qt0 = wmin & ~31;
    const int n_tiles = (wmax - qt0 + 31) / 32;
    stage_tile<D>(k_s, fp.k + (int64_t)kvh * p.k_sh, p.k_st, kb * 32, p.total_k - 1, lane);
    stage_tile<D>(v_s, fp.v + (int64_t)kvh * p.v_sh, p.v_st, kb * 32, p.total_k - 1, lane);
    f32x16_t dk_acc[DT], dv_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk_acc[dt][r] = 0.f; dv_acc[dt][r] = 0.f; }
    const float c2 = p.scale_log2;
    for (int rep = 0; rep < p.n_rep; ++rep) {       // fixed order: bit-reproducible sums over the group's query heads
        const int head = kvh * p.n_rep + rep;
        for (int t = 0; t < n_tiles; ++t) {
            const int qt = qt0 + 32 * t;
            __syncthreads();
            stage_tile<D>(q_s, fp.q + (int64_t)head * p.q_sh, p.q_st, qt, p.total_q - 1, lane);
            stage_tile<D>(do_s, fp.d_o + (int64_t)head * p.o_sh, p.o_st, qt, p.total_q - 1, lane);
            if (lane < 32) {
                const int tok = min(qt + lane, p.total_q - 1);
                lse_s[lane] = fp.lse[(int64_t)head * p.total_q + tok] * kLog2eF;
                delta_s[lane] = fp.delta[(int64_t)head * p.total_q + tok];
            }
            __syncthreads();
            f32x16_t s = rows_product<D>(q_s, k_s, l32, g);        // rows = queries, column = this lane's key
            f32x16_t dp = rows_product<D>(do_s, v_s, l32, g);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = acc_row(r, g), q = qt + row;
                const float pv = (q >= qlo && q < qhi) ? fast_exp2(s[r] * c2 - lse_s[row]) : 0.f;
                s[r] = pv;
                dp[r] = pv * (dp[r] - delta_s[row]);
            }
            cols_product<D>(dv_acc, do_s, s, l32, g);
            cols_product<D>(dk_acc, q_s, dp, l32, g);
        }
    }
    if (key < p.total_k) {
        store_rows<D>(fp.dk + (int64_t)key * p.dk_st + (int64_t)kvh * p.dk_sh, dk_acc, p.scale, g);
        store_rows<D>(fp.dv + (int64_t)key * p.dv_st + (int64_t)kvh * p.dv_sh, dv_acc, 1.0f, g);
    }
}

// ---- dQ: a wavefront owns 32 queries of one head: S^T = K Q^T, dP^T = V dO^T (lane = query), dQ^T += K^T dS^T -------
template <int D>
__global__ __launch_bounds__(64) void attn_f32_dq_kernel(const F32Params fp) {
    constexpr int LD = D + 1, DT = D / 32;
    __shared__ float q_s[32 * LD], do_s[32 * LD], k_s[32 * LD], v_s[32 * LD];
    const AttnParams& p = fp.m;
    const int lane = threadIdx.x, l32 = lane & 31, g = lane >> 5;
    const int head = blockIdx.x % p.nq, qb = blockIdx.x / p.nq;
    const int kvh = head / p.n_rep;
    const int tq = qb * 32 + l32;
    int klo, khi;
    key_range(p, tq, klo, khi);
    int wmin = khi > klo ? klo : 0x7fffffff, wmax = khi > klo ? khi : 0;
    wave_min_max(wmin, wmax);
    if (wmax <= wmin) { wmin = 0; wmax = 0; }
    const int kt0 = wmin & ~31;
    const int n_tiles = (wmax - kt0 + 31) / 32;
    stage_tile<D>(q_s, fp.q + (int64_t)head * p.q_sh, p.q_st, qb * 32, p.total_q - 1, lane);
    stage_tile<D>(do_s, fp.d_o + (int64_t)head * p.o_sh, p.o_st, qb * 32, p.total_q - 1, lane);
    const int tl = tq < p.total_q ? tq : p.total_q - 1;
    const float lse2 = fp.lse[(int64_t)head * p.total_q + tl] * kLog2eF;
    const float delta = fp.delta[(int64_t)head * p.total_q + tl];
    f32x16_t dq_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[dt][r] = 0.f;
    const float c2 = p.scale_log2;
    for (int t = 0; t < n_tiles; ++t) {
        const int kt = kt0 + 32 * t;
        __syncthreads();
        stage_tile<D>(k_s, fp.k + (int64_t)kvh * p.k_sh, p.k_st, kt, p.total_k - 1, lane);
        stage_tile<D>(v_s, fp.v + (int64_t)kvh * p.v_sh, p.v_st, kt, p.total_k - 1, lane);
        __syncthreads();
        f32x16_t s = rows_product<D>(k_s, q_s, l32, g);            // rows = keys, column = this lane's query
        f32x16_t dp = rows_product<D>(v_s, do_s, l32, g);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k_idx = kt + acc_row(r, g);
            const float pv = (k_idx >= klo && k_idx < khi) ? fast_exp2(s[r] * c2 - lse2) : 0.f;
            dp[r] = pv * (dp[r] - delta);
        }
        cols_product<D>(dq_acc, k_s, dp, l32, g);
    }
    if (tq < p.total_q) store_rows<D>(fp.dq + (int64_t)tq * p.q_st + (int64_t)head * p.q_sh, dq_acc, p.scale, g);
}

int validate_f32(const mi_attn_args* a, const char* who) {
    int rc = mi_attn_validate(a, who, MI_F32, 4);
    if (rc != MI_OK) return rc;
    if (a->rotary_cos || a->rotary_sin) return mi_fail(MI_E_DTYPE, "%s: the fused rotary takes bf16 / f16 tensors; rotate fp32 q and k with mi_rotary first", who);
    if (a->dropout_p > 0.f) return mi_fail(MI_E_DTYPE, "%s: attention-probability dropout takes bf16 / f16 tensors", who);
    return MI_OK;
}

void fill(const mi_attn_args* a, F32Params* fp) {
    *fp = F32Params{};
    mi_attn_fill_params(a, &fp->m);
    fp->q = (const float*)a->q; fp->k = (const float*)a->k; fp->v = (const float*)a->v;
    fp->o = (float*)a->o; fp->lse = a->lse;
}

}  // namespace

int mi_attn_fwd_impl_f32(const mi_attn_args* a) {
    int rc = validate_f32(a, "attn_fwd");
    if (rc != MI_OK) return rc;
    if (!a->o) return mi_fail(MI_E_NULL, "attn_fwd: o is null");
    if (!mi_aligned16(a->o) || a->o_stride_token % 4 || a->o_stride_head % 4)
        return mi_fail(MI_E_ALIGN, "attn_fwd: o must be 16-byte aligned with strides multiple of 4");
    if (a->total_q == 0) return MI_OK;
    F32Params fp;
    fill(a, &fp);
    const int64_t grid = ((a->total_q + 31) / 32) * a->n_q_heads;
    if (grid > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "attn_fwd: too many work items");
    hipStream_t st = (hipStream_t)a->stream;
    switch (a->head_dim) {
        case 32: attn_f32_fwd_kernel<32><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp); break;
        case 64: attn_f32_fwd_kernel<64><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp); break;
        case 96: attn_f32_fwd_kernel<96><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp); break;
        case 128: attn_f32_fwd_kernel<128><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp); break;
        default: return mi_fail(MI_E_SHAPE, "attn_fwd: head_dim %d unsupported (32, 64, 96, 128)", a->head_dim);
    }
    return mi_check_launch("attn_fwd (f32)");
}

template <int D> static int launch_bwd_f32(const F32Params& fp, int flags, hipStream_t st) {
    const AttnParams& p = fp.m;
    const int stages = flags & (MI_ATTN_BWD_DELTA | MI_ATTN_BWD_DKDV | MI_ATTN_BWD_DQ);
    const bool all = stages == 0;
    if (all || (stages & MI_ATTN_BWD_DELTA)) {
        const int64_t rows = (int64_t)p.total_q * p.nq;
        attn_f32_delta_kernel<D><<<dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, st>>>(fp);
        int rc = mi_check_launch("attn_bwd_delta (f32)");
        if (rc != MI_OK) return rc;
    }
    if (all || (stages & MI_ATTN_BWD_DKDV)) {
        const int64_t grid = (((int64_t)p.total_k + 31) / 32) * p.nkv;
        attn_f32_dkdv_kernel<D><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp);
        int rc = mi_check_launch("attn_bwd_dkdv (f32)");
        if (rc != MI_OK) return rc;
    }
    if (all || (stages & MI_ATTN_BWD_DQ)) {
        const int64_t grid = (((int64_t)p.total_q + 31) / 32) * p.nq;
        attn_f32_dq_kernel<D><<<dim3((unsigned)grid), dim3(64), 0, st>>>(fp);
        return mi_check_launch("attn_bwd_dq (f32)");
    }
    return MI_OK;
}

int mi_attn_bwd_impl_f32(const mi_attn_bwd_args* b) {
    if (!b) return mi_fail(MI_E_NULL, "attn_bwd: args is null");
    const mi_attn_args* a = &b->fwd;
    int rc = validate_f32(a, "attn_bwd");
    if (rc != MI_OK) return rc;
    if (!a->o || !a->lse || !b->d_o || !b->dq || !b->dk || !b->dv)
        return mi_fail(MI_E_NULL, "attn_bwd: o, lse, d_o, dq, dk, dv are required");
    if (!mi_aligned16(a->o) || !mi_aligned16(b->d_o) || !mi_aligned16(b->dq) || !mi_aligned16(b->dk) || !mi_aligned16(b->dv))
        return mi_fail(MI_E_ALIGN, "attn_bwd: tensors must be 16-byte aligned");
    if (a->o_stride_token % 4 || a->o_stride_head % 4 || b->dk_stride_token % 4 || b->dk_stride_head % 4 ||
        b->dv_stride_token % 4 || b->dv_stride_head % 4)
        return mi_fail(MI_E_ALIGN, "attn_bwd: strides must be multiples of 4 elements");
    if (a->total_q == 0) return MI_OK;
    const size_t need = (size_t)a->total_q * (size_t)a->n_q_heads * sizeof(float);
    if (!b->workspace || b->workspace_bytes < need || !mi_aligned16(b->workspace))
        return mi_fail(MI_E_WORKSPACE, "attn_bwd: workspace needs %zu bytes (16-byte aligned), got %zu", need, b->workspace_bytes);
    if ((((int64_t)a->total_q + 31) / 32) * a->n_q_heads > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "attn_bwd: too many work items");
    F32Params fp;
    fill(a, &fp);
    fp.d_o = (const float*)b->d_o; fp.dq = (float*)b->dq; fp.dk = (float*)b->dk; fp.dv = (float*)b->dv;
    fp.m.dk_st = b->dk_stride_token; fp.m.dk_sh = b->dk_stride_head;
    fp.m.dv_st = b->dv_stride_token; fp.m.dv_sh = b->dv_stride_head;
    fp.delta = (float*)b->workspace;
    hipStream_t st = (hipStream_t)a->stream;
    switch (a->head_dim) {
        case 32: return launch_bwd_f32<32>(fp, a->flags, st);
        case 64: return launch_bwd_f32<64>(fp, a->flags, st);
        case 96: return launch_bwd_f32<96>(fp, a->flags, st);
        case 128: return launch_bwd_f32<128>(fp, a->flags, st);
        default: return mi_fail(MI_E_SHAPE, "attn_bwd: head_dim %d unsupported", a->head_dim);
    }
}
