// Decode attention over a pre-allocated KV cache for gfx950: one query token per sequence, HBM-bound.
//
// Grid = batch x KV heads x key splits.  All query heads of a GQA group are processed by the same
// workgroup, so every cached K/V element is read from HBM exactly once.  Each wavefront streams its
// own 32-key chunks:
//     S^T[key][head]  = K * Q^T     v_mfma_f32_16x16x32_bf16, A = K rows loaded straight from global
//                                   memory in operand layout, B = Q^T (heads of the group, zero padded)
//     online softmax over keys      the lane's column is a head; 8 in-lane keys + 2 lane exchanges
//     O^T[d][head]   += V^T * P^T   A = V^T read from a transposed per-wavefront LDS copy of the chunk
// Partial (max, sum, O) per split go to a workspace and are merged by a second kernel.
// A small first kernel appends the new K/V row in place (instead of the reference's torch.cat) and
// applies rotary to it; the query is rotated while its fragments are loaded.
#include "attn_common.h"

typedef float f32x4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int kChunk = 32;           // keys per wavefront and iteration
constexpr int kMaxSplits = 32;

struct DecodeParams {
    const elem_t* q; elem_t* kc; elem_t* vc; elem_t* o;
    const int32_t* ctx_len;
    const elem_t* k_new; const elem_t* v_new;
    const elem_t* cos; const elem_t* sin; const int64_t* pos; int table_rows;
    const float* cos32; const float* sin32;   // interleaved-pair rotary: fp32 tables [table_rows, D / 2]
    int batch, max_ctx, nq, nkv, n_rep, n_splits;
    int n_hc;      // chunks of up to 16 query heads per KV head (a workgroup serves one chunk)
    int64_t c_sb, c_st, c_sh;
    int64_t q_sb, kn_sb, vn_sb;   // element strides between sequences of q / k_new / v_new
    float scale_log2;
    float* ws_o;   // [batch][nq][n_splits][D]
    float* ws_ml;  // [batch][nq][n_splits][2]
};

__device__ __forceinline__ f32x4v mfma_16x16x32(elem8_t a, elem8_t b, f32x4v c) {
#ifdef MI_ELEM_F16
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
#else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
#endif
}

// ---- in-place append of the new K/V row (optionally rotated) -------------------------------------
template <int D>
__global__ void decode_append_kernel(const DecodeParams p) {
    // one thread per (batch, kv head, 8-feature vector of the first half)
    constexpr int HV = D / 16;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= p.batch * p.nkv * HV) return;
    const int c = idx % HV, kvh = (idx / HV) % p.nkv, b = idx / (HV * p.nkv);
    const int ctx = p.ctx_len[b];
    if (ctx < 1 || ctx > p.max_ctx) return;
    const int64_t src = (int64_t)b * p.kn_sb + (int64_t)kvh * D + 8 * c;
    const int64_t src_v = (int64_t)b * p.vn_sb + (int64_t)kvh * D + 8 * c;
    const int64_t dst = (int64_t)b * p.c_sb + (int64_t)(ctx - 1) * p.c_st + (int64_t)kvh * p.c_sh + 8 * c;
    uint4 lo = *reinterpret_cast<const uint4*>(p.k_new + src);
    uint4 hi = *reinterpret_cast<const uint4*>(p.k_new + src + D / 2);
    if (p.cos != nullptr) {
        int64_t pos = p.pos[b];
        pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
        const uint4 cv = *reinterpret_cast<const uint4*>(p.cos + pos * D + 8 * c);
        const uint4 sv = *reinterpret_cast<const uint4*>(p.sin + pos * D + 8 * c);
        rotate_pair(lo, hi, cv, sv, 1.0f);
    } else if (p.cos32 != nullptr) {
        int64_t pos = p.pos[b];
        pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
        const float* cr = p.cos32 + pos * (D / 2) + 4 * c;   // features 8 c .. + 8 = pairs 4 c .. + 4
        const float* sr = p.sin32 + pos * (D / 2) + 4 * c;
        rotate_interleaved(lo, ld128(cr), ld128(sr), 1.0f);
        rotate_interleaved(hi, ld128(cr + D / 4), ld128(sr + D / 4), 1.0f);
    }
    *reinterpret_cast<uint4*>(p.kc + dst) = lo;
    *reinterpret_cast<uint4*>(p.kc + dst + D / 2) = hi;
    *reinterpret_cast<uint4*>(p.vc + dst) = *reinterpret_cast<const uint4*>(p.v_new + src_v);
    *reinterpret_cast<uint4*>(p.vc + dst + D / 2) = *reinterpret_cast<const uint4*>(p.v_new + src_v + D / 2);
}

// ---- split kernel ----------------------------------------------------------------------------------
// NWV wavefronts (4 or 8) share the keys of one (batch, KV head, split); with a single split the merged result
// is the attention output and goes straight to `o`, otherwise the partial goes to the workspace.
// ROT: 0 = q as it is, 1 = rotate-half rotary on the q load, 2 = interleaved-pair rotary on the q load.
template <int D, int ROT, int NWV>
__global__ __launch_bounds__(64 * NWV, 2) void decode_split_kernel(const DecodeParams p) {
    constexpr int kThreads = 64 * NWV;
    constexpr int KS = D / 32;          // contraction steps of Q K^T (32 features each)
    constexpr int DT = D / 16;          // 16-row tiles of O^T
    constexpr int VSTR = 2 * D + 32;    // bytes per key row of the staged V chunk: transpose reads of 8 rows x 32 bytes hit 256 distinct bytes
    constexpr int V_ITEMS = 8 * (D / 8);  // (key quad, feature group) items of a 32-key chunk
    constexpr int V_PER_LANE = (V_ITEMS + 63) / 64;   // head_dim 32 / 96: the last round is partly empty

    __shared__ __attribute__((aligned(16))) char v_lds[NWV][kChunk * VSTR];
    __shared__ float wm_lds[NWV][16];
    __shared__ float wl_lds[NWV][16];
    __shared__ float wo_lds[NWV][16][D + 1];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, l16 = lane & 15, G = lane >> 4;

    const int split = blockIdx.x % p.n_splits;
    const int kv_hc = (blockIdx.x / p.n_splits) % (p.nkv * p.n_hc);
    const int kvh = kv_hc / p.n_hc, hc = kv_hc - kvh * p.n_hc;
    const int b = blockIdx.x / (p.n_splits * p.nkv * p.n_hc);
    // this workgroup's query heads: head0 .. head0 + n_heads of the group (groups of more than 16 heads take
    // several workgroups, each reading the group's K / V once)
    const int head0 = kvh * p.n_rep + 16 * hc;
    const int n_heads = min(16, p.n_rep - 16 * hc);

    int ctx = p.ctx_len[b];
    ctx = ctx < 0 ? 0 : (ctx > p.max_ctx ? p.max_ctx : ctx);
    // keys of this split: [s0, s1), split length rounded up to whole workgroup iterations
    int per = (ctx + p.n_splits - 1) / p.n_splits;
    per = (per + NWV * kChunk - 1) / (NWV * kChunk) * (NWV * kChunk);
    const int s0 = split * per;
    const int s1 = min(ctx, s0 + per);
    const int n_iter = s1 > s0 ? (s1 - s0 + NWV * kChunk - 1) / (NWV * kChunk) : 0;

    // Q^T fragments: column = head slot l16 (valid when < n_rep), contraction = features 32*ks + 8*G + i
    elem8_t qf[KS];
    {
        const int hs = l16 < n_heads ? l16 : 0;
        const elem_t* qr = p.q + (int64_t)b * p.q_sb + (int64_t)(head0 + hs) * D + 8 * G;
        uint4 raw[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) raw[ks] = *reinterpret_cast<const uint4*>(qr + 32 * ks);
        if constexpr (ROT == 1) {
            int64_t pos = p.pos[b];
            pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
#pragma unroll
            for (int ks = 0; ks < KS / 2; ++ks) {
                const uint4 cv = *reinterpret_cast<const uint4*>(p.cos + pos * D + 32 * ks + 8 * G);
                const uint4 sv = *reinterpret_cast<const uint4*>(p.sin + pos * D + 32 * ks + 8 * G);
                rotate_pair(raw[ks], raw[ks + KS / 2], cv, sv, 1.0f);
            }
        } else if constexpr (ROT == 2) {
            int64_t pos = p.pos[b];
            pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {   // features 32 ks + 8 G .. + 8 = pairs 16 ks + 4 G .. + 4
                const float* cr = p.cos32 + pos * (D / 2) + 16 * ks + 4 * G;
                const float* sr = p.sin32 + pos * (D / 2) + 16 * ks + 4 * G;
                rotate_interleaved(raw[ks], ld128(cr), ld128(sr), 1.0f);
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (l16 >= n_heads) raw[ks] = make_uint4(0, 0, 0, 0);
            qf[ks] = __builtin_bit_cast(elem8_t, raw[ks]);
        }
    }

    f32x4v o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o_acc[dt] = f32x4v{0.f, 0.f, 0.f, 0.f};
    float m_i = -INFINITY, l_i = 0.f;

    const elem_t* kbase = p.kc + (int64_t)b * p.c_sb + (int64_t)kvh * p.c_sh;
    const elem_t* vbase = p.vc + (int64_t)b * p.c_sb + (int64_t)kvh * p.c_sh;
    char* vt = v_lds[wave];
    // transpose-read base of this lane: keys 4G + (l16 >> 2), features 4 * (l16 & 3) (+ 16 per feature tile, + 16 keys for the second half)
    const char* vt_lane = vt + (4 * G + (l16 >> 2)) * VSTR + 8 * (l16 & 3);

    // K fragments and V rows of a chunk; two sets so that the loads of chunk i+1 are in flight while
    // chunk i is being processed
    struct ChunkRegs {
        elem8_t kf[2][KS];
        uint4 vraw[V_PER_LANE][4];
    };
    auto load_chunk = [&](ChunkRegs& c, int it) {
        const int key0 = s0 + (NWV * it + wave) * kChunk;
        if (key0 >= s1) return;
        const int last = s1 - 1;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int tok = min(key0 + 16 * t + l16, last);
            const elem_t* kr = kbase + (int64_t)tok * p.c_st + 8 * G;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) c.kf[t][ks] = __builtin_bit_cast(elem8_t, ldg_nt(reinterpret_cast<const uint4*>(kr + 32 * ks)));
        }
#pragma unroll
        for (int j = 0; j < V_PER_LANE; ++j) {
            const int item = lane + 64 * j;
            if (V_ITEMS % 64 != 0 && item >= V_ITEMS) break;
            const int quad = item / (D / 8), dg = item % (D / 8);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int tok = min(key0 + 4 * quad + r, last);
                c.vraw[j][r] = ldg_nt(reinterpret_cast<const uint4*>(vbase + (int64_t)tok * p.c_st + 8 * dg));
            }
        }
    };
    auto process_chunk = [&](const ChunkRegs& c, int it) {
        const int key0 = s0 + (NWV * it + wave) * kChunk;
        const bool active = key0 < s1;          // wave-uniform
        // Each wavefront owns its LDS chunk; the LDS pipeline executes one wavefront's accesses in program
        // order, so wavefront-scope fences (compiler ordering only) are enough and the wavefronts of a
        // workgroup never wait for each other inside the loop.
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        elem8_t pf;
        float alpha = 1.f;
        if (active) {
            f32x4v s_acc[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s_acc[t] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) s_acc[t] = mfma_16x16x32(c.kf[t][ks], qf[ks], s_acc[t]);
            }
            // rows: keys key0 + 16*t + 4*G + r; column: head slot l16
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (key0 + 16 * t + 4 * G + r >= s1) s_acc[t][r] = -INFINITY;
                    mx = fmaxf(mx, s_acc[t][r]);
                }
            mx = quad_max(mx);
            const float m_new = fmaxf(m_i, mx * p.scale_log2);   // finite: the chunk holds >= 1 valid key
            alpha = fast_exp2(m_i - m_new);
            m_i = m_new;
            float rs = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = fast_exp2(s_acc[t][r] * p.scale_log2 - m_new);
                    rs += e;
                    pf[4 * t + r] = (elem_t)e;   // slot (G, i): key 16*(i/4) + 4*G + (i%4)
                }
            l_i = l_i * alpha + rs;
            // key-major copy of the V chunk (rows as loaded); the PV operand is read back transposed
#pragma unroll
            for (int j = 0; j < V_PER_LANE; ++j) {
                const int item = lane + 64 * j;
                if (V_ITEMS % 64 != 0 && item >= V_ITEMS) break;
                const int quad = item / (D / 8), dg = item % (D / 8);
#pragma unroll
                for (int r = 0; r < 4; ++r) st128(vt + (4 * quad + r) * VSTR + 16 * dg, c.vraw[j][r]);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        if (active) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                // slots 0-3: keys 4G..4G+3, slots 4-7: keys 16+4G..16+4G+3 (the order of pf)
                const elem8_t a = tr_pair(vt_lane + 32 * dt, vt_lane + 16 * VSTR + 32 * dt);
                o_acc[dt] = o_acc[dt] * alpha;
                o_acc[dt] = mfma_16x16x32(a, pf, o_acc[dt]);
            }
        }
    };

    ChunkRegs ra, rb;
    if (n_iter > 0) load_chunk(ra, 0);
    for (int it = 0; it < n_iter; it += 2) {
        if (it + 1 < n_iter) load_chunk(rb, it + 1);
        process_chunk(ra, it);
        if (it + 1 < n_iter) {
            if (it + 2 < n_iter) load_chunk(ra, it + 2);
            process_chunk(rb, it + 1);
        }
    }

    // ---- merge the four wavefronts, emit the split partial -----------------------------------------
    l_i = quad_sum(l_i);
    __syncthreads();
    if (G == 0) { wm_lds[wave][l16] = m_i; wl_lds[wave][l16] = l_i; }
    if (l16 < n_heads) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) wo_lds[wave][l16][16 * dt + 4 * G + r] = o_acc[dt][r];
    }
    __syncthreads();
    for (int idx = tid; idx < n_heads * D; idx += kThreads) {
        const int hs = idx / D, d = idx % D;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < NWV; ++w) M = fmaxf(M, wm_lds[w][hs]);
        float L = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; ++w) {
            const float wm = wm_lds[w][hs];
            const float f = wm == -INFINITY ? 0.f : fast_exp2(wm - M);
            L += f * wl_lds[w][hs];
            O += f * wo_lds[w][hs][d];
        }
        const int64_t bh = (int64_t)b * p.nq + head0 + hs;
        if (p.n_splits == 1) {
            p.o[bh * D + d] = (elem_t)(L > 0.f ? O / L : 0.f);
        } else {
            const int64_t slot = bh * p.n_splits + split;
            p.ws_o[slot * D + d] = O;
            if (d == 0) { p.ws_ml[slot * 2] = M; p.ws_ml[slot * 2 + 1] = L; }
        }
    }
}

// ---- merge of the splits ------------------------------------------------------------------------------
template <int D>
__global__ void decode_merge_kernel(const DecodeParams p) {
    // one thread per (batch, head, feature)
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.batch * p.nq * D) return;
    const int d = (int)(idx % D);
    const int64_t bh = idx / D;
    float M = -INFINITY;
    for (int s = 0; s < p.n_splits; ++s) M = fmaxf(M, p.ws_ml[(bh * p.n_splits + s) * 2]);
    float L = 0.f, O = 0.f;
    for (int s = 0; s < p.n_splits; ++s) {
        const float m = p.ws_ml[(bh * p.n_splits + s) * 2];
        const float f = m == -INFINITY ? 0.f : fast_exp2(m - M);
        L += f * p.ws_ml[(bh * p.n_splits + s) * 2 + 1];
        O += f * p.ws_o[(bh * p.n_splits + s) * D + d];
    }
    p.o[bh * D + d] = (elem_t)(L > 0.f ? O / L : 0.f);
}

// 8-wavefront workgroups (one per compute unit) once there is a (batch, KV head) pair for most of the 256
// compute units: then one split does and the merge kernel is not launched; otherwise 4-wavefront workgroups
// and enough splits for about two workgroups per compute unit.
bool wide_blocks(int batch, int nkv) { return (int64_t)batch * nkv >= 192; }

int choose_splits(int batch, int nkv, int max_ctx) {
    const int64_t pairs = (int64_t)batch * nkv;
    if (wide_blocks(batch, nkv)) return 1;
    // one workgroup per compute unit: measured best or within a few percent of it for batch 1 - 16 at contexts
    // of 1k - 16k (two per compute unit, the earlier choice, cost 5 - 10 % in merge work at batch 4 - 16)
    int64_t s = (256 + pairs - 1) / pairs;
    const int64_t by_len = ((int64_t)max_ctx + 4 * kChunk - 1) / (4 * kChunk);
    if (s > by_len) s = by_len;
    if (s > kMaxSplits) s = kMaxSplits;
    if (s < 1) s = 1;
    return (int)s;
}

// rot: 0 = none, 1 = rotate-half, 2 = interleaved pairs
template <int D, int NWV> int launch_split(const DecodeParams& p, int rot, hipStream_t st) {
    const unsigned grid = (unsigned)p.batch * p.nkv * p.n_hc * p.n_splits;
    if (rot == 2) decode_split_kernel<D, 2, NWV><<<dim3(grid), dim3(64 * NWV), 0, st>>>(p);
    else if (rot == 1) {
        // rotate-half pairs feature i with i + D / 2: the same lane holds both only when D / 32 is even
        if constexpr (D == 64 || D == 128) decode_split_kernel<D, 1, NWV><<<dim3(grid), dim3(64 * NWV), 0, st>>>(p);
        else return mi_fail(MI_E_SHAPE, "attn_decode: fused rotate-half rotary needs head_dim 64 or 128");
    } else decode_split_kernel<D, 0, NWV><<<dim3(grid), dim3(64 * NWV), 0, st>>>(p);
    return mi_check_launch("decode_split");
}

template <int D> int launch_decode(const DecodeParams& p, bool append, int rot, hipStream_t st) {
    if (append) {
        const int n = p.batch * p.nkv * (D / 16);
        decode_append_kernel<D><<<dim3((n + 127) / 128), dim3(128), 0, st>>>(p);
        int rc = mi_check_launch("decode_append");
        if (rc != MI_OK) return rc;
    }
    const int rc = wide_blocks(p.batch, p.nkv * p.n_hc) ? launch_split<D, 8>(p, rot, st) : launch_split<D, 4>(p, rot, st);
    if (rc != MI_OK || p.n_splits == 1) return rc;
    const int64_t n = (int64_t)p.batch * p.nq * D;
    decode_merge_kernel<D><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(p);
    return mi_check_launch("decode_merge");
}

}  // namespace

#ifndef MI_ELEM_F16
extern "C" size_t mi_attn_decode_workspace_bytes(int32_t batch, int32_t n_q_heads, int32_t head_dim, int32_t max_ctx) {
    (void)max_ctx;
    if (batch <= 0 || n_q_heads <= 0 || head_dim <= 0) return 0;
    return (size_t)batch * n_q_heads * kMaxSplits * (size_t)(head_dim + 2) * sizeof(float);
}
#endif

namespace {
// Validation and launches shared by the two entry points; `ws` / `ws_bytes` is the scratch for the per-split partial
// results (the caller's workspace, or the library's own static array for mi_attn_decode_static).
int decode_entry(const mi_decode_args* a, void* ws, size_t ws_bytes, bool static_ws) {
    if (!a) return mi_fail(MI_E_NULL, "attn_decode: args is null");
    if (!a->q || !a->k_cache || !a->v_cache || !a->o || !a->ctx_len) return mi_fail(MI_E_NULL, "attn_decode: q, caches, o and ctx_len are required");
    if (a->dtype != MI_ELEM_DTYPE) return mi_fail(MI_E_DTYPE, "attn_decode: the decode kernels take bf16 or f16 tensors (dtype code %d)", a->dtype);
    if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 96 && a->head_dim != 128)
        return mi_fail(MI_E_SHAPE, "attn_decode: head_dim %d unsupported (32, 64, 96, 128)", a->head_dim);
    if (a->batch <= 0 || a->max_ctx <= 0 || a->n_q_heads <= 0 || a->n_kv_heads <= 0 || a->n_q_heads % a->n_kv_heads != 0)
        return mi_fail(MI_E_SHAPE, "attn_decode: bad batch/head configuration");
    if ((a->k_new == nullptr) != (a->v_new == nullptr)) return mi_fail(MI_E_NULL, "attn_decode: k_new and v_new go together");
    const bool rot = a->rotary_cos != nullptr || a->rotary_sin != nullptr;
    if (rot && (!a->rotary_cos || !a->rotary_sin || !a->position_ids || a->rotary_table_rows <= 0))
        return mi_fail(MI_E_NULL, "attn_decode: fused rotary needs cos, sin, position ids and the table size");
    if (rot && !a->rotary_interleaved && a->head_dim != 64 && a->head_dim != 128)
        return mi_fail(MI_E_SHAPE, "attn_decode: fused rotate-half rotary needs head_dim 64 or 128");
    if (!mi_aligned16(a->q) || !mi_aligned16(a->k_cache) || !mi_aligned16(a->v_cache) || !mi_aligned16(a->o) ||
        (a->k_new && (!mi_aligned16(a->k_new) || !mi_aligned16(a->v_new))) ||
        (rot && (!mi_aligned16(a->rotary_cos) || !mi_aligned16(a->rotary_sin))))
        return mi_fail(MI_E_ALIGN, "attn_decode: tensors must be 16-byte aligned");
    if (a->cache_stride_batch % 8 || a->cache_stride_token % 8 || a->cache_stride_head % 8 || a->q_stride_batch % 8 ||
        a->k_new_stride_batch % 8 || a->v_new_stride_batch % 8)
        return mi_fail(MI_E_ALIGN, "attn_decode: strides must be multiples of 8 elements");
    if ((a->q_stride_batch && a->q_stride_batch < (int64_t)a->n_q_heads * a->head_dim) ||
        (a->k_new_stride_batch && a->k_new_stride_batch < (int64_t)a->n_kv_heads * a->head_dim) ||
        (a->v_new_stride_batch && a->v_new_stride_batch < (int64_t)a->n_kv_heads * a->head_dim))
        return mi_fail(MI_E_SHAPE, "attn_decode: a sequence stride is smaller than heads * head_dim");
    if (!(a->softmax_scale > 0.f)) return mi_fail(MI_E_SHAPE, "attn_decode: softmax_scale must be positive");
    const int n_hc = (a->n_q_heads / a->n_kv_heads + 15) / 16;
    int splits = a->n_splits > 0 ? a->n_splits : choose_splits(a->batch, a->n_kv_heads * n_hc, a->max_ctx);
    if (splits > kMaxSplits) splits = kMaxSplits;
    const size_t need = (size_t)a->batch * a->n_q_heads * splits * (size_t)(a->head_dim + 2) * sizeof(float);
    if (static_ws && need > ws_bytes)
        return mi_fail(MI_E_WORKSPACE, "attn_decode_static: batch %d x %d query heads x %d key splits x head_dim %d needs %zu bytes of "
                       "scratch, the library's static array holds %zu; use mi_attn_decode with a caller workspace",
                       a->batch, a->n_q_heads, splits, a->head_dim, need, ws_bytes);
    if (!ws || ws_bytes < need || !mi_aligned16(ws))
        return mi_fail(MI_E_WORKSPACE, "attn_decode: workspace needs %zu bytes (16-byte aligned), got %zu", need, ws_bytes);
    DecodeParams p{};
    p.q = (const elem_t*)a->q; p.kc = (elem_t*)a->k_cache; p.vc = (elem_t*)a->v_cache; p.o = (elem_t*)a->o;
    p.ctx_len = a->ctx_len; p.k_new = (const elem_t*)a->k_new; p.v_new = (const elem_t*)a->v_new;
    if (a->rotary_interleaved) {
        p.cos32 = (const float*)a->rotary_cos; p.sin32 = (const float*)a->rotary_sin;
    } else {
        p.cos = (const elem_t*)a->rotary_cos; p.sin = (const elem_t*)a->rotary_sin;
    }
    p.pos = a->position_ids;
    p.table_rows = (int)a->rotary_table_rows;
    p.batch = a->batch; p.max_ctx = a->max_ctx; p.nq = a->n_q_heads; p.nkv = a->n_kv_heads;
    p.n_rep = a->n_q_heads / a->n_kv_heads; p.n_splits = splits; p.n_hc = n_hc;
    p.c_sb = a->cache_stride_batch; p.c_st = a->cache_stride_token; p.c_sh = a->cache_stride_head;
    p.q_sb = a->q_stride_batch ? a->q_stride_batch : (int64_t)a->n_q_heads * a->head_dim;
    p.kn_sb = a->k_new_stride_batch ? a->k_new_stride_batch : (int64_t)a->n_kv_heads * a->head_dim;
    p.vn_sb = a->v_new_stride_batch ? a->v_new_stride_batch : (int64_t)a->n_kv_heads * a->head_dim;
    p.scale_log2 = a->softmax_scale * 1.4426950408889634f;
    p.ws_o = (float*)ws;
    p.ws_ml = p.ws_o + (size_t)a->batch * a->n_q_heads * splits * a->head_dim;
    hipStream_t st = (hipStream_t)a->stream;
    const int rot_mode = rot ? (a->rotary_interleaved ? 2 : 1) : 0;
    switch (a->head_dim) {
        case 32: return launch_decode<32>(p, a->k_new != nullptr, rot_mode, st);
        case 64: return launch_decode<64>(p, a->k_new != nullptr, rot_mode, st);
        case 96: return launch_decode<96>(p, a->k_new != nullptr, rot_mode, st);
        default: return launch_decode<128>(p, a->k_new != nullptr, rot_mode, st);
    }
}
}  // namespace

int MI_ENTRY(mi_attn_decode_impl)(const mi_decode_args* a, bool static_ws) {
    if (!a) return mi_fail(MI_E_NULL, "attn_decode: args is null");
    if (!static_ws) return decode_entry(a, a->workspace, a->workspace_bytes, false);
    // the entry point that allocates nothing: partial results go to the library's static device array
    void* ws = nullptr;
    size_t bytes = 0;
    const int rc = mi_static_scratch(&ws, &bytes);
    if (rc != MI_OK) return rc;
    return decode_entry(a, ws, bytes, true);
}
