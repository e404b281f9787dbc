// Stand-alone rotary embedding (rotate-half pairing) for gfx950: one pass, 128-bit accesses.
//
// One thread owns a 128-bit vector of the first half of the rotated span and its partner vector
// rot_dim/2 further on, so both outputs of every (i, i + rot_dim/2) pair come from one thread.  The
// features beyond rot_dim are copied.  A scalar kernel covers head sizes that do not vectorise.
#include "common.h"

namespace {

constexpr int kBlock = 256;

struct RotaryParams {
    const void* x; void* out; const void* cos; const void* sin; const int64_t* pos;
    int64_t n_tokens; int n_heads; int head_dim; int rot_dim;
    int64_t xs_t, xs_h, os_t, os_h;
    int64_t table_rows, seq_len_null; float sign;
};

__device__ __forceinline__ int64_t table_row(const RotaryParams& p, int64_t t) {
    int64_t r = p.pos ? p.pos[t] : (t % p.seq_len_null);
    if (r < 0) r = 0;
    if (r >= p.table_rows) r = p.table_rows - 1;
    return r;
}

// reads N consecutive table values (N = 4 or 8) starting at a 16-byte aligned address
template <typename TT, int N> __device__ __forceinline__ void load_table(const TT* ptr, float* f) {
    if constexpr (sizeof(TT) == 4) {
#pragma unroll
        for (int j = 0; j < N / 4; ++j) Elem<float>::unpack(reinterpret_cast<const uint4*>(ptr)[j], f + 4 * j);
    } else {
        static_assert(N == 8, "16-bit tables are read 8 values at a time");
        Elem<TT>::unpack(*reinterpret_cast<const uint4*>(ptr), f);
    }
}

// T: data type, TT: table type.  Work item = (token, head, vec) with vec over half the rotated span
// followed by the vectors of the unrotated tail.
template <typename T, typename TT>
__global__ __launch_bounds__(kBlock) void rotary_vec_kernel(RotaryParams p) {
    constexpr int V = Elem<T>::kVec;
    const int half_vecs = p.rot_dim / 2 / V;
    const int tail_vecs = (p.head_dim - p.rot_dim) / V;
    const int per_head = half_vecs + tail_vecs;
    const int64_t per_token = (int64_t)per_head * p.n_heads;
    const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= per_token * p.n_tokens) return;
    const int64_t t = item / per_token;
    const int rem = (int)(item % per_token);
    const int h = rem / per_head;
    const int v = rem % per_head;
    const T* xrow = (const T*)p.x + t * p.xs_t + (int64_t)h * p.xs_h;
    T* orow = (T*)p.out + t * p.os_t + (int64_t)h * p.os_h;
    if (v >= half_vecs) {  // unrotated tail
        const int c = p.rot_dim + (v - half_vecs) * V;
        if ((const void*)xrow != (const void*)orow)
            stg_nt(reinterpret_cast<uint4*>(orow + c), *reinterpret_cast<const uint4*>(xrow + c));
        return;
    }
    const int c0 = v * V, c1 = c0 + p.rot_dim / 2;
    const int64_t r = table_row(p, t);
    const TT* cr = (const TT*)p.cos + r * p.rot_dim;
    const TT* sr = (const TT*)p.sin + r * p.rot_dim;
    float x0[V], x1[V], o0[V], o1[V], cA[V], sA[V], cB[V], sB[V];
    Elem<T>::unpack(ldg_nt(reinterpret_cast<const uint4*>(xrow + c0)), x0);
    Elem<T>::unpack(ldg_nt(reinterpret_cast<const uint4*>(xrow + c1)), x1);
    load_table<TT, V>(cr + c0, cA);
    load_table<TT, V>(sr + c0, sA);
    load_table<TT, V>(cr + c1, cB);
    load_table<TT, V>(sr + c1, sB);
#pragma unroll
    for (int i = 0; i < V; ++i) {
        o0[i] = x0[i] * cA[i] - x1[i] * (p.sign * sA[i]);
        o1[i] = x1[i] * cB[i] + x0[i] * (p.sign * sB[i]);
    }
    stg_nt(reinterpret_cast<uint4*>(orow + c0), Elem<T>::pack(o0));
    stg_nt(reinterpret_cast<uint4*>(orow + c1), Elem<T>::pack(o1));
}

template <typename T, typename TT>
__global__ __launch_bounds__(kBlock) void rotary_scalar_kernel(RotaryParams p) {
    const int half = p.rot_dim / 2;
    const int per_head = half + (p.head_dim - p.rot_dim);
    const int64_t per_token = (int64_t)per_head * p.n_heads;
    const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= per_token * p.n_tokens) return;
    const int64_t t = item / per_token;
    const int rem = (int)(item % per_token);
    const int h = rem / per_head;
    const int i = rem % per_head;
    const T* xrow = (const T*)p.x + t * p.xs_t + (int64_t)h * p.xs_h;
    T* orow = (T*)p.out + t * p.os_t + (int64_t)h * p.os_h;
    if (i >= half) {
        const int c = p.rot_dim + (i - half);
        Elem<T>::store1(orow + c, Elem<T>::load1(xrow + c));
        return;
    }
    const int64_t r = table_row(p, t);
    const TT* cr = (const TT*)p.cos + r * p.rot_dim;
    const TT* sr = (const TT*)p.sin + r * p.rot_dim;
    const float x0 = Elem<T>::load1(xrow + i), x1 = Elem<T>::load1(xrow + i + half);
    const float o0 = x0 * Elem<TT>::load1(cr + i) - x1 * (p.sign * Elem<TT>::load1(sr + i));
    const float o1 = x1 * Elem<TT>::load1(cr + i + half) + x0 * (p.sign * Elem<TT>::load1(sr + i + half));
    Elem<T>::store1(orow + i, o0);
    Elem<T>::store1(orow + i + half, o1);
}

// Interleaved ("complex") pairing (2i, 2i+1) over the whole head, fp32 tables [rows, head_dim/2].
// One thread owns one 128-bit vector = V/2 complete pairs.
template <typename T>
__global__ __launch_bounds__(kBlock) void rotary_complex_kernel(RotaryParams p) {
    constexpr int V = Elem<T>::kVec;
    const int vec_per_head = p.head_dim / V;
    const int64_t per_token = (int64_t)vec_per_head * p.n_heads;
    const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= per_token * p.n_tokens) return;
    const int64_t t = item / per_token;
    const int rem = (int)(item % per_token);
    const int h = rem / vec_per_head, v = rem % vec_per_head;
    const T* xrow = (const T*)p.x + t * p.xs_t + (int64_t)h * p.xs_h + v * V;
    T* orow = (T*)p.out + t * p.os_t + (int64_t)h * p.os_h + v * V;
    const int64_t r = table_row(p, t);
    const float* cr = (const float*)p.cos + r * (p.head_dim / 2) + v * (V / 2);
    const float* sr = (const float*)p.sin + r * (p.head_dim / 2) + v * (V / 2);
    float x[V], o[V];
    Elem<T>::unpack(*reinterpret_cast<const uint4*>(xrow), x);
#pragma unroll
    for (int i = 0; i < V / 2; ++i) {
        o[2 * i] = x[2 * i];
        o[2 * i + 1] = x[2 * i + 1];
        rotate_complex_pair(o[2 * i], o[2 * i + 1], cr[i], p.sign * sr[i]);
    }
    stg_nt(reinterpret_cast<uint4*>(orow), Elem<T>::pack(o));
}

template <typename T, typename TT> int launch(const RotaryParams& p, hipStream_t st) {
    constexpr int V = Elem<T>::kVec;
    const bool vec_ok = (p.rot_dim / 2) % V == 0 && (p.head_dim - p.rot_dim) % V == 0 && p.xs_t % V == 0 &&
                        p.xs_h % V == 0 && p.os_t % V == 0 && p.os_h % V == 0 && mi_aligned16(p.x) && mi_aligned16(p.out) &&
                        mi_aligned16(p.cos) && mi_aligned16(p.sin) && (sizeof(TT) == 4 || V == 8);
    int64_t per_head = vec_ok ? (p.rot_dim / 2 / V + (p.head_dim - p.rot_dim) / V) : (p.rot_dim / 2 + p.head_dim - p.rot_dim);
    const int64_t items = per_head * p.n_heads * p.n_tokens;
    const int64_t blocks = (items + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "rotary: too many elements");
    if (vec_ok)
        rotary_vec_kernel<T, TT><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(p);
    else
        rotary_scalar_kernel<T, TT><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(p);
    return mi_check_launch("rotary");
}

}  // namespace

extern "C" int mi_rotary(const void* x, void* out, const void* cos, const void* sin, const int64_t* position_ids,
                         int64_t n_tokens, int32_t n_heads, int32_t head_dim, int32_t rot_dim, int64_t x_stride_token,
                         int64_t x_stride_head, int64_t out_stride_token, int64_t out_stride_head, int64_t table_rows,
                         int64_t seq_len_for_null_ids, int inverse, int dtype, int table_dtype, void* stream) {
    if (n_tokens == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !out || !cos || !sin) return mi_fail(MI_E_NULL, "rotary: null pointer");
    if (n_tokens < 0 || n_heads <= 0 || head_dim <= 0 || rot_dim <= 1 || rot_dim > head_dim || (rot_dim & 1) || table_rows <= 0)
        return mi_fail(MI_E_SHAPE, "rotary: bad shape tokens=%lld heads=%d head_dim=%d rot_dim=%d table_rows=%lld",
                       (long long)n_tokens, n_heads, head_dim, rot_dim, (long long)table_rows);
    if (!position_ids && seq_len_for_null_ids <= 0) return mi_fail(MI_E_SHAPE, "rotary: need position ids or a sequence length");
    if (table_dtype != dtype && table_dtype != MI_F32) return mi_fail(MI_E_DTYPE, "rotary: table dtype must equal the data dtype or be fp32");
    RotaryParams p{x, out, cos, sin, position_ids, n_tokens, n_heads, head_dim, rot_dim, x_stride_token, x_stride_head,
                   out_stride_token, out_stride_head, table_rows, seq_len_for_null_ids, inverse ? -1.0f : 1.0f};
    MI_DISPATCH_DTYPE(dtype, {
        if (table_dtype == dtype) return launch<T, T>(p, (hipStream_t)stream);
        return launch<T, float>(p, (hipStream_t)stream);
    });
    return MI_OK;
}

extern "C" int mi_rotary_complex(const void* x, void* out, const float* cos, const float* sin, const int64_t* position_ids,
                                 int64_t n_tokens, int32_t n_heads, int32_t head_dim, int64_t x_stride_token,
                                 int64_t x_stride_head, int64_t out_stride_token, int64_t out_stride_head,
                                 int64_t table_rows, int64_t seq_len_for_null_ids, int inverse, int dtype, void* stream) {
    if (n_tokens == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !out || !cos || !sin) return mi_fail(MI_E_NULL, "rotary_complex: null pointer");
    if (n_tokens < 0 || n_heads <= 0 || head_dim <= 0 || table_rows <= 0)
        return mi_fail(MI_E_SHAPE, "rotary_complex: bad shape tokens=%lld heads=%d head_dim=%d", (long long)n_tokens, n_heads, head_dim);
    if (!position_ids && seq_len_for_null_ids <= 0) return mi_fail(MI_E_SHAPE, "rotary_complex: need position ids or a sequence length");
    RotaryParams p{x, out, cos, sin, position_ids, n_tokens, n_heads, head_dim, head_dim, x_stride_token, x_stride_head,
                   out_stride_token, out_stride_head, table_rows, seq_len_for_null_ids, inverse ? -1.0f : 1.0f};
    MI_DISPATCH_DTYPE(dtype, {
        constexpr int V = Elem<T>::kVec;
        if (head_dim % V || x_stride_token % V || x_stride_head % V || out_stride_token % V || out_stride_head % V ||
            !mi_aligned16(x) || !mi_aligned16(out))
            return mi_fail(MI_E_ALIGN, "rotary_complex: head_dim and strides must be multiples of %d elements, pointers 16-byte aligned", V);
        const int64_t items = (int64_t)(head_dim / V) * n_heads * n_tokens;
        const int64_t blocks = (items + kBlock - 1) / kBlock;
        if (blocks > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "rotary_complex: too many elements");
        rotary_complex_kernel<T><<<dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream>>>(p);
    });
    return mi_check_launch("rotary_complex");
}
