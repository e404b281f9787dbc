// Shared pieces of the gfx950 attention kernels: parameter block, document lookup, mask ranges,
// MFMA wrapper and the LDS layouts used to feed v_mfma_f32_32x32x16_bf16.
//
// MFMA 32x32x16 (bf16) register layout, wavefront of 64 lanes, lane = 32*g + l32:
//   A operand (32 x 16): lane holds row l32,    k = 8*g + 0..7   (8 bf16 = 4 VGPRs)
//   B operand (16 x 32): lane holds column l32, k = 8*g + 0..7
//   C / D     (32 x 32): lane holds column l32, rows 8*(r/4) + 4*g + (r%4) for r = 0..15 (16 fp32 VGPRs)
// Because A and B use the same k assignment, any permutation of the contraction index that is applied
// to both operands leaves the product unchanged.  The kernels rely on that: a C tile is re-used
// directly as the B operand of the next product (contraction over its rows) with the k slot (g, i)
// standing for row 8*(i/4) + 4*g + (i%4) of a 16-row chunk, and the matching A operand is stored in
// LDS in exactly that order ("chunk order", see chunk_pos below).
#pragma once
#include "common.h"

struct AttnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; __bf16* o; float* lse;
    const int32_t* cu_q; const int32_t* cu_k;
    int n_docs; int causal;
    int total_q; int total_k;
    int nq; int nkv; int n_rep;
    int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;
    float scale_log2;   // softmax_scale * log2(e)
    const __bf16* cos; const __bf16* sin; const int64_t* pos_q; const int64_t* pos_k; int table_rows;
    // backward only
    const __bf16* d_o; __bf16* dq; __bf16* dk; __bf16* dv; float* delta;
    int64_t dk_st, dk_sh, dv_st, dv_sh;
    float scale;        // softmax_scale
};

__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// index j with cu[j] <= t < cu[j+1]  (cu has n_docs + 1 non-decreasing entries, cu[0] = 0)
__device__ __forceinline__ int find_doc(const int32_t* __restrict__ cu, int n_docs, int t) {
    int lo = 0, hi = n_docs;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

// allowed keys of query token t: [klo, khi) on the flattened key axis (empty when khi <= klo)
__device__ __forceinline__ void key_range(const AttnParams& p, int t, int& klo, int& khi) {
    if (t >= p.total_q) { klo = 0; khi = 0; return; }
    const int j = find_doc(p.cu_q, p.n_docs, t);
    const int qs = p.cu_q[j], qe = p.cu_q[j + 1];
    const int ks = p.cu_k[j], ke = p.cu_k[j + 1];
    klo = ks;
    khi = ke;
    if (p.causal) {
        const int lim = ks + (t - qs) + (ke - ks) - (qe - qs) + 1;
        khi = lim < ke ? lim : ke;
    }
    if (khi < klo) khi = klo;
}

// allowed queries of key token u: [qlo, qhi) on the flattened query axis (mirror image of key_range)
__device__ __forceinline__ void query_range(const AttnParams& p, int u, int& qlo, int& qhi) {
    if (u >= p.total_k) { qlo = 0; qhi = 0; return; }
    const int j = find_doc(p.cu_k, p.n_docs, u);
    const int qs = p.cu_q[j], qe = p.cu_q[j + 1];
    const int ks = p.cu_k[j], ke = p.cu_k[j + 1];
    qlo = qs;
    qhi = qe;
    if (p.causal) {
        // (u - ks) <= (t - qs) + (len_k - len_q)   <=>   t >= qs + (u - ks) - (len_k - len_q)
        const int lim = qs + (u - ks) - ((ke - ks) - (qe - qs));
        qlo = lim > qs ? lim : qs;
    }
    if (qlo > qhi) qlo = qhi;
}

// ---- "chunk order" LDS layout for operands whose contraction index is the row index of a C tile ----
// A [R rows][64 contraction] matrix is stored row-major (128 bytes per row) with the 16-byte units of a
// row XOR-swizzled; inside each 16-wide chunk the contraction indices are permuted so that lane group
// g finds its 8 k-slots contiguous: unit (2*m + g) of row r holds indices 16*m + {4g..4g+3, 8+4g..8+4g+3}.
// The swizzle depends on (row & 31) only, so the address of (row + 32*dt) is the address of row plus
// an immediate, and 16 consecutive rows read by one lane group hit 16 different bank quads.
__device__ __forceinline__ int swz(int row) { return ((row >> 1) & 7) ^ ((row >> 3) & 3); }

// byte offset of the 8-byte group holding contraction indices 4*quad .. 4*quad+3 (quad = index / 4)
template <int N> __device__ __forceinline__ int chunk_quad_offset(int row, int quad) {
    static_assert(N == 64, "one row = 8 swizzled units of 16 bytes");
    const int m = quad >> 2, kq = quad & 3;
    const int unit = 2 * m + (kq & 1);
    return row * (N * 2) + ((unit ^ swz(row)) << 4) + ((kq >> 1) << 3);
}

// byte offset of the 16-byte unit read by lane group g for chunk m of row `row`
template <int N> __device__ __forceinline__ int chunk_unit_offset(int row, int m, int g) {
    static_assert(N == 64, "one row = 8 swizzled units of 16 bytes");
    return row * (N * 2) + (((2 * m + g) ^ swz(row)) << 4);
}

// 4 tokens x 8 features held as 4 row vectors -> for feature dd the 4 token values as one 8-byte group
__device__ __forceinline__ uint2 transpose_quad(const uint4 (&raw)[4], int dd) {
    const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&raw[0]);
    const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&raw[1]);
    const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&raw[2]);
    const uint32_t* w3 = reinterpret_cast<const uint32_t*>(&raw[3]);
    const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;   // high / low halves of the two words
    return make_uint2(__builtin_amdgcn_perm(w1[dd >> 1], w0[dd >> 1], sel),
                      __builtin_amdgcn_perm(w3[dd >> 1], w2[dd >> 1], sel));
}

// ---- LDS transpose read (gfx950 ds_read_b64_tr_b16) ---------------------------------------------------
// Within each block of 16 lanes the instruction loads 16 x 8 bytes and hands lane j the j-th 16-bit element
// of each of the four 32-byte rows formed by lanes {0..3}, {4..7}, {8..11}, {12..15}.  With a token-major
// [token][feature] tile in LDS, pointing lane i of a block at token (t0 + i/4), features (f0 + 4*(i%4) ..)
// returns to lane j the values of tokens t0..t0+3 at feature f0 + j: the transposed A operand of an MFMA
// whose contraction index is the token, without a transposed copy of the tile.
// Row stride: 4 rows x 2 feature halves of 32 bytes are touched per 32 lanes; a stride of 64 (mod 256)
// bytes puts them on disjoint banks (measured: no conflicts), whereas 16-byte-odd strides conflict.
typedef short v4i16_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i16_t lds_read_tr16_b64(const void* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) v4i16_t*)(__attribute__((address_space(3))) void*)p);
}

// A operand (32 rows = features f0 + l32, 16-token chunk m in chunk order) of a token-major tile with
// `stride_bytes` per token: lane_base = tr_lane_base(lane, stride_bytes), then for chunk m and feature tile
// dt the two halves are at lane_base + (16*m + 8*half) * stride_bytes + 64*dt.
__device__ __forceinline__ int tr_lane_base(int lane, int stride_bytes) {
    const int g = lane >> 5, i = lane & 15, blk = (lane >> 4) & 1;
    return (4 * g + (i >> 2)) * stride_bytes + (16 * blk + 4 * (i & 3)) * 2;
}

__device__ __forceinline__ bf16x8_t tr_operand(const char* tile, int lane_base, int stride_bytes, int m, int dt) {
    const v4i16_t lo = lds_read_tr16_b64(tile + lane_base + (16 * m) * stride_bytes + 64 * dt);
    const v4i16_t hi = lds_read_tr16_b64(tile + lane_base + (16 * m + 8) * stride_bytes + 64 * dt);
    typedef short v8i16_t __attribute__((ext_vector_type(8)));
    const v8i16_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
}

// 128-bit load / store through a native vector type.  Copying a uint4 (a struct) between address spaces
// becomes a memcpy that keeps staging arrays in scratch memory; building the value element-wise lets
// them live in registers.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ld128(const void* p) {
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(p);
    return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void st128(void* p, const uint4& x) {
    u32x4_t v;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    *reinterpret_cast<u32x4_t*>(p) = v;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2_t p;
    p[0] = (__bf16)lo;
    p[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// rotate-half rotary applied to a (first-half, second-half) pair of 8-element vectors; cos/sin hold
// the table values of the first-half columns (both table halves are equal by construction)
__device__ __forceinline__ void rotate_pair(uint4& lo, uint4& hi, const uint4& c, const uint4& s, float sign) {
    uint32_t* l = reinterpret_cast<uint32_t*>(&lo);
    uint32_t* h = reinterpret_cast<uint32_t*>(&hi);
    const uint32_t* cw = reinterpret_cast<const uint32_t*>(&c);
    const uint32_t* sw = reinterpret_cast<const uint32_t*>(&s);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float x0a = bf16_lo(l[i]), x0b = bf16_hi(l[i]);
        const float x1a = bf16_lo(h[i]), x1b = bf16_hi(h[i]);
        const float ca = bf16_lo(cw[i]), cb = bf16_hi(cw[i]);
        const float sa = sign * bf16_lo(sw[i]), sb = sign * bf16_hi(sw[i]);
        l[i] = pack_bf16x2(x0a * ca - x1a * sa, x0b * cb - x1b * sb);
        h[i] = pack_bf16x2(x1a * ca + x0a * sa, x1b * cb + x0b * sb);
    }
}

// maps the linear workgroup id to a work item so that the workgroups an XCD receives (ids congruent
// modulo 8) form one contiguous range of work items (neighbouring items share K/V in that XCD's L2)
__device__ __forceinline__ int xcd_remap(int linear, int total) {
    if ((total & 7) != 0) return linear;
    return (linear & 7) * (total >> 3) + (linear >> 3);
}
