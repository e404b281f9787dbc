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

#include <type_traits>

// Element type of q / k / v / o and of every MFMA operand.  Each attention source file is compiled twice: as is for
// bfloat16 and with MI_ELEM_F16 for float16 (half-precision MFMA, same tilings); the bfloat16 objects export the C
// entry points and hand float16 calls to the MI_ENTRY(...)-named functions of the float16 objects.
#ifdef MI_ELEM_F16
typedef _Float16 elem_t;
typedef _Float16 elem2_t __attribute__((ext_vector_type(2)));
typedef _Float16 elem4_t __attribute__((ext_vector_type(4)));
typedef _Float16 elem8_t __attribute__((ext_vector_type(8)));
#define MI_ELEM_DTYPE MI_F16
#else
typedef __bf16 elem_t;
typedef bf16x2_t elem2_t;
typedef bf16x4_t elem4_t;
typedef bf16x8_t elem8_t;
#define MI_ELEM_DTYPE MI_BF16
#endif

struct AttnParams {
    const elem_t* q; const elem_t* k; const elem_t* v; elem_t* o; float* lse;
    const int32_t* cu_q; const int32_t* cu_k;
    int n_docs; int causal;
    int total_q; int total_k;
    int nq; int nkv; int n_rep;
    int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;
    float scale_log2;   // softmax_scale * log2(e)
    const elem_t* cos; const elem_t* sin; const int64_t* pos_q; const int64_t* pos_k; int table_rows;
    const float* cos32; const float* sin32;   // interleaved-pair rotary: fp32 tables [table_rows, head_dim / 2]
    // backward only
    const elem_t* d_o; elem_t* dq; elem_t* dk; elem_t* dv; float* delta;
    int64_t dk_st, dk_sh, dv_st, dv_sh;
    float scale;        // softmax_scale
    // dropout on the attention probabilities (0 = off): an element is dropped iff its random byte < drop_thr,
    // kept probabilities are scaled by drop_rscale = 256 / (256 - drop_thr)
    uint32_t drop_thr; float drop_rscale; uint32_t drop_seed;
    // blocks per document on the query / key axis when the workgroups are to be handed out across documents
    // (see block_for_rank), 0 for the order along the flattened axis; set by the host entry points
    int across_q, across_k;
    // documents of different lengths: hand the blocks out longest-processing-time first, by the order that every
    // workgroup derives from the cumulative lengths itself (see lpt_order); set by the host entry points where the
    // hand-out across documents pays (same conditions as across_q / across_k) and the batch does not look equal-length
    int lpt_q, lpt_k;
    // dK/dV with fewer than 8 KV heads: the query heads of a group are split over hsplit workgroups per key block,
    // each writing fp32 partial sums [hsplit][total_k][nkv][head_dim] that a reduce launch adds up (1 = no split)
    int hsplit; float* dk_part; float* dv_part;
    // forward: optional copy of the rotated q (fused rotary), same strides as q
    elem_t* q_rot;
    // backward with rotary: q / k are the rotated tensors; dq / dk leave the kernels rotated back (0 = no rotary,
    // 1 = rotate-half with tables in the I/O dtype, 2 = interleaved pairs with fp32 tables)
    int unrotate;
};

// ---- dropout mask ---------------------------------------------------------------------------------------
// The random byte of element (query q, key k) of a head is a pure function of (seed, head, q, k), so the
// forward and both backward kernels regenerate the same mask whatever their tiling:
//   x = head_base + (q >> 1) * C1 + (k >> 1) * C2          (mod 2^32)
//   h = lowbias32(x)                                       (two multiply / xor-shift rounds)
//   byte = (h >> (16 * (q & 1) + 8 * (k & 1))) & 0xff
// One hash serves a 2 x 2 block of elements, two of which any lane of either score-tile layout holds.
constexpr uint32_t kDropC1 = 0x9E3779B1u, kDropC2 = 0x85EBCA77u;

__host__ __device__ __forceinline__ uint32_t lowbias32(uint32_t x) {
    x ^= x >> 16; x *= 0x7FEB352Du;
    x ^= x >> 15; x *= 0x846CA68Bu;
    x ^= x >> 16;
    return x;
}

__device__ __forceinline__ uint32_t drop_head_base(uint32_t seed, int head) {
    return lowbias32(seed ^ lowbias32((uint32_t)head * 0x9E3779B9u + 0x7F4A7C15u));
}

// byte `field` (0..3) of the block hash
__device__ __forceinline__ uint32_t drop_byte(uint32_t h, uint32_t shift) { return __builtin_amdgcn_ubfe(h, shift, 8); }

__device__ __forceinline__ f32x16_t mfma_32x32x16(elem8_t a, elem8_t b, f32x16_t c) {
#ifdef MI_ELEM_F16
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#endif
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max / sum of a value with that of the lane 32 further on (lane ^ 32), exchanged inside the VALU by v_permlane32_swap
// (afterwards every lane holds the pair (value of the low lane, value of the high lane)) instead of through the LDS
// crossbar, whose round trip would sit in the middle of the softmax chain of every tile
__device__ __forceinline__ float pair_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// the same over the four lanes l16, l16 + 16, l16 + 32, l16 + 48 (v_permlane16_swap pairs the rows of 16 lanes)
__device__ __forceinline__ float quad_max(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return pair_max(fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])));
}
__device__ __forceinline__ float pair_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float quad_sum(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return pair_sum(__uint_as_float(r[0]) + __uint_as_float(r[1]));
}

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

// "Chunk order": a 32x32 accumulator tile holds, for lane group g, rows 8*(r/4) + 4g + r%4 in register r.
// Used as the B operand of the next product (contraction over those rows), k-slot i of lane group g of
// 16-row chunk m is row 16m + 8*(i/4) + 4g + i%4, so the matching A operand takes tokens
// 16m + 4g + {0..3} (first transpose read) and 16m + 8 + 4g + {0..3} (second).
typedef short v8i16_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ elem8_t tr_pair(const char* lo_addr, const char* hi_addr) {
    const v4i16_t lo = lds_read_tr16_b64(lo_addr);
    const v4i16_t hi = lds_read_tr16_b64(hi_addr);
    const v8i16_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(elem8_t, both);
}

// ---- token-major LDS tile filled by direct global -> LDS loads ------------------------------------------
// 64 tokens, unpadded rows of UPR 16-byte units (head_dim 96 uses rows of 16 units, 12 of them live).
// A direct load instruction writes 64 x 16 bytes to consecutive LDS addresses (lane i -> base + 16 i), so
// padding is impossible; instead the unit index of row r is XORed with f(r), chosen so that
//   row operand   (lane = token, 16 bytes per k-step): 16 consecutive rows at one k-step hit 16 different
//                 16-byte bank groups,
//   transposed    (ds_read_b64_tr_b16; lane = feature, k-slots = tokens): the 4 rows x 2 x 32 bytes touched by
//                 32 lanes cover 256 distinct bytes (mod 256),
// and a loader lane simply fetches the logical unit (physical ^ f(row)) of its row from global memory.
// Rows of an operand start at a multiple of 16, so f is fixed per lane.
template <int D> struct LdsTile {
    static_assert(D == 32 || D == 64 || D == 96 || D == 128, "head_dim");
    static constexpr int UPR = (D == 96) ? 16 : D / 8;   // physical units per row
    static constexpr int RB = 16 * UPR;                  // bytes per row
    static constexpr int kInstrs = UPR;                  // direct-load instructions per 64-token tile
    static constexpr int kBytes = 64 * RB;

    static __device__ __forceinline__ int f(int r) {
        if constexpr (UPR == 16) return ((r & 3) << 2) | ((r >> 2) & 3);
        else if constexpr (UPR == 8) return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
        else return (r >> 2) & 3;
    }
    // byte offset of logical 16-byte unit c of row r (register-staged stores)
    static __device__ __forceinline__ int unit_offset(int r, int c) { return r * RB + ((c ^ f(r)) << 4); }
    // direct-load instruction n of a tile, lane -> source row and logical unit (unit >= D/8: nothing to fetch)
    static __device__ __forceinline__ void dma_src(int n, int lane, int& row, int& unit) {
        const int u = 64 * n + lane;
        row = u / UPR;
        unit = (u % UPR) ^ f(row);
    }
    // row operand of lane (row, g): k-step ks is at (row_base ^ (ks << 5))
    static __device__ __forceinline__ int row_base(int row, int g) { return row * RB + ((g ^ f(row)) << 4); }
    // transposed operand: 16-token chunk m (chunk order), feature tile dt:
    //   tr_pair(tile + (h0 ^ (dt << 6)) + 16*m*RB, tile + (h1 ^ (dt << 6)) + 16*m*RB)
    static __device__ __forceinline__ void tr_bases(int lane, int& h0, int& h1) {
        const int g = lane >> 5, i = lane & 15, blk = (lane >> 4) & 1;
        const int j = i >> 2, e = (i >> 1) & 1, hb = i & 1;
        const int r0 = 4 * g + j, r1 = 8 + 4 * g + j;
        h0 = r0 * RB + (((2 * blk + e) ^ f(r0)) << 4) + 8 * hb;
        h1 = r1 * RB + (((2 * blk + e) ^ f(r1)) << 4) + 8 * hb;
    }
};

// Direct global -> LDS loads of 64-token tiles by one wavefront: instructions [n0, n0 + COUNT) of each tile.
// The per-lane byte offsets inside a tile are fixed for the kernel, so a tile costs COUNT instructions with
// a scalar base address and no vector arithmetic; only a tile that runs past the last token recomputes its
// offsets (rows past the end repeat the last token).
// Issued through inline assembly on purpose: the compiler would otherwise wait for every outstanding
// direct load (vmcnt(0)) before each barrier and LDS read, which serialises the ring; completion is
// tracked by the explicit wait_vmcnt below instead.
template <int D, int COUNT> struct DmaPlan {
    using T = LdsTile<D>;
    uint32_t off[COUNT];     // byte offset of this lane's 16 bytes from the first token of a full tile
    int n0, lane;

    __device__ __forceinline__ static void src_of(int n, int lane_, int& row, int& unit_off) {
        int unit;
        T::dma_src(n, lane_, row, unit);
        if (D == 96 && unit >= D / 8) unit = 0;          // dead physical units of the padded row
        unit_off = 16 * unit;
    }
    __device__ __forceinline__ void init(int first_instr, int lane_, int64_t tok_stride) {
        n0 = first_instr;
        lane = lane_;
#pragma unroll
        for (int j = 0; j < COUNT; ++j) {
            int row, unit_off;
            src_of(n0 + j, lane, row, unit_off);
            off[j] = (uint32_t)(row * (int)tok_stride * 2 + unit_off);
        }
    }
    __device__ __forceinline__ static void issue_one(uint32_t voff, const void* sbase, char* dst_lds) {
        const uint32_t dst = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)dst_lds;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(dst)) : "memory", "m0");
    }
    // All COUNT instructions of the tile whose first token is tok0, straight-line when the tile is full.
    // tile: wave-uniform LDS address of the stage; base + tok0 * tok_stride must be wave-uniform too.
    __device__ __forceinline__ void issue(const elem_t* base, int64_t tok_stride, int tok0, int last_tok, char* tile) const {
        char* dst = tile + 1024 * n0;
        if (tok0 + 63 <= last_tok) {
            const elem_t* tile_base = base + (int64_t)tok0 * tok_stride;
#pragma unroll
            for (int j = 0; j < COUNT; ++j) issue_one(off[j], tile_base, dst + 1024 * j);
        } else {
            const int first = min(tok0, last_tok);            // the lane offsets below must not be negative
            const elem_t* tile_base = base + (int64_t)first * tok_stride;
            int l = lane;
            asm volatile("" : "+v"(l));   // opaque: keeps this rarely used arithmetic from being hoisted out of the caller's loop
#pragma unroll
            for (int j = 0; j < COUNT; ++j) {
                int row, unit_off;
                src_of(n0 + j, l, row, unit_off);
                const int r = min(row, last_tok - first);
                issue_one((uint32_t)(r * (int)tok_stride * 2 + unit_off), tile_base, dst + 1024 * j);
            }
        }
    }
};

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index is a constant
// expression inside the body
template <int N, int I = 0, class F> __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// waits until at most n (wave-uniform, run-time) vector memory loads are outstanding; large n waits for less
// than asked only in the sense of waiting for everything older than the newest 24
template <int N> __device__ __forceinline__ void wait_vmcnt();
__device__ __forceinline__ void wait_vmcnt_dyn(int n) {
    switch (n) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<1>(); break;
        case 2: wait_vmcnt<2>(); break;
        case 3: wait_vmcnt<3>(); break;
        case 4: wait_vmcnt<4>(); break;
        case 5: wait_vmcnt<5>(); break;
        case 6: wait_vmcnt<6>(); break;
        case 7: wait_vmcnt<7>(); break;
        case 8: wait_vmcnt<8>(); break;
        case 9: case 10: case 11: wait_vmcnt<9>(); break;
        case 12: case 13: case 14: case 15: wait_vmcnt<12>(); break;
        default: if (n >= 16) wait_vmcnt<16>(); else wait_vmcnt<0>(); break;
    }
}

// waits until at most N of this wavefront's vector memory loads are outstanding (N compile-time)
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// 128-bit load / store through a native vector type.  Copying a uint4 (a struct) between address spaces
// becomes a memcpy that keeps staging arrays in scratch memory; building the value element-wise lets
// them live in registers.
__device__ __forceinline__ uint4 ld128(const void* p) {
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(p);
    return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void st128(void* p, const uint4& x) {
    u32x4_t v;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    *reinterpret_cast<u32x4_t*>(p) = v;
}

__device__ __forceinline__ uint32_t pack_elem2(float lo, float hi) {
    elem2_t p;
    p[0] = (elem_t)lo;
    p[1] = (elem_t)hi;
    return __builtin_bit_cast(uint32_t, p);
}

#ifdef MI_ELEM_F16
__device__ __forceinline__ float elem_lo(uint32_t w) { return (float)__builtin_bit_cast(elem2_t, w)[0]; }
__device__ __forceinline__ float elem_hi(uint32_t w) { return (float)__builtin_bit_cast(elem2_t, w)[1]; }
#else
__device__ __forceinline__ float elem_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float elem_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
#endif

// rotate-half rotary applied to a (first-half, second-half) pair of 8-element vectors; cos/sin hold
// the table values of the first-half columns (both table halves are equal by construction)
__device__ __forceinline__ void rotate_pair(uint4& lo, uint4& hi, const uint4& c, const uint4& s, float sign) {
    uint32_t* l = reinterpret_cast<uint32_t*>(&lo);
    uint32_t* h = reinterpret_cast<uint32_t*>(&hi);
    const uint32_t* cw = reinterpret_cast<const uint32_t*>(&c);
    const uint32_t* sw = reinterpret_cast<const uint32_t*>(&s);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float x0a = elem_lo(l[i]), x0b = elem_hi(l[i]);
        const float x1a = elem_lo(h[i]), x1b = elem_hi(h[i]);
        const float ca = elem_lo(cw[i]), cb = elem_hi(cw[i]);
        const float sa = sign * elem_lo(sw[i]), sb = sign * elem_hi(sw[i]);
        l[i] = pack_elem2(x0a * ca - x1a * sa, x0b * cb - x1b * sb);
        h[i] = pack_elem2(x1a * ca + x0a * sa, x1b * cb + x0b * sb);
    }
}

// interleaved-pair rotary of one 8-element vector = 4 pairs (2i, 2i+1); c / s hold the 4 fp32 table values
__device__ __forceinline__ void rotate_interleaved(uint4& v, const uint4& c, const uint4& s, float sign) {
    uint32_t* w = reinterpret_cast<uint32_t*>(&v);
    const uint32_t* cw = reinterpret_cast<const uint32_t*>(&c);
    const uint32_t* sw = reinterpret_cast<const uint32_t*>(&s);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float x0 = elem_lo(w[i]), x1 = elem_hi(w[i]);
        rotate_complex_pair(x0, x1, __uint_as_float(cw[i]), sign * __uint_as_float(sw[i]));
        w[i] = pack_elem2(x0, x1);
    }
}

// Inverse rotary (rotation by minus the position's angles) of one token's gradient row held in accumulator layout:
// acc[dt][4 a + c] is feature 32 dt + 8 a + 4 g + c of the lane's token.  Rotate-half pairs feature f with f + D / 2
// (accumulators dt and dt + D / 64, same register), the interleaved form pairs registers (4 a, 4 a + 1) and
// (4 a + 2, 4 a + 3).  fp32 throughout; the caller rounds once afterwards.
template <int D>
__device__ __forceinline__ void unrotate_acc(f32x16_t (&acc)[D / 32], const AttnParams& p, int64_t pos, int g) {
    static_assert(D == 64 || D == 128, "fused rotary covers head_dim 64 and 128");
    constexpr int DT = D / 32;
    pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
    if (p.unrotate == 1) {
        const elem_t* cr = p.cos + pos * D + 4 * g;
        const elem_t* sr = p.sin + pos * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT / 2; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const uint2 cw = *reinterpret_cast<const uint2*>(cr + 32 * dt + 8 * a);
                const uint2 sw = *reinterpret_cast<const uint2*>(sr + 32 * dt + 8 * a);
                const float c4[4] = {elem_lo(cw.x), elem_hi(cw.x), elem_lo(cw.y), elem_hi(cw.y)};
                const float s4[4] = {elem_lo(sw.x), elem_hi(sw.x), elem_lo(sw.y), elem_hi(sw.y)};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float x0 = acc[dt][4 * a + c], x1 = acc[dt + DT / 2][4 * a + c];
                    acc[dt][4 * a + c] = x0 * c4[c] + x1 * s4[c];
                    acc[dt + DT / 2][4 * a + c] = x1 * c4[c] - x0 * s4[c];
                }
            }
    } else {
        const float* cr = p.cos32 + pos * (D / 2) + 2 * g;
        const float* sr = p.sin32 + pos * (D / 2) + 2 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const float2 c2 = *reinterpret_cast<const float2*>(cr + 16 * dt + 4 * a);
                const float2 s2 = *reinterpret_cast<const float2*>(sr + 16 * dt + 4 * a);
                float x0 = acc[dt][4 * a], x1 = acc[dt][4 * a + 1], y0 = acc[dt][4 * a + 2], y1 = acc[dt][4 * a + 3];
                rotate_complex_pair(x0, x1, c2.x, -s2.x);
                rotate_complex_pair(y0, y1, c2.y, -s2.y);
                acc[dt][4 * a] = x0; acc[dt][4 * a + 1] = x1; acc[dt][4 * a + 2] = y0; acc[dt][4 * a + 3] = y1;
            }
    }
}

// Work item (query head, rank of its query block) of workgroup `linear` in a grid of n_heads * n_blocks workgroups
// that hands an XCD the workgroups congruent to it modulo 8: every XCD gets whole heads (n_heads / 8 neighbouring
// ones, which share K / V within a GQA group) with all their blocks, heaviest rank first, so the XCDs carry equal
// work whatever the number of KV heads.  (Giving an XCD a contiguous slice of a kv-head-major item list, the
// earlier scheme, coincides with this for 8 or more KV heads and leaves one XCD with all the long blocks for fewer:
// multi-query attention ran 1.7x slower.)  Without a head count divisible by 8: head fastest, no XCD grouping.
__device__ __forceinline__ void head_and_rank(int linear, int n_heads, int& head, int& rank) {
    if ((n_heads & 7) == 0) {
        const int hpx = n_heads >> 3, j = linear >> 3;
        rank = j / hpx;
        head = (linear & 7) * hpx + (j - rank * hpx);
    } else {
        rank = linear / n_heads;
        head = linear - rank * n_heads;
    }
}

// Block of the token axis that is handed out rank-th: longest first under a causal mask, where a query block has
// the more work the later it sits in its document (late_first) and a key block the earlier.  By position on the
// whole axis (exact for one document) or, with per_doc != 0, the r-th longest blocks of all documents before the
// (r + 1)-th longest, for n_docs documents of per_doc blocks each.  Always a permutation of the blocks.
__device__ __forceinline__ int block_for_rank(int rank, int n_blocks, int n_docs, int per_doc, bool late_first) {
    if (per_doc != 0) {
        const int pos = rank / n_docs, doc = rank - pos * n_docs;
        return doc * per_doc + (late_first ? per_doc - 1 - pos : pos);
    }
    return late_first ? n_blocks - 1 - rank : rank;
}

// Longest-processing-time-first order of the blocks of a token axis whose documents differ in length: perm_lds[r] =
// block that is handed out r-th.  A block's work is estimated as the extent of the union of the allowed ranges of its
// first and its last token (exact for causal and bidirectional documents whose q and k lengths agree); ties go to the
// lower block index, so the result is a permutation whatever the estimate.  Every workgroup computes the same table
// from the cumulative lengths (two interval lookups per block, then a rank by counting: n_blocks <= kLptMax keeps
// that under a microsecond), so no extra launch, workspace or host read-back is involved.  All threads of the
// workgroup must call; ends with a barrier.
constexpr int kLptMax = 128;
template <bool KEY_BLOCKS>
__device__ __forceinline__ void lpt_order(const AttnParams& p, int n_blocks, int block, int* w_lds, int* perm_lds) {
    for (int b = threadIdx.x; b < n_blocks; b += blockDim.x) {
        const int t0 = b * block, t1 = min(t0 + block, KEY_BLOCKS ? p.total_k : p.total_q) - 1;
        int lo0, hi0, lo1, hi1;
        if constexpr (KEY_BLOCKS) { query_range(p, t0, lo0, hi0); query_range(p, t1, lo1, hi1); }
        else { key_range(p, t0, lo0, hi0); key_range(p, t1, lo1, hi1); }
        int lo = 0x7fffffff, hi = 0;
        if (hi0 > lo0) { lo = min(lo, lo0); hi = max(hi, hi0); }
        if (hi1 > lo1) { lo = min(lo, lo1); hi = max(hi, hi1); }
        w_lds[b] = hi > lo ? hi - lo : 0;
    }
    __syncthreads();
    for (int b = threadIdx.x; b < n_blocks; b += blockDim.x) {
        const int wb = w_lds[b];
        int r = 0;
        for (int j = 0; j < n_blocks; ++j) {
            const int wj = w_lds[j];
            r += (wj > wb || (wj == wb && j < b)) ? 1 : 0;
        }
        perm_lds[r] = b;
    }
    __syncthreads();
}

// Host side: whether lpt_order applies (several documents that do not look equal-length, few enough blocks)
static inline int mi_use_lpt(int64_t total_tokens, int n_docs, int block, int across) {
    if (n_docs <= 1 || across != 0) return 0;
    const int64_t n_blocks = (total_tokens + block - 1) / block;
    return n_blocks > 1 && n_blocks <= kLptMax ? 1 : 0;
}

// Host side of the above: blocks per document if the batch looks like n_docs documents of one length that is a
// multiple of the block size (all that can be told without reading the cumulative lengths; a wrong guess only costs
// balance), else 0.  Handing out across documents balances the tail of the launch but separates blocks of one
// document that would share operands in L2, so the entry points ask for it only where that sharing does not exist
// (forward / dQ: every query head has its own K / V) or the launch has few workgroups per compute unit (dK/dV)
// (measured on batches of 3 - 16 sequences of 512 - 2048 tokens: 10 - 25 % either way).
static inline int mi_blocks_per_doc(int64_t total_tokens, int n_docs, int block) {
    if (n_docs <= 1 || total_tokens % n_docs != 0 || (total_tokens / n_docs) % block != 0) return 0;
    return (int)(total_tokens / n_docs / block);
}

// maps the linear workgroup id to a work item so that the workgroups an XCD receives (ids congruent
// modulo 8) form one contiguous range of work items (neighbouring items share K/V in that XCD's L2)
__device__ __forceinline__ int xcd_remap(int linear, int total) {
    if ((total & 7) != 0) return linear;
    return (linear & 7) * (total >> 3) + (linear >> 3);
}

// ---- host side: argument checking and parameter block shared by the attention entry points -----------------
#ifdef MI_ELEM_F16
#define MI_ENTRY(name) name##_f16
#else
#define MI_ENTRY(name) name##_bf16
#endif
int mi_compute_units();
int mi_static_scratch(void** out, size_t* bytes);

// want_dtype / vec: the element type this build of the kernels takes and its elements per 128-bit access
static inline int mi_attn_validate(const mi_attn_args* a, const char* who, int want_dtype = MI_ELEM_DTYPE, int vec = 8) {
    if (!a) return mi_fail(MI_E_NULL, "%s: args is null", who);
    if (!a->q || !a->k || !a->v || !a->cu_seqlens_q) return mi_fail(MI_E_NULL, "%s: q, k, v and cu_seqlens_q are required", who);
    if (a->dtype != want_dtype) return mi_fail(MI_E_DTYPE, "%s: dtype code %d does not match the kernels of this entry point (%d)", who, a->dtype, want_dtype);
    if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 96 && a->head_dim != 128)
        return mi_fail(MI_E_SHAPE, "%s: head_dim %d unsupported (32, 64, 96, 128)", who, a->head_dim);
    if (a->n_q_heads <= 0 || a->n_kv_heads <= 0 || a->n_q_heads % a->n_kv_heads != 0)
        return mi_fail(MI_E_SHAPE, "%s: n_q_heads=%d must be a positive multiple of n_kv_heads=%d", who, a->n_q_heads, a->n_kv_heads);
    if (a->total_q < 0 || a->total_k < 0 || a->total_q > 0x7fffffffLL || a->total_k > 0x7fffffffLL || a->n_docs < 0)
        return mi_fail(MI_E_SHAPE, "%s: bad token counts q=%lld k=%lld docs=%d", who, (long long)a->total_q, (long long)a->total_k, a->n_docs);
    if (a->total_q > 0 && (a->n_docs < 1 || a->total_k < 1))
        return mi_fail(MI_E_SHAPE, "%s: non-empty query needs at least one document and one key", who);
    if (!mi_aligned16(a->q) || !mi_aligned16(a->k) || !mi_aligned16(a->v))
        return mi_fail(MI_E_ALIGN, "%s: q, k, v must be 16-byte aligned", who);
    if (a->q_stride_token % vec || a->q_stride_head % vec || a->k_stride_token % vec || a->k_stride_head % vec ||
        a->v_stride_token % vec || a->v_stride_head % vec)
        return mi_fail(MI_E_ALIGN, "%s: strides must be multiples of %d elements", who, vec);
    if (!(a->softmax_scale > 0.f)) return mi_fail(MI_E_SHAPE, "%s: softmax_scale must be positive", who);
    if (a->rotary_cos || a->rotary_sin) {
        if (!a->rotary_cos || !a->rotary_sin || !a->position_ids_q)
            return mi_fail(MI_E_NULL, "%s: fused rotary needs cos, sin and the query position ids", who);
        if (a->head_dim != 64 && a->head_dim != 128) return mi_fail(MI_E_SHAPE, "%s: fused rotary needs head_dim 64 or 128", who);
        if (a->rotary_table_rows <= 0 || a->rotary_table_rows > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "%s: bad rotary table size", who);
        if (!mi_aligned16(a->rotary_cos) || !mi_aligned16(a->rotary_sin)) return mi_fail(MI_E_ALIGN, "%s: rotary tables must be 16-byte aligned", who);
    }
    if (!(a->dropout_p >= 0.f) || a->dropout_p >= 1.f) return mi_fail(MI_E_SHAPE, "%s: dropout_p must be in [0, 1)", who);
    return MI_OK;
}

static inline void mi_attn_fill_params(const mi_attn_args* a, AttnParams* p) {
    *p = AttnParams{};
    p->q = (const elem_t*)a->q; p->k = (const elem_t*)a->k; p->v = (const elem_t*)a->v;
    p->o = (elem_t*)a->o; p->lse = a->lse;
    p->cu_q = a->cu_seqlens_q; p->cu_k = a->cu_seqlens_k ? a->cu_seqlens_k : a->cu_seqlens_q;
    p->n_docs = a->n_docs; p->causal = a->causal;
    p->total_q = (int)a->total_q; p->total_k = (int)a->total_k;
    p->nq = a->n_q_heads; p->nkv = a->n_kv_heads; p->n_rep = a->n_q_heads / a->n_kv_heads;
    p->q_st = a->q_stride_token; p->q_sh = a->q_stride_head;
    p->k_st = a->k_stride_token; p->k_sh = a->k_stride_head;
    p->v_st = a->v_stride_token; p->v_sh = a->v_stride_head;
    p->o_st = a->o_stride_token; p->o_sh = a->o_stride_head;
    p->scale = a->softmax_scale;
    p->scale_log2 = a->softmax_scale * 1.4426950408889634f;
    if (a->rotary_interleaved) {
        p->cos32 = (const float*)a->rotary_cos; p->sin32 = (const float*)a->rotary_sin;
    } else {
        p->cos = (const elem_t*)a->rotary_cos; p->sin = (const elem_t*)a->rotary_sin;
    }
    p->pos_q = a->position_ids_q; p->pos_k = a->position_ids_k; p->table_rows = (int)a->rotary_table_rows;
    if (a->dropout_p > 0.f) {
        int t = (int)(a->dropout_p * 256.0f + 0.5f);
        t = t < 1 ? 1 : (t > 255 ? 255 : t);
        p->drop_thr = (uint32_t)t;
        p->drop_rscale = 256.0f / (float)(256 - t);
        p->drop_seed = (uint32_t)(a->dropout_seed & 0xffffffffu) ^ (uint32_t)(a->dropout_seed >> 32);
    }
}

