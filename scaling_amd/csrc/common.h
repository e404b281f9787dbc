// Shared device/host helpers for the gfx950 kernels of libmi355_layer.so.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/mi355_layer.h"

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define MI_WAVE 64

// ---- host side error plumbing -------------------------------------------------------------
void mi_set_error(const char* fmt, ...);
int mi_fail(int status, const char* fmt, ...);
int mi_check_launch(const char* what);

static inline bool mi_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- element type traits: 8 x 16-bit or 4 x fp32 per 128-bit access --------------------------
template <typename T> struct Elem;

template <> struct Elem<__bf16> {
    static constexpr int kVec = 8;
    static __device__ __forceinline__ void unpack(const uint4& u, float* f) {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ uint4 pack(const float* f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bf16x2_t p;
            p[0] = (__bf16)f[2 * i];
            p[1] = (__bf16)f[2 * i + 1];
            w[i] = __builtin_bit_cast(uint32_t, p);
        }
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
    static __device__ __forceinline__ float load1(const __bf16* p) { return (float)*p; }
    static __device__ __forceinline__ void store1(__bf16* p, float v) { *p = (__bf16)v; }
};

template <> struct Elem<_Float16> {
    static constexpr int kVec = 8;
    static __device__ __forceinline__ void unpack(const uint4& u, float* f) {
        f16x8_t h = __builtin_bit_cast(f16x8_t, u);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
    }
    static __device__ __forceinline__ uint4 pack(const float* f) {
        f16x8_t h;
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (_Float16)f[i];
        return __builtin_bit_cast(uint4, h);
    }
    static __device__ __forceinline__ float load1(const _Float16* p) { return (float)*p; }
    static __device__ __forceinline__ void store1(_Float16* p, float v) { *p = (_Float16)v; }
};

template <> struct Elem<float> {
    static constexpr int kVec = 4;
    static __device__ __forceinline__ void unpack(const uint4& u, float* f) {
        f[0] = __uint_as_float(u.x); f[1] = __uint_as_float(u.y);
        f[2] = __uint_as_float(u.z); f[3] = __uint_as_float(u.w);
    }
    static __device__ __forceinline__ uint4 pack(const float* f) {
        return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
    }
    static __device__ __forceinline__ float load1(const float* p) { return *p; }
    static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};

// ---- streaming 128-bit global accesses -------------------------------------------------------
// Non-temporal hint for tensors a launch touches exactly once.  Which side to hint was measured per kernel
// (8192 x 4096 and 8192 x 14336 bf16 tensors): kernels that read more streams than they write gain from hinted
// loads (SwiGLU forward 5.7 -> 6.6 TB/s, GELU backward 5.6 -> 6.7, decode attention 5.8 -> 6.3), one-in one-out
// kernels from hinted stores (GELU forward 5.8 -> 6.8, RMSNorm forward 5.9 -> 6.4) and, for the norm forward
// kernels and rotary, from hinted loads on top (+ 1 - 5 %; a plain 1 GiB copy: 5.6 TB/s without hints, 5.75 with
// hinted stores, 6.2 with both), and the norm backward kernels lose with any hint.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ldg_nt(const uint4* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void stg_nt(uint4* p, const uint4& x) {
    u32x4_t v;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(p));
}

// One pair of the interleaved ("complex") rotary: (x0 + i x1) * (c + i s).  The roundings are spelled out so
// that every kernel that applies the rotation (stand-alone or fused into an attention load) gives the same bits.
__device__ __forceinline__ void rotate_complex_pair(float& x0, float& x1, float c, float s) {
    const float re = __builtin_fmaf(x0, c, -(x1 * s));
    const float im = __builtin_fmaf(x0, s, x1 * c);
    x0 = re;
    x1 = im;
}

// ---- wavefront reductions (64 lanes) -------------------------------------------------------
// Sum over aligned groups of WIDTH lanes, every lane receiving the total, without going through the LDS crossbar
// (six dependent ds_bpermute round trips per 64-lane sum otherwise): DPP lane selects inside a row of 16 lanes
// (quad permutes, then the mirror images of 8 and of 16 lanes, which pair every partial sum with the one it still
// lacks), v_permlane16_swap across the rows of a half and v_permlane32_swap across the halves.
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32 || WIDTH == 64, "group width");
    if constexpr (WIDTH >= 2) v += dpp_mov<0xB1>(v);     // quad_perm [1, 0, 3, 2]
    if constexpr (WIDTH >= 4) v += dpp_mov<0x4E>(v);     // quad_perm [2, 3, 0, 1]
    if constexpr (WIDTH >= 8) v += dpp_mov<0x141>(v);    // row_half_mirror
    if constexpr (WIDTH >= 16) v += dpp_mov<0x140>(v);   // row_mirror
    if constexpr (WIDTH >= 32) {
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    if constexpr (WIDTH >= 64) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    return v;
}

// The same lane pairing for any associative, commutative operation on 32-bit values (maximum, integer minimum, ...).
template <int WIDTH, class Op> __device__ __forceinline__ uint32_t group_reduce_bits(uint32_t v, Op op) {
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32 || WIDTH == 64, "group width");
    auto dpp = [](uint32_t x, auto ctrl) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, decltype(ctrl)::value, 0xf, 0xf, true);
    };
    if constexpr (WIDTH >= 2) v = op(v, dpp(v, std::integral_constant<int, 0xB1>{}));
    if constexpr (WIDTH >= 4) v = op(v, dpp(v, std::integral_constant<int, 0x4E>{}));
    if constexpr (WIDTH >= 8) v = op(v, dpp(v, std::integral_constant<int, 0x141>{}));
    if constexpr (WIDTH >= 16) v = op(v, dpp(v, std::integral_constant<int, 0x140>{}));
    if constexpr (WIDTH >= 32) {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        v = op(r[0], r[1]);
    }
    if constexpr (WIDTH >= 64) {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        v = op(r[0], r[1]);
    }
    return v;
}
template <int WIDTH> __device__ __forceinline__ float group_max(float v) {
    return __uint_as_float(group_reduce_bits<WIDTH>(__float_as_uint(v), [](uint32_t a, uint32_t b) {
        return __float_as_uint(fmaxf(__uint_as_float(a), __uint_as_float(b)));
    }));
}
template <int WIDTH> __device__ __forceinline__ int group_min(int v) {
    return (int)group_reduce_bits<WIDTH>((uint32_t)v, [](uint32_t a, uint32_t b) { return (uint32_t)min((int)a, (int)b); });
}
template <int WIDTH> __device__ __forceinline__ int group_max(int v) {
    return (int)group_reduce_bits<WIDTH>((uint32_t)v, [](uint32_t a, uint32_t b) { return (uint32_t)max((int)a, (int)b); });
}

#define MI_DISPATCH_DTYPE(dtype, ...)                                       \
    switch (dtype) {                                                        \
        case MI_BF16: { using T = __bf16; __VA_ARGS__; break; }             \
        case MI_F16: { using T = _Float16; __VA_ARGS__; break; }            \
        case MI_F32: { using T = float; __VA_ARGS__; break; }               \
        default: return mi_fail(MI_E_DTYPE, "unsupported dtype code %d", (int)(dtype)); \
    }
