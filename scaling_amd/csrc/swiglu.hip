// Activation kernels for gfx950 (SwiGLU, exact GELU), forward / backward: elementwise, 128-bit accesses, fp32 math.
#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 2;  // 128-bit vectors per thread and tensor

__device__ __forceinline__ float sigmoid_f(float a) { return 1.0f / (1.0f + __expf(-a)); }

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_fwd_kernel(const T* __restrict__ a, const T* __restrict__ g,
                                                             T* __restrict__ out, int64_t n_vec, int64_t n_elem) {
    constexpr int V = Elem<T>::kVec;
    const int64_t base = ((int64_t)blockIdx.x * kBlock) * kUnroll + threadIdx.x;
    uint4 ra[kUnroll], rg[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            ra[u] = ldg_nt(reinterpret_cast<const uint4*>(a) + v);
            rg[u] = ldg_nt(reinterpret_cast<const uint4*>(g) + v);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            float fa[V], fg[V];
            Elem<T>::unpack(ra[u], fa);
            Elem<T>::unpack(rg[u], fg);
#pragma unroll
            for (int i = 0; i < V; ++i) fa[i] = (fa[i] * sigmoid_f(fa[i])) * fg[i];
            reinterpret_cast<uint4*>(out)[v] = Elem<T>::pack(fa);
        }
    }
    // scalar tail (n_elem not a multiple of the vector width): handled by the last block
    if (blockIdx.x == gridDim.x - 1) {
        for (int64_t i = n_vec * V + threadIdx.x; i < n_elem; i += kBlock) {
            const float x = Elem<T>::load1(a + i);
            Elem<T>::store1(out + i, (x * sigmoid_f(x)) * Elem<T>::load1(g + i));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_bwd_kernel(const T* __restrict__ a, const T* __restrict__ g,
                                                             const T* __restrict__ dout, T* __restrict__ da,
                                                             T* __restrict__ dg, int64_t n_vec, int64_t n_elem) {
    constexpr int V = Elem<T>::kVec;
    const int64_t base = ((int64_t)blockIdx.x * kBlock) * kUnroll + threadIdx.x;
    uint4 ra[kUnroll], rg[kUnroll], rd[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            ra[u] = ldg_nt(reinterpret_cast<const uint4*>(a) + v);
            rg[u] = ldg_nt(reinterpret_cast<const uint4*>(g) + v);
            rd[u] = ldg_nt(reinterpret_cast<const uint4*>(dout) + v);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            float fa[V], fg[V], fd[V], oa[V], og[V];
            Elem<T>::unpack(ra[u], fa);
            Elem<T>::unpack(rg[u], fg);
            Elem<T>::unpack(rd[u], fd);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float s = sigmoid_f(fa[i]);
                oa[i] = fd[i] * fg[i] * s * (1.0f + fa[i] * (1.0f - s));
                og[i] = fd[i] * (fa[i] * s);
            }
            stg_nt(reinterpret_cast<uint4*>(da) + v, Elem<T>::pack(oa));   // three streams in, two out: both sides hinted
            stg_nt(reinterpret_cast<uint4*>(dg) + v, Elem<T>::pack(og));
        }
    }
    if (blockIdx.x == gridDim.x - 1) {
        for (int64_t i = n_vec * V + threadIdx.x; i < n_elem; i += kBlock) {
            const float x = Elem<T>::load1(a + i), gg = Elem<T>::load1(g + i), d = Elem<T>::load1(dout + i);
            const float s = sigmoid_f(x);
            Elem<T>::store1(da + i, d * gg * s * (1.0f + x * (1.0f - s)));
            Elem<T>::store1(dg + i, d * (x * s));
        }
    }
}

// exact (erf) GELU, the reference's default activation (torch.nn.functional.gelu with approximate='none').
// fp32 tensors use erff.  16-bit tensors use a branch-free form: with z = |x| / sqrt(2),
//   0.5 * erfc(z) = 0.5 * t * (a1 + t * (a2 + t * (a3 + t * (a4 + t * a5)))) * exp(-z * z),  t = 1 / (1 + p * z)
// (Abramowitz & Stegun 7.1.26, absolute error <= 1.5e-7 on erfc, far below half a bf16 / fp16 ulp of the
// result), so Phi(x) = x >= 0 ? 1 - h : h needs one reciprocal and one exponential, and the same
// exponential is the Gaussian density of the derivative.
template <bool FAST> struct GeluMath {
    // cdf = Phi(x), pdf_e = exp(-x * x / 2)
    static __device__ __forceinline__ void parts(float x, float& cdf, float& pdf_e) {
        if constexpr (FAST) {
            const float z = fabsf(x) * 0.7071067811865476f;
            const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
            pdf_e = __builtin_amdgcn_exp2f(x * x * -0.7213475204444817f);
            float poly = 1.061405429f;
            poly = poly * t - 1.453152027f;
            poly = poly * t + 1.421413741f;
            poly = poly * t - 0.284496736f;
            poly = poly * t + 0.254829592f;
            const float h = 0.5f * poly * t * pdf_e;
            cdf = x >= 0.f ? 1.0f - h : h;
        } else {
            cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
            pdf_e = __expf(-0.5f * x * x);
        }
    }
    static __device__ __forceinline__ float value(float x) {
        float cdf, e;
        parts(x, cdf, e);
        return x * cdf;
    }
    static __device__ __forceinline__ float grad(float x) {
        float cdf, e;
        parts(x, cdf, e);
        return cdf + x * 0.3989422804014327f * e;
    }
};

// BWD = false: y = gelu(x) (dy unused);  BWD = true: y = dy * gelu'(x)
template <typename T, bool BWD>
__global__ __launch_bounds__(kBlock) void gelu_kernel(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ y,
                                                       int64_t n_vec, int64_t n_elem) {
    constexpr int V = Elem<T>::kVec;
    using G = GeluMath<sizeof(T) == 2>;
    const int64_t base = ((int64_t)blockIdx.x * kBlock) * kUnroll + threadIdx.x;
    uint4 rx[kUnroll], rd[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            // the side with more streams carries the hint: the loads of the backward, the store of the forward
            rx[u] = BWD ? ldg_nt(reinterpret_cast<const uint4*>(x) + v) : reinterpret_cast<const uint4*>(x)[v];
            if (BWD) rd[u] = ldg_nt(reinterpret_cast<const uint4*>(dy) + v);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = base + (int64_t)u * kBlock;
        if (v < n_vec) {
            float fx[V], fd[V];
            Elem<T>::unpack(rx[u], fx);
            if (BWD) Elem<T>::unpack(rd[u], fd);
#pragma unroll
            for (int i = 0; i < V; ++i) fx[i] = BWD ? fd[i] * G::grad(fx[i]) : G::value(fx[i]);
            if (BWD) reinterpret_cast<uint4*>(y)[v] = Elem<T>::pack(fx);
            else stg_nt(reinterpret_cast<uint4*>(y) + v, Elem<T>::pack(fx));
        }
    }
    if (blockIdx.x == gridDim.x - 1) {
        for (int64_t i = n_vec * V + threadIdx.x; i < n_elem; i += kBlock) {
            const float a = Elem<T>::load1(x + i);
            Elem<T>::store1(y + i, BWD ? Elem<T>::load1(dy + i) * G::grad(a) : G::value(a));
        }
    }
}

template <typename T> unsigned grid_for(int64_t n_elem, int64_t* n_vec) {
    *n_vec = n_elem / Elem<T>::kVec;
    int64_t blocks = (*n_vec + (int64_t)kBlock * kUnroll - 1) / ((int64_t)kBlock * kUnroll);
    if (blocks < 1) blocks = 1;
    return (unsigned)blocks;
}

}  // namespace

extern "C" {

int mi_swiglu_fwd(const void* a, const void* gate, void* out, int64_t n_elem, int dtype, void* stream) {
    if (n_elem == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!a || !gate || !out) return mi_fail(MI_E_NULL, "swiglu_fwd: null pointer");
    if (n_elem < 0) return mi_fail(MI_E_SHAPE, "swiglu_fwd: negative size");
    if (!mi_aligned16(a) || !mi_aligned16(gate) || !mi_aligned16(out)) return mi_fail(MI_E_ALIGN, "swiglu_fwd: pointers must be 16-byte aligned");
    if (n_elem / 4 / (kBlock * kUnroll) > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "swiglu_fwd: too many elements");
    MI_DISPATCH_DTYPE(dtype, {
        int64_t n_vec;
        const unsigned grid = grid_for<T>(n_elem, &n_vec);
        swiglu_fwd_kernel<T><<<dim3(grid), dim3(kBlock), 0, (hipStream_t)stream>>>((const T*)a, (const T*)gate, (T*)out, n_vec, n_elem);
    });
    return mi_check_launch("swiglu_fwd");
}

int mi_swiglu_bwd(const void* a, const void* gate, const void* dout, void* da, void* dgate, int64_t n_elem, int dtype,
                  void* stream) {
    if (n_elem == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!a || !gate || !dout || !da || !dgate) return mi_fail(MI_E_NULL, "swiglu_bwd: null pointer");
    if (n_elem < 0) return mi_fail(MI_E_SHAPE, "swiglu_bwd: negative size");
    if (!mi_aligned16(a) || !mi_aligned16(gate) || !mi_aligned16(dout) || !mi_aligned16(da) || !mi_aligned16(dgate))
        return mi_fail(MI_E_ALIGN, "swiglu_bwd: pointers must be 16-byte aligned");
    if (n_elem / 4 / (kBlock * kUnroll) > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "swiglu_bwd: too many elements");
    MI_DISPATCH_DTYPE(dtype, {
        int64_t n_vec;
        const unsigned grid = grid_for<T>(n_elem, &n_vec);
        swiglu_bwd_kernel<T><<<dim3(grid), dim3(kBlock), 0, (hipStream_t)stream>>>((const T*)a, (const T*)gate, (const T*)dout,
                                                                                  (T*)da, (T*)dgate, n_vec, n_elem);
    });
    return mi_check_launch("swiglu_bwd");
}

int mi_gelu_fwd(const void* x, void* y, int64_t n_elem, int dtype, void* stream) {
    if (n_elem == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !y) return mi_fail(MI_E_NULL, "gelu_fwd: null pointer");
    if (n_elem < 0) return mi_fail(MI_E_SHAPE, "gelu_fwd: negative size");
    if (!mi_aligned16(x) || !mi_aligned16(y)) return mi_fail(MI_E_ALIGN, "gelu_fwd: pointers must be 16-byte aligned");
    if (n_elem / 4 / (kBlock * kUnroll) > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "gelu_fwd: too many elements");
    MI_DISPATCH_DTYPE(dtype, {
        int64_t n_vec;
        const unsigned grid = grid_for<T>(n_elem, &n_vec);
        gelu_kernel<T, false><<<dim3(grid), dim3(kBlock), 0, (hipStream_t)stream>>>((const T*)x, nullptr, (T*)y, n_vec, n_elem);
    });
    return mi_check_launch("gelu_fwd");
}

int mi_gelu_bwd(const void* x, const void* dy, void* dx, int64_t n_elem, int dtype, void* stream) {
    if (n_elem == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !dy || !dx) return mi_fail(MI_E_NULL, "gelu_bwd: null pointer");
    if (n_elem < 0) return mi_fail(MI_E_SHAPE, "gelu_bwd: negative size");
    if (!mi_aligned16(x) || !mi_aligned16(dy) || !mi_aligned16(dx)) return mi_fail(MI_E_ALIGN, "gelu_bwd: pointers must be 16-byte aligned");
    if (n_elem / 4 / (kBlock * kUnroll) > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "gelu_bwd: too many elements");
    MI_DISPATCH_DTYPE(dtype, {
        int64_t n_vec;
        const unsigned grid = grid_for<T>(n_elem, &n_vec);
        gelu_kernel<T, true><<<dim3(grid), dim3(kBlock), 0, (hipStream_t)stream>>>((const T*)x, (const T*)dy, (T*)dx, n_vec, n_elem);
    });
    return mi_check_launch("gelu_bwd");
}

}  // extern "C"
