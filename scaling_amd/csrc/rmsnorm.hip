// RMSNorm forward / backward for gfx950: single pass over HBM, 128-bit accesses, fp32 math.
//
// A row is owned by TPR threads (16 / 64 lanes of one wavefront, or a whole 256-thread block for very
// wide rows); each thread keeps CH 128-bit vectors of the row in registers, so x (and dy) are read
// from HBM exactly once.  Rows handled by a wavefront need no block barrier, so the memory pipeline
// stays full.  The weight gradient is accumulated in registers across a block's rows, combined in
// LDS in a fixed order, written as one fp32 partial row per block and reduced by a second kernel.
#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kMaxBwdBlocks = 512;

template <int TPR> __device__ __forceinline__ float row_sum(float v, float* lds) {
    if constexpr (TPR <= 64) {
        return group_sum<TPR>(v);
    } else {
        v = group_sum<64>(v);
        const int wave = threadIdx.x >> 6;
        __syncthreads();  // protect lds from the previous use
        if ((threadIdx.x & 63) == 0) lds[wave] = v;
        __syncthreads();
        return lds[0] + lds[1] + lds[2] + lds[3];
    }
}

// ADD: the row that is normalised is x + residual, rounded to T and also stored to sum_out (which may alias x or
// residual): the residual add of the layer fused into the norm that follows it.
template <typename T, int TPR, int CH, bool ADD = false>
__global__ __launch_bounds__(kBlock) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                              T* __restrict__ y, float* __restrict__ rstd_out,
                                                              int64_t n_rows, int hidden, float eps,
                                                              const T* residual = nullptr, T* sum_out = nullptr) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kBlock / TPR;
    __shared__ float lds[4];
    const int tr = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
    const bool row_ok = row < n_rows;
    const int vecs = hidden / V;
    const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
    uint4 raw[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int v = c * TPR + tr;
        raw[c] = (row_ok && v < vecs) ? (ADD ? xr[v] : ldg_nt(xr + v)) : make_uint4(0, 0, 0, 0);
        if constexpr (ADD) {
            if (row_ok && v < vecs) {
                float a[V], r[V];
                Elem<T>::unpack(raw[c], a);
                Elem<T>::unpack(reinterpret_cast<const uint4*>(residual + row * hidden)[v], r);
#pragma unroll
                for (int i = 0; i < V; ++i) a[i] += r[i];
                raw[c] = Elem<T>::pack(a);            // the norm sees the sum as it is stored
                reinterpret_cast<uint4*>(sum_out + row * hidden)[v] = raw[c];
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float f[V];
        Elem<T>::unpack(raw[c], f);
#pragma unroll
        for (int i = 0; i < V; ++i) ss += f[i] * f[i];
    }
    ss = row_sum<TPR>(ss, lds);
    const float rstd = rsqrtf(ss / (float)hidden + eps);
    if (rstd_out != nullptr && row_ok && tr == 0) rstd_out[row] = rstd;
    if (!row_ok) return;
    const uint4* wr = reinterpret_cast<const uint4*>(w);
    uint4* yr = reinterpret_cast<uint4*>(y + row * hidden);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int v = c * TPR + tr;
        if (v < vecs) {
            float f[V], g[V];
            Elem<T>::unpack(raw[c], f);
            Elem<T>::unpack(wr[v], g);
#pragma unroll
            for (int i = 0; i < V; ++i) f[i] = (f[i] * rstd) * g[i];
            if constexpr (ADD) yr[v] = Elem<T>::pack(f);
            else stg_nt(yr + v, Elem<T>::pack(f));
        }
    }
}

template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kBlock) void rmsnorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                              const T* __restrict__ dy, T* __restrict__ dx,
                                                              float* __restrict__ dw_partial, int64_t n_rows,
                                                              int hidden, float eps) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kBlock / TPR;
    extern __shared__ float dw_lds[];  // [hidden]
    __shared__ float lds[4];
    const int tr = threadIdx.x % TPR;
    const int rg = threadIdx.x / TPR;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;

    float wf[CH][V];
    float acc[CH][V];
    const uint4* wr = reinterpret_cast<const uint4*>(w);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int v = c * TPR + tr;
        uint4 u = (v < vecs) ? wr[v] : make_uint4(0, 0, 0, 0);
        Elem<T>::unpack(u, wf[c]);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[c][i] = 0.f;
    }

    const int64_t row_step = (int64_t)gridDim.x * RPB;
    // every thread of the block runs the same number of iterations (barriers inside row_sum for TPR=256)
    const int64_t iters = (n_rows + row_step - 1) / row_step;
    for (int64_t it = 0; it < iters; ++it) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + (row_ok ? row : 0) * hidden);
        uint4 xraw[CH], graw[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            const bool ok = row_ok && v < vecs;
            xraw[c] = ok ? xr[v] : make_uint4(0, 0, 0, 0);
            graw[c] = ok ? gr[v] : make_uint4(0, 0, 0, 0);
        }
        float ss = 0.f, dot = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float xf[V], gf[V];
            Elem<T>::unpack(xraw[c], xf);
            Elem<T>::unpack(graw[c], gf);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                ss += xf[i] * xf[i];
                dot += gf[i] * wf[c][i] * xf[i];
            }
        }
        ss = row_sum<TPR>(ss, lds);
        dot = row_sum<TPR>(dot, lds);
        const float rstd = rsqrtf(ss * inv_h + eps);
        const float coef = dot * inv_h * rstd * rstd * rstd;
        if (row_ok) {
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * hidden);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
                    float xf[V], gf[V], o[V];
                    Elem<T>::unpack(xraw[c], xf);
                    Elem<T>::unpack(graw[c], gf);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        o[i] = rstd * (gf[i] * wf[c][i]) - xf[i] * coef;
                        acc[c][i] += gf[i] * (xf[i] * rstd);
                    }
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
    }

    // combine the row groups of this block in a fixed order, then emit one partial row
    for (int i = threadIdx.x; i < hidden; i += kBlock) dw_lds[i] = 0.f;
    __syncthreads();
    for (int g = 0; g < RPB; ++g) {
        if (rg == g) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
#pragma unroll
                    for (int i = 0; i < V; ++i) dw_lds[v * V + i] += acc[c][i];
                }
            }
        }
        __syncthreads();
    }
    float* out = dw_partial + (int64_t)blockIdx.x * hidden;
    for (int i = threadIdx.x; i < hidden; i += kBlock) out[i] = dw_lds[i];
}

// Backward for wide rows: 1024 threads per block, TPR (256 or 512) threads per row, so 4 or 2 rows are in
// flight per block and the per-thread slices (raw row vectors, fp32 dweight) are small enough for 16
// wavefronts per compute unit; one block per compute unit keeps the number of dweight partial rows <= 256.
// One barrier per row step (both row sums travel through a double-buffered LDS slot).
constexpr int kWideBlock = 512;     // LayerNorm backward: two blocks per compute unit (two barriers per row step)
constexpr int kRmsWideBlock = 1024; // RMSNorm backward: one block per compute unit, half as many partial dweight rows
constexpr int kWideMaxBlocks = 256;
constexpr int kLnMaxBlocks = 512;     // partial dweight / dbias rows of the LayerNorm backward

template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kRmsWideBlock) void rmsnorm_bwd_wide_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                          const T* __restrict__ dy, T* __restrict__ dx,
                                                                          float* __restrict__ dw_partial, int64_t n_rows,
                                                                          int hidden, float eps) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kRmsWideBlock / TPR;
    constexpr int WPR = TPR / 64;      // wavefronts per row
    extern __shared__ float dw_lds[];  // [hidden] dweight combine buffer, then [hidden] fp32 copy of the weight
    __shared__ float2 part[2][16];     // [parity][wavefront]
    float* w_lds = dw_lds + hidden;
    const int tr = threadIdx.x % TPR;
    const int rg = threadIdx.x / TPR;
    const int wave = threadIdx.x >> 6;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;

    // the weight is read from LDS where it is used: keeping it in registers would cost as many registers
    // as the dweight accumulator and halve the number of resident wavefronts
    float acc[CH][V];
    for (int i = threadIdx.x; i < hidden; i += kRmsWideBlock) w_lds[i] = Elem<T>::load1(w + i);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < V; ++i) acc[c][i] = 0.f;
    __syncthreads();
    const int64_t row_step = (int64_t)gridDim.x * RPB;
    const int64_t iters = (n_rows + row_step - 1) / row_step;
    // the rows of iteration it + 1 are fetched while iteration it is reduced, so loads stay in flight
    // across the block-wide reductions
    uint4 xraw[CH], graw[CH], xnext[CH], gnext[CH];
    auto fetch = [&](int64_t it, uint4 (&xv)[CH], uint4 (&gv)[CH]) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + (row_ok ? row : 0) * hidden);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            const bool ok = row_ok && v < vecs;
            xv[c] = ok ? xr[v] : make_uint4(0, 0, 0, 0);
            gv[c] = ok ? gr[v] : make_uint4(0, 0, 0, 0);
        }
    };
    // one row step: reduce the two row sums over the row's wavefronts (one barrier), write dx, add to dweight
    auto process = [&](int64_t it, const uint4 (&xv)[CH], const uint4 (&gv)[CH]) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        float ss = 0.f, dot = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float xf[V], gf[V], wf[V];
            Elem<T>::unpack(xv[c], xf);
            Elem<T>::unpack(gv[c], gf);
            const int v0 = (c * TPR + tr < vecs ? c * TPR + tr : 0) * V;
#pragma unroll
            for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v0 + i);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                ss += xf[i] * xf[i];
                dot += gf[i] * wf[i] * xf[i];
            }
        }
        ss = group_sum<64>(ss);
        dot = group_sum<64>(dot);
        const int par = (int)(it & 1);
        if ((threadIdx.x & 63) == 0) part[par][wave] = make_float2(ss, dot);
        __syncthreads();
        ss = 0.f;
        dot = 0.f;
#pragma unroll
        for (int j = 0; j < WPR; ++j) {
            const float2 pj = part[par][WPR * rg + j];
            ss += pj.x;
            dot += pj.y;
        }
        const float rstd = rsqrtf(ss * inv_h + eps);
        const float coef = dot * inv_h * rstd * rstd * rstd;
        if (row_ok) {
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * hidden);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
                    float xf[V], gf[V], wf[V], o[V];
                    Elem<T>::unpack(xv[c], xf);
                    Elem<T>::unpack(gv[c], gf);
#pragma unroll
                    for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v * V + i);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        o[i] = rstd * (gf[i] * wf[i]) - xf[i] * coef;
                        acc[c][i] += gf[i] * (xf[i] * rstd);
                    }
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
    };
    // Three register sets rotate: the rows of steps it + 1 and it + 2 are in flight while step it is reduced (two
    // steps of loads outstanding per compute unit cover the memory latency; with one, the block-wide barrier
    // made every wavefront issue its loads at the same moment and the memory pipe ran dry in between).  The loop
    // is unrolled by three so that every set is addressed statically; `iters` is the same for the whole block.
    constexpr bool kDeep = CH == 1;       // three register sets fit without spilling only for one vector per thread
    if constexpr (kDeep) {
        uint4 x2[CH], g2[CH];
        if (iters > 0) fetch(0, xraw, graw);
        if (iters > 1) fetch(1, xnext, gnext);
        for (int64_t it = 0; it < iters; it += 3) {
            if (it + 2 < iters) fetch(it + 2, x2, g2);
            process(it, xraw, graw);
            if (it + 1 < iters) {
                if (it + 3 < iters) fetch(it + 3, xraw, graw);
                process(it + 1, xnext, gnext);
            }
            if (it + 2 < iters) {
                if (it + 4 < iters) fetch(it + 4, xnext, gnext);
                process(it + 2, x2, g2);
            }
        }
    } else if constexpr (CH <= 2) {       // two sets: the rows of step it + 1 are in flight while step it is reduced
        if (iters > 0) fetch(0, xraw, graw);
        for (int64_t it = 0; it < iters; it += 2) {
            if (it + 1 < iters) fetch(it + 1, xnext, gnext);
            process(it, xraw, graw);
            if (it + 1 < iters) {
                if (it + 2 < iters) fetch(it + 2, xraw, graw);
                process(it + 1, xnext, gnext);
            }
        }
    } else {
        for (int64_t it = 0; it < iters; ++it) {
            fetch(it, xraw, graw);
            process(it, xraw, graw);
        }
    }
    for (int i = threadIdx.x; i < hidden; i += kRmsWideBlock) dw_lds[i] = 0.f;
    __syncthreads();
    for (int g = 0; g < RPB; ++g) {
        if (rg == g) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
#pragma unroll
                    for (int i = 0; i < V; ++i) dw_lds[v * V + i] += acc[c][i];
                }
            }
        }
        __syncthreads();
    }
    float* out = dw_partial + (int64_t)blockIdx.x * hidden;
    for (int i = threadIdx.x; i < hidden; i += kRmsWideBlock) out[i] = dw_lds[i];
}

// dw[col] = sum_p partial[p][col]; 32 columns x 8 row groups per block (a row group reads 128 contiguous bytes of a
// partial row: with 16 columns the 64-byte pieces cost twice their size in fetched sectors), fixed summation order.
constexpr int kDwCols = 32, kDwGroups = kBlock / kDwCols;
template <typename T>
__global__ __launch_bounds__(kBlock) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, T* __restrict__ dw,
                                                                    int n_partial, int hidden, T* __restrict__ dw2 = nullptr) {
    // blockIdx.y == 1 (LayerNorm): the second set of partial rows, stored after the first, goes to dw2
    if (blockIdx.y == 1) {
        partial += (int64_t)n_partial * hidden;
        dw = dw2;
    }
    __shared__ float lds[kDwGroups][kDwCols + 1];
    const int cl = threadIdx.x % kDwCols, pg = threadIdx.x / kDwCols;
    const int col = blockIdx.x * kDwCols + cl;
    float s = 0.f;
    if (col < hidden) {
        // the launch is latency bound (a few MB, one short dependent chain per thread): 16 loads are requested
        // before the first is used, so 256 partial rows cost two memory round trips
        constexpr int K = 16;
        float acc[K];
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = 0.f;
        int p = pg;
        for (; p + kDwGroups * (K - 1) < n_partial; p += kDwGroups * K) {
            float v[K];
#pragma unroll
            for (int k = 0; k < K; ++k) v[k] = partial[(int64_t)(p + kDwGroups * k) * hidden + col];
#pragma unroll
            for (int k = 0; k < K; ++k) acc[k] += v[k];
        }
        for (; p < n_partial; p += kDwGroups) acc[0] += partial[(int64_t)p * hidden + col];
#pragma unroll
        for (int w = K / 2; w > 0; w >>= 1)          // fixed pairwise order
#pragma unroll
            for (int k = 0; k < w; ++k) acc[k] += acc[k + w];
        s = acc[0];
    }
    lds[pg][cl] = s;
    __syncthreads();
    if (pg == 0 && col < hidden) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < kDwGroups; ++i) t += lds[i][cl];
        Elem<T>::store1(dw + col, t);
    }
}

struct Plan { int tpr; int ch; };

template <typename T> bool make_plan(int64_t hidden, Plan* p) {
    constexpr int V = Elem<T>::kVec;
    if (hidden <= 0 || hidden % V != 0) return false;
    const int64_t vecs = hidden / V;
    int tpr, ch;
    if (vecs <= 16) { tpr = 16; ch = 1; }
    else if (vecs <= 64 * 8) { tpr = 64; ch = (int)((vecs + 63) / 64); }
    else if (vecs <= 256 * 8) { tpr = 256; ch = (int)((vecs + 255) / 256); }
    else return false;
    int c = 1;
    while (c < ch) c *= 2;
    p->tpr = tpr; p->ch = c;
    return true;
}

int bwd_blocks(int64_t n_rows, int tpr) {
    const int64_t rpb = kBlock / tpr;
    int64_t b = (n_rows + rpb - 1) / rpb;
    if (b > kMaxBwdBlocks) b = kMaxBwdBlocks;
    if (b < 1) b = 1;
    return (int)b;
}

template <int TPRV, int CHV> struct PlanTag { static constexpr int TPR = TPRV; static constexpr int CH = CHV; };

// calls f(PlanTag<tpr, ch>{}) for the instantiated (threads per row, vectors per thread) pair
template <typename F> bool dispatch_plan(const Plan& plan, F&& f) {
#define RMS_CASE(TPRV, CHV) if (plan.tpr == TPRV && plan.ch == CHV) { f(PlanTag<TPRV, CHV>{}); return true; }
    RMS_CASE(16, 1)
    RMS_CASE(64, 1) RMS_CASE(64, 2) RMS_CASE(64, 4) RMS_CASE(64, 8)
    RMS_CASE(256, 1) RMS_CASE(256, 2) RMS_CASE(256, 4) RMS_CASE(256, 8)
#undef RMS_CASE
    return false;
}

template <typename T>
int launch_fwd(const void* x, const void* w, void* y, float* rstd, int64_t n_rows, int64_t hidden, float eps,
               hipStream_t st, const void* residual = nullptr, void* sum_out = nullptr) {
    Plan plan;
    if (!make_plan<T>(hidden, &plan))
        return mi_fail(MI_E_SHAPE, "rmsnorm: hidden=%lld unsupported (must be a multiple of %d and <= %d)",
                       (long long)hidden, Elem<T>::kVec, 256 * 8 * Elem<T>::kVec);
    // few rows (a decode step): a whole block per row, so that the launch is not eight blocks of long serial threads
    const int64_t vecs = hidden / Elem<T>::kVec;
    if (plan.tpr == 64 && plan.ch >= 2 && n_rows <= 1024) {
        plan.tpr = 256;
        plan.ch = vecs <= 256 ? 1 : 2;
    }
    const bool launched = dispatch_plan(plan, [&](auto tag) {
        constexpr int TPR = decltype(tag)::TPR;
        constexpr int CH = decltype(tag)::CH;
        const int rpb = kBlock / TPR;
        const unsigned grid = (unsigned)((n_rows + rpb - 1) / rpb);
        if (residual != nullptr)
            rmsnorm_fwd_kernel<T, TPR, CH, true><<<dim3(grid), dim3(kBlock), 0, st>>>((const T*)x, (const T*)w, (T*)y, rstd, n_rows,
                                                                                      (int)hidden, eps, (const T*)residual, (T*)sum_out);
        else
            rmsnorm_fwd_kernel<T, TPR, CH><<<dim3(grid), dim3(kBlock), 0, st>>>((const T*)x, (const T*)w, (T*)y, rstd, n_rows,
                                                                                (int)hidden, eps);
    });
    if (!launched) return mi_fail(MI_E_SHAPE, "rmsnorm: no kernel for hidden=%lld", (long long)hidden);
    return mi_check_launch("rmsnorm_fwd");
}

template <typename T>
int launch_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, void* ws, size_t ws_bytes,
               int64_t n_rows, int64_t hidden, float eps, hipStream_t st) {
    Plan plan;
    if (!make_plan<T>(hidden, &plan))
        return mi_fail(MI_E_SHAPE, "rmsnorm: hidden=%lld unsupported", (long long)hidden);
    const int64_t vecs = hidden / Elem<T>::kVec;
    const bool wide = vecs >= 256;
    // wide rows: 256 threads per row up to 512 vectors (4 rows per block and step), 512 up to 1024, the whole block
    // beyond: at most two vectors per thread, so that the next step's rows always fit in registers next to this
    // step's (four vectors per thread without that prefetch ran at 1.9 TB/s at hidden 12288)
    const int wide_tpr = vecs <= 256 ? 256 : (vecs <= 1024 ? 512 : 1024);
    // wide rows: a single round of blocks (two per compute unit), each amortising its epilogue over many rows
    const int wide_rpb = kRmsWideBlock / wide_tpr;
    const int64_t wide_blocks = (n_rows + wide_rpb - 1) / wide_rpb;
    const int blocks = wide ? (int)(wide_blocks > kWideMaxBlocks ? kWideMaxBlocks : (wide_blocks < 1 ? 1 : wide_blocks))
                            : bwd_blocks(n_rows, plan.tpr);
    if (ws == nullptr || ws_bytes < (size_t)blocks * hidden * sizeof(float))
        return mi_fail(MI_E_WORKSPACE, "rmsnorm_bwd: workspace needs %zu bytes, got %zu",
                       (size_t)blocks * hidden * sizeof(float), ws_bytes);
    if (wide) {
        const int ch = (int)((vecs + wide_tpr - 1) / wide_tpr);
        const size_t lds = 2 * hidden * sizeof(float);
#define RMS_WIDE(TPRV, CHV) rmsnorm_bwd_wide_kernel<T, TPRV, CHV><<<dim3(blocks), dim3(kRmsWideBlock), lds, st>>>( \
            (const T*)x, (const T*)w, (const T*)dy, (T*)dx, (float*)ws, n_rows, (int)hidden, eps)
        if (wide_tpr == 256) { if (ch <= 1) RMS_WIDE(256, 1); else RMS_WIDE(256, 2); }
        else if (wide_tpr == 512) { if (ch <= 1) RMS_WIDE(512, 1); else RMS_WIDE(512, 2); }
        else RMS_WIDE(1024, 2);
#undef RMS_WIDE
        int rcw = mi_check_launch("rmsnorm_bwd_wide");
        if (rcw != MI_OK) return rcw;
        rmsnorm_dw_reduce_kernel<T><<<dim3((unsigned)((hidden + kDwCols - 1) / kDwCols)), dim3(kBlock), 0, st>>>((const float*)ws, (T*)dw,
                                                                                                   blocks, (int)hidden);
        return mi_check_launch("rmsnorm_dw_reduce");
    }
    const bool launched = dispatch_plan(plan, [&](auto tag) {
        constexpr int TPR = decltype(tag)::TPR;
        constexpr int CH = decltype(tag)::CH;
        rmsnorm_bwd_kernel<T, TPR, CH><<<dim3(blocks), dim3(kBlock), hidden * sizeof(float), st>>>(
            (const T*)x, (const T*)w, (const T*)dy, (T*)dx, (float*)ws, n_rows, (int)hidden, eps);
    });
    if (!launched) return mi_fail(MI_E_SHAPE, "rmsnorm: no kernel for hidden=%lld", (long long)hidden);
    int rc = mi_check_launch("rmsnorm_bwd");
    if (rc != MI_OK) return rc;
    rmsnorm_dw_reduce_kernel<T><<<dim3((unsigned)((hidden + kDwCols - 1) / kDwCols)), dim3(kBlock), 0, st>>>((const float*)ws, (T*)dw,
                                                                                               blocks, (int)hidden);
    return mi_check_launch("rmsnorm_dw_reduce");
}

// ---- LayerNorm (weight and optional bias) -----------------------------------------------------------------
// Same row ownership as the RMSNorm kernels.  Mean and variance are taken in fp32 from the register copy of
// the row (two passes over registers, one over HBM).
template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kBlock) void layernorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                const T* __restrict__ b, T* __restrict__ y,
                                                                float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                                int64_t n_rows, int hidden, float eps) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kBlock / TPR;
    __shared__ float lds[4];
    const int tr = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
    const bool row_ok = row < n_rows;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;
    const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
    float f[CH][V];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int v = c * TPR + tr;
        const uint4 raw = (row_ok && v < vecs) ? ldg_nt(xr + v) : make_uint4(0, 0, 0, 0);
        Elem<T>::unpack(raw, f[c]);
#pragma unroll
        for (int i = 0; i < V; ++i) sum += f[c][i];
    }
    const float mean = row_sum<TPR>(sum, lds) * inv_h;
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool live = c * TPR + tr < vecs;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const float dlt = live ? f[c][i] - mean : 0.f;
            sq += dlt * dlt;
        }
    }
    const float rstd = rsqrtf(row_sum<TPR>(sq, lds) * inv_h + eps);
    if (!row_ok) return;
    if (mean_out != nullptr && tr == 0) { mean_out[row] = mean; rstd_out[row] = rstd; }
    const uint4* wr = reinterpret_cast<const uint4*>(w);
    const uint4* br = reinterpret_cast<const uint4*>(b);
    uint4* yr = reinterpret_cast<uint4*>(y + row * hidden);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int v = c * TPR + tr;
        if (v < vecs) {
            float g[V], bb[V], o[V];
            Elem<T>::unpack(wr[v], g);
            if (b != nullptr) Elem<T>::unpack(br[v], bb);
#pragma unroll
            for (int i = 0; i < V; ++i) o[i] = (f[c][i] - mean) * rstd * g[i] + (b != nullptr ? bb[i] : 0.f);
            stg_nt(yr + v, Elem<T>::pack(o));
        }
    }
}

// dx = rstd * (g*w - mean(g*w) - xhat * mean(g*w*xhat)),  dw = sum_rows g * xhat,  db = sum_rows g
// partial rows: [gridDim.x][hidden] of dw followed by [gridDim.x][hidden] of db
template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kBlock) void layernorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                const T* __restrict__ dy, T* __restrict__ dx,
                                                                float* __restrict__ partial, int64_t n_rows, int hidden,
                                                                float eps) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kBlock / TPR;
    extern __shared__ float comb_lds[];  // [2][hidden]
    __shared__ float lds[4];
    const int tr = threadIdx.x % TPR;
    const int rg = threadIdx.x / TPR;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;
    const uint4* wr = reinterpret_cast<const uint4*>(w);

    float acc_w[CH][V], acc_b[CH][V];
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < V; ++i) { acc_w[c][i] = 0.f; acc_b[c][i] = 0.f; }

    const int64_t row_step = (int64_t)gridDim.x * RPB;
    const int64_t iters = (n_rows + row_step - 1) / row_step;   // same count in every thread (barriers in row_sum)
    for (int64_t it = 0; it < iters; ++it) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + (row_ok ? row : 0) * hidden);
        float xf[CH][V], gw[CH][V];
        uint4 graw[CH];
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            const bool ok = row_ok && v < vecs;
            const uint4 xraw = ok ? xr[v] : make_uint4(0, 0, 0, 0);
            graw[c] = ok ? gr[v] : make_uint4(0, 0, 0, 0);
            Elem<T>::unpack(xraw, xf[c]);
#pragma unroll
            for (int i = 0; i < V; ++i) sum += xf[c][i];
        }
        const float mean = row_sum<TPR>(sum, lds) * inv_h;
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const bool live = row_ok && c * TPR + tr < vecs;
#pragma unroll
            for (int i = 0; i < V; ++i) {
                xf[c][i] = live ? xf[c][i] - mean : 0.f;
                sq += xf[c][i] * xf[c][i];
            }
        }
        const float rstd = rsqrtf(row_sum<TPR>(sq, lds) * inv_h + eps);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            float gf[V], wf[V];
            Elem<T>::unpack(graw[c], gf);
            Elem<T>::unpack(v < vecs ? wr[v] : make_uint4(0, 0, 0, 0), wf);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                xf[c][i] *= rstd;                       // xhat
                gw[c][i] = gf[i] * wf[i];
                s1 += gw[c][i];
                s2 += gw[c][i] * xf[c][i];
                acc_w[c][i] += gf[i] * xf[c][i];
                acc_b[c][i] += gf[i];
            }
        }
        s1 = row_sum<TPR>(s1, lds) * inv_h;
        s2 = row_sum<TPR>(s2, lds) * inv_h;
        if (row_ok) {
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * hidden);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
                    float o[V];
#pragma unroll
                    for (int i = 0; i < V; ++i) o[i] = rstd * (gw[c][i] - s1 - xf[c][i] * s2);
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
    }

    // combine the row groups of this block in a fixed order, then emit one partial row each for dw and db
    for (int i = threadIdx.x; i < 2 * hidden; i += kBlock) comb_lds[i] = 0.f;
    __syncthreads();
    for (int g = 0; g < RPB; ++g) {
        if (rg == g) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        comb_lds[v * V + i] += acc_w[c][i];
                        comb_lds[hidden + v * V + i] += acc_b[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    float* out_w = partial + (int64_t)blockIdx.x * hidden;
    float* out_b = partial + ((int64_t)gridDim.x + blockIdx.x) * hidden;
    for (int i = threadIdx.x; i < hidden; i += kBlock) { out_w[i] = comb_lds[i]; out_b[i] = comb_lds[hidden + i]; }
}

// Backward for wide rows, laid out like rmsnorm_bwd_wide_kernel: 512 threads per block, TPR (256 or 512)
// threads per row, the fp32 weight in LDS, the rows of the next step in flight while this step is reduced.
// A row step takes two block-wide reductions (the mean, then the centred sums), each through its own
// double-buffered LDS slot, so two barriers per step.
template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kWideBlock, 4) void layernorm_bwd_wide_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                            const T* __restrict__ dy, T* __restrict__ dx,
                                                                            float* __restrict__ partial, int64_t n_rows,
                                                                            int hidden, float eps) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kWideBlock / TPR;
    constexpr int WPR = TPR / 64;
    extern __shared__ float comb_lds[];   // [hidden] dweight, [hidden] dbias, then [hidden] fp32 copy of the weight
    __shared__ float part_mean[2][8];
    __shared__ float part_sq[2][8], part_s1[2][8], part_s2[2][8];
    float* w_lds = comb_lds + 2 * hidden;
    const int tr = threadIdx.x % TPR;
    const int rg = threadIdx.x / TPR;
    const int wave = threadIdx.x >> 6;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;

    float acc_w[CH][V], acc_b[CH][V];
    for (int i = threadIdx.x; i < hidden; i += kWideBlock) w_lds[i] = Elem<T>::load1(w + i);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < V; ++i) { acc_w[c][i] = 0.f; acc_b[c][i] = 0.f; }
    __syncthreads();
    const int64_t row_step = (int64_t)gridDim.x * RPB;
    const int64_t iters = (n_rows + row_step - 1) / row_step;
    uint4 xraw[CH], graw[CH], xnext[CH], gnext[CH];
    auto fetch = [&](int64_t it, uint4 (&xv)[CH], uint4 (&gv)[CH]) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + (row_ok ? row : 0) * hidden);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            const bool ok = row_ok && v < vecs;
            xv[c] = ok ? xr[v] : make_uint4(0, 0, 0, 0);
            gv[c] = ok ? gr[v] : make_uint4(0, 0, 0, 0);
        }
    };
    if (iters > 0) fetch(0, xraw, graw);
    for (int64_t it = 0; it < iters; ++it) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        if (it + 1 < iters) fetch(it + 1, xnext, gnext);
        const int par = (int)(it & 1);
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float xf[V];
            Elem<T>::unpack(xraw[c], xf);
#pragma unroll
            for (int i = 0; i < V; ++i) sum += xf[i];
        }
        sum = group_sum<64>(sum);
        if ((threadIdx.x & 63) == 0) part_mean[par][wave] = sum;
        __syncthreads();
        sum = 0.f;
#pragma unroll
        for (int j = 0; j < WPR; ++j) sum += part_mean[par][WPR * rg + j];
        const float mean = sum * inv_h;
        float sq = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float xf[V], gf[V], wf[V];
            Elem<T>::unpack(xraw[c], xf);
            Elem<T>::unpack(graw[c], gf);
            const bool live = c * TPR + tr < vecs;
            const int v0 = (live ? c * TPR + tr : 0) * V;
#pragma unroll
            for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v0 + i);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float xc = live ? xf[i] - mean : 0.f;
                const float gw = gf[i] * wf[i];       // zero where the row or the vector is out of range
                sq += xc * xc;
                s1 += gw;
                s2 += gw * xc;
            }
        }
        sq = group_sum<64>(sq);
        s1 = group_sum<64>(s1);
        s2 = group_sum<64>(s2);
        if ((threadIdx.x & 63) == 0) { part_sq[par][wave] = sq; part_s1[par][wave] = s1; part_s2[par][wave] = s2; }
        __syncthreads();
        sq = 0.f; s1 = 0.f; s2 = 0.f;
#pragma unroll
        for (int j = 0; j < WPR; ++j) {
            sq += part_sq[par][WPR * rg + j];
            s1 += part_s1[par][WPR * rg + j];
            s2 += part_s2[par][WPR * rg + j];
        }
        const float rstd = rsqrtf(sq * inv_h + eps);
        s1 *= inv_h;
        s2 *= inv_h * rstd;                           // mean(gw * xhat)
        if (row_ok) {
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * hidden);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
                    float xf[V], gf[V], wf[V], o[V];
                    Elem<T>::unpack(xraw[c], xf);
                    Elem<T>::unpack(graw[c], gf);
#pragma unroll
                    for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v * V + i);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const float xhat = (xf[i] - mean) * rstd;
                        o[i] = rstd * (gf[i] * wf[i] - s1 - xhat * s2);
                        acc_w[c][i] += gf[i] * xhat;
                        acc_b[c][i] += gf[i];
                    }
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) { xraw[c] = xnext[c]; graw[c] = gnext[c]; }
    }
    for (int i = threadIdx.x; i < 2 * hidden; i += kWideBlock) comb_lds[i] = 0.f;
    __syncthreads();
    for (int g = 0; g < RPB; ++g) {
        if (rg == g) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        comb_lds[v * V + i] += acc_w[c][i];
                        comb_lds[hidden + v * V + i] += acc_b[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    float* out_w = partial + (int64_t)blockIdx.x * hidden;
    float* out_b = partial + ((int64_t)gridDim.x + blockIdx.x) * hidden;
    for (int i = threadIdx.x; i < hidden; i += kWideBlock) { out_w[i] = comb_lds[i]; out_b[i] = comb_lds[hidden + i]; }
}

// Backward for wide rows when the forward pass saved mean and rstd: the two row sums (g*w and g*w*xhat) no
// longer wait for the statistics, so a row step takes one block-wide reduction, as in rmsnorm_bwd_wide_kernel
// (same block shape: kRmsWideBlock threads, one block per compute unit, one barrier per row step).
template <typename T, int TPR, int CH>
__global__ __launch_bounds__(kRmsWideBlock) void layernorm_bwd_stats_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                             const T* __restrict__ dy,
                                                                             const float* __restrict__ mean_in,
                                                                             const float* __restrict__ rstd_in, T* __restrict__ dx,
                                                                             float* __restrict__ partial, int64_t n_rows,
                                                                             int hidden) {
    constexpr int V = Elem<T>::kVec;
    constexpr int RPB = kRmsWideBlock / TPR;
    constexpr int WPR = TPR / 64;
    extern __shared__ float comb_lds[];   // [hidden] dweight, [hidden] dbias, then [hidden] fp32 copy of the weight
    __shared__ float2 part[2][16];        // [parity][wavefront]: sum g*w, sum g*w*xhat
    float* w_lds = comb_lds + 2 * hidden;
    const int tr = threadIdx.x % TPR;
    const int rg = threadIdx.x / TPR;
    const int wave = threadIdx.x >> 6;
    const int vecs = hidden / V;
    const float inv_h = 1.0f / (float)hidden;

    float acc_w[CH][V], acc_b[CH][V];
    for (int i = threadIdx.x; i < hidden; i += kRmsWideBlock) w_lds[i] = Elem<T>::load1(w + i);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < V; ++i) { acc_w[c][i] = 0.f; acc_b[c][i] = 0.f; }
    __syncthreads();
    const int64_t row_step = (int64_t)gridDim.x * RPB;
    const int64_t iters = (n_rows + row_step - 1) / row_step;
    uint4 xraw[CH], graw[CH], xnext[CH], gnext[CH];
    float mean = 0.f, rstd = 0.f, mean_next = 0.f, rstd_next = 0.f;
    auto fetch = [&](int64_t it, uint4 (&xv)[CH], uint4 (&gv)[CH], float& mu, float& rs) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        const uint4* xr = reinterpret_cast<const uint4*>(x + (row_ok ? row : 0) * hidden);
        const uint4* gr = reinterpret_cast<const uint4*>(dy + (row_ok ? row : 0) * hidden);
        mu = mean_in[row_ok ? row : 0];
        rs = rstd_in[row_ok ? row : 0];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int v = c * TPR + tr;
            const bool ok = row_ok && v < vecs;
            xv[c] = ok ? xr[v] : make_uint4(0, 0, 0, 0);
            gv[c] = ok ? gr[v] : make_uint4(0, 0, 0, 0);
        }
    };
    if (iters > 0) fetch(0, xraw, graw, mean, rstd);
    for (int64_t it = 0; it < iters; ++it) {
        const int64_t row = it * row_step + (int64_t)blockIdx.x * RPB + rg;
        const bool row_ok = row < n_rows;
        if (it + 1 < iters) fetch(it + 1, xnext, gnext, mean_next, rstd_next);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float xf[V], gf[V], wf[V];
            Elem<T>::unpack(xraw[c], xf);
            Elem<T>::unpack(graw[c], gf);
            const int v0 = (c * TPR + tr < vecs ? c * TPR + tr : 0) * V;
#pragma unroll
            for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v0 + i);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float gw = gf[i] * wf[i];       // zero where the row or the vector is out of range
                s1 += gw;
                s2 += gw * ((xf[i] - mean) * rstd);
            }
        }
        s1 = group_sum<64>(s1);
        s2 = group_sum<64>(s2);
        const int par = (int)(it & 1);
        if ((threadIdx.x & 63) == 0) part[par][wave] = make_float2(s1, s2);
        __syncthreads();
        s1 = 0.f;
        s2 = 0.f;
#pragma unroll
        for (int j = 0; j < WPR; ++j) {
            const float2 pj = part[par][WPR * rg + j];
            s1 += pj.x;
            s2 += pj.y;
        }
        s1 *= inv_h;
        s2 *= inv_h;
        if (row_ok) {
            uint4* dxr = reinterpret_cast<uint4*>(dx + row * hidden);
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
                    float xf[V], gf[V], wf[V], o[V];
                    Elem<T>::unpack(xraw[c], xf);
                    Elem<T>::unpack(graw[c], gf);
#pragma unroll
                    for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4_t*>(wf + i) = *reinterpret_cast<const f32x4_t*>(w_lds + v * V + i);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const float xhat = (xf[i] - mean) * rstd;
                        o[i] = rstd * (gf[i] * wf[i] - s1 - xhat * s2);
                        acc_w[c][i] += gf[i] * xhat;
                        acc_b[c][i] += gf[i];
                    }
                    dxr[v] = Elem<T>::pack(o);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) { xraw[c] = xnext[c]; graw[c] = gnext[c]; }
        mean = mean_next;
        rstd = rstd_next;
    }
    for (int i = threadIdx.x; i < 2 * hidden; i += kRmsWideBlock) comb_lds[i] = 0.f;
    __syncthreads();
    for (int g = 0; g < RPB; ++g) {
        if (rg == g) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int v = c * TPR + tr;
                if (v < vecs) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        comb_lds[v * V + i] += acc_w[c][i];
                        comb_lds[hidden + v * V + i] += acc_b[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    float* out_w = partial + (int64_t)blockIdx.x * hidden;
    float* out_b = partial + ((int64_t)gridDim.x + blockIdx.x) * hidden;
    for (int i = threadIdx.x; i < hidden; i += kRmsWideBlock) { out_w[i] = comb_lds[i]; out_b[i] = comb_lds[hidden + i]; }
}

template <typename T>
int launch_ln_fwd(const void* x, const void* w, const void* b, void* y, float* mean, float* rstd, int64_t n_rows,
                  int64_t hidden, float eps, hipStream_t st) {
    Plan plan;
    if (!make_plan<T>(hidden, &plan))
        return mi_fail(MI_E_SHAPE, "layernorm: hidden=%lld unsupported (must be a multiple of %d and <= %d)",
                       (long long)hidden, Elem<T>::kVec, 256 * 8 * Elem<T>::kVec);
    const bool launched = dispatch_plan(plan, [&](auto tag) {
        constexpr int TPR = decltype(tag)::TPR;
        constexpr int CH = decltype(tag)::CH;
        const int rpb = kBlock / TPR;
        const unsigned grid = (unsigned)((n_rows + rpb - 1) / rpb);
        layernorm_fwd_kernel<T, TPR, CH><<<dim3(grid), dim3(kBlock), 0, st>>>((const T*)x, (const T*)w, (const T*)b, (T*)y,
                                                                              mean, rstd, n_rows, (int)hidden, eps);
    });
    if (!launched) return mi_fail(MI_E_SHAPE, "layernorm: no kernel for hidden=%lld", (long long)hidden);
    return mi_check_launch("layernorm_fwd");
}

template <typename T>
int launch_ln_bwd(const void* x, const void* w, const void* dy, const float* mean, const float* rstd, void* dx, void* dw,
                  void* db, void* ws, size_t ws_bytes, int64_t n_rows, int64_t hidden, float eps, hipStream_t st) {
    Plan plan;
    if (!make_plan<T>(hidden, &plan)) return mi_fail(MI_E_SHAPE, "layernorm: hidden=%lld unsupported", (long long)hidden);
    const int64_t vecs = hidden / Elem<T>::kVec;
    // rows beyond 1024 vectors take the whole 1024-thread block, which only the saved-statistics kernel has
    const bool lds_fits = (size_t)3 * hidden * sizeof(float) <= 159 * 1024;
    const bool wide = vecs >= 256 && lds_fits && (vecs <= 1024 || (vecs <= 2048 && mean != nullptr));
    const int wide_tpr = vecs <= 512 ? 256 : (vecs <= 1024 ? 512 : 1024);
    // saved statistics (wide rows only; narrower rows recompute them, which costs them nothing measurable)
    const bool stats = wide && mean != nullptr;
    const int wide_rpb = (stats ? kRmsWideBlock : kWideBlock) / wide_tpr;
    const int wide_max = stats ? kWideMaxBlocks : kLnMaxBlocks;
    const int64_t wide_blocks = (n_rows + wide_rpb - 1) / wide_rpb;
    int blocks = wide ? (int)(wide_blocks > wide_max ? wide_max : (wide_blocks < 1 ? 1 : wide_blocks))
                      : bwd_blocks(n_rows, plan.tpr);
    if (blocks > kLnMaxBlocks) blocks = kLnMaxBlocks;
    if (ws == nullptr || ws_bytes < (size_t)2 * blocks * hidden * sizeof(float))
        return mi_fail(MI_E_WORKSPACE, "layernorm_bwd: workspace needs %zu bytes, got %zu",
                       (size_t)2 * blocks * hidden * sizeof(float), ws_bytes);
    bool launched = true;
    if (stats) {
        const int ch = (int)((vecs + wide_tpr - 1) / wide_tpr);
        const size_t lds = 3 * hidden * sizeof(float);
#define LN_STATS(TPRV, CHV) layernorm_bwd_stats_kernel<T, TPRV, CHV><<<dim3(blocks), dim3(kRmsWideBlock), lds, st>>>( \
            (const T*)x, (const T*)w, (const T*)dy, mean, rstd, (T*)dx, (float*)ws, n_rows, (int)hidden)
        if (wide_tpr == 256) { if (ch <= 1) LN_STATS(256, 1); else LN_STATS(256, 2); }
        else if (wide_tpr == 512) LN_STATS(512, 2);
        else LN_STATS(1024, 2);
#undef LN_STATS
    } else if (wide) {
        const int ch = (int)((vecs + wide_tpr - 1) / wide_tpr);
        const size_t lds = 3 * hidden * sizeof(float);
#define LN_WIDE(TPRV, CHV) layernorm_bwd_wide_kernel<T, TPRV, CHV><<<dim3(blocks), dim3(kWideBlock), lds, st>>>( \
            (const T*)x, (const T*)w, (const T*)dy, (T*)dx, (float*)ws, n_rows, (int)hidden, eps)
        if (wide_tpr == 256) { if (ch <= 1) LN_WIDE(256, 1); else LN_WIDE(256, 2); }
        else LN_WIDE(512, 2);
#undef LN_WIDE
    } else {
        launched = dispatch_plan(plan, [&](auto tag) {
            constexpr int TPR = decltype(tag)::TPR;
            constexpr int CH = decltype(tag)::CH;
            layernorm_bwd_kernel<T, TPR, CH><<<dim3(blocks), dim3(kBlock), 2 * hidden * sizeof(float), st>>>(
                (const T*)x, (const T*)w, (const T*)dy, (T*)dx, (float*)ws, n_rows, (int)hidden, eps);
        });
    }
    if (!launched) return mi_fail(MI_E_SHAPE, "layernorm: no kernel for hidden=%lld", (long long)hidden);
    int rc = mi_check_launch("layernorm_bwd");
    if (rc != MI_OK) return rc;
    const unsigned rgrid = (unsigned)((hidden + kDwCols - 1) / kDwCols);
    rmsnorm_dw_reduce_kernel<T><<<dim3(rgrid, db != nullptr ? 2 : 1), dim3(kBlock), 0, st>>>((const float*)ws, (T*)dw, blocks,
                                                                                             (int)hidden, (T*)db);
    return mi_check_launch("layernorm_dw_reduce");
}

}  // namespace

extern "C" {

int mi_rmsnorm_fwd(const void* x, const void* weight, void* y, float* rstd, int64_t n_rows, int64_t hidden, float eps,
                   int dtype, void* stream) {
    if (n_rows == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !weight || !y) return mi_fail(MI_E_NULL, "rmsnorm_fwd: null pointer");
    if (n_rows < 0 || hidden <= 0) return mi_fail(MI_E_SHAPE, "rmsnorm_fwd: bad shape [%lld, %lld]", (long long)n_rows, (long long)hidden);
    if (!mi_aligned16(x) || !mi_aligned16(weight) || !mi_aligned16(y)) return mi_fail(MI_E_ALIGN, "rmsnorm_fwd: pointers must be 16-byte aligned");
    MI_DISPATCH_DTYPE(dtype, return launch_fwd<T>(x, weight, y, rstd, n_rows, hidden, eps, (hipStream_t)stream));
    return MI_OK;
}

int mi_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* sum_out, void* y, int64_t n_rows,
                       int64_t hidden, float eps, int dtype, void* stream) {
    if (n_rows == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !residual || !weight || !sum_out || !y) return mi_fail(MI_E_NULL, "add_rmsnorm_fwd: null pointer");
    if (n_rows < 0 || hidden <= 0) return mi_fail(MI_E_SHAPE, "add_rmsnorm_fwd: bad shape [%lld, %lld]", (long long)n_rows, (long long)hidden);
    if (!mi_aligned16(x) || !mi_aligned16(residual) || !mi_aligned16(weight) || !mi_aligned16(sum_out) || !mi_aligned16(y))
        return mi_fail(MI_E_ALIGN, "add_rmsnorm_fwd: pointers must be 16-byte aligned");
    if (y == sum_out || y == x || y == residual) return mi_fail(MI_E_SHAPE, "add_rmsnorm_fwd: y must not alias the other tensors");
    MI_DISPATCH_DTYPE(dtype, return launch_fwd<T>(x, weight, y, nullptr, n_rows, hidden, eps, (hipStream_t)stream, residual, sum_out));
    return MI_OK;
}

size_t mi_rmsnorm_bwd_workspace_bytes(int64_t n_rows, int64_t hidden) {
    (void)n_rows;
    return (size_t)kMaxBwdBlocks * (size_t)(hidden > 0 ? hidden : 0) * sizeof(float);
}

int mi_rmsnorm_bwd(const void* x, const void* weight, const void* dy, void* dx, void* dweight, void* workspace,
                   size_t workspace_bytes, int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream) {
    if (!x || !weight || !dy || !dx || !dweight) return mi_fail(MI_E_NULL, "rmsnorm_bwd: null pointer");
    if (n_rows <= 0 || hidden <= 0) return mi_fail(MI_E_SHAPE, "rmsnorm_bwd: bad shape [%lld, %lld]", (long long)n_rows, (long long)hidden);
    if (!mi_aligned16(x) || !mi_aligned16(weight) || !mi_aligned16(dy) || !mi_aligned16(dx) || !mi_aligned16(workspace))
        return mi_fail(MI_E_ALIGN, "rmsnorm_bwd: pointers must be 16-byte aligned");
    if (2 * hidden * sizeof(float) > 160 * 1024 - 256) return mi_fail(MI_E_SHAPE, "rmsnorm_bwd: hidden too large for LDS");
    MI_DISPATCH_DTYPE(dtype, return launch_bwd<T>(x, weight, dy, dx, dweight, workspace, workspace_bytes, n_rows, hidden,
                                                  eps, (hipStream_t)stream));
    return MI_OK;
}

int mi_layernorm_fwd(const void* x, const void* weight, const void* bias, void* y, float* mean, float* rstd,
                     int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream) {
    if (n_rows == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!x || !weight || !y) return mi_fail(MI_E_NULL, "layernorm_fwd: null pointer");
    if ((mean == nullptr) != (rstd == nullptr)) return mi_fail(MI_E_NULL, "layernorm_fwd: mean and rstd go together");
    if (n_rows < 0 || hidden <= 0) return mi_fail(MI_E_SHAPE, "layernorm_fwd: bad shape [%lld, %lld]", (long long)n_rows, (long long)hidden);
    if (!mi_aligned16(x) || !mi_aligned16(weight) || !mi_aligned16(y) || (bias && !mi_aligned16(bias)))
        return mi_fail(MI_E_ALIGN, "layernorm_fwd: pointers must be 16-byte aligned");
    MI_DISPATCH_DTYPE(dtype, return launch_ln_fwd<T>(x, weight, bias, y, mean, rstd, n_rows, hidden, eps, (hipStream_t)stream));
    return MI_OK;
}

size_t mi_layernorm_bwd_workspace_bytes(int64_t n_rows, int64_t hidden) {
    (void)n_rows;
    return (size_t)2 * kLnMaxBlocks * (size_t)(hidden > 0 ? hidden : 0) * sizeof(float);
}

int mi_layernorm_bwd(const void* x, const void* weight, const void* dy, const float* mean, const float* rstd, void* dx,
                     void* dweight, void* dbias, void* workspace, size_t workspace_bytes, int64_t n_rows, int64_t hidden,
                     float eps, int dtype, void* stream) {
    if (!x || !weight || !dy || !dx || !dweight) return mi_fail(MI_E_NULL, "layernorm_bwd: null pointer");
    if ((mean == nullptr) != (rstd == nullptr)) return mi_fail(MI_E_NULL, "layernorm_bwd: mean and rstd go together");
    if (n_rows <= 0 || hidden <= 0) return mi_fail(MI_E_SHAPE, "layernorm_bwd: bad shape [%lld, %lld]", (long long)n_rows, (long long)hidden);
    if (!mi_aligned16(x) || !mi_aligned16(weight) || !mi_aligned16(dy) || !mi_aligned16(dx) || !mi_aligned16(workspace))
        return mi_fail(MI_E_ALIGN, "layernorm_bwd: pointers must be 16-byte aligned");
    if (2 * hidden * sizeof(float) > 160 * 1024 - 256) return mi_fail(MI_E_SHAPE, "layernorm_bwd: hidden too large for LDS");
    MI_DISPATCH_DTYPE(dtype, return launch_ln_bwd<T>(x, weight, dy, mean, rstd, dx, dweight, dbias, workspace, workspace_bytes,
                                                     n_rows, hidden, eps, (hipStream_t)stream));
    return MI_OK;
}

}  // extern "C"
