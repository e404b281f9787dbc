// Token-level cross entropy over vocabulary rows for gfx950: loss, log-sum-exp, argmax and (optionally) the
// gradient with respect to the logits in one launch.  HBM-bound: a row is read once and, when the gradient is
// asked for, written once.
//
// Three kernels:
//   ce_row_kernel     gradient asked for: 1024-thread workgroups (one per compute unit) walk the rows; a row stays in
//                     registers (up to 16 x 128-bit vectors per thread, i.e. 131072 16-bit or 65536 fp32 logits), so
//                     max, sum of exponentials and the gradient all come from the single read; of rows longer than
//                     9216 vectors the first 9 vectors per thread of the next row are fetched into LDS meanwhile
//   ce_fwd_kernel     no gradient: 512-thread workgroups stream a row once with a running (max, sum)
//   ce_stream_kernel  anything else (rows that do not fit, unaligned rows, vocab not a multiple of the vector width):
//                     scalar accesses, the row is re-read for each of three passes
#include "common.h"

#include <type_traits>

namespace {

constexpr int kCeBlock = 1024;
constexpr int kCeWaves = kCeBlock / 64;
constexpr int kCeResident = 256;   // compute units
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct RowStats {
    float mx;       // row maximum
    float sum;      // sum exp(x - mx)
    int arg;        // first index of the maximum
};

// Block-wide (max, first index of max); every thread receives the result.
__device__ __forceinline__ void block_argmax(float& v, int& idx, float* lds_v, int* lds_i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, MI_WAVE);
        const int oi = __shfl_xor(idx, off, MI_WAVE);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { lds_v[wave] = v; lds_i[wave] = idx; }
    __syncthreads();
    v = lds_v[0];
    idx = lds_i[0];
#pragma unroll
    for (int w = 1; w < kCeWaves; ++w) {
        const float ov = lds_v[w];
        const int oi = lds_i[w];
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
}

__device__ __forceinline__ float block_sum(float v, float* lds) {
    v = group_sum<64>(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kCeWaves; ++w) s += lds[w];
    return s;
}

// 128 bits of -inf in the logits' type: a register that holds no part of the row
template <typename T> __device__ __forceinline__ uint4 neg_inf_vec();
template <> __device__ __forceinline__ uint4 neg_inf_vec<__bf16>() { return make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u); }
template <> __device__ __forceinline__ uint4 neg_inf_vec<_Float16>() { return make_uint4(0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u); }
template <> __device__ __forceinline__ uint4 neg_inf_vec<float>() { return make_uint4(0xff800000u, 0xff800000u, 0xff800000u, 0xff800000u); }

// Keeps the three passes from sharing one unpacked fp32 copy of the row (it would need eight times the registers):
// after this the compiler knows nothing about the value.
__device__ __forceinline__ void forget(uint4& u) { asm volatile("" : "+v"(u.x), "+v"(u.y), "+v"(u.z), "+v"(u.w)); }

struct CeArgs {
    const void* logits;
    const int64_t* targets;
    const float* row_scale;    // nullable: gradient scale per row (loss weight / sum of weights), 1 when null
    float* losses;             // nullable
    float* lse;                // nullable
    int32_t* argmax;           // nullable
    void* dlogits;             // nullable, may alias logits
    int64_t logits_stride, dlogits_stride;
    int vocab;
};

// Finishes a row once max / sum are known: scalar outputs by thread 0, returns (lse, scale) for the gradient.
template <typename T>
__device__ __forceinline__ void row_outputs(const CeArgs& a, int64_t row, const RowStats& st, int64_t target, bool ignored,
                                            float x_target, float& lse, float& scale) {
    lse = st.mx + __builtin_amdgcn_logf(st.sum) * kLn2;
    scale = ignored ? 0.f : (a.row_scale != nullptr ? a.row_scale[row] : 1.0f);
    if (threadIdx.x == 0) {
        if (a.losses != nullptr) a.losses[row] = ignored ? 0.f : lse - x_target;
        if (a.lse != nullptr) a.lse[row] = lse;
        if (a.argmax != nullptr) a.argmax[row] = st.arg;
    }
    (void)target;
}

// One logit as raw bits (16-bit types zero-extended): a single load instruction with no arithmetic behind it, so
// that nothing waits for the load where it is issued; bits_to_float converts where the value is used.
template <typename T> __device__ __forceinline__ uint32_t load1_bits(const T* p) {
    if constexpr (sizeof(T) == 2) return *reinterpret_cast<const uint16_t*>(p);
    else return *reinterpret_cast<const uint32_t*>(p);
}
template <typename T> __device__ __forceinline__ float bits_to_float(uint32_t b) {
    if constexpr (std::is_same<T, __bf16>::value) return __uint_as_float(b << 16);
    else if constexpr (std::is_same<T, _Float16>::value) return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
    else return __uint_as_float(b);
}

// NL > 0: the first NL vectors per thread of the next row are fetched into LDS by direct global -> LDS loads.  They
// need no register, so they are in flight during the second pass and the reduction of the current row, when the
// registers still hold that row and nothing else could be requested; only the remaining NV - NL vectors per thread
// are requested when the gradient pass frees their registers.
template <typename T, int NV, int NL>
__global__ __launch_bounds__(kCeBlock) void ce_row_kernel(const CeArgs a, int n_rows) {
    constexpr int V = Elem<T>::kVec;
    static_assert(NL >= 0 && NL <= NV && NL * kCeBlock * 16 <= 152 * 1024, "staging area within the LDS");
    // reduction slots, double-buffered by row parity so that one barrier per row is enough
    __shared__ float lds_m[2][kCeWaves], lds_s[2][kCeWaves];
    __shared__ int lds_i[2][kCeWaves];
    __shared__ __attribute__((aligned(1024))) u32x4_t stage[NL > 0 ? NL : 1][kCeBlock];
    const int vecs = a.vocab / V;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool lane0 = (threadIdx.x & 63) == 0;
    // LDS byte address of this wavefront's 64 slots of staged vector 0
    const uint32_t stage_base = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)&stage[0][0]) + (uint32_t)wave * 1024u;

    // A workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ...  The vectors of the next row that are not
    // staged are requested as soon as the gradient pass over the current row has consumed the register they land
    // in, so the read of row r + 1 (and the write of row r) overlap the arithmetic of row r.  Registers past the end
    // of the row are never loaded and stay at -inf, which every pass treats as "no element" (max ignores it, exp
    // gives 0).  Staged vectors are whole: the launch asks for vecs >= NL * kCeBlock.
    uint4 raw[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) raw[j] = neg_inf_vec<T>();
    auto row_ptr = [&](int64_t r) { return reinterpret_cast<const T*>(a.logits) + r * a.logits_stride; };
    auto in_row = [&](int j) { return j < NL || j * kCeBlock + (int)threadIdx.x < vecs; };
    auto load_vec = [&](int64_t r, int j) {
        if (in_row(j)) raw[j] = ldg_nt(reinterpret_cast<const uint4*>(row_ptr(r)) + j * kCeBlock + threadIdx.x);
    };
    // Direct load of vector j of row r into this thread's staging slot.  A wavefront writes and later reads only its
    // own 64 slots of a vector, so its own wait for the loads is all the ordering the staging needs.  The compiler
    // does not count these loads.  Vector memory operations complete in order, so a wait it places for one of its
    // own loads still covers that load; it waits for the direct loads as well when they are older, which is why
    // they are issued where no tracked load is consumed before the explicit wait.  The barrier of the reduction
    // must not wait for them either, hence the hand-written one.
    auto stage_vec = [&](int64_t r, int j) {
        const uint32_t dst = stage_base + (uint32_t)j * (kCeBlock * 16u);
        const uint4* src = reinterpret_cast<const uint4*>(row_ptr(r)) + j * kCeBlock;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :: "v"((uint32_t)threadIdx.x * 16u), "s"(src), "s"(dst) : "memory", "m0");
    };
    auto take_staged = [&](int j) {
        const u32x4_t x = stage[j][threadIdx.x];
        raw[j] = make_uint4(x[0], x[1], x[2], x[3]);
    };
    auto block_barrier = [&]() {
        if constexpr (NL > 0) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else __syncthreads();
    };
    // Target and target logit of the next row are requested at the start of the gradient pass, where nothing else is
    // in flight, the target a row before its logit (whose address it gives): waiting for either at the top of a row
    // would wait for every older load, i.e. for the whole row in flight.  The index passes through a register the
    // compiler knows nothing about, or it would move the (uniform) target into scalar registers right behind the
    // load, which waits on the spot; to_scalar does that a row later.
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    auto load_target = [&](int64_t r) { return a.targets[r + lane_zero]; };
    auto to_scalar = [](int64_t t) {
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)t);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)t >> 32));
        return (int64_t)(((uint64_t)hi << 32) | lo);
    };
    auto is_ignored = [&](int64_t t) { return t < 0 || t >= a.vocab; };
    auto load_x_bits = [&](int64_t r, int64_t t) {      // read before an in-place gradient overwrites it
        return is_ignored(t) ? 0u : load1_bits<T>(row_ptr(r) + t);
    };
    auto emit_argmax = [&](int64_t r, int par) {      // thread 0, after a barrier that follows the slot writes
        if (a.argmax == nullptr) return;
        int best = lds_i[par][0];
#pragma unroll
        for (int w = 1; w < kCeWaves; ++w) best = min(best, lds_i[par][w]);
        a.argmax[r] = best;
    };

    int64_t row = blockIdx.x;
    if (row >= n_rows) return;
#pragma unroll
    for (int j = 0; j < NV; ++j) load_vec(row, j);
    int64_t target = to_scalar(load_target(row));
    int64_t target_pending = -1;              // of the next row, in flight until the gradient pass
    if (row + gridDim.x < n_rows) target_pending = load_target(row + gridDim.x);
    uint32_t x_bits = load_x_bits(row, target), x_bits_next = 0;

    int par = 0;
    int64_t prev_row = -1;
    for (; row < n_rows; row += gridDim.x, par ^= 1) {
        const int64_t next = row + gridDim.x;
        const bool has_next = next < n_rows;
        // pass 1: this thread's maximum.  The vectors that came from memory first; once they are here nothing the
        // compiler tracks is in flight, and the staged part of the next row is requested.
        float mt = -INFINITY;
        auto max_vec = [&](int j) {
            float f[V];
            forget(raw[j]);
            Elem<T>::unpack(raw[j], f);
#pragma unroll
            for (int i = 0; i < V; ++i) mt = fmaxf(mt, f[i]);
            if (j & 1) __builtin_amdgcn_sched_barrier(0);    // two vectors at a time: unpacking further ahead only costs registers
        };
#pragma unroll
        for (int j = NL; j < NV; ++j) max_vec(j);
        if constexpr (NL > 0) {
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the slots have been read before they are refilled
            if (has_next) {
#pragma unroll
                for (int j = 0; j < NL; ++j) stage_vec(next, j);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NL; ++j) max_vec(j);
        }
        // pass 2: this thread's sum of exponentials relative to its own maximum
        const float mt2 = (mt == -INFINITY ? 0.f : mt) * kLog2e;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            float f[V];
            forget(raw[j]);
            Elem<T>::unpack(raw[j], f);
#pragma unroll
            for (int i = 0; i < V; i += 2) {
                s0 += __builtin_amdgcn_exp2f(f[i] * kLog2e - mt2);
                s1 += __builtin_amdgcn_exp2f(f[i + 1] * kLog2e - mt2);
            }
            if (j & 1) __builtin_amdgcn_sched_barrier(0);
        }
        // merge (maximum, sum) pairs: wavefront, then block
        const float wm = group_max<64>(mt);
        float ws = (mt == -INFINITY) ? 0.f : (s0 + s1) * __builtin_amdgcn_exp2f((mt - wm) * kLog2e);
        ws = group_sum<64>(ws);
        if (lane0) { lds_m[par][wave] = wm; lds_s[par][wave] = ws; }
        block_barrier();
        if (threadIdx.x == 0 && prev_row >= 0) emit_argmax(prev_row, par ^ 1);   // slots of the previous row are complete
        // every row of 16 lanes merges the 16 slots, one slot per lane
        static_assert(kCeWaves == 16, "one slot per lane of a 16-lane row");
        const float m_w = lds_m[par][threadIdx.x & 15], s_w = lds_s[par][threadIdx.x & 15];
        const float mx = group_max<16>(m_w);
        const float sum = group_sum<16>((m_w == -INFINITY) ? 0.f : s_w * __builtin_amdgcn_exp2f((m_w - mx) * kLog2e));
        // first position of the maximum: only the wavefronts with a thread that holds it look, walking their register
        // copy once more (a few hundred instructions for one wavefront; re-reading the vectors from memory instead
        // put a chain of dependent loads, each behind everything else in flight, on the critical path of the row)
        int arg = 0x7fffffff;
        if (__any(mt == mx)) {
#pragma unroll
            for (int j = NV - 1; j >= 0; --j) {
                float f[V];
                forget(raw[j]);
                Elem<T>::unpack(raw[j], f);
                const int e0 = (j * kCeBlock + (int)threadIdx.x) * V;
#pragma unroll
                for (int i = V - 1; i >= 0; --i)
                    if (f[i] == mx) arg = e0 + i;
                if (j & 1) __builtin_amdgcn_sched_barrier(0);
            }
            arg = group_min<64>(arg);
        }
        if (lane0) lds_i[par][wave] = arg;

        // ---- gradient pass.  Everything requested so far is waited for here: the staged part of the next row, the
        // target of the next row and the target logit of this one.
        if constexpr (NL > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        const int64_t target_next = to_scalar(target_pending);
        if (has_next) x_bits_next = load_x_bits(next, target_next);
        if (next + gridDim.x < n_rows) target_pending = load_target(next + gridDim.x);

        const bool ignored = is_ignored(target);
        asm volatile("" : "+v"(x_bits));
        const float x_target = bits_to_float<T>(x_bits);
        const float lse = mx + __builtin_amdgcn_logf(sum) * kLn2;
        const float scale = ignored ? 0.f : (a.row_scale != nullptr ? a.row_scale[row] : 1.0f);
        if (threadIdx.x == 0) {
            if (a.losses != nullptr) a.losses[row] = ignored ? 0.f : lse - x_target;
            if (a.lse != nullptr) a.lse[row] = lse;
        }
        // the thread that stores the vector holding the target patches that element right after (two stores of one
        // thread to one address keep their order)
        T* dx = reinterpret_cast<T*>(a.dlogits) + row * a.dlogits_stride;
        const float l2 = lse * kLog2e;
        const int v_target = ignored ? -1 : (int)(target / V);
        auto grad_vec = [&](int j) {
            if (in_row(j)) {
                const int v = j * kCeBlock + threadIdx.x;
                float f[V];
                forget(raw[j]);
                Elem<T>::unpack(raw[j], f);
#pragma unroll
                for (int i = 0; i < V; ++i) f[i] = __builtin_amdgcn_exp2f(f[i] * kLog2e - l2) * scale;
                stg_nt(reinterpret_cast<uint4*>(dx) + v, Elem<T>::pack(f));
                if (v == v_target)
                    Elem<T>::store1(dx + target, (__builtin_amdgcn_exp2f(x_target * kLog2e - l2) - 1.0f) * scale);
            }
        };
#pragma unroll
        for (int j = NL; j < NV; ++j) {
            grad_vec(j);
            if (has_next) load_vec(next, j);
            if (j & 1) __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            grad_vec(j);
            if (has_next) take_staged(j);
            if (j & 1) __builtin_amdgcn_sched_barrier(0);
        }
        prev_row = row;
        target = target_next;
        x_bits = x_bits_next;
    }
    block_barrier();
    if (threadIdx.x == 0) emit_argmax(prev_row, par ^ 1);
}

// Forward only (no gradient asked for): nothing of the row has to be kept, so each thread streams its vectors
// once with a running (max, sum) pair and the pairs are merged at the end.  512 threads per row and several
// rows per compute unit keep loads in flight under the arithmetic.
constexpr int kFwdBlock = 512;
constexpr int kFwdDepth = 4;        // vectors in flight per thread

// A row as [head scalars][whole aligned 16-byte vectors][tail scalars].
struct RowSplit {
    int head, vecs, tail0, vocab;
    // index of the scalar element thread t takes, -1 for none
    __device__ __forceinline__ int scalar_index(int t) const {
        if (t < head) return t;
        const int i = tail0 + (t - head);
        return i < vocab ? i : -1;
    }
};

template <typename T> __device__ __forceinline__ RowSplit split_row(const T* x, int vocab) {
    constexpr int V = Elem<T>::kVec;
    RowSplit r;
    const int to_boundary = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(x) & 15u)) & 15u) / sizeof(T));
    r.head = to_boundary < vocab ? to_boundary : vocab;
    r.vecs = (vocab - r.head) / V;
    r.tail0 = r.head + r.vecs * V;
    r.vocab = vocab;
    return r;
}

template <typename T>
__global__ __launch_bounds__(kFwdBlock) void ce_fwd_kernel(const CeArgs a) {
    constexpr int V = Elem<T>::kVec;
    constexpr int NW = kFwdBlock / 64;
    __shared__ float lds_m[NW], lds_s[NW];
    __shared__ int lds_i[NW];
    const int64_t row = blockIdx.x;
    const T* x = reinterpret_cast<const T*>(a.logits) + row * a.logits_stride;
    // rows need not start on a 16-byte boundary nor hold a whole number of vectors: the elements before the first
    // aligned vector and after the last whole one (at most V - 1 each) are taken one per thread
    const RowSplit rs = split_row<T>(x, a.vocab);
    const uint4* xr = reinterpret_cast<const uint4*>(x + rs.head);
    const int vecs = rs.vecs;
    const int64_t target = a.targets[row];
    const bool ignored = target < 0 || target >= a.vocab;
    const float x_target = ignored ? 0.f : Elem<T>::load1(x + target);
    const int sc_idx = rs.scalar_index(threadIdx.x);
    const float sc = sc_idx >= 0 ? Elem<T>::load1(x + sc_idx) : -INFINITY;

    float m = -INFINITY, s = 0.f;     // running maximum (natural units) and sum of exp(x - m)
    uint4 buf[kFwdDepth];
#pragma unroll
    for (int d = 0; d < kFwdDepth; ++d) {
        const int v = threadIdx.x + d * kFwdBlock;
        buf[d] = v < vecs ? ldg_nt(xr + v) : neg_inf_vec<T>();
    }
    for (int v0 = threadIdx.x; v0 < vecs; v0 += kFwdDepth * kFwdBlock) {
#pragma unroll
        for (int d = 0; d < kFwdDepth; ++d) {
            float f[V];
            Elem<T>::unpack(buf[d], f);
            const int vn = v0 + (d + kFwdDepth) * kFwdBlock;
            buf[d] = vn < vecs ? ldg_nt(xr + vn) : neg_inf_vec<T>();
            float vm = f[0];
#pragma unroll
            for (int i = 1; i < V; ++i) vm = fmaxf(vm, f[i]);
            if (vm > m) {             // rare after the first vectors
                s *= __builtin_amdgcn_exp2f((m - vm) * kLog2e);
                m = vm;
            }
            const float m2 = m * kLog2e;
            if (m > -INFINITY) {
#pragma unroll
                for (int i = 0; i < V; ++i) s += __builtin_amdgcn_exp2f(f[i] * kLog2e - m2);
            }
        }
    }
    if (sc > m) {
        s *= __builtin_amdgcn_exp2f((m - sc) * kLog2e);
        m = sc;
    }
    if (sc_idx >= 0 && m > -INFINITY) s += __builtin_amdgcn_exp2f((sc - m) * kLog2e);
    // merge the (m, s) pairs of the block
    float bm = m;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) bm = fmaxf(bm, __shfl_xor(bm, off, MI_WAVE));
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds_m[wave] = bm;
    __syncthreads();
    bm = lds_m[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) bm = fmaxf(bm, lds_m[w]);
    float part = (m > -INFINITY) ? s * __builtin_amdgcn_exp2f((m - bm) * kLog2e) : 0.f;
    part = group_sum<64>(part);
    if ((threadIdx.x & 63) == 0) lds_s[wave] = part;
    // first position of the maximum: the threads whose running maximum equals it re-read their vectors
    int arg = 0x7fffffff;
    if (m == bm) {
#pragma unroll 1
        for (int v = threadIdx.x; v < vecs && arg == 0x7fffffff; v += kFwdBlock) {
            float f[V];
            Elem<T>::unpack(xr[v], f);
#pragma unroll
            for (int i = V - 1; i >= 0; --i)
                if (f[i] == bm) arg = rs.head + v * V + i;
        }
        if (sc_idx >= 0 && sc == bm) arg = min(arg, sc_idx);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) arg = min(arg, __shfl_xor(arg, off, MI_WAVE));
    if ((threadIdx.x & 63) == 0) lds_i[wave] = arg;
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = 0.f;
        int best = 0x7fffffff;
#pragma unroll
        for (int w = 0; w < NW; ++w) { sum += lds_s[w]; best = min(best, lds_i[w]); }
        const float lse = bm + __builtin_amdgcn_logf(sum) * kLn2;
        if (a.losses != nullptr) a.losses[row] = ignored ? 0.f : lse - x_target;
        if (a.lse != nullptr) a.lse[row] = lse;
        if (a.argmax != nullptr) a.argmax[row] = best;
    }
}

// Any vocabulary size, stride and alignment: three passes over the row with scalar accesses.
template <typename T>
__global__ __launch_bounds__(kCeBlock) void ce_stream_kernel(const CeArgs a) {
    __shared__ float lds_v[kCeWaves];
    __shared__ int lds_i[kCeWaves];
    __shared__ float lds_s[kCeWaves];
    const int64_t row = blockIdx.x;
    const T* x = reinterpret_cast<const T*>(a.logits) + row * a.logits_stride;
    const int64_t target = a.targets[row];
    const bool ignored = target < 0 || target >= a.vocab;
    const float x_target = ignored ? 0.f : Elem<T>::load1(x + target);
    float mx = -INFINITY;
    int arg = 0x7fffffff;
    for (int i = threadIdx.x; i < a.vocab; i += kCeBlock) {
        const float f = Elem<T>::load1(x + i);
        if (f > mx) { mx = f; arg = i; }
    }
    block_argmax(mx, arg, lds_v, lds_i);
    const float m2 = mx * kLog2e;
    float sum = 0.f;
    for (int i = threadIdx.x; i < a.vocab; i += kCeBlock) sum += __builtin_amdgcn_exp2f(Elem<T>::load1(x + i) * kLog2e - m2);
    sum = block_sum(sum, lds_s);
    RowStats st{mx, sum, arg};
    float lse, scale;
    row_outputs<T>(a, row, st, target, ignored, x_target, lse, scale);
    if (a.dlogits == nullptr) return;
    T* dx = reinterpret_cast<T*>(a.dlogits) + row * a.dlogits_stride;
    const float l2 = lse * kLog2e;
    for (int i = threadIdx.x; i < a.vocab; i += kCeBlock) {
        const float p = __builtin_amdgcn_exp2f(Elem<T>::load1(x + i) * kLog2e - l2);
        Elem<T>::store1(dx + i, (p - ((int64_t)i == target ? 1.0f : 0.f)) * scale);
    }
}

// Gradient pass for vocabularies whose rows do not fit the registers of one workgroup (more than 16 vectors per
// thread): an elementwise launch after the streaming forward kernel, which has left the log-sum-exp of every row in
// a.lse.  dlogits = (softmax - onehot(target)) * scale; in place is fine (a vector is read and written by one thread).
constexpr int kGradBlock = 256;
constexpr int kGradUnroll = 2;

template <typename T>
__global__ __launch_bounds__(kGradBlock) void ce_grad_kernel(const CeArgs a) {
    constexpr int V = Elem<T>::kVec;
    const int64_t row = blockIdx.y;
    const T* x0 = reinterpret_cast<const T*>(a.logits) + row * a.logits_stride;
    T* dx0 = reinterpret_cast<T*>(a.dlogits) + row * a.dlogits_stride;
    const RowSplit rs = split_row<T>(x0, a.vocab);       // dx0 sits at the same offset from a 16-byte boundary (host check)
    const int vecs = rs.vecs;
    const T* x = x0 + rs.head;
    T* dx = dx0 + rs.head;
    const int64_t target_abs = a.targets[row];
    const bool ignored = target_abs < 0 || target_abs >= a.vocab;
    const int64_t target = target_abs - rs.head;         // relative to the first whole vector
    const float scale = ignored ? 0.f : (a.row_scale != nullptr ? a.row_scale[row] : 1.0f);
    const float l2 = a.lse[row] * kLog2e;
    const int v_target = (ignored || target < 0) ? -1 : (int)(target / V);
    const int base = blockIdx.x * (kGradBlock * kGradUnroll) + threadIdx.x;
    if (blockIdx.x == 0) {                                // the scalar elements of the row
        const int i = rs.scalar_index(threadIdx.x);
        if (i >= 0) {
            const float p = __builtin_amdgcn_exp2f(Elem<T>::load1(x0 + i) * kLog2e - l2);
            Elem<T>::store1(dx0 + i, (p - ((int64_t)i == target_abs && !ignored ? 1.0f : 0.f)) * scale);
        }
    }
    uint4 raw[kGradUnroll];
#pragma unroll
    for (int u = 0; u < kGradUnroll; ++u) {
        const int v = base + u * kGradBlock;
        if (v < vecs) raw[u] = ldg_nt(reinterpret_cast<const uint4*>(x) + v);
    }
#pragma unroll
    for (int u = 0; u < kGradUnroll; ++u) {
        const int v = base + u * kGradBlock;
        if (v < vecs) {
            float f[V];
            Elem<T>::unpack(raw[u], f);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float p = __builtin_amdgcn_exp2f(f[i] * kLog2e - l2);
                f[i] = (p - ((v == v_target && i == (int)(target - (int64_t)v * V)) ? 1.0f : 0.f)) * scale;
            }
            reinterpret_cast<uint4*>(dx)[v] = Elem<T>::pack(f);
        }
    }
}

template <typename T>
int launch_ce(const CeArgs& a, int64_t n_rows, hipStream_t st) {
    constexpr int V = Elem<T>::kVec;
    const bool vec_ok = a.vocab % V == 0 && a.logits_stride % V == 0 && mi_aligned16(a.logits) &&
                        (a.dlogits == nullptr || (a.dlogits_stride % V == 0 && mi_aligned16(a.dlogits)));
    const int64_t vecs = a.vocab / V;
    const int nv = (int)((vecs + kCeBlock - 1) / kCeBlock);
    const dim3 grid((unsigned)n_rows), block(kCeBlock);
    // the streaming kernels take any row alignment; for the gradient launch logits and dlogits rows have to sit
    // at the same offset from a 16-byte boundary
    const bool same_phase = a.dlogits != nullptr &&
        ((reinterpret_cast<uintptr_t>(a.logits) ^ reinterpret_cast<uintptr_t>(a.dlogits)) & 15u) == 0 &&
        ((a.logits_stride - a.dlogits_stride) * (int64_t)sizeof(T)) % 16 == 0;
    if (a.dlogits == nullptr) {
        ce_fwd_kernel<T><<<grid, dim3(kFwdBlock), 0, st>>>(a);
    } else if (vec_ok && nv <= 16) {
        // one resident workgroup per compute unit, each walking its share of the rows
        const dim3 pgrid((unsigned)(n_rows < kCeResident ? n_rows : kCeResident));
        const int nr = (int)n_rows;
        if (nv <= 1) ce_row_kernel<T, 1, 0><<<pgrid, block, 0, st>>>(a, nr);
        else if (nv <= 2) ce_row_kernel<T, 2, 0><<<pgrid, block, 0, st>>>(a, nr);
        else if (nv <= 4) ce_row_kernel<T, 4, 0><<<pgrid, block, 0, st>>>(a, nr);
        else if (nv <= 8) ce_row_kernel<T, 8, 0><<<pgrid, block, 0, st>>>(a, nr);
        else if (vecs >= 9 * kCeBlock) ce_row_kernel<T, 16, 9><<<pgrid, block, 0, st>>>(a, nr);
        else ce_row_kernel<T, 16, 0><<<pgrid, block, 0, st>>>(a, nr);
    } else if (same_phase && a.lse != nullptr && n_rows <= 65535) {
        // rows too long for the register-resident kernel, not a whole number of vectors or not 16-byte aligned:
        // streaming forward, then an elementwise gradient launch
        CeArgs f = a;
        f.dlogits = nullptr;
        ce_fwd_kernel<T><<<grid, dim3(kFwdBlock), 0, st>>>(f);
        const int rc = mi_check_launch("cross_entropy");
        if (rc != MI_OK) return rc;
        const unsigned gx = (unsigned)((vecs + 1 + kGradBlock * kGradUnroll - 1) / (kGradBlock * kGradUnroll));
        ce_grad_kernel<T><<<dim3(gx, (unsigned)n_rows), dim3(kGradBlock), 0, st>>>(a);
    } else {
        ce_stream_kernel<T><<<grid, block, 0, st>>>(a);
    }
    return mi_check_launch("cross_entropy");
}

}  // namespace

extern "C" {

int mi_cross_entropy(const void* logits, const int64_t* targets, const float* row_scale, float* losses, float* lse,
                     int32_t* argmax, void* dlogits, int64_t n_rows, int64_t vocab, int64_t logits_row_stride,
                     int64_t dlogits_row_stride, int dtype, void* stream) {
    if (n_rows < 0 || vocab <= 0 || vocab > 0x7fffffffLL)
        return mi_fail(MI_E_SHAPE, "cross_entropy: bad shape [%lld, %lld]", (long long)n_rows, (long long)vocab);
    if (n_rows == 0) return MI_OK;       // nothing to do (an empty tensor may come with a null pointer)
    if (!logits || !targets) return mi_fail(MI_E_NULL, "cross_entropy: null pointer");
    if (n_rows > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "cross_entropy: too many rows");
    if (logits_row_stride < vocab || (dlogits != nullptr && dlogits_row_stride < vocab))
        return mi_fail(MI_E_SHAPE, "cross_entropy: row stride smaller than the vocabulary");
    CeArgs a;
    a.logits = logits; a.targets = targets; a.row_scale = row_scale; a.losses = losses; a.lse = lse; a.argmax = argmax;
    a.dlogits = dlogits; a.logits_stride = logits_row_stride; a.dlogits_stride = dlogits_row_stride; a.vocab = (int)vocab;
    MI_DISPATCH_DTYPE(dtype, return launch_ce<T>(a, n_rows, (hipStream_t)stream));
    return MI_OK;
}

}  // extern "C"
