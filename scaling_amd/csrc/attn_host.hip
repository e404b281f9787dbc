// Entry points of the attention kernels: the kernels are compiled once per element type (bf16, f16); the C entry points
// here pick the build that matches args->dtype.  Also home of the few things that exist once per library.
#include "attn_common.h"

#include <mutex>

int mi_attn_fwd_impl_bf16(const mi_attn_args* a);
int mi_attn_fwd_impl_f16(const mi_attn_args* a);
int mi_attn_bwd_impl_bf16(const mi_attn_bwd_args* b);
int mi_attn_bwd_impl_f16(const mi_attn_bwd_args* b);
int mi_attn_fwd_impl_f32(const mi_attn_args* a);
int mi_attn_bwd_impl_f32(const mi_attn_bwd_args* b);
int mi_attn_decode_impl_bf16(const mi_decode_args* a, bool static_ws);
int mi_attn_decode_impl_f16(const mi_decode_args* a, bool static_ws);

extern "C" int mi_attn_fwd(const mi_attn_args* a) {
    if (!a) return mi_fail(MI_E_NULL, "attn_fwd: args is null");
    if (a->total_q == 0 && a->total_k == 0) return MI_OK;     // no tokens (an empty tensor may come with a null pointer)
    if (a->dtype == MI_F32) return mi_attn_fwd_impl_f32(a);
    return a->dtype == MI_F16 ? mi_attn_fwd_impl_f16(a) : mi_attn_fwd_impl_bf16(a);
}

extern "C" int mi_attn_bwd(const mi_attn_bwd_args* b) {
    if (!b) return mi_fail(MI_E_NULL, "attn_bwd: args is null");
    if (b->fwd.total_q == 0 && b->fwd.total_k == 0) return MI_OK;
    if (b->fwd.dtype == MI_F32) return mi_attn_bwd_impl_f32(b);
    return b->fwd.dtype == MI_F16 ? mi_attn_bwd_impl_f16(b) : mi_attn_bwd_impl_bf16(b);
}

extern "C" int mi_attn_decode(const mi_decode_args* a) {
    if (!a) return mi_fail(MI_E_NULL, "attn_decode: args is null");
    return a->dtype == MI_F16 ? mi_attn_decode_impl_f16(a, false) : mi_attn_decode_impl_bf16(a, false);
}

extern "C" int mi_attn_decode_static(const mi_decode_args* a) {
    if (!a) return mi_fail(MI_E_NULL, "attn_decode_static: args is null");
    return a->dtype == MI_F16 ? mi_attn_decode_impl_f16(a, true) : mi_attn_decode_impl_bf16(a, true);
}

// ---- scratch of the entry point that allocates nothing -----------------------------------------------------------
// The per-split partial results of mi_attn_decode_static live in a file-scope device array instead of a caller
// workspace.  Every GPU the library's code object is loaded on holds its own copy of the array at its own address,
// obtained once per device with hipGetSymbolAddress (the array's name is only a host-side handle, not a device
// address) and kept in g_scratch_ptr.
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];        // per device; written once, under g_scratch_mutex
std::mutex g_scratch_mutex;
}  // namespace

int mi_static_scratch(void** out, size_t* bytes) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return mi_fail(MI_E_LAUNCH, "attn_decode_static: hipGetDevice failed or device index %d out of range (%s)", dev, hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return mi_fail(MI_E_LAUNCH, "attn_decode_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    *bytes = kStaticScratchBytes;
    return MI_OK;
}

extern "C" size_t mi_attn_decode_static_scratch_bytes(void) { return kStaticScratchBytes; }

// Compute units of the current device (256 on an MI355X), asked once per device.
int mi_compute_units() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}
