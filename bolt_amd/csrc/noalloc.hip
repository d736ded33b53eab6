// The one entry point that allocates nothing: dynamic fp32 -> u8 / s8 quantisation with the scale kept on the
// device, for callers that cannot call hipMalloc (code under HIP graph capture, tight serving loops, harnesses that
// forbid allocation). It is bolt_gfx950_quantize_f32_async with the partial-maximum slots -- the scratch words that
// entry point takes from the library's allocation -- in a file-scope device array instead.
//
// In host code the array's NAME is a host-side stand-in, not a device address: it must never be passed to a kernel
// or a memory routine. Its device address is looked up once per device with hipGetSymbolAddress (each GPU holds its
// own copy of the array at its own address) and only that pointer is used below.
#include <hip/hip_runtime.h>
#include <mutex>

#include "../../include/bolt_gfx950.h"
#include "kernels.h"

using namespace bg;

namespace {

// 64 slots of one 64-byte line each (kWsWords words = 4 KiB). Every GPU the library runs on holds this until the
// process ends.
static __device__ __align__(256) uint32_t scratch[kWsWords];

constexpr int kMaxDevices = 64;
std::mutex g_mu;
uint32_t *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device i; null until looked up

// Device address of the scratch array on the CURRENT device (looked up on first use, with that device current).
EE scratch_on_current_device(uint32_t **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        api_set_error("hipGetDevice", e);
        return UNKNOWN;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        api_set_error("quantize_f32_noalloc: device ordinal beyond 63", hipSuccess);
        return NOT_SUPPORTED;
    }
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            api_set_error("hipGetSymbolAddress(scratch)", e);
            return UNKNOWN;
        }
        g_scratch_ptr[dev] = (uint32_t *)p;
    }
    *out = g_scratch_ptr[dev];
    return SUCCESS;
}

}  // namespace

namespace bg {

// called by the library's init with the device it initialises on current
int noalloc_init_current_device()
{
    uint32_t *p = nullptr;
    return (int)scratch_on_current_device(&p);
}

}  // namespace bg

extern "C" EE bolt_gfx950_quantize_f32_noalloc(const float *data, U32 n, DataType qdt, void *q, float *dscale, int mode)
{
    if (qdt != DT_I8 && qdt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    if (!data || !q || !dscale) {
        return NULL_POINTER;
    }
    if (n > BOLT_GFX950_NOALLOC_MAX_ELEMENTS) {
        api_set_error("quantize_f32_noalloc: more than BOLT_GFX950_NOALLOC_MAX_ELEMENTS (2^30) elements", hipSuccess);
        return NOT_SUPPORTED;
    }
    if (((uintptr_t)data & 3) || ((uintptr_t)dscale & 3)) {
        api_set_error("quantize_f32_noalloc: data / dscale must be 4-byte aligned", hipSuccess);
        return NOT_SUPPORTED;
    }
    uint32_t *ws = nullptr;
    EE e = scratch_on_current_device(&ws);
    if (e != SUCCESS) {
        return e;
    }
    hipStream_t st = api_stream();
    // The slots keep the last call's maxima: launch_absmax_f32 clears them first (a fill kernel, not a memset node:
    // safe to record into a graph), then folds max|x| into them; the quantiser reads them and the caller's scale.
    hipError_t he = launch_absmax_f32(data, n, ws, st);
    if (he == hipSuccess) {
        he = launch_quantize_f32(data, n, q, qdt == DT_U8_Q, ws, 0.0f, dscale, mode, dscale, st);
    }
    if (he != hipSuccess) {
        api_set_error("quantize_f32_noalloc launch", he);
        return UNKNOWN;
    }
    return SUCCESS;
}
