// C-ABI entry points, first part: the runtime (per-thread contexts, options, counters, copies, timers), the eleven
// blas_enhance functions, the quantize family, FullyConnected and the forms that keep their scales in device memory.
// The other operator families live in api_conv.hip, api_conv_ext.hip, api_deconv.hip, api_depthwise.hip, api_ops.hip
// (matmul, pooling, concatenation, LSTM cell), api_encoder.hip and api_ptq.hip; api_internal.h holds what they share.
// Argument validation, Bolt's tmp / offsetC / scale conventions, host <-> device staging for the host-pointer mode,
// and dispatch to the kernels. No arithmetic on tensor data happens on the CPU here except the load-time weight pack
// in host-pointer mode.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <chrono>
#include <mutex>
#include <string>
#include <vector>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

namespace {

struct CtxPool {
    std::mutex mu;
    std::vector<Ctx *> idle;
};

CtxPool &ctx_pool()
{
    static CtxPool *p = new CtxPool;  // never destroyed: threads may end after static destructors have run
    return *p;
}

struct CtxLease {
    Ctx *c = nullptr;
    ~CtxLease()
    {
        if (c) {
            CtxPool &p = ctx_pool();
            std::lock_guard<std::mutex> lk(p.mu);
            c->stream = nullptr;
            c->reused = true;
            p.idle.push_back(c);
        }
    }
};

}  // namespace

namespace bgapi {

Ctx &ctx()
{
    thread_local CtxLease lease;
    if (!lease.c) {
        CtxPool &p = ctx_pool();
        std::lock_guard<std::mutex> lk(p.mu);
        if (!p.idle.empty()) {
            lease.c = p.idle.back();
            p.idle.pop_back();
        } else {
            lease.c = new Ctx;
        }
    }
    return *lease.c;
}

// counters behind bolt_gfx950_get_counter
std::atomic<unsigned long long> g_fused_fallbacks{0};

}  // namespace bgapi

namespace bg {

hipStream_t api_stream()
{
    return ctx().stream;
}

void api_set_error(const char *what, hipError_t he)
{
    Ctx &c = ctx();
    c.err = what;
    if (he != hipSuccess) {
        c.err += ": ";
        c.err += hipGetErrorString(he);
    }
}

}  // namespace bg

namespace bgapi {

EE fail(EE code, const char *what, hipError_t he)
{
    bg::api_set_error(what, he);
    return code;
}

}  // namespace bgapi

namespace bgapi {

// 1-bit convolution: 2 = matrix cores with E2M1 operands where the shape has that kernel, else int8 (default);
// 1 = matrix cores with int8 operands; 0 = vector-ALU xor / popcount route
int g_bnn_mfma = 2;
// int8 convolution through the filter-panel kernel: gather from the caller's tensor in place for int32 / fp32 results
// (1, default) or for every result type (2); 0 = always re-lay the input as a padded s8 image first
int g_conv_direct = 1;
// u8 convolution through the filter-panel kernel: 1 = one pass where every workgroup fits the device at once (the
// tensor-wide maximum is agreed on with the accumulators in registers; default), 0 = always two passes
int g_conv_onepass = 1;
// LSTM cell: from this many batch rows on, a weight that carries the GEMM packing goes through the matrix cores
int g_lstm_gemm_rows = 4;
// dynamic quantisation through the public entry points: 1 = one launch that reads the tensor once where
// it fits (default), 0 = always the two-pass form (scratch fill, abs-max, quantise)
int g_quantize_fused = 1;
// encoder layer: 1 = the FullyConnected in front of the GELU also applies the GELU and quantises its result for the
// next FullyConnected, in one launch (where the shape allows; default); 0 = separate kernels, fp32 intermediate kept
int g_encoder_fused = 1;

}  // namespace bgapi

namespace bgapi {

EE ensure_init()
{
    Ctx &c = ctx();
    if (c.ready) {
        if (c.reused) {
            // this context served a thread that has ended; whatever that thread enqueued last must not overlap with
            // this thread's use of the same scratch words (its stream may be gone: wait for the device)
            c.reused = false;
            hipError_t e = hipDeviceSynchronize();
            if (e != hipSuccess) {
                return fail(UNKNOWN, "hipDeviceSynchronize", e);
            }
        }
        return SUCCESS;
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        return fail(NOT_SUPPORTED, "no HIP device available", e);
    }
    if (!c.ws) {
        e = hipMalloc((void **)&c.ws, (kWsWords + 64 + 4 * kWsWords + 2 * kWsWords) * sizeof(uint32_t));
        if (e != hipSuccess) {
            c.ws = nullptr;
            return fail(ALLOC_FAILED, "hipMalloc(scratch words)", e);
        }
    }
    c.enc_ws = c.ws + kWsWords + 64;
    c.conv_ws[0] = c.enc_ws + 4 * kWsWords;
    c.conv_ws[1] = c.conv_ws[0] + kWsWords;
    if (!c.fsync.slots) {
        void *p = nullptr;
        e = hipMalloc(&p, kFusedSyncBytes);
        if (e == hipSuccess) {
            e = hipMemset(p, 0, kFusedSyncBytes);
        }
        if (e != hipSuccess) {
            return fail(ALLOC_FAILED, "hipMalloc(quantiser sync area)", e);
        }
        c.fsync.slots = (unsigned long long *)p;
        c.fsync.release = (unsigned long long *)((uint8_t *)p + kGridSyncMaxBlocks * 8);
    }
    if (!c.hscale) {
        e = hipHostMalloc((void **)&c.hscale, 64, hipHostMallocMapped);
        if (e == hipSuccess) {
            e = hipHostGetDevicePointer((void **)&c.hscale_dev, c.hscale, 0);
        }
        if (e != hipSuccess) {
            c.hscale = nullptr;
            return fail(ALLOC_FAILED, "hipHostMalloc(scale word)", e);
        }
    }
    if (noalloc_init_current_device() != SUCCESS) {
        return UNKNOWN;  // the text is already set
    }
    c.ready = true;
    return SUCCESS;
}

// A scale that a kernel computes and the interface returns through a host pointer: the host arms the pinned
// word with a pattern no scale can have, the kernel's first thread stores the scale there, and the host
// takes it as soon as it shows up -- the rest of the call stays ordered on the stream like every other
// device-pointer call, and no copy command or stream drain sits between two calls. If the word has not
// changed after 2 ms the stream is drained instead (a launch that produced nothing must not hang the caller).
constexpr uint32_t kScaleUnset = 0xffffffffu;

void arm_scale(Ctx &c)
{
    *(volatile uint32_t *)c.hscale = kScaleUnset;
}

EE take_scale(Ctx &c, float *dst, bool *gave_up)
{
    volatile uint32_t *w = (volatile uint32_t *)c.hscale;
    const auto t0 = std::chrono::steady_clock::now();
    uint32_t spins = 0;
    while (*w == kScaleUnset) {
        if ((++spins & 0x3ff) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) {
            HIP_TRY(hipStreamSynchronize(c.stream));
            break;
        }
    }
    const uint32_t bits = *w;
    if (bits == kScaleUnset) {
        return fail(UNKNOWN, "the kernel did not produce a scale");
    }
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
        // NaN: the one-launch quantiser's bounded wait for its grid expired. Every workgroup of that launch then
        // skipped its stores; the caller runs the two-pass form instead (gave_up), or reports it.
        if (gave_up) {
            *gave_up = true;
            return SUCCESS;
        }
        return fail(UNKNOWN, "the quantiser's grid barrier timed out");
    }
    memcpy(dst, &bits, 4);
    return SUCCESS;
}

}  // namespace bgapi

namespace bgapi {

EE get2d(TensorDesc d, DataType *dt, DataFormat *df, U32 *rows, U32 *cols)
{
    if (d.nDims != 2) {
        return NOT_MATCH;
    }
    *dt = d.dt;
    *df = d.df;
    *cols = d.dims[0];
    *rows = d.dims[1];
    return SUCCESS;
}

EE get1d(TensorDesc d, DataType *dt, U32 *len)
{
    if (d.nDims != 1) {
        return NOT_MATCH;
    }
    *dt = d.dt;
    *len = d.dims[0];
    return SUCCESS;
}

// element count of a desc in 64 bits (the reference's tensorNumElements multiplies in 32 bits and wraps)
uint64_t elements64(TensorDesc d)
{
    if (d.nDims == 0) {
        return 0;
    }
    uint64_t r = 1;
    for (U32 i = 0; i < d.nDims && i < DIM_LEN; i++) {
        r *= d.dims[i];
    }
    return r;
}

// Element count for the element-wise operators, whose kernels walk a tensor with 32-bit indices in grid strides: false
// for more than kMaxElementwise elements (a stride added to an index that close to 2^32 would wrap).
bool elementwise_count(TensorDesc d, U32 *n)
{
    const uint64_t e = elements64(d);
    if (e > kMaxElementwise) {
        return false;
    }
    *n = (U32)e;
    return true;
}

uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

bool aligned4(const void *p)
{
    return ((uintptr_t)p & 3) == 0;
}

Epilogue epi_from_scale(const F32 *scale)
{
    Epilogue e;
    memset(&e, 0, sizeof(e));
    if (scale == nullptr) {
        e.mode = EPI_I32;
    } else if (scale[0] < 0) {
        e.mode = EPI_U8;
        e.factor = scale[1];
    } else {
        e.mode = EPI_F32;
        e.factor = 1 / scale[0];
    }
    return e;
}

// ---- host-side weight pack (host-pointer mode, load time) ----------------------------------------
void pack_host(bool mmm, const INT8 *src, size_t sk, size_t sn, U32 K, U32 N, INT8 *dst, I32 *comp)
{
    const U32 Kp = align_up(K, 8), N16 = align_up(N, 16);
    memset(dst, 0, (size_t)N16 * Kp);
    for (U32 n = 0; n < N; ++n) {
        I32 s = 0;
        for (U32 k = 0; k < K; ++k) {
            const INT8 v = src[k * sk + n * sn];
            s += v;
            dst[mmm ? mmm_packed_offset(n, k, Kp) : mvm_packed_offset(n, k, Kp)] = v;
        }
        comp[n] = s * (-128);
    }
}

// bytes of the packed matrix part for an N x K weight
U32 packed_matrix_bytes(U32 N, U32 K)
{
    return align_up(N, 16) * align_up(K, 8);
}

// ---- GEMM core (device pointers) -----------------------------------------------------------------
EE mmm_device(U32 M, U32 N, U32 K, DataFormat adf, const void *A, DataFormat bdf, const void *B, void *tmp,
    DataType cdt, void *C, const F32 *scale)
{
    Ctx &c = ctx();
    const INT8 *Bp = (const INT8 *)B;
    U8 *t = (U8 *)tmp;
    const U32 rhs = packed_matrix_bytes(N, K);
    if (bdf != DF_NKNxKx) {
        // on-the-fly transform into tmp, then tmp advances past the packed matrix so that its
        // first N int32 are the compensation vector the transform just wrote (mmm.cpp:207-219)
        const bool tr = (bdf == DF_TRANSPOSE);
        HIP_TRY(launch_pack_mmm((const int8_t *)B, tr ? 1 : N, tr ? K : 1, K, N, (int8_t *)t, (int32_t *)(t + rhs),
            c.stream));
        Bp = (const INT8 *)t;
        t += rhs;
    }
    if (cdt == DT_I32) {
        scale = nullptr;  // mmm.cpp:222-224
    }
    GemmArgs g;
    memset(&g, 0, sizeof(g));  // every field a kernel may look at, including the ones this caller does not use
    g.A = (const uint8_t *)A;
    g.transA = (adf == DF_TRANSPOSE);
    g.lda = g.transA ? M : K;
    g.Bp = (const int8_t *)Bp;
    g.M = M;
    g.N = N;
    g.K = K;
    g.ob = (const int32_t *)t;
    g.comp = (const int32_t *)(Bp + rhs);
    g.C = C;
    g.epi = epi_from_scale(scale);
    g.add_cin = (g.epi.mode != EPI_U8);
    HIP_TRY(launch_gemm_u8s8(g, c.stream));
    return SUCCESS;
}

EE mvm_device(U32 N, U32 K, DataType mdt, DataFormat mdf, const void *W, const void *x, void *tmp, void *y,
    const F32 *scale)
{
    Ctx &c = ctx();
    Epilogue epi = epi_from_scale(scale);
    if (mdt == DT_U8_Q) {
        // u8 matrix x s8 vector; N = rows of the matrix
        const bool tr = (mdf == DF_TRANSPOSE);
        HIP_TRY(launch_gemv_u8s8((const uint8_t *)W, tr ? 1 : K, tr ? N : 1, (const int8_t *)x, K, N, y, epi,
            c.stream));
        return SUCCESS;
    }
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    const U32 mat = packed_matrix_bytes(N, K);
    if (mdf != DF_NKN32K4) {
        // unpacked: tmp = [compensation N*4][packed matrix], as mvm.cpp:176-182 lays it out
        U8 *t = (U8 *)tmp;
        const bool tr = (mdf == DF_TRANSPOSE);
        HIP_TRY(launch_pack_mvm((const int8_t *)W, tr ? N : 1, tr ? 1 : K, K, N, (int8_t *)(t + (size_t)N * 4),
            (int32_t *)t, c.stream));
        g.W = (const int8_t *)(t + (size_t)N * 4);
        g.comp = (const int32_t *)t;
    } else {
        g.W = (const int8_t *)W;
        g.comp = (const int32_t *)((const U8 *)W + mat);
    }
    g.ldw = align_up(K, 8);
    g.x = (const uint8_t *)x;
    g.K = K;
    g.N = N;
    g.ob = (const int32_t *)tmp;
    g.y = y;
    g.epi = epi;
    g.add_yin = (epi.mode != EPI_U8);
    HIP_TRY(launch_gemv_s8u8(g, c.stream));
    return SUCCESS;
}

U32 out_elem_bytes(const F32 *scale)
{
    return (scale && scale[0] < 0) ? 1 : 4;
}

}  // namespace bgapi

extern "C" {

// ---- runtime -------------------------------------------------------------------------------------
EE bolt_gfx950_init(void)
{
    return ensure_init();
}

EE bolt_gfx950_set_stream(void *stream)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    if (c.stream != (hipStream_t)stream) {
        // the scratch words and the quantiser's sync area are shared by every call: work enqueued on the old stream
        // must not overlap with what the new stream will run
        HIP_TRY(hipStreamSynchronize(c.stream));
        c.stream = (hipStream_t)stream;
    }
    return SUCCESS;
}

EE bolt_gfx950_synchronize(void)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipStreamSynchronize(ctx().stream));
    return SUCCESS;
}

const char *bolt_gfx950_last_error(void)
{
    return ctx().err.c_str();
}

EE bolt_gfx950_set_option(const char *name, int value)
{
    if (!name) {
        return NULL_POINTER;
    }
    if (strcmp(name, "gemm_tile") == 0) {
        gemm_force_tile(value);
        return SUCCESS;
    }
    if (strcmp(name, "bnn_mfma") == 0) {
        if (value < 0 || value > 2) {
            return NOT_MATCH;
        }
        g_bnn_mfma = value;
        return SUCCESS;
    }
    if (strcmp(name, "lstm_gemm_rows") == 0) {
        if (value < 1) {
            return NOT_MATCH;
        }
        g_lstm_gemm_rows = value;
        return SUCCESS;
    }
    if (strcmp(name, "quantize_fused_spin") == 0) {
        // polls of the one-launch quantiser's bounded wait before a workgroup gives up; tests set it to 1 so that the
        // launch gives up and the two-pass form takes over. 0 restores the default (about a second). Per thread.
        if (value < 0) {
            return NOT_MATCH;
        }
        ctx().fsync.spin_limit = value ? (uint32_t)value : kFusedSpinDefault;
        return SUCCESS;
    }
    if (strcmp(name, "encoder_fused") == 0) {
        if (value != 0 && value != 1) {
            return NOT_MATCH;
        }
        g_encoder_fused = value;
        return SUCCESS;
    }
    if (strcmp(name, "quantize_fused") == 0) {
        if (value != 0 && value != 1) {
            return NOT_MATCH;
        }
        g_quantize_fused = value;
        return SUCCESS;
    }
    if (strcmp(name, "conv_direct") == 0) {
        if (value < 0 || value > 2) {
            return NOT_MATCH;
        }
        g_conv_direct = value;
        return SUCCESS;
    }
    if (strcmp(name, "conv_onepass") == 0) {
        if (value != 0 && value != 1) {
            return NOT_MATCH;
        }
        g_conv_onepass = value;
        return SUCCESS;
    }
    if (strcmp(name, "conv_panel") == 0) {
        if (value != 0 && value != 2 && value != 4) {
            return NOT_MATCH;
        }
        conv_force_panel(value);
        return SUCCESS;
    }
    return NOT_FOUND;
}

EE bolt_gfx950_get_counter(const char *name, unsigned long long *value)
{
    if (!name || !value) {
        return NULL_POINTER;
    }
    if (strcmp(name, "quantize_fused_fallbacks") == 0) {
        *value = g_fused_fallbacks.load();
        return SUCCESS;
    }
    return NOT_FOUND;
}

void *bolt_gfx950_malloc(size_t bytes)
{
    if (ensure_init() != SUCCESS) {
        return nullptr;
    }
    void *p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 4) != hipSuccess) {
        return nullptr;
    }
    return p;
}

void bolt_gfx950_free(void *p)
{
    if (p) {
        (void)hipFree(p);
    }
}

EE bolt_gfx950_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx().stream));
    HIP_TRY(hipStreamSynchronize(ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_memcpy_d2d(void *dst, const void *src, size_t bytes)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx().stream));  // ordered on the library's stream
    return SUCCESS;
}

EE bolt_gfx950_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx().stream));
    HIP_TRY(hipStreamSynchronize(ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_timer_start(void)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    if (!c.ev0) {
        HIP_TRY(hipEventCreate(&c.ev0));
        HIP_TRY(hipEventCreate(&c.ev1));
    }
    HIP_TRY(hipEventRecord(c.ev0, c.stream));
    return SUCCESS;
}

EE bolt_gfx950_timer_stop(float *ms)
{
    Ctx &c = ctx();
    if (!c.ev0 || !ms) {
        return fail(NULL_POINTER, "timer_stop without timer_start");
    }
    HIP_TRY(hipEventRecord(c.ev1, c.stream));
    HIP_TRY(hipEventSynchronize(c.ev1));
    HIP_TRY(hipEventElapsedTime(ms, c.ev0, c.ev1));
    return SUCCESS;
}

// ---- axpby ---------------------------------------------------------------------------------------
// y = a * x + b * y (compute/blas_enhance/src/axpby.cpp:24-60). The x86 build supports DT_F32 only.
EE vector_vector_axpby_gfx950(F32 a, TensorDesc xDesc, const void *x, F32 b, TensorDesc yDesc, void *y, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!x || !y) {
        return NULL_POINTER;
    }
    DataType xdt, ydt;
    U32 xn, yn;
    if (get1d(xDesc, &xdt, &xn) != SUCCESS || get1d(yDesc, &ydt, &yn) != SUCCESS || xdt != ydt || xn != yn) {
        return NOT_MATCH;
    }
    if (xdt != DT_F32) {
        return NOT_SUPPORTED;
    }
    if (xn == 0) {
        return SUCCESS;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    if (arch == AMD_GFX950_DEVICE) {
        if (!aligned4(x) || !aligned4(y)) {
            return fail(NOT_SUPPORTED, "device x / y must be 4-byte aligned");
        }
        HIP_TRY(launch_axpby_f32(xn, a, (const float *)x, b, (float *)y, c.stream));
        return SUCCESS;
    }
    Stage st;
    const size_t bytes = (size_t)xn * 4;
    void *dx = st.get(bytes), *dy = st.get(bytes);
    if (!dx || !dy) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dx, x, bytes, hipMemcpyHostToDevice, c.stream));
    HIP_TRY(hipMemcpyAsync(dy, y, bytes, hipMemcpyHostToDevice, c.stream));
    HIP_TRY(launch_axpby_f32(xn, a, (const float *)dx, b, (float *)dy, c.stream));
    HIP_TRY(hipMemcpyAsync(y, dy, bytes, hipMemcpyDeviceToHost, c.stream));
    HIP_TRY(hipStreamSynchronize(c.stream));
    return SUCCESS;
}

// ---- GEMM ----------------------------------------------------------------------------------------
DataFormat matrix_matrix_multiply_rhs_format_gfx950(DataType dt)
{
    (void)dt;
    return DF_NKNxKx;
}

// Sizes follow mmm_avx512_vnni.cpp:22-58 exactly so a caller sized for the x86 path fits.
EE matrix_matrix_multiply_transform_rhs_bytes_gfx950(TensorDesc desc, U32 *bytes, U32 *rhsBytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    DataType dt;
    DataFormat df;
    U32 K, N;
    EE e = get2d(desc, &dt, &df, &K, &N);
    if (e != SUCCESS) {
        return e;
    }
    if (dt != DT_I8 && dt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    if (df == DF_TRANSPOSE) {
        std::swap(K, N);
    }
    U32 matrix = 0, total = 0;
    if (df != DF_NKNxKx) {
        // a weight whose blob does not fit the interface's 32-bit byte count is refused, not wrapped
        const uint64_t m64 = (uint64_t)align_up(N, 16) * align_up(K, 8), t64 = (uint64_t)N * 4 + m64 + 64;
        if (t64 > 0xffffffffull) {
            return NOT_SUPPORTED;
        }
        matrix = (U32)m64;
        total = (U32)t64;
    }
    if (rhsBytes) {
        *rhsBytes = matrix;
    }
    if (bytes) {
        *bytes = total;
    }
    return SUCCESS;
}

EE matrix_matrix_multiply_tmp_bytes_gfx950(TensorDesc matrixADesc, TensorDesc matrixBDesc, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    DataType adt, bdt;
    DataFormat adf, bdf;
    U32 M, K, K2, N;
    EE e = get2d(matrixADesc, &adt, &adf, &M, &K);
    if (e != SUCCESS) {
        return e;
    }
    e = get2d(matrixBDesc, &bdt, &bdf, &K2, &N);
    if (e != SUCCESS) {
        return e;
    }
    if (adf == DF_TRANSPOSE) {
        std::swap(M, K);
    }
    if (bdf == DF_TRANSPOSE) {
        std::swap(K2, N);
    }
    if (adt != DT_U8_Q && adt != DT_I8) {
        return NOT_SUPPORTED;
    }
    e = matrix_matrix_multiply_transform_rhs_bytes_gfx950(matrixBDesc, bytes, nullptr, arch);
    if (e != SUCCESS) {
        return e;
    }
    if (adf == DF_NORMAL) {
        *bytes += 32 * K;
        if (K % 8 != 0) {
            *bytes += align_up(M, 24) * 8;
        }
    } else if (adf == DF_TRANSPOSE) {
        *bytes += align_up(M, 24) * std::min<U32>(4096, align_up(K, 8));
    } else {
        return NOT_SUPPORTED;
    }
    *bytes += N * 4;
    *bytes += 64;
    return SUCCESS;
}

EE matrix_matrix_multiply_transform_rhs_gfx950(TensorDesc desc, const void *src, TensorDesc *descTran, void *dst,
    Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (desc.df == DF_NKNxKx) {
        return SUCCESS;  // already packed: descTran and dst stay untouched (x86/mmm.cpp:135-137)
    }
    if (desc.dt != DT_I8 || (desc.df != DF_NORMAL && desc.df != DF_TRANSPOSE)) {
        return NOT_SUPPORTED;
    }
    if (!src || !dst || !descTran) {
        return NULL_POINTER;
    }
    DataType dt;
    DataFormat df;
    U32 rows, cols;
    EE e = get2d(desc, &dt, &df, &rows, &cols);
    if (e != SUCCESS) {
        return e;
    }
    const bool tr = (df == DF_TRANSPOSE);
    const U32 K = tr ? cols : rows, N = tr ? rows : cols;
    const U32 mat = packed_matrix_bytes(N, K);
    if (arch == AMD_GFX950) {
        pack_host(true, (const INT8 *)src, tr ? 1 : N, tr ? K : 1, K, N, (INT8 *)dst, (I32 *)((U8 *)dst + mat));
    } else {
        e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        if (!aligned4(dst)) {
            return fail(NOT_SUPPORTED, "device dst must be 4-byte aligned");
        }
        HIP_TRY(launch_pack_mmm((const int8_t *)src, tr ? 1 : N, tr ? K : 1, K, N, (int8_t *)dst,
            (int32_t *)((U8 *)dst + mat), ctx().stream));
    }
    *descTran = desc;
    descTran->df = DF_NKNxKx;
    if (tr) {
        std::swap(descTran->dims[0], descTran->dims[1]);
    }
    return SUCCESS;
}

EE matrix_matrix_multiply_gfx950(TensorDesc matrixADesc, const void *matrixA, TensorDesc matrixBDesc,
    const void *matrixB, U32 bytes, void *tmp, TensorDesc matrixCDesc, void *matrixC, const F32 *scale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (bytes != 0 && tmp == nullptr) {
        return NULL_POINTER;
    }
    if (!matrixA || !matrixB || !matrixC) {
        return NULL_POINTER;
    }
    if (tensorNumElements(matrixCDesc) == 0) {
        return SUCCESS;
    }
    DataType adt, bdt, cdt;
    DataFormat adf, bdf, cdf;
    U32 M, K, K2, N, CM, CN;
    if (get2d(matrixADesc, &adt, &adf, &M, &K) != SUCCESS || get2d(matrixBDesc, &bdt, &bdf, &K2, &N) != SUCCESS ||
        get2d(matrixCDesc, &cdt, &cdf, &CM, &CN) != SUCCESS) {
        return NOT_MATCH;
    }
    if (adt != bdt && !(adt == DT_U8_Q && bdt == DT_I8)) {
        return NOT_MATCH;
    }
    if (adf == DF_TRANSPOSE) {
        std::swap(M, K);
    }
    if (bdf == DF_TRANSPOSE) {
        std::swap(K2, N);
    }
    if (M != CM || N != CN || K != K2) {
        return NOT_MATCH;
    }
    if (bdt != DT_I8 || (adf != DF_NORMAL && adf != DF_TRANSPOSE) ||
        (bdf != DF_NORMAL && bdf != DF_TRANSPOSE && bdf != DF_NKNxKx)) {
        return NOT_SUPPORTED;
    }
    if (tmp == nullptr) {
        return NULL_POINTER;  // the first N int32 of tmp carry offsetC (x86/mmm.cpp path)
    }
    U32 need = 0;
    if (bdf != DF_NKNxKx) {
        need = packed_matrix_bytes(N, K);
        if (bytes < need + N * 4) {
            return NOT_MATCH;
        }
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    const F32 *sc = (cdt == DT_I32) ? nullptr : scale;
    if (arch == AMD_GFX950_DEVICE) {
        if (!aligned4(tmp) || !aligned4(matrixC) || !aligned4(matrixB)) {
            return fail(NOT_SUPPORTED, "device tmp / B / C must be 4-byte aligned");
        }
        return mmm_device(M, N, K, adf, matrixA, bdf, matrixB, tmp, cdt, matrixC, sc);
    }
    // host-pointer mode
    Ctx &c = ctx();
    Stage st;
    const size_t aBytes = (size_t)M * K;
    const size_t bBytes = (bdf == DF_NKNxKx) ? (size_t)packed_matrix_bytes(N, K) + (size_t)N * 4 : (size_t)K * N;
    const size_t tBytes = (size_t)need + (size_t)N * 4;
    const size_t cBytes = (size_t)M * N * out_elem_bytes(sc);
    void *dA = st.get(aBytes), *dB = st.get(bBytes), *dT = st.get(tBytes), *dC = st.get(cBytes);
    if (!dA || !dB || !dT || !dC) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dA, matrixA, aBytes, hipMemcpyHostToDevice, c.stream));
    HIP_TRY(hipMemcpyAsync(dB, matrixB, bBytes, hipMemcpyHostToDevice, c.stream));
    if (bdf == DF_NKNxKx) {
        HIP_TRY(hipMemcpyAsync(dT, tmp, (size_t)N * 4, hipMemcpyHostToDevice, c.stream));
    }
    if (out_elem_bytes(sc) == 4) {
        HIP_TRY(hipMemcpyAsync(dC, matrixC, cBytes, hipMemcpyHostToDevice, c.stream));
    }
    e = mmm_device(M, N, K, adf, dA, bdf, dB, dT, cdt, dC, sc);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(matrixC, dC, cBytes, hipMemcpyDeviceToHost, c.stream));
    HIP_TRY(hipStreamSynchronize(c.stream));
    return SUCCESS;
}

// ---- GEMV ----------------------------------------------------------------------------------------
DataFormat matrix_vector_multiply_weight_format_gfx950(DataType dt)
{
    return (dt == DT_U8_Q) ? DF_NK : DF_NKN32K4;  // mvm.cpp:51-77
}

static EE mvm_bytes(TensorDesc matrixDesc, U32 *bytes)
{
    DataType dt;
    DataFormat df;
    U32 row, col;
    EE e = get2d(matrixDesc, &dt, &df, &row, &col);
    if (e != SUCCESS) {
        return e;
    }
    if (df == DF_TRANSPOSE) {
        std::swap(row, col);
    }
    if (dt != DT_I8 && dt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    // x86/mvm.cpp:23-42
    uint64_t b = 0;
    if (dt == DT_I8) {
        b += (uint64_t)row * 4;
    }
    if (dt == DT_U8_Q && col % 32 != 0) {
        b += 32ull * ((uint64_t)row + 1);
    }
    if (df != matrix_vector_multiply_weight_format_gfx950(dt)) {
        b += (uint64_t)align_up(row, 16) * align_up(col, 8);
        b += 32;
    }
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;  // does not fit the interface's 32-bit byte count
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE matrix_vector_multiply_transform_weight_bytes_gfx950(TensorDesc desc, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    return mvm_bytes(desc, bytes);
}

EE matrix_vector_multiply_tmp_bytes_gfx950(TensorDesc matrixDesc, TensorDesc vectorDesc, U32 *bytes, Arch arch)
{
    (void)vectorDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    return mvm_bytes(matrixDesc, bytes);  // x86/mvm.cpp:77-100: same formula
}

EE matrix_vector_multiply_transform_weight_gfx950(TensorDesc desc, const void *src, TensorDesc *descTran, void *dst,
    Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (desc.df == matrix_vector_multiply_weight_format_gfx950(desc.dt)) {
        return SUCCESS;  // x86/mvm.cpp:47-49
    }
    if (desc.dt != DT_I8 || (desc.df != DF_NORMAL && desc.df != DF_TRANSPOSE)) {
        return NOT_SUPPORTED;
    }
    if (!src || !dst || !descTran) {
        return NULL_POINTER;
    }
    DataType dt;
    DataFormat df;
    U32 rows, cols;
    EE e = get2d(desc, &dt, &df, &rows, &cols);
    if (e != SUCCESS) {
        return e;
    }
    const bool tr = (df == DF_TRANSPOSE);
    const U32 N = tr ? cols : rows, K = tr ? rows : cols;
    const U32 mat = packed_matrix_bytes(N, K);
    if (arch == AMD_GFX950) {
        pack_host(false, (const INT8 *)src, tr ? N : 1, tr ? 1 : K, K, N, (INT8 *)dst, (I32 *)((U8 *)dst + mat));
    } else {
        e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        if (!aligned4(dst)) {
            return fail(NOT_SUPPORTED, "device dst must be 4-byte aligned");
        }
        HIP_TRY(launch_pack_mvm((const int8_t *)src, tr ? N : 1, tr ? 1 : K, K, N, (int8_t *)dst,
            (int32_t *)((U8 *)dst + mat), ctx().stream));
    }
    *descTran = desc;
    if (tr) {
        std::swap(descTran->dims[0], descTran->dims[1]);
    }
    descTran->df = DF_NKN32K4;
    return SUCCESS;
}

EE matrix_vector_multiply_gfx950(TensorDesc matrixDesc, const void *matrix, TensorDesc vectorDesc, const void *vector,
    U32 bytes, void *tmp, TensorDesc resultDesc, void *result, const F32 *scale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if ((bytes != 0 && tmp == nullptr) || !matrix || !vector || !result) {
        return NULL_POINTER;
    }
    DataType mdt, vdt, rdt;
    DataFormat mdf;
    U32 row, col, vlen, rlen;
    if (get2d(matrixDesc, &mdt, &mdf, &row, &col) != SUCCESS || get1d(vectorDesc, &vdt, &vlen) != SUCCESS ||
        get1d(resultDesc, &rdt, &rlen) != SUCCESS) {
        return NOT_MATCH;
    }
    if (mdf == DF_TRANSPOSE) {
        std::swap(row, col);
    }
    if (row != rlen || col != vlen) {
        return NOT_MATCH;
    }
    if (mdt == DT_U8_Q && mdf == DF_NK) {
        return NOT_SUPPORTED;  // mvm.cpp:172-175
    }
    if (mdt != DT_I8 && mdt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    if (mdt == DT_I8 && mdf != DF_NORMAL && mdf != DF_TRANSPOSE && mdf != DF_NKN32K4) {
        return NOT_SUPPORTED;
    }
    if (mdt == DT_U8_Q && mdf != DF_NORMAL && mdf != DF_TRANSPOSE) {
        return NOT_SUPPORTED;
    }
    if (row == 0) {
        return SUCCESS;
    }
    const U32 N = row, K = col;
    const bool unpacked = (mdt == DT_I8 && mdf != DF_NKN32K4);
    if (mdt == DT_I8 && tmp == nullptr) {
        return NULL_POINTER;  // CHECK_REQUIREMENT(offsetCBias != nullptr), x86/mvm.cpp:121
    }
    if (unpacked && bytes < N * 4 + packed_matrix_bytes(N, K)) {
        return NOT_MATCH;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    if (arch == AMD_GFX950_DEVICE) {
        if ((mdt == DT_I8 && !aligned4(tmp)) || !aligned4(result) || (mdt == DT_I8 && !aligned4(matrix))) {
            return fail(NOT_SUPPORTED, "device tmp / matrix / result must be 4-byte aligned");
        }
        return mvm_device(N, K, mdt, mdf, matrix, vector, tmp, result, scale);
    }
    Ctx &c = ctx();
    Stage st;
    const size_t wBytes = (mdt == DT_I8 && !unpacked) ? (size_t)packed_matrix_bytes(N, K) + (size_t)N * 4 : (size_t)N * K;
    const size_t tBytes = (size_t)N * 4 + (unpacked ? packed_matrix_bytes(N, K) : 0);
    const size_t yBytes = (size_t)N * out_elem_bytes(scale);
    void *dW = st.get(wBytes), *dX = st.get(K), *dT = st.get(tBytes), *dY = st.get(yBytes);
    if (!dW || !dX || !dT || !dY) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dW, matrix, wBytes, hipMemcpyHostToDevice, c.stream));
    HIP_TRY(hipMemcpyAsync(dX, vector, K, hipMemcpyHostToDevice, c.stream));
    if (mdt == DT_I8 && !unpacked) {
        HIP_TRY(hipMemcpyAsync(dT, tmp, (size_t)N * 4, hipMemcpyHostToDevice, c.stream));
    }
    if (out_elem_bytes(scale) == 4) {
        HIP_TRY(hipMemcpyAsync(dY, result, yBytes, hipMemcpyHostToDevice, c.stream));
    }
    e = mvm_device(N, K, mdt, mdf, dW, dX, dT, dY, scale);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(result, dY, yBytes, hipMemcpyDeviceToHost, c.stream));
    HIP_TRY(hipStreamSynchronize(c.stream));
    return SUCCESS;
}

// ---- quantize family -----------------------------------------------------------------------------
EE quantize_gfx950(TensorDesc dDesc, const void *data, TensorDesc *qDesc, void *qData, F32 *scale, int mode, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!qDesc) {
        return NULL_POINTER;
    }
    const DataType ddt = dDesc.dt, qdt = qDesc->dt;
    const bool f32in = (ddt == DT_F32 || ddt == DT_F32_8Q);
    const bool ok = (f32in && (qdt == DT_I8 || qdt == DT_U8_Q)) || (ddt == DT_U8_Q && qdt == DT_I8) ||
        (ddt == DT_I32 && (qdt == DT_I8 || qdt == DT_U8_Q));
    if (!ok) {
        return NOT_SUPPORTED;
    }
    const bool needs_scale = !(ddt == DT_U8_Q);
    if (needs_scale && scale == nullptr) {
        return NOT_MATCH;  // avx512/quantize.cpp:123-125
    }
    U32 n;
    if (!elementwise_count(dDesc, &n)) {
        return NOT_SUPPORTED;
    }
    if (n != 0 && (!data || !qData)) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const void *dIn = data;
    void *dOut = qData;
    const size_t inBytes = (size_t)n * bytesOf(ddt);
    if (arch == AMD_GFX950) {
        void *a = st.get(inBytes), *b = st.get(n);
        if (!a || !b) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, data, inBytes, hipMemcpyHostToDevice, c.stream));
        dIn = a;
        dOut = b;
    } else if (!aligned4(data) && ddt != DT_U8_Q) {
        return fail(NOT_SUPPORTED, "device data must be 4-byte aligned");
    }
    // Only a call that returns a freshly computed scale lets its kernel write the pinned word (and waits for it
    // below). A static-scale kernel that wrote it too would do so at some later time, without the host waiting,
    // and could land its value after the NEXT call has armed the word.
    const bool f32dyn = f32in && (!mode || *scale <= 0);
    const bool i32dyn = (ddt == DT_I32) && (scale[0] < 0 && scale[1] > 0);
    const bool read_back = f32dyn || i32dyn;
    const F32 s0 = scale ? scale[0] : 0.0f, s1 = (ddt == DT_I32) ? scale[1] : 0.0f;
    // attempt 0 may be the one-launch form; if its bounded wait for the grid gives up (another stream held the CUs)
    // every workgroup has skipped its stores and attempt 1 runs the two-pass form on the same stream
    for (int attempt = 0; attempt < 2; ++attempt) {
        float *dscale = nullptr;
        if (read_back) {
            arm_scale(c);
            dscale = c.hscale_dev;
        }
        bool fused = false;
        if (f32in) {
            if (f32dyn && g_quantize_fused && attempt == 0) {  // one launch, one read, where the tensor fits a resident grid's registers
                HIP_TRY(launch_quantize_fused(dIn, n, dOut, 0, qdt == DT_U8_Q, c.fsync, s0, dscale, c.stream, &fused));
            }
            if (!fused) {
                if (f32dyn) {
                    HIP_TRY(launch_absmax_f32((const float *)dIn, n, c.ws, c.stream));
                }
                HIP_TRY(launch_quantize_f32((const float *)dIn, n, dOut, qdt == DT_U8_Q, c.ws, s0, nullptr, mode, dscale,
                    c.stream));
            }
        } else if (ddt == DT_U8_Q) {
            HIP_TRY(launch_u8_to_i8((const uint8_t *)dIn, n, (int8_t *)dOut, c.stream));
        } else {
            if (i32dyn && g_quantize_fused && attempt == 0) {
                HIP_TRY(launch_quantize_fused(dIn, n, dOut, 1, qdt == DT_U8_Q, c.fsync, s1, dscale, c.stream, &fused));
            }
            if (!fused) {
                if (i32dyn) {
                    HIP_TRY(launch_absmax_i32((const int32_t *)dIn, n, c.ws, c.stream));
                }
                HIP_TRY(launch_requant_i32((const int32_t *)dIn, n, dOut, qdt == DT_U8_Q, c.ws, s0, s1, dscale, c.stream));
            }
        }
        if (!read_back) {
            break;
        }
        // the scale is a host value in this interface: the call completes before returning it
        bool gave_up = false;
        EE te = take_scale(c, scale, fused ? &gave_up : nullptr);
        if (te != SUCCESS) {
            return te;
        }
        if (!gave_up) {
            break;
        }
        g_fused_fallbacks.fetch_add(1);
    }
    if (arch == AMD_GFX950 && n) {
        HIP_TRY(hipMemcpyAsync(qData, dOut, n, hipMemcpyDeviceToHost, c.stream));
    }
    if (arch == AMD_GFX950) {
        HIP_TRY(hipStreamSynchronize(c.stream));  // host-pointer mode: the copy of the result must have landed
    }
    return SUCCESS;
}

EE dequantize_gfx950(TensorDesc qDesc, void *qData, const F32 *scale, TensorDesc bDesc, void *bData, TensorDesc dDesc,
    void *dData, Arch arch)
{
    (void)bDesc;
    (void)bData;  // the x86 path ignores the bias argument (cpu/x86/dequantize.cpp:19-48)
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (dDesc.dt != DT_F32 || (qDesc.dt != DT_I32 && qDesc.dt != DT_U8_Q)) {
        return NOT_SUPPORTED;
    }
    if (!scale) {
        return NULL_POINTER;
    }
    U32 n;
    if (!elementwise_count(dDesc, &n)) {
        return NOT_SUPPORTED;
    }
    if (n == 0) {
        return SUCCESS;
    }
    if (!qData || !dData) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const void *dIn = qData;
    void *dOut = dData;
    const size_t inBytes = (size_t)n * bytesOf(qDesc.dt);
    if (arch == AMD_GFX950) {
        void *a = st.get(inBytes), *b = st.get((size_t)n * 4);
        if (!a || !b) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, qData, inBytes, hipMemcpyHostToDevice, c.stream));
        dIn = a;
        dOut = b;
    }
    if (qDesc.dt == DT_I32) {
        HIP_TRY(launch_dequant_i32((const int32_t *)dIn, n, nullptr, *scale, (float *)dOut, c.stream));
    } else {
        HIP_TRY(launch_dequant_u8((const uint8_t *)dIn, n, nullptr, *scale, (float *)dOut, c.stream));
    }
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(dData, dOut, (size_t)n * 4, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

static bool native_filter_format(DataFormat df)
{
    return df == DF_NCHW || df == DF_NHWC || df == DF_MTK || df == DF_NORMAL || df == DF_TRANSPOSE;
}

EE quantize_bias_offsetC_gfx950(const void *bias, TensorDesc biasDesc, DataType qType, const void *filter,
    TensorDesc filterDesc, const F32 *scale, void *offsetCBias, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (qType != DT_I32 || (bias && biasDesc.dt != DT_F32 && biasDesc.dt != DT_I32)) {
        return NOT_SUPPORTED;
    }
    if (!bias && !filter) {
        return SUCCESS;  // avx512/quantize.cpp:246-248
    }
    if (!offsetCBias) {
        return NULL_POINTER;
    }
    U32 N = bias ? tensorNumElements(biasDesc) : 0;
    const bool no_bias = (!bias || N == 0);
    if (no_bias) {
        N = std::max(filterDesc.dims[0], filterDesc.dims[1]);
    }
    // `filter` points at the compensation vector of a packed blob; native formats carry none
    const bool add_off = filter && !native_filter_format(filterDesc.df);
    if (!no_bias && biasDesc.dt == DT_F32 && !scale) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const void *dBias = no_bias ? nullptr : bias;
    const void *dOff = add_off ? filter : nullptr;
    void *dOut = offsetCBias;
    if (arch == AMD_GFX950) {
        dOut = st.get((size_t)N * 4);
        if (dBias) {
            void *b = st.get((size_t)N * 4);
            HIP_TRY(hipMemcpyAsync(b, bias, (size_t)N * 4, hipMemcpyHostToDevice, c.stream));
            dBias = b;
        }
        if (dOff) {
            void *o = st.get((size_t)N * 4);
            HIP_TRY(hipMemcpyAsync(o, filter, (size_t)N * 4, hipMemcpyHostToDevice, c.stream));
            dOff = o;
        }
    }
    if (!no_bias && biasDesc.dt == DT_I32) {
        // integer bias (cpu/x86/quantize.cpp:100-110) has no caller on the int8 FullyConnected /
        // Convolution path
        return fail(NOT_SUPPORTED, "DT_I32 bias is not supported");
    }
    HIP_TRY(launch_bias_offsetC((const float *)dBias, N, (const int32_t *)dOff, nullptr, scale ? scale[0] : 1.0f,
        (int32_t *)dOut, c.stream));
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(offsetCBias, dOut, (size_t)N * 4, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

EE requantize_gfx950(TensorDesc inputDesc, INT8 *input, F32 inputScale, TensorDesc outputDesc, INT8 *output,
    F32 outputScale, Arch arch)
{
    (void)inputDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    U32 n;
    if (!elementwise_count(outputDesc, &n)) {
        return NOT_SUPPORTED;
    }
    if (n == 0) {
        return SUCCESS;
    }
    if (!input || !output) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    if (arch == AMD_GFX950) {
        if (outputScale == inputScale) {
            memcpy(output, input, n);
            return SUCCESS;
        }
        Stage st;
        void *a = st.get(n), *b = st.get(n);
        if (!a || !b) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, input, n, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(launch_requantize_i8((const int8_t *)a, n, outputScale / inputScale, (int8_t *)b, c.stream));
        HIP_TRY(hipMemcpyAsync(output, b, n, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
        return SUCCESS;
    }
    if (outputScale == inputScale) {
        HIP_TRY(hipMemcpyAsync(output, input, n, hipMemcpyDeviceToDevice, c.stream));
        return SUCCESS;
    }
    HIP_TRY(launch_requantize_i8(input, n, outputScale / inputScale, output, c.stream));
    return SUCCESS;
}

// ---- int8 FullyConnected (x86 branch of compute/tensor/src/fully_connected.cpp:372-495) ------------
// false: a tensor of 2^32 elements or more, which the interface's 32-bit sizes cannot describe
static bool fc_dims(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, U32 *M, U32 *K, U32 *N)
{
    const uint64_t in = elements64(inputDesc), fl = elements64(filterDesc), out = elements64(outputDesc);
    if (in > 0xffffffffull || fl > 0xffffffffull || out > 0xffffffffull) {
        return false;
    }
    *N = outputDesc.dims[0];                       // fw, fully_connected.cpp:370
    *K = (*N) ? (U32)(fl / (*N)) : 0;              // fh
    *M = (*K) ? (U32)(in / (*K)) : 0;
    return true;
}

EE fully_connected_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    if (filterDesc.nDims != 2) {
        return NOT_MATCH;
    }
    U32 M, K, N;
    if (!fc_dims(inputDesc, filterDesc, outputDesc, &M, &K, &N)) {
        return NOT_SUPPORTED;
    }
    EE e;
    if (M != 1) {
        e = matrix_matrix_multiply_tmp_bytes_gfx950(tensor2df(inputDesc.dt, DF_NORMAL, M, K), filterDesc, bytes, arch);
    } else {
        e = matrix_vector_multiply_tmp_bytes_gfx950(filterDesc, tensor1d(inputDesc.dt, K), bytes, arch);
    }
    if (e != SUCCESS) {
        return e;
    }
    if (filterDesc.dt == DT_I8) {  // fully_connected.cpp:149-156
        // the reference sums these in 32 bits and wraps; a tmp that size would be overrun, so a shape whose tmp does
        // not fit the interface's 32-bit byte count is refused
        uint64_t total = *bytes;
        if (inputDesc.dt != DT_I8) {
            total += (uint64_t)M * K * bytesOf(inputDesc.dt);
        }
        total += (uint64_t)N * 4;
        total += (uint64_t)M * N * 4;
        if (total > 0xffffffffull) {
            return NOT_SUPPORTED;
        }
        *bytes = (U32)total;
    }
    return SUCCESS;
}

// all pointers are device pointers here
static EE fc_device(U32 M, U32 K, U32 N, const void *input, F32 scaleI, DataFormat fdf, const void *filter, F32 scaleW,
    const void *bias, void *tmp, DataType odt, void *output, F32 *outputScale)
{
    Ctx &c = ctx();
    F32 scaleO = scaleI * scaleW;  // :396
    F32 sarr[2] = {-1, -1};
    const F32 *scale = nullptr;
    DataType cdt = odt;
    if (odt == DT_F32) {
        scale = &scaleO;  // :381-382
    } else if (odt == DT_U8_Q) {
        if (*outputScale > 0) {
            sarr[1] = *outputScale / scaleO;  // :383-387, :408-410
            scale = sarr;
        } else {
            cdt = DT_I32;  // :388
        }
    }
    U8 *t = (U8 *)tmp;
    void *dst = output;
    if (cdt != odt) {
        dst = t;  // int32 result parked at the head of tmp, offsetC behind it (:400-403, :432-436)
        t += (size_t)M * N * 4;
    }
    const U32 mat = packed_matrix_bytes(N, K);
    const bool packed = (fdf == DF_NKNxKx || fdf == DF_NKN32K4);
    // :404-406 -- round(bias * scaleO) is added to the compensation vector behind the packed matrix; the kernels do
    // that fold themselves for the columns they own (same arithmetic as quantize_bias_offsetC), so there is no
    // separate launch and nothing is parked in tmp
    if (!packed) {
        return fail(NOT_SUPPORTED, "FullyConnected expects a pre-packed filter (transform_filter)");
    }
    const int32_t *fcomp = (const int32_t *)((const U8 *)filter + mat);
    // the reference zeroes the result (:458) and the product accumulates into it; starting the
    // accumulation from zero without reading the buffer is the same result
    EE e;
    if (M == 1 && fdf != DF_NKNxKx) {  // :461-469
        if (fdf != DF_NKN32K4) {
            return fail(NOT_SUPPORTED, "FullyConnected expects a pre-packed filter (transform_filter)");
        }
        GemvArgs g;
        memset(&g, 0, sizeof(g));
        g.W = (const int8_t *)filter;
        g.ldw = align_up(K, 8);
        g.x = (const uint8_t *)input;
        g.K = K;
        g.N = N;
        g.ob = fcomp;
        g.comp = fcomp;
        g.fold_bias = (const float *)bias;
        g.fold_scale = scaleO;
        g.y = dst;
        g.epi = epi_from_scale(cdt == DT_I32 ? nullptr : scale);
        HIP_TRY(launch_gemv_s8u8(g, c.stream));
    } else {
        if (fdf != DF_NKNxKx) {
            return fail(NOT_SUPPORTED, "FullyConnected expects a pre-packed filter (transform_filter)");
        }
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = (const uint8_t *)input;
        g.lda = K;
        g.Bp = (const int8_t *)filter;
        g.M = M;
        g.N = N;
        g.K = K;
        g.ob = fcomp;
        g.comp = fcomp;
        g.fold_bias = (const float *)bias;
        g.fold_scale = scaleO;
        g.C = dst;
        g.epi = epi_from_scale(cdt == DT_I32 ? nullptr : scale);
        HIP_TRY(launch_gemm_u8s8(g, c.stream));
    }
    e = SUCCESS;
    if (cdt != odt) {  // :477-486 -- dynamic requantisation of the int32 result
        arm_scale(c);
        HIP_TRY(launch_absmax_i32((const int32_t *)dst, M * N, c.ws, c.stream));
        HIP_TRY(launch_requant_i32((const int32_t *)dst, M * N, output, 1, c.ws, *outputScale, scaleO, c.hscale_dev,
            c.stream));
        EE te = take_scale(c, outputScale);  // the output scale is a host value in this interface
        if (te != SUCCESS) {
            return te;
        }
    } else if (odt == DT_F32 || odt == DT_I32) {
        *outputScale = scaleO;
    }
    return e;
}

EE fully_connected_gfx950(TensorDesc inputDesc, const void *input, F32 inputScale, TensorDesc filterDesc,
    const void *filter, F32 filterScale, TensorDesc biasDesc, const void *bias, U32 tmpBytes, void *tmp,
    TensorDesc outputDesc, void *output, F32 *outputScale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !outputScale) {
        return NULL_POINTER;
    }
    if (filterDesc.nDims != 2) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_I8) {
        return NOT_SUPPORTED;
    }
    if (inputDesc.dt != DT_U8_Q) {
        return NOT_MATCH;  // CHECK_REQUIREMENT(idt == qIDesc.dt), fully_connected.cpp:395
    }
    const DataType odt = outputDesc.dt;
    if (odt != DT_F32 && odt != DT_U8_Q && odt != DT_I32) {
        return NOT_SUPPORTED;
    }
    U32 M, K, N;
    if (!fc_dims(inputDesc, filterDesc, outputDesc, &M, &K, &N)) {
        return NOT_SUPPORTED;
    }
    if (M == 0 || N == 0 || K == 0) {
        return NOT_MATCH;
    }
    if (bias) {
        if (biasDesc.nDims != 1 || biasDesc.dims[0] != N) {
            return NOT_MATCH;  // fully_connected.cpp:444-446
        }
    }
    U32 need = 0;
    EE e = fully_connected_infer_forward_tmp_bytes_gfx950(inputDesc, filterDesc, outputDesc, &need, arch);
    if (e != SUCCESS) {
        return e;
    }
    if (!tmp || tmpBytes < N * 4 + ((odt == DT_U8_Q && *outputScale <= 0) ? M * N * 4 : 0)) {
        return tmp ? NOT_MATCH : NULL_POINTER;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    if (arch == AMD_GFX950_DEVICE) {
        if (!aligned4(tmp) || !aligned4(output) || !aligned4(filter)) {
            return fail(NOT_SUPPORTED, "device tmp / filter / output must be 4-byte aligned");
        }
        return fc_device(M, K, N, input, inputScale, filterDesc.df, filter, filterScale, bias, tmp, odt, output,
            outputScale);
    }
    Ctx &c = ctx();
    Stage st;
    const size_t inB = (size_t)M * K, fB = (size_t)packed_matrix_bytes(N, K) + (size_t)N * 4;
    const size_t outB = (size_t)M * N * (odt == DT_U8_Q ? 1 : 4);
    const size_t tB = (size_t)M * N * 4 + (size_t)N * 4 + 256;
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = bias ? st.get((size_t)N * 4) : nullptr, *dT = st.get(tB),
         *dO = st.get(outB);
    if (!dIn || !dF || !dT || !dO || (bias && !dB)) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, input, inB, hipMemcpyHostToDevice, c.stream));
    HIP_TRY(hipMemcpyAsync(dF, filter, fB, hipMemcpyHostToDevice, c.stream));
    if (bias) {
        HIP_TRY(hipMemcpyAsync(dB, bias, (size_t)N * 4, hipMemcpyHostToDevice, c.stream));
    }
    e = fc_device(M, K, N, dIn, inputScale, filterDesc.df, dF, filterScale, dB, dT, odt, dO, outputScale);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(output, dO, outB, hipMemcpyDeviceToHost, c.stream));
    HIP_TRY(hipStreamSynchronize(c.stream));
    return SUCCESS;
}

// ---- device-resident-scale forms ------------------------------------------------------------------
EE bolt_gfx950_quantize_f32_async(const float *data, U32 n, DataType qdt, void *q, float *dscale, int mode)
{
    if (qdt != DT_I8 && qdt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    if (!data || !q || !dscale) {
        return NULL_POINTER;
    }
    if (n > kMaxElementwise) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    // the caller's scale lives on the device, so whether it asks for a dynamic scale is only known
    // there: the |max| pass always runs.
    HIP_TRY(launch_absmax_f32(data, n, c.ws, c.stream));
    HIP_TRY(launch_quantize_f32(data, n, q, qdt == DT_U8_Q, c.ws, 0.0f, dscale, mode, dscale, c.stream));
    return SUCCESS;
}

EE bolt_gfx950_mmm_int8_perchannel(U32 M, U32 N, U32 K, const void *A, const void *packedB, const I32 *offsetC,
    float *C, const float *dscaleI, const float *scaleW, const float *bias)
{
    if (!A || !packedB || !offsetC || !C || !dscaleI || !scaleW) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = (const uint8_t *)A;
    g.lda = K;
    g.Bp = (const int8_t *)packedB;
    g.M = M;
    g.N = N;
    g.K = K;
    g.ob = offsetC;
    g.comp = (const int32_t *)((const U8 *)packedB + packed_matrix_bytes(N, K));
    g.C = C;
    g.epi.mode = EPI_F32_CH;
    g.epi.scaleI = dscaleI;
    g.epi.scaleW = scaleW;
    g.epi.bias = bias;
    HIP_TRY(launch_gemm_u8s8(g, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_mmm_int8_perchannel_u8(U32 M, U32 N, U32 K, const void *A, const void *packedB, const I32 *offsetC,
    void *C, const float *dscaleI, const float *scaleW, const float *bias, F32 outputScale)
{
    if (!A || !packedB || !offsetC || !C || !dscaleI || !scaleW) {
        return NULL_POINTER;
    }
    if (!(outputScale > 0)) {
        return fail(NOT_MATCH, "the output scale must be positive (this epilogue is the static form)");
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = (const uint8_t *)A;
    g.lda = K;
    g.Bp = (const int8_t *)packedB;
    g.M = M;
    g.N = N;
    g.K = K;
    g.ob = offsetC;
    g.comp = (const int32_t *)((const U8 *)packedB + packed_matrix_bytes(N, K));
    g.C = C;
    g.epi.mode = EPI_U8_CH;
    g.epi.scaleI = dscaleI;
    g.epi.scaleW = scaleW;
    g.epi.bias = bias;
    g.epi.factor = outputScale;
    HIP_TRY(launch_gemm_u8s8(g, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_mvm_int8_perchannel(U32 N, U32 K, const void *packedW, const void *x, const I32 *offsetC, float *y,
    const float *dscaleI, const float *scaleW, const float *bias)
{
    if (!packedW || !x || !offsetC || !y || !dscaleI || !scaleW) {
        return NULL_POINTER;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.W = (const int8_t *)packedW;
    g.ldw = align_up(K, 8);
    g.x = (const uint8_t *)x;
    g.K = K;
    g.N = N;
    g.ob = offsetC;
    g.comp = (const int32_t *)((const U8 *)packedW + packed_matrix_bytes(N, K));
    g.y = y;
    g.epi.mode = EPI_F32_CH;
    g.epi.scaleI = dscaleI;
    g.epi.scaleW = scaleW;
    g.epi.bias = bias;
    HIP_TRY(launch_gemv_s8u8(g, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_mvm_int8_strided_batch(U32 batch, U32 N, U32 K, const void *packedW, size_t weightStride,
    U32 weightCopies, const void *x, float *y, const float *dscaleI, const float *scaleW, const float *bias)
{
    if (!packedW || !x || !y || !dscaleI || !scaleW) {
        return NULL_POINTER;
    }
    if (batch == 0 || N == 0) {
        return SUCCESS;
    }
    const size_t blob = (size_t)packed_matrix_bytes(N, K) + (size_t)N * 4;
    if (weightCopies == 0 || batch > 65535 || (weightCopies > 1 && (weightStride < blob || (weightStride & 3)))) {
        return NOT_MATCH;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.W = (const int8_t *)packedW;
    g.ldw = align_up(K, 8);
    g.x = (const uint8_t *)x;
    g.K = K;
    g.N = N;
    g.comp = (const int32_t *)((const U8 *)packedW + packed_matrix_bytes(N, K));
    g.ob = g.comp;  // no folded bias: offsetC is each blob's own compensation vector
    g.y = y;
    g.epi.mode = EPI_F32_CH;
    g.epi.scaleI = dscaleI;
    g.epi.scaleW = scaleW;
    g.epi.bias = bias;
    g.batch.count = batch;
    g.batch.wcopies = weightCopies;
    g.batch.wstride = weightStride;
    g.batch.xstride = K;
    g.batch.ystride = N * 4;
    g.batch.ob_in_blob = 1;
    HIP_TRY(launch_gemv_s8u8(g, ctx().stream));
    return SUCCESS;
}

}  // extern "C"
