// C-ABI entry points: argument validation, Bolt's tmp / offsetC / scale conventions, host <-> device
// staging for the host-pointer mode, and dispatch to the kernels. No arithmetic on tensor data
// happens on the CPU here except the load-time weight pack in host-pointer mode.
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

namespace {

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

}  // namespace

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

namespace {

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

}  // namespace

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
        matrix = packed_matrix_bytes(N, K);
        total = N * 4 + matrix + 64;
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
    *bytes = 0;
    if (dt == DT_I8) {
        *bytes += row * 4;
    }
    if (dt == DT_U8_Q && col % 32 != 0) {
        *bytes += 32 * (row + 1);
    }
    if (df != matrix_vector_multiply_weight_format_gfx950(dt)) {
        *bytes += align_up(row, 16) * align_up(col, 8);
        *bytes += 32;
    }
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
    const U32 n = tensorNumElements(dDesc);
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
    const U32 n = tensorNumElements(dDesc);
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
    const U32 n = tensorNumElements(outputDesc);
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
static void fc_dims(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, U32 *M, U32 *K, U32 *N)
{
    *N = outputDesc.dims[0];                                     // fw, fully_connected.cpp:370
    *K = (*N) ? tensorNumElements(filterDesc) / (*N) : 0;        // fh
    *M = (*K) ? tensorNumElements(inputDesc) / (*K) : 0;
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
    fc_dims(inputDesc, filterDesc, outputDesc, &M, &K, &N);
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
        if (inputDesc.dt != DT_I8) {
            *bytes += tensorNumBytes(inputDesc);
        }
        *bytes += N * 4;
        *bytes += tensorNumElements(outputDesc) * 4;
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
    fc_dims(inputDesc, filterDesc, outputDesc, &M, &K, &N);
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

// ---- int8 convolution (compute/tensor/src/cpu/x86/int8/convolution.cpp:97-150) ---------------------
extern "C++" {
namespace bgapi {

EE get4d(TensorDesc d, U32 *n, U32 *c, U32 *h, U32 *w)
{
    if (d.nDims != 4) {
        return NOT_MATCH;
    }
    *w = d.dims[0];
    *h = d.dims[1];
    *c = d.dims[2];
    *n = d.dims[3];
    return SUCCESS;
}

EE conv_shape(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, const ConvolutionParamSpec &p,
    ConvShape *s)
{
    U32 on, fc;
    if (get4d(inputDesc, &s->n, &s->ic, &s->ih, &s->iw) != SUCCESS || get4d(filterDesc, &s->oc, &fc, &s->fh, &s->fw) != SUCCESS ||
        get4d(outputDesc, &on, &s->oc, &s->oh, &s->ow) != SUCCESS) {
        return NOT_MATCH;
    }
    if (p.group != 1) {
        return NOT_SUPPORTED;  // depthwise / grouped int8 convolution is a different reference kernel
    }
    // a transformed filter's desc carries the channel count rounded up to 16 (convolution_transform.cpp:70-87)
    if ((fc != s->ic && fc != align_up(s->ic, 16)) || on != s->n || s->ic % 8 != 0 || s->oc % 8 != 0) {
        return NOT_MATCH;
    }
    s->sh = p.stride_h;
    s->sw = p.stride_w;
    s->pt = p.pad_top;
    s->pb = p.pad_bottom;
    s->pl = p.pad_left;
    s->pr = p.pad_right;
    s->dh = p.dilatedRate_h ? p.dilatedRate_h : 1;
    s->dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (s->sh == 0 || s->sw == 0) {
        return NOT_MATCH;
    }
    s->Hp = s->ih + s->pt + s->pb;
    s->Wp = s->iw + s->pl + s->pr;
    s->ICp = align_up(s->ic, 16);
    s->Kp = align_up(s->fh * s->fw * s->ICp, 64);
    s->N16 = align_up(s->oc, 16);
    const U32 eh = (s->fh - 1) * s->dh + 1, ew = (s->fw - 1) * s->dw + 1;
    if (s->Hp < eh || s->Wp < ew || (s->Hp - eh) / s->sh + 1 < s->oh || (s->Wp - ew) / s->sw + 1 < s->ow) {
        return NOT_MATCH;  // the output must fit the padded input (every gather stays inside it)
    }
    return SUCCESS;
}

size_t conv_padded_bytes(const ConvShape &s)
{
    return ((size_t)s.n * s.Hp * s.Wp * s.ICp + 255) / 256 * 256;
}

// tmp = [padded s8 image][offsetC + folded bias, oc int32]
size_t conv_tmp_layout(const ConvShape &s, size_t *off)
{
    size_t b = (conv_padded_bytes(s) + 255) / 256 * 256;
    *off = b;
    b += (size_t)s.oc * 4;
    return b + 32;
}

void conv_pack_filter_host(const INT8 *src, const ConvShape &s, I32 *offsetC, INT8 *dst)
{
    const U32 fhw = s.fh * s.fw;
    memset(dst, 0, (size_t)s.N16 * s.Kp);
    for (U32 n = 0; n < s.oc; ++n) {
        I32 sum = 0;
        for (U32 c = 0; c < s.ic; ++c) {
            for (U32 t = 0; t < fhw; ++t) {
                const INT8 v = src[((size_t)n * s.ic + c) * fhw + t];
                sum += v;
                dst[mmm_packed_offset(n, t * s.ICp + c, s.Kp)] = v;
            }
        }
        offsetC[n] = -128 * sum;
    }
}

// all pointers device
EE conv_device(const ConvShape &s, DataFormat idf, const void *input, const void *eltwise, const void *filter,
    const void *bias, void *tmp, DataType odt, DataFormat odf, void *output, F32 *scale, int relu)
{
    Ctx &c = ctx();
    size_t offOff;
    conv_tmp_layout(s, &offOff);
    U8 *t = (U8 *)tmp;
    const F32 scaleO = scale[0] * scale[2];  // convolution_direct.cpp:2687
    // The filter-panel kernel (few output channels, short K) gathers from the caller's tensor itself when the channel
    // count is a multiple of 16; every other shape first re-lays the input as a zero-padded s8 image in tmp. The
    // in-place gather costs the kernel about as much as half a padding pass (bounds tests, and two 8-byte loads per
    // fragment from NCHWC8), so by default (1) it is taken where the convolution runs once -- int32 and fp32
    // results -- and not for u8 results, whose two passes share one padded image; 2 takes it always.
    const bool gather_ok = conv_panel_ok(s.oc, s.Kp) && s.ic % 16 == 0 && (((uintptr_t)input) & 15) == 0;
    // u8 result in ONE pass of the filter-panel kernel when all its workgroups are resident at once: they agree on
    // max|acc| with the accumulators still in registers and requantise from there. The convolution then runs once,
    // so it also gathers from the caller's tensor in place where it can.
    const uint32_t M_pix = s.n * s.oh * s.ow;
    bool onepass = odt == DT_U8_Q && g_conv_onepass && conv_panel_ok(s.oc, s.Kp) &&
        conv_panel_grid(M_pix) <= conv_onepass_max_grid(s.Kp);
    const bool direct = g_conv_direct && (g_conv_direct == 2 || odt != DT_U8_Q || onepass) && gather_ok;
    if (!direct) {
        HIP_TRY(launch_conv_pad((const uint8_t *)input, s.n, s.ic, s.ih, s.iw, idf == DF_NCHWC16 ? 16 : 8, s.pt, s.pb, s.pl,
            s.pr, (int8_t *)t, c.stream, odt == DT_U8_Q ? c.ws : nullptr));  // u8 results: also clears the max slots
    }
    // filter blob = [offsetC oc*4][packed matrix] (convolution_transform.cpp:36-44 keeps the vector in front)
    const int32_t *offC = (const int32_t *)filter;
    const int8_t *mat = (const int8_t *)filter + (size_t)s.oc * 4;
    // offsetC + round(bias * scaleO) (convolution_direct.cpp:2687-2700) is formed inside the kernel for the columns
    // it owns: no separate launch
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = direct ? (const uint8_t *)input : (const uint8_t *)t;
    if (direct) {
        g.conv.in_c = idf == DF_NCHWC16 ? 16 : 8;
        g.conv.H = s.ih;
        g.conv.W = s.iw;
        g.conv.IC = s.ic;
        g.conv.pt = s.pt;
        g.conv.pl = s.pl;
    }
    g.Bp = mat;
    g.M = s.n * s.oh * s.ow;
    g.N = s.oc;
    g.K = s.Kp;
    g.ob = offC;
    g.comp = offC;
    g.fold_bias = (const float *)bias;
    g.fold_scale = scaleO;
    g.conv.OHW = s.oh * s.ow;
    g.conv.OW = s.ow;
    g.conv.sh = s.sh;
    g.conv.sw = s.sw;
    g.conv.Hp = s.Hp;
    g.conv.Wp = s.Wp;
    g.conv.ICp = s.ICp;
    g.conv.fh = s.fh;
    g.conv.fw = s.fw;
    g.conv.dh = s.dh;
    g.conv.dw = s.dw;
    g.conv.out_c = (odf == DF_NCHWC8) ? 8 : 16;
    g.conv.relu = relu;
    if (odt == DT_F32) {
        g.C = output;
        g.epi.mode = EPI_F32;
        g.epi.factor = 1 / scaleO;  // :2700-2703
        g.conv.eltwise = (const float *)eltwise;
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        scale[1] = scaleO;
        return SUCCESS;
    }
    g.epi.mode = EPI_I32;
    if (odt == DT_I32) {
        g.C = output;
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        scale[1] = scaleO;
        return SUCCESS;
    }
    // u8 with the tensor-wide dynamic output scale (:2797-2806). The reference parks int32 accumulators
    // in tmp, takes their abs-max and requantises; here the convolution runs twice instead -- once
    // folding max|acc| into the scratch slots without storing anything, once writing u8 with the scale
    // that maximum gives. The arithmetic per element is the same; the int32 tensor (4 bytes per output,
    // written and read back) never exists, which is worth more than the repeated matrix work.
    if (onepass) {
        g.C = output;
        g.epi.mode = EPI_U8;
        g.conv.scaleO = scaleO;
        g.conv.dscale_out = c.hscale_dev;
        g.sync = c.fsync.next(conv_panel_grid(M_pix));
        arm_scale(c);
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        bool gave_up = false;
        EE te = take_scale(c, &scale[1], &gave_up);
        if (te != SUCCESS || !gave_up) {
            return te;
        }
        // the bounded wait of the one-pass form expired (the CUs were held by other work): nothing was stored;
        // the two passes below redo the convolution
        g_fused_fallbacks.fetch_add(1);
        memset(&g.sync, 0, sizeof(g.sync));
        g.epi.mode = EPI_I32;
        g.conv.dscale_out = nullptr;
    }
    g.C = nullptr;
    g.conv.absmax = c.ws;
    if (direct || onepass) {  // otherwise the padding kernel has cleared the slots
        HIP_TRY(launch_fill_u32(c.ws, kWsWords, 0, c.stream));
    }
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    g.C = output;
    g.epi.mode = EPI_U8;
    g.conv.scaleO = scaleO;
    g.conv.dscale_out = c.hscale_dev;  // the new output scale goes straight into pinned host memory
    arm_scale(c);
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    return take_scale(c, &scale[1]);
}

}  // namespace bgapi
}  // extern "C++"

EE convolution_infer_output_size_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, ConvolutionParamSpec p,
    TensorDesc *outputDesc, DataType targetDataType, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!outputDesc) {
        return NULL_POINTER;
    }
    U32 in, ic, ih, iw, fn, fc, fh, fw;
    if (get4d(inputDesc, &in, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_SUPPORTED;  // 5-D (3-D convolution) is not on the int8 path
    }
    EE ret = SUCCESS;
    if (fh < 1 || fw < 1) {
        ret = NOT_SUPPORTED;
    }
    const U32 dh = p.dilatedRate_h ? p.dilatedRate_h : 1, dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (p.stride_h == 0 || p.stride_w == 0) {
        return NOT_MATCH;
    }
    const I32 fhD = (I32)((fh - 1) * dh + 1), fwD = (I32)((fw - 1) * dw + 1);
    I32 oh, ow;
    switch (p.round_mode) {  // convolution.cpp:62-82
        case ROUND_SAME_UPPER:
            oh = (I32)((ih + p.stride_h - 1) / p.stride_h);
            ow = (I32)((iw + p.stride_w - 1) / p.stride_w);
            break;
        case ROUND_SAME_LOWER:
            oh = (I32)(ih / p.stride_h);
            ow = (I32)(iw / p.stride_w);
            break;
        default: {
            // unsigned arithmetic like the reference's (U32 operands): a window larger than the padded image wraps
            const U32 th = ih + p.pad_top + p.pad_bottom - (U32)fhD, tw = iw + p.pad_left + p.pad_right - (U32)fwD;
            oh = (I32)(th / p.stride_h + 1);
            ow = (I32)(tw / p.stride_w + 1);
            break;
        }
    }
    if (oh < 0 || ow < 0) {
        ret = NOT_MATCH;
    }
    if (fn % 8 != 0) {
        return NOT_SUPPORTED;  // :93-95
    }
    DataFormat odf = DF_NCHWC8;
    if (targetDataType == DT_U8_Q && fn != 8) {
        odf = DF_NCHWC16;  // :97-101
    }
    *outputDesc = tensor4df(targetDataType, odf, in, fn, (U32)oh, (U32)ow);
    return ret;
}

EE convolution_infer_forward_algorithm_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm, DataType targetDataType,
    ActivationParamSpec activationDesc, Arch arch)
{
    (void)outputDesc;
    (void)p;
    (void)policy;
    (void)activationDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!algorithm) {
        return NULL_POINTER;
    }
    if (*algorithm != CONVOLUTION_ALGORITHM_NULL) {
        return SUCCESS;  // cpu/x86/convolution.cpp:39-41
    }
    if (targetDataType != DT_U8_Q && targetDataType != DT_I8) {
        return NOT_SUPPORTED;  // only the quantised convolution runs here
    }
    U32 in, ic, ih, iw, fn, fc, fh, fw;
    if (get4d(inputDesc, &in, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_SUPPORTED;
    }
    *algorithm = (fh == 1 && fw == 1) ? CONVOLUTION_ALGORITHM_POINTWISE : CONVOLUTION_ALGORITHM_DIRECT;  // :79-82, :101
    return SUCCESS;
}

EE convolution_transform_filter_bytes_gfx950(TensorDesc filterDesc, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (p.group != 1 || filterDesc.dt != DT_I8) {
        return NOT_SUPPORTED;
    }
    *bytes = fn * 4 + align_up(fn, 16) * align_up(fh * fw * align_up(fc, 16), 64) + 32;
    return SUCCESS;
}

EE convolution_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, TensorDesc *ftmDesc, void *filterTransformed, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;
    }
    if (filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHW || p.group != 1) {
        return NOT_SUPPORTED;
    }
    ConvShape s;
    memset(&s, 0, sizeof(s));
    if (get4d(filterDesc, &s.oc, &s.ic, &s.fh, &s.fw) != SUCCESS) {
        return NOT_MATCH;
    }
    s.ICp = align_up(s.ic, 16);
    s.Kp = align_up(s.fh * s.fw * s.ICp, 64);
    s.N16 = align_up(s.oc, 16);
    if (arch == AMD_GFX950) {
        conv_pack_filter_host((const INT8 *)filter, s, (I32 *)filterTransformed, (INT8 *)filterTransformed + (size_t)s.oc * 4);
    } else {
        EE e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        HIP_TRY(launch_conv_pack_filter((const int8_t *)filter, s.oc, s.ic, s.fh, s.fw, (int32_t *)filterTransformed,
            (int8_t *)filterTransformed + (size_t)s.oc * 4, ctx().stream));
    }
    *ftmDesc = filterDesc;
    ftmDesc->df = DF_NCHWC2NxC4;  // convolution_transform.cpp:207-211
    ftmDesc->dims[2] = s.ICp;      // channels rounded up to the 16 of the packed layout (:70-87)
    return SUCCESS;
}

EE convolution_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    ConvShape s;
    EE e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    size_t off;
    const size_t total = conv_tmp_layout(s, &off);
    if (total > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)total;
    return SUCCESS;
}

EE convolution_gfx950(TensorDesc inputDesc, const void *input, const void *eltwiseInput, TensorDesc filterDesc,
    const void *filter, ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, F32 *scale,
    ActivationParamSpec activationDesc, Arch arch)
{
    (void)algorithm;
    (void)biasDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !bias || !tmp || !scale) {
        return NULL_POINTER;  // x86/int8/convolution.cpp:114-117
    }
    if (outputDesc.df != DF_NCHWC16 && outputDesc.df != DF_NCHWC8) {
        return NOT_MATCH;  // :128-130
    }
    if (inputDesc.dt != DT_U8_Q || filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHWC2NxC4) {
        return NOT_MATCH;  // convolution_direct.cpp:2613-2615 (activations arrive quantised on this path)
    }
    if (inputDesc.df != DF_NCHWC8 && inputDesc.df != DF_NCHWC16) {
        return NOT_SUPPORTED;
    }
    const DataType odt = outputDesc.dt;
    if (odt != DT_F32 && odt != DT_U8_Q && odt != DT_I32) {
        return NOT_SUPPORTED;
    }
    if (activationDesc.mode != ACTIVATION_NULL && activationDesc.mode != ACTIVATION_RELU) {
        return NOT_SUPPORTED;
    }
    if (eltwiseInput && odt != DT_F32) {
        return NOT_SUPPORTED;
    }
    ConvShape s;
    EE e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    size_t off;
    const size_t need = conv_tmp_layout(s, &off);
    if (tmpBytes < need) {
        return NOT_MATCH;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    const int relu = (activationDesc.mode == ACTIVATION_RELU);
    if (arch == AMD_GFX950_DEVICE) {
        if (((uintptr_t)tmp & 15) || ((uintptr_t)filter & 15) || ((uintptr_t)output & 15) || ((uintptr_t)input & 7)) {
            return fail(NOT_SUPPORTED, "device tmp / filter / output must be 16-byte aligned, input 8-byte aligned");
        }
        return conv_device(s, inputDesc.df, input, eltwiseInput, filter, bias, tmp, odt, outputDesc.df, output, scale,
            relu);
    }
    Ctx &cx = ctx();
    Stage st;
    const size_t inB = (size_t)s.n * s.ic * s.ih * s.iw;
    const size_t fB = (size_t)s.oc * 4 + (size_t)s.N16 * s.Kp;
    const size_t outN = (size_t)s.n * s.oc * s.oh * s.ow;
    const size_t outB = outN * (odt == DT_U8_Q ? 1 : 4);
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = st.get((size_t)s.oc * 4), *dT = st.get(need), *dO = st.get(outB);
    void *dE = eltwiseInput ? st.get(outN * 4) : nullptr;
    if (!dIn || !dF || !dB || !dT || !dO || (eltwiseInput && !dE)) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, input, inB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dF, filter, fB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dB, bias, (size_t)s.oc * 4, hipMemcpyHostToDevice, cx.stream));
    if (dE) {
        HIP_TRY(hipMemcpyAsync(dE, eltwiseInput, outN * 4, hipMemcpyHostToDevice, cx.stream));
    }
    e = conv_device(s, inputDesc.df, dIn, dE, dF, dB, dT, odt, outputDesc.df, dO, scale, relu);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(output, dO, outB, hipMemcpyDeviceToHost, cx.stream));
    HIP_TRY(hipStreamSynchronize(cx.stream));
    return SUCCESS;
}

// ---- 1-bit convolution (compute/tensor/src/cpu/arm/bnn/convolution.cpp:16-72) ----------------------
// Transformed-filter blob: [bit-packed filter, fn * fc * fh * fw / 8 bytes rounded up to 256 (the vector-ALU
// route)][the same filter expanded to int8 in the GEMM's packed right-hand-side layout, K = fh * fw * fc padded
// to 64 (the matrix-core route)]
static size_t bnn_blob_bits_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return ((size_t)fn * fc * fh * fw / 8 + 255) / 256 * 256;
}

static size_t bnn_blob_i8_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return ((size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16) + 255) / 256 * 256;
}

// ... followed by the filter as E2M1 pairs (K bytes = fh * fw * fc / 2 padded to 64) for the fp4 form of that route
static size_t bnn_blob_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return bnn_blob_bits_bytes(fn, fc, fh, fw) + bnn_blob_i8_bytes(fn, fc, fh, fw) +
        (size_t)align_up(fh * fw * fc / 2, 64) * align_up(fn, 16);
}

EE convolution_transform_filter_bytes_bnn_gfx950(TensorDesc filterDesc, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_BIN01 && filterDesc.dt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    const size_t b = bnn_blob_bytes(fn, fc, fh, fw);
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE convolution_transform_filter_bnn_gfx950(TensorDesc filterDesc, const void *filter, TensorDesc *ftmDesc,
    void *filterTransformed, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;  // convolution_transform_bnn.h:38-40
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_BIN01 && filterDesc.dt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    if (filterDesc.df != DF_NCHW && filterDesc.df != DF_NCHWN16C8) {
        return NOT_MATCH;  // :83-84
    }
    if (fn % 32 != 0 || fc % 32 != 0) {
        return NOT_SUPPORTED;  // kernel structure of the reference (convolution_xnor_A76.cpp:109,665)
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    const size_t bytes = (size_t)fn * fc * fh * fw / 8, bits = bnn_blob_bits_bytes(fn, fc, fh, fw),
                 total = bnn_blob_bytes(fn, fc, fh, fw);
    const int fmt = (filterDesc.df == DF_NCHWN16C8) ? 1 : 0;
    const int xnor = (filterDesc.dt == DT_BIN11);
    if (arch == AMD_GFX950) {
        Stage st;
        void *a = st.get(bytes);
        U8 *b = (U8 *)st.get(total);
        if (!a || !b) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, filter, bytes, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemsetAsync(b, 0, bits, c.stream));
        HIP_TRY(launch_bnn_pack_filter((const uint8_t *)a, fmt, fn, fc, fh * fw, (uint32_t *)b, c.stream));
        HIP_TRY(launch_bnn_expand_filter((const uint32_t *)b, fn, fc, fh * fw, xnor, (int8_t *)(b + bits), c.stream));
        HIP_TRY(hipMemsetAsync(b + bits + (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), 0,
            bnn_blob_i8_bytes(fn, fc, fh, fw) - (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), c.stream));
        HIP_TRY(launch_bnn_expand_filter_fp4((const uint32_t *)b, fn, fc, fh * fw, xnor,
            b + bits + bnn_blob_i8_bytes(fn, fc, fh, fw), c.stream));
        HIP_TRY(hipMemcpyAsync(filterTransformed, b, total, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    } else {
        if (((uintptr_t)filterTransformed & 15) != 0) {
            return fail(NOT_SUPPORTED, "device filterTransformed must be 16-byte aligned");
        }
        U8 *b = (U8 *)filterTransformed;
        if (bits > bytes / 4 * 4) {  // the padding behind the bits, so that equal filters give equal blobs
            HIP_TRY(launch_fill_u32((uint32_t *)(b + bytes / 4 * 4), (U32)((bits - bytes / 4 * 4) / 4), 0, c.stream));
        }
        HIP_TRY(launch_bnn_pack_filter((const uint8_t *)filter, fmt, fn, fc, fh * fw, (uint32_t *)b, c.stream));
        HIP_TRY(launch_bnn_expand_filter((const uint32_t *)b, fn, fc, fh * fw, xnor, (int8_t *)(b + bits), c.stream));
        const size_t i8 = (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), i8p = bnn_blob_i8_bytes(fn, fc, fh, fw);
        if (i8p > i8) {
            HIP_TRY(launch_fill_u32((uint32_t *)(b + bits + i8), (U32)((i8p - i8) / 4), 0, c.stream));
        }
        HIP_TRY(launch_bnn_expand_filter_fp4((const uint32_t *)b, fn, fc, fh * fw, xnor, b + bits + i8p, c.stream));
    }
    *ftmDesc = filterDesc;
    ftmDesc->df = DF_NCHWN16C8;  // the tag the operator layer checks; the byte order inside is this library's
    return SUCCESS;
}

EE convolution_infer_forward_tmp_bytes_bnn_gfx950(TensorDesc inputDesc, ConvolutionParamSpec p, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 n, ic, ih, iw;
    if (get4d(inputDesc, &n, &ic, &ih, &iw) != SUCCESS) {
        return NOT_MATCH;
    }
    const size_t Hp = ih + p.pad_top + p.pad_bottom, Wp = iw + p.pad_left + p.pad_right;
    // vector-ALU route: the bit-packed padded image. Matrix-core route: the image expanded to one byte per value.
    const size_t bits = (size_t)n * Hp * Wp * (ic / 8) + 32;
    const size_t img = (size_t)n * Hp * Wp * ic + 32;
    const size_t b = std::max(bits, img);
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE convolution_bnn_gfx950(TensorDesc inputDesc, const void *input, TensorDesc filterDesc, const void *filter,
    ConvolutionParamSpec p, TensorDesc scaleDesc, const void *scale, TensorDesc biasDesc, const void *bias, U32 tmpBytes,
    void *tmp, TensorDesc outputDesc, void *output, ActivationParamSpec activationDesc, Arch arch)
{
    (void)scaleDesc;
    (void)biasDesc;
    (void)activationDesc;  // ignored by the reference as well (bnn/convolution.cpp:35)
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !scale || !bias || !tmp) {
        return NULL_POINTER;  // bnn/convolution.cpp:32-35
    }
    U32 n, ic, ih, iw, fn, fc, fh, fw, on, oc, oh, ow;
    if (get4d(inputDesc, &n, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS ||
        get4d(outputDesc, &on, &oc, &oh, &ow) != SUCCESS) {
        return NOT_MATCH;
    }
    const DataType fdt = filterDesc.dt, idt = inputDesc.dt, odt = outputDesc.dt;
    if (fdt != DT_BIN01 && fdt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    // fp32 stands where the reference has fp16; bit-packed activations of the filter's type are also taken
    if ((idt != DT_F32 && idt != fdt) || (odt != DT_F32 && odt != DT_I32)) {
        return NOT_MATCH;
    }
    if ((idt == DT_F32 && inputDesc.df != DF_NCHWC8) || outputDesc.df != DF_NCHWC8 || filterDesc.df != DF_NCHWN16C8) {
        return NOT_MATCH;  // :45-53
    }
    if (fc != ic || fn != oc || on != n || ic % 32 != 0 || oc % 32 != 0 || p.group != 1 || p.stride_h == 0 ||
        p.stride_w == 0) {
        return NOT_MATCH;
    }
    if ((p.dilatedRate_h > 1) || (p.dilatedRate_w > 1)) {
        return NOT_SUPPORTED;
    }
    const U32 Hp = ih + p.pad_top + p.pad_bottom, Wp = iw + p.pad_left + p.pad_right;
    if (Hp < fh || Wp < fw || (Hp - fh) / p.stride_h + 1 < oh || (Wp - fw) / p.stride_w + 1 < ow) {
        return NOT_MATCH;
    }
    U32 need = 0;
    EE e = convolution_infer_forward_tmp_bytes_bnn_gfx950(inputDesc, p, &need, arch);
    if (e != SUCCESS) {
        return e;
    }
    if (tmpBytes < need) {
        return NOT_MATCH;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const size_t inB = (idt == DT_F32) ? (size_t)n * ic * ih * iw * 4 : (size_t)n * ic * ih * iw / 8;
    const size_t fB = bnn_blob_bytes(oc, ic, fh, fw);
    const size_t outN = (size_t)n * oc * oh * ow;
    const void *dIn = input, *dF = filter, *dS = scale, *dB = bias;
    void *dT = tmp, *dO = output;
    if (arch == AMD_GFX950) {
        void *a = st.get(inB), *f = st.get(fB), *s = st.get((size_t)oc * 4), *b = st.get((size_t)oc * 4);
        dT = st.get(need);
        dO = st.get(outN * 4);
        if (!a || !f || !s || !b || !dT || !dO) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, input, inB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(f, filter, fB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(s, scale, (size_t)oc * 4, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(b, bias, (size_t)oc * 4, hipMemcpyHostToDevice, c.stream));
        dIn = a;
        dF = f;
        dS = s;
        dB = b;
    } else if (!aligned4(tmp) || ((uintptr_t)output & 15) || !aligned4(filter)) {
        return fail(NOT_SUPPORTED, "device tmp / filter must be 4-byte aligned, output 16-byte aligned");
    }
    const int xnor = (fdt == DT_BIN11);
    if (g_bnn_mfma && (((uintptr_t)dT | (uintptr_t)dF) & 15) == 0) {
        // matrix-core route: the image expanded to int8 (or E2M1 pairs), the filter already expanded in the blob,
        // then the implicit-GEMM convolution with fma(S, scale, bias) (or the raw sums) as its epilogue
        const bool fp4 = g_bnn_mfma == 2 && conv_fp4_ok(n * oh * ow, oc);
        int8_t *img = (int8_t *)dT;
        const int8_t *flt = (const int8_t *)dF + bnn_blob_bits_bytes(oc, ic, fh, fw) + (fp4 ? bnn_blob_i8_bytes(oc, ic, fh, fw) : 0);
        if (fp4) {
            HIP_TRY(launch_bnn_expand_input_fp4(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left,
                p.pad_right, xnor ? 0.0f : 0.5f, xnor, (uint8_t *)img, c.stream));
        } else {
            HIP_TRY(launch_bnn_expand_input(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left,
                p.pad_right, xnor ? 0.0f : 0.5f, xnor, img, c.stream));
        }
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = (const uint8_t *)img;
        g.Bp = flt;
        g.M = n * oh * ow;
        g.N = oc;
        g.K = fp4 ? align_up(fh * fw * ic / 2, 64) : align_up(fh * fw * ic, 64);  // in operand bytes
        g.fp4 = fp4 ? 1 : 0;
        g.ob = (const int32_t *)flt;  // ob == comp: no offset, the sums are exact as they are
        g.comp = (const int32_t *)flt;
        g.C = dO;
        g.conv.OHW = oh * ow;
        g.conv.OW = ow;
        g.conv.sh = p.stride_h;
        g.conv.sw = p.stride_w;
        g.conv.Hp = Hp;
        g.conv.Wp = Wp;
        g.conv.ICp = fp4 ? ic / 2 : ic;  // bytes per pixel
        g.conv.fh = fh;
        g.conv.fw = fw;
        g.conv.dh = 1;
        g.conv.dw = 1;
        g.conv.out_c = 8;
        if (odt == DT_I32) {
            g.epi.mode = EPI_I32;
        } else {
            g.epi.mode = EPI_F32_CH;
            g.epi.scaleW = (const float *)dS;
            g.epi.bias = (const float *)dB;
        }
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        if (arch == AMD_GFX950) {
            HIP_TRY(hipMemcpyAsync(output, dO, outN * 4, hipMemcpyDeviceToHost, c.stream));
            HIP_TRY(hipStreamSynchronize(c.stream));
        }
        return SUCCESS;
    }
    HIP_TRY(launch_bnn_pack_input(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left, p.pad_right,
        xnor ? 0.0f : 0.5f, (uint32_t *)dT, c.stream));
    BnnArgs a;
    memset(&a, 0, sizeof(a));
    a.x = (const uint32_t *)dT;
    a.w = (const uint32_t *)dF;
    a.M = n * oh * ow;
    a.OHW = oh * ow;
    a.OW = ow;
    a.sh = p.stride_h;
    a.sw = p.stride_w;
    a.Hp = Hp;
    a.Wp = Wp;
    a.IC = ic;
    a.OC = oc;
    a.fh = fh;
    a.fw = fw;
    a.scale = (const float *)dS;
    a.bias = (const float *)dB;
    if (odt == DT_I32) {
        a.sums = (int32_t *)dO;
    } else {
        a.out = (float *)dO;
    }
    HIP_TRY(launch_bnn_conv(a, xnor, c.stream));
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(output, dO, outN * 4, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

// ---- tensor_computing: int8 matmul (compute/tensor/src/matmul.cpp:203-300, 302-576, x86 branch) --------
namespace {
struct MatmulShape {
    U32 M, K, N, batch, batchA, batchB;
    size_t elemsA, elemsB;
    size_t offQA, offQB, offBlob, offScale, total;  // tmp layout
};

EE matmul_shape(TensorDesc a, bool tA, TensorDesc b, bool tB, TensorDesc c, MatmulShape *s)
{
    if (a.nDims < 2 || b.nDims < 2 || c.nDims < 2) {
        return NOT_SUPPORTED;
    }
    s->M = tA ? a.dims[0] : a.dims[1];
    s->K = tA ? a.dims[1] : a.dims[0];
    const U32 kb = tB ? b.dims[0] : b.dims[1];
    s->N = tB ? b.dims[1] : b.dims[0];
    if (kb != s->K || c.dims[0] != s->N || c.dims[1] != s->M) {
        return NOT_MATCH;
    }
    auto lead = [](const TensorDesc &d) {
        U32 n = 1;
        for (U32 i = 2; i < d.nDims; ++i) {
            n *= d.dims[i];
        }
        return n;
    };
    s->batchA = lead(a);
    s->batchB = lead(b);
    s->batch = lead(c);
    // a 2-D operand is shared by every slice (matmul.cpp:505-528 with all leading dims 1)
    if ((s->batchA != s->batch && s->batchA != 1) || (s->batchB != s->batch && s->batchB != 1)) {
        return NOT_SUPPORTED;
    }
    s->elemsA = (size_t)s->batchA * s->M * s->K;
    s->elemsB = (size_t)s->batchB * s->K * s->N;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += (bytes + 255) / 256 * 256;
        return at;
    };
    s->offQA = take(s->elemsA);
    s->offQB = take(s->elemsB);
    // the operand that gets packed per slice: B (N x K) for a matrix result; A (M x K) when B is a single
    // column (matrix_vector_multiply packs its unpacked matrix into tmp, mvm.cpp:176-182); nothing for M == 1
    const U32 rowsP = (s->M != 1 && s->N == 1) ? s->M : s->N;
    s->offBlob = take((size_t)rowsP * 4 + packed_matrix_bytes(rowsP, s->K) + 64);
    s->offScale = take(64);
    s->total = off;
    return SUCCESS;
}
}  // namespace

EE matmul_infer_forward_tmp_bytes_gfx950(TensorDesc matrixADesc, bool transposeA, TensorDesc matrixBDesc, bool transposeB,
    TensorDesc matrixCDesc, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    MatmulShape s;
    EE e = matmul_shape(matrixADesc, transposeA, matrixBDesc, transposeB, matrixCDesc, &s);
    if (e != SUCCESS) {
        return e;
    }
    if (s.total > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)s.total;
    return SUCCESS;
}

EE matmul_gfx950(TensorDesc matrixADesc, bool transposeA, const void *matrixA, F32 scaleA, TensorDesc matrixBDesc,
    bool transposeB, const void *matrixB, F32 scaleB, U32 tmpBytes, void *tmp, TensorDesc matrixCDesc, void *matrixC,
    Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!matrixA || !matrixB || !matrixC) {
        return NULL_POINTER;  // matmul.cpp:322-324
    }
    MatmulShape s;
    EE e = matmul_shape(matrixADesc, transposeA, matrixBDesc, transposeB, matrixCDesc, &s);
    if (e != SUCCESS) {
        return e;
    }
    const DataType adt = matrixADesc.dt, bdt = matrixBDesc.dt, cdt = matrixCDesc.dt;
    const bool af32 = (adt == DT_F32 || adt == DT_F32_8Q), bf32 = (bdt == DT_F32 || bdt == DT_F32_8Q);
    // A vector result goes through matrix_vector_multiply with the operands quantised the other way
    // round: A -> I8, B -> U8_Q (matmul.cpp:374-382, :531-548).
    const bool vec = (s.M == 1 || s.N == 1);
    const DataType qadt = vec ? DT_I8 : DT_U8_Q, qbdt = vec ? DT_U8_Q : DT_I8;
    if ((!af32 && adt != qadt) || (!bf32 && bdt != qbdt) || (cdt != DT_F32 && cdt != DT_I32)) {
        return NOT_SUPPORTED;
    }
    if ((!af32 && scaleA <= 0) || (!bf32 && scaleB <= 0)) {
        return NOT_MATCH;
    }
    if (s.batch == 0 || s.M == 0 || s.N == 0) {
        return SUCCESS;
    }
    if (!tmp || tmpBytes < s.total) {
        return tmp ? NOT_MATCH : NULL_POINTER;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const void *dA = matrixA, *dB = matrixB;
    void *dC = matrixC;
    U8 *dT = (U8 *)tmp;
    const size_t aB = s.elemsA * bytesOf(adt), bB = s.elemsB * bytesOf(bdt), cB = (size_t)s.batch * s.M * s.N * 4;
    if (arch == AMD_GFX950) {
        void *a = st.get(aB), *b = st.get(bB);
        dC = st.get(cB);
        dT = (U8 *)st.get(s.total);
        if (!a || !b || !dC || !dT) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, matrixA, aB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(b, matrixB, bB, hipMemcpyHostToDevice, c.stream));
        dA = a;
        dB = b;
    } else if (!aligned4(matrixA) || !aligned4(matrixB) || !aligned4(matrixC) || ((uintptr_t)tmp & 15)) {
        return fail(NOT_SUPPORTED, "device operands must be 4-byte aligned, tmp 16-byte aligned");
    }
    float *sc = (float *)(dT + s.offScale);  // [0] = scale of A, [1] = scale of B, [2] = their product
    const uint8_t *qA = (const uint8_t *)dA;
    const int8_t *qB = (const int8_t *)dB;
    // Whole-tensor quantisation, the caller's scale as the floor (quantize_cpu with its default mode,
    // matmul.cpp:401-421): A -> U8_Q, B -> I8.
    if (af32) {
        HIP_TRY(launch_absmax_f32((const float *)dA, (U32)s.elemsA, c.ws, c.stream));
        HIP_TRY(launch_quantize_f32((const float *)dA, (U32)s.elemsA, dT + s.offQA, vec ? 0 : 1, c.ws, scaleA, nullptr, 0,
            sc + 0, c.stream));
        qA = dT + s.offQA;
    } else {
        HIP_TRY(launch_fill_u32((uint32_t *)(sc + 0), 1, f32_bits(scaleA), c.stream));
    }
    if (bf32) {
        HIP_TRY(launch_absmax_f32((const float *)dB, (U32)s.elemsB, c.ws, c.stream));
        HIP_TRY(launch_quantize_f32((const float *)dB, (U32)s.elemsB, dT + s.offQB, vec ? 1 : 0, c.ws, scaleB, nullptr, 0,
            sc + 1, c.stream));
        qB = (const int8_t *)(dT + s.offQB);
    } else {
        HIP_TRY(launch_fill_u32((uint32_t *)(sc + 1), 1, f32_bits(scaleB), c.stream));
    }
    HIP_TRY(launch_mul_scalars(sc + 2, sc + 0, sc + 1, c.stream));  // scaleO = sA * sB (:411-420)

    // One slice at a time, B packed into tmp per slice exactly as matrix_matrix_multiply does for an
    // unpacked right-hand side (mmm.cpp:206-218).
    int8_t *blob = (int8_t *)(dT + s.offBlob);
    int32_t *comp = (int32_t *)((U8 *)blob + packed_matrix_bytes(s.N, s.K));
    for (U32 ic = 0; ic < s.batch && vec; ++ic) {
        const U8 *as = qA + (s.batchA == 1 ? 0 : (size_t)ic * s.M * s.K);
        const U8 *bs = (const U8 *)qB + (s.batchB == 1 ? 0 : (size_t)ic * s.K * s.N);
        void *cs = (U8 *)dC + (size_t)ic * s.M * s.N * 4;
        Epilogue epi;
        memset(&epi, 0, sizeof(epi));
        epi.mode = (cdt == DT_F32) ? EPI_F32 : EPI_I32;
        epi.dfactor = (cdt == DT_F32) ? sc + 2 : nullptr;
        if (s.M == 1) {
            // u8 matrix B (stored [K][N], or [N][K] if transposed) times the s8 row vector A (:531-539)
            HIP_TRY(launch_gemv_u8s8(bs, transposeB ? s.K : 1, transposeB ? 1 : s.N, (const int8_t *)as, s.K, s.N, cs, epi,
                c.stream));
        } else {
            // s8 matrix A (stored [M][K], or [K][M] if transposed) times the u8 column vector B (:540-548);
            // the matrix is packed into tmp with its compensation in front, the result starts from zero
            int32_t *vcomp = (int32_t *)blob;
            int8_t *vmat = (int8_t *)blob + (size_t)s.M * 4;
            if (ic == 0 || s.batchA != 1) {
                HIP_TRY(launch_pack_mvm((const int8_t *)as, transposeA ? s.M : 1, transposeA ? 1 : s.K, s.K, s.M, vmat, vcomp,
                    c.stream));
            }
            GemvArgs g;
            memset(&g, 0, sizeof(g));
            g.W = vmat;
            g.ldw = align_up(s.K, 8);
            g.x = bs;
            g.K = s.K;
            g.N = s.M;
            g.ob = vcomp;
            g.comp = vcomp;
            g.y = cs;
            g.epi = epi;
            HIP_TRY(launch_gemv_s8u8(g, c.stream));
        }
    }
    for (U32 ic = 0; ic < s.batch && !vec; ++ic) {
        const int8_t *bs = qB + (s.batchB == 1 ? 0 : (size_t)ic * s.K * s.N);
        if (ic == 0 || s.batchB != 1) {
            HIP_TRY(launch_pack_mmm(bs, transposeB ? 1 : s.N, transposeB ? s.K : 1, s.K, s.N, blob, comp, c.stream));
        }
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = qA + (s.batchA == 1 ? 0 : (size_t)ic * s.M * s.K);
        g.lda = transposeA ? s.M : s.K;
        g.transA = transposeA ? 1 : 0;
        g.Bp = blob;
        g.M = s.M;
        g.N = s.N;
        g.K = s.K;
        g.comp = comp;
        g.ob = comp;
        g.C = (U8 *)dC + (size_t)ic * s.M * s.N * 4;
        if (cdt == DT_F32) {
            g.epi.mode = EPI_F32;
            g.epi.dfactor = sc + 2;
        } else {
            g.epi.mode = EPI_I32;
        }
        HIP_TRY(launch_gemm_u8s8(g, c.stream));
    }
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(matrixC, dC, cB, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

// ---- u8 pooling (compute/tensor/src/cpu/x86/int8/avx512/pooling_int8.cpp:316-429) ---------------------
EE pooling_gfx950(TensorDesc inputDesc, const void *input, PoolingParamSpec p, void *scale, TensorDesc outputDesc,
    void *output, void *idx, Arch arch)
{
    (void)idx;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !output) {
        return NULL_POINTER;
    }
    U32 n, ic, ih, iw, on, oc, oh, ow;
    if (get4d(inputDesc, &n, &ic, &ih, &iw) != SUCCESS || get4d(outputDesc, &on, &oc, &oh, &ow) != SUCCESS) {
        return NOT_MATCH;
    }
    if (inputDesc.dt != DT_U8_Q) {
        return NOT_SUPPORTED;   // pooling_x86 routes only DT_U8_Q to the quantised kernels
    }
    if (outputDesc.dt != DT_U8_Q || n != on || ic != oc || inputDesc.df != DF_NCHWC16 || outputDesc.df != DF_NCHWC16 ||
        ic % 16 != 0) {
        return NOT_MATCH;
    }
    if (p.mode != POOLING_MAX && p.mode != POOLING_MEAN) {
        return NOT_SUPPORTED;
    }
    // a zero kernel extent means the whole image (update_param, compute/tensor/src/pooling.cpp:107-131)
    if (p.kernel_w == 0) {
        p.kernel_w = iw;
    }
    if (p.kernel_h == 0) {
        p.kernel_h = ih;
    }
    if (p.kernel_h == 0 || p.kernel_w == 0 || p.stride_h == 0 || p.stride_w == 0 || p.pad_top >= p.kernel_h ||
        p.pad_left >= p.kernel_w) {
        return NOT_SUPPORTED;
    }
    const unsigned long long window = (unsigned long long)p.kernel_h * p.kernel_w;
    if (window > 65536ull) {
        return NOT_SUPPORTED;   // 65536 / window < 1
    }
    const U32 factor = 65536u / (U32)window;
    const size_t inB = (size_t)n * ic * ih * iw, outB = (size_t)n * ic * oh * ow;
    if (outB == 0) {
        return SUCCESS;
    }
    if (inB == 0 || outB / 16 > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    // the last window in each direction must still start inside the image
    if ((unsigned long long)(oh - 1) * p.stride_h >= (unsigned long long)ih + p.pad_top ||
        (unsigned long long)(ow - 1) * p.stride_w >= (unsigned long long)iw + p.pad_left) {
        return NOT_SUPPORTED;
    }
    if (scale) {
        F32 *sc = (F32 *)scale;
        if (p.mode == POOLING_MAX) {
            sc[1] = sc[0];
        } else {
            sc[1] = sc[0] * (F32)(I32)factor * (F32)(U32)window / (F32)65536;
        }
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    bg::PoolArgs a;
    a.total = (uint32_t)(outB / 16);
    a.IH = ih;
    a.IW = iw;
    a.OH = oh;
    a.OW = ow;
    a.kh = p.kernel_h;
    a.kw = p.kernel_w;
    a.sh = p.stride_h;
    a.sw = p.stride_w;
    a.pt = p.pad_top;
    a.pl = p.pad_left;
    a.mean = p.mode == POOLING_MEAN;
    a.count_include_pad = p.count_include_pad ? 1 : 0;
    a.pool_full = factor;
    if (arch == AMD_GFX950) {
        Stage st;
        void *di = st.get(inB), *dout = st.get(outB);
        if (!di || !dout) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(di, input, inB, hipMemcpyHostToDevice, c.stream));
        a.in = (const uint8_t *)di;
        a.out = (uint8_t *)dout;
        HIP_TRY(bg::launch_pool_u8_c16(a, c.stream));
        HIP_TRY(hipMemcpyAsync(output, dout, outB, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
        return SUCCESS;
    }
    a.in = (const uint8_t *)input;
    a.out = (uint8_t *)output;
    HIP_TRY(bg::launch_pool_u8_c16(a, c.stream));
    return SUCCESS;
}

// ---- concatenation with a common scale (compute/tensor/src/cpu/concat.cpp:90-189) -----------------------
EE concat_infer_forward_tmp_bytes_gfx950(U32 num, const TensorDesc *inputDesc, TensorDesc outputDesc, U32 *bytes,
    Arch arch)
{
    (void)num;
    (void)inputDesc;
    (void)outputDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    *bytes = 0;   // no format conversion is done here, so nothing is staged
    return SUCCESS;
}

EE concat_gfx950(U32 num, const TensorDesc *inputDesc, void *const *input, const F32 *inputScale, ConcatParamSpec p,
    void *tmp, TensorDesc outputDesc, void *output, F32 *outputScale, Arch arch)
{
    (void)tmp;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!output || (num && (!inputDesc || !input))) {
        return NULL_POINTER;
    }
    const bool rescale = outputDesc.dt == DT_I8 && inputScale && outputScale;
    F32 oscale = 0;
    if (rescale && num > 0) {
        oscale = inputScale[0];
        for (U32 j = 1; j < num; ++j) {
            oscale = std::min(inputScale[j], oscale);
        }
        *outputScale = oscale;
    }
    const int dim = (int)outputDesc.nDims;
    if (dim < 1 || dim > (int)DIM_LEN) {
        return NOT_MATCH;
    }
    int axis = ((p.axis % dim) + dim) % dim;
    axis = dim - 1 - axis;   // index into dims[], which runs innermost first
    size_t tile = bytesOf(outputDesc.dt);
    for (int i = 0; i < axis; ++i) {
        tile *= outputDesc.dims[i];
    }
    size_t loops = 1;
    for (int i = axis + 1; i < dim; ++i) {
        loops *= outputDesc.dims[i];
    }
    const U32 cblock = outputDesc.df == DF_NCHWC8 ? 8 : outputDesc.df == DF_NCHWC16 ? 16 : 1;
    const bool blocked = cblock > 1 && dim == 4;
    if (blocked && axis < dim - 2) {
        tile *= cblock;   // joined along h or w: a "row" of the copy spans the channel block as well
        loops /= cblock;
    }
    // validate: same type / format / rank, same extents off the axis, extents on the axis add up
    U32 sum = 0;
    for (U32 j = 0; j < num; ++j) {
        if (!input[j] || tensorNumElements(inputDesc[j]) == 0) {
            continue;
        }
        const TensorDesc &d = inputDesc[j];
        if (d.dt != outputDesc.dt || (int)d.nDims != dim) {
            return NOT_MATCH;
        }
        if (d.df != outputDesc.df) {
            return NOT_SUPPORTED;
        }
        for (int i = 0; i < dim; ++i) {
            if (i != axis && d.dims[i] != outputDesc.dims[i]) {
                return NOT_MATCH;
            }
        }
        if (blocked && axis == dim - 2 && d.dims[axis] % cblock != 0) {
            return NOT_SUPPORTED;
        }
        sum += d.dims[axis];
    }
    if (sum == 0) {
        return SUCCESS;
    }
    if (sum != outputDesc.dims[axis]) {
        return NOT_MATCH;
    }
    if (loops > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    const size_t ostride = (size_t)sum * tile;
    const size_t outB = ostride * loops;
    Stage st;
    uint8_t *dout = (uint8_t *)output;
    if (arch == AMD_GFX950) {
        dout = (uint8_t *)st.get(outB);
        if (!dout) {
            return fail(ALLOC_FAILED, "device staging");
        }
    }
    // gather the inputs that take part; in host-pointer mode they are staged on the device first
    std::vector<const void *> srcs;
    std::vector<size_t> lens;
    std::vector<float> factors;
    std::vector<char> scaled;
    for (U32 j = 0; j < num; ++j) {
        if (!input[j] || tensorNumElements(inputDesc[j]) == 0) {
            continue;
        }
        const size_t len = (size_t)inputDesc[j].dims[axis] * tile;
        if (len > 0xffffffffull) {
            return NOT_SUPPORTED;
        }
        const void *src = input[j];
        if (arch == AMD_GFX950) {
            void *d = st.get(len * loops);
            if (!d) {
                return fail(ALLOC_FAILED, "device staging");
            }
            HIP_TRY(hipMemcpyAsync(d, input[j], len * loops, hipMemcpyHostToDevice, c.stream));
            src = d;
        }
        const bool rs = rescale && inputScale[j] != oscale;
        srcs.push_back(src);
        lens.push_back(len);
        factors.push_back(rs ? oscale / inputScale[j] : 1.0f);
        scaled.push_back(rs ? 1 : 0);
    }
    bg::ConcatMulti cm;
    if (srcs.size() <= 8) {
        size_t off = 0;
        for (size_t j = 0; j < srcs.size(); ++j) {
            cm.in[j] = (const uint8_t *)srcs[j];
            cm.len[j] = (uint32_t)lens[j];
            cm.off[j] = off;
            cm.r[j] = factors[j];
            cm.rescale[j] = (uint8_t)scaled[j];
            off += lens[j];
        }
        cm.num = (uint32_t)srcs.size();
        cm.rows = (uint32_t)loops;
        cm.ostride = ostride;
        cm.out = dout;
    }
    if (cm.num && bg::concat_multi_fits(cm)) {
        HIP_TRY(bg::launch_concat_i8_multi(cm, c.stream));
    } else {
        size_t off = 0;
        for (size_t j = 0; j < srcs.size(); ++j) {
            HIP_TRY(bg::launch_concat_i8(srcs[j], dout + off, (uint32_t)loops, (uint32_t)lens[j], ostride,
                scaled[j], factors[j], c.stream));
            off += lens[j];
        }
    }
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(output, dout, outB, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

// ---- int8 LSTM cell (compute/tensor/src/cpu/x86/int8/lstm.cpp:20-179) -----------------------------------
namespace {
struct LstmShape {
    U32 batch, xDim, hDim, column, N, K;  // column = num_projection when there is one (lstm.cpp:60-62), else hDim
    size_t quantOff, dscaleOff, scaleWOff, interOff, actOff, total;
};

EE lstm_shape(TensorDesc xDesc, RNNParamSpec p, LstmShape *s)
{
    DataType dt;
    DataFormat df;
    if (get2d(xDesc, &dt, &df, &s->batch, &s->xDim) != SUCCESS) {
        return NOT_MATCH;
    }
    if (p.mode != RNN_LSTM) {
        return NOT_SUPPORTED;
    }
    s->hDim = p.num_outputs;
    s->column = p.num_projection > 0 ? p.num_projection : s->hDim;
    if (p.num_projection > 0 && s->hDim % 32 != 0) {
        return NOT_SUPPORTED;  // the projection matrix comes in blocks of 32 rows (DF_NKN32)
    }
    s->N = 4 * s->column;
    s->K = s->xDim + s->hDim;
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    s->quantOff = 0;
    s->dscaleOff = up((size_t)s->batch * s->K);
    s->scaleWOff = s->dscaleOff + up((size_t)s->batch * 4);
    s->interOff = s->scaleWOff + up((size_t)s->N * 4);
    s->actOff = s->interOff + up((size_t)s->batch * s->N * 4);
    s->total = s->actOff + (p.num_projection > 0 ? up((size_t)s->batch * s->column * 4) : 0);
    return SUCCESS;
}
}  // namespace

// Cell weight for both routes: [matrix-vector blob | the same matrix in the GEMM's packed layout]
EE rnn_transform_filter_bytes_gfx950(TensorDesc filterDesc, RNNParamSpec p, U32 *bytes, Arch arch)
{
    (void)p;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    DataType dt;
    DataFormat df;
    U32 N, K;
    if (get2d(filterDesc, &dt, &df, &N, &K) != SUCCESS || dt != DT_I8) {
        return NOT_MATCH;
    }
    if (df == DF_NKNx_NKN32) {
        *bytes = 0;   // already transformed
        return SUCCESS;
    }
    const size_t b = 2 * (size_t)packed_matrix_bytes(N, K) + (size_t)N * 4;
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE rnn_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, RNNParamSpec p, TensorDesc *ftmDesc,
    void *filterTransformed, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;
    }
    DataType dt;
    DataFormat df;
    U32 N, K;
    if (get2d(filterDesc, &dt, &df, &N, &K) != SUCCESS || dt != DT_I8 || df != DF_NORMAL) {
        return NOT_MATCH;   // s8 [4 * column][xDim + num_outputs], row-major (column = num_projection or num_outputs)
    }
    if (p.mode != RNN_LSTM || N != 4 * (p.num_projection > 0 ? p.num_projection : p.num_outputs)) {
        return NOT_SUPPORTED;
    }
    const size_t mat = packed_matrix_bytes(N, K), mvmB = mat + (size_t)N * 4;
    *ftmDesc = tensor2df(DT_I8, DF_NKNx_NKN32, N, K);
    if (N == 0 || K == 0) {
        return SUCCESS;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    U8 *dst = (U8 *)filterTransformed;
    if (arch == AMD_GFX950) {
        std::vector<I32> comp(N);
        pack_host(false, (const INT8 *)filter, 1, K, K, N, (INT8 *)dst, (I32 *)(dst + mat));
        pack_host(true, (const INT8 *)filter, 1, K, K, N, (INT8 *)(dst + mvmB), comp.data());
        return SUCCESS;
    }
    // the GEMM packing's compensation vector is the same as the matrix-vector one: it lands there twice
    HIP_TRY(launch_pack_mvm((const int8_t *)filter, 1, K, K, N, (int8_t *)dst, (int32_t *)(dst + mat), c.stream));
    HIP_TRY(launch_pack_mmm((const int8_t *)filter, 1, K, K, N, (int8_t *)(dst + mvmB), (int32_t *)(dst + mat),
        c.stream));
    return SUCCESS;
}

EE rnncell_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    RNNParamSpec p, U32 *bytes, Arch arch)
{
    (void)filterDesc;
    (void)outputDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    LstmShape s;
    EE e = lstm_shape(inputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    if (s.total > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)s.total;
    return SUCCESS;
}

EE rnncell_gfx950(TensorDesc xDesc, const void *currentX, const TensorDesc *filterDesc, const void **filter,
    const TensorDesc *biasDesc, const void **bias, F32 *scale, void *state, U32 tmpBytes, void *tmp, RNNParamSpec p,
    U32 batchStrideX, U32 batchStrideH, TensorDesc hDesc, void *output, Arch arch)
{
    (void)biasDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !bias || !state || !tmp || !output || !filterDesc || !scale || !filter[0] || !bias[0]) {
        return NULL_POINTER;
    }
    LstmShape s;
    EE e = lstm_shape(xDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    DataType fdt, odt;
    DataFormat fdf, odf;
    U32 fn, fk, on, oh;
    if (get2d(filterDesc[0], &fdt, &fdf, &fn, &fk) != SUCCESS || get2d(hDesc, &odt, &odf, &on, &oh) != SUCCESS) {
        return NOT_MATCH;
    }
    if (fdf != DF_NKN32 && fdf != DF_NKNx_NKN32) {
        return NOT_MATCH;   // lstm.cpp:54-56
    }
    if (xDesc.dt != DT_F32 || fdt != DT_I8 || odt != DT_F32 || fn != s.N || fk != s.K || on != s.batch || oh != s.hDim) {
        return NOT_MATCH;   // lstm.cpp:65-70 (an fp32 filter is another back end's)
    }
    if (p.activation_type != ACTIVATION_TANH) {
        return NOT_SUPPORTED;
    }
    if (s.batch == 0 || s.hDim == 0) {
        return SUCCESS;
    }
    if (s.xDim > 0 && !currentX) {
        return NULL_POINTER;
    }
    if (tmpBytes < s.total) {
        return NOT_MATCH;
    }
    if (s.batch > 65535 || batchStrideH < s.hDim || (s.xDim > 0 && batchStrideX < s.xDim)) {
        return NOT_SUPPORTED;
    }
    const U32 steps = batchStrideH / s.hDim / (p.bi_direction ? 2 : 1);   // lstm.cpp:64
    const size_t biasStride = (size_t)steps * s.N;
    if (biasStride > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const size_t blobB = (size_t)packed_matrix_bytes(s.N, s.K) + (size_t)s.N * 4;   // matrix-vector part
    const size_t filterB = blobB + (fdf == DF_NKNx_NKN32 ? (size_t)packed_matrix_bytes(s.N, s.K) : 0);
    const size_t stateB = (size_t)s.batch * (s.column + s.hDim) * 4;
    const bool projected = p.num_projection > 0;
    const size_t projB = projected ? (size_t)s.hDim * s.column * 4 : 0;
    if (projected && (!filter[1] || filterDesc[1].dt != DT_F32)) {
        return fail(NOT_MATCH, "a projection needs filter[1]: fp32, DF_NKN32 layout [num_outputs / 32][num_projection][32]");
    }
    bg::LstmArgs a;
    a.batch = s.batch;
    a.xdim = s.xDim;
    a.hdim = s.hDim;
    a.column = s.column;
    a.scale_in = scale[0];
    a.forget_bias = p.forget_bias;
    a.zoneout_cell = p.zoneout_cell;
    a.zoneout_output = p.zoneout_output;
    const void *dW = filter[0];
    U8 *dT = (U8 *)tmp;
    float *dOut = nullptr, *dState = nullptr;
    if (arch == AMD_GFX950) {
        // host pointers: rows are gathered into compact device copies
        float *dx = (float *)st.get((size_t)s.batch * std::max<U32>(s.xDim, 1) * 4);
        float *db = (float *)st.get((size_t)s.batch * s.N * 4);
        void *w = st.get(filterB);
        dState = (float *)st.get(stateB);
        dOut = (float *)st.get((size_t)s.batch * s.hDim * 4);
        dT = (U8 *)st.get(s.total);
        float *dP = projected ? (float *)st.get(projB) : nullptr;
        if (!dx || !db || !w || !dState || !dOut || !dT || (projected && !dP)) {
            return fail(ALLOC_FAILED, "device staging");
        }
        if (projected) {
            HIP_TRY(hipMemcpyAsync(dP, filter[1], projB, hipMemcpyHostToDevice, c.stream));
            a.proj = dP;
        }
        for (U32 m = 0; m < s.batch; ++m) {
            if (s.xDim) {
                HIP_TRY(hipMemcpyAsync(dx + (size_t)m * s.xDim, (const float *)currentX + (size_t)m * batchStrideX,
                    (size_t)s.xDim * 4, hipMemcpyHostToDevice, c.stream));
            }
            HIP_TRY(hipMemcpyAsync(db + (size_t)m * s.N, (const float *)bias[0] + m * biasStride, (size_t)s.N * 4,
                hipMemcpyHostToDevice, c.stream));
        }
        HIP_TRY(hipMemcpyAsync(w, filter[0], filterB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(dState, state, stateB, hipMemcpyHostToDevice, c.stream));
        dW = w;
        a.x = dx;
        a.x_stride = s.xDim;
        a.bias = db;
        a.bias_stride = s.N;
        a.state = dState;
        a.out = dOut;
        a.out_stride = s.hDim;
    } else {
        a.x = (const float *)currentX;
        a.x_stride = batchStrideX;
        a.bias = (const float *)bias[0];
        a.bias_stride = (uint32_t)biasStride;
        a.state = (float *)state;
        a.out = (float *)output;
        a.out_stride = batchStrideH;
        a.proj = projected ? (const float *)filter[1] : nullptr;
    }
    a.quant = dT + s.quantOff;
    a.dscale = (float *)(dT + s.dscaleOff);
    float *scaleW = (float *)(dT + s.scaleWOff);
    float *inter = (float *)(dT + s.interOff);
    a.inter = inter;
    a.act = projected ? (float *)(dT + s.actOff) : nullptr;
    if (fdf == DF_NKNx_NKN32 && s.batch >= (U32)g_lstm_gemm_rows) {
        // enough rows to share one pass over the weight: all rows through the matrix cores as one GEMM with exact
        // int32 results; the gates kernel dequantises them with each row's own scale, in the arithmetic of the
        // matrix-vector epilogue
        HIP_TRY(bg::launch_lstm_xh_quant(a, c.stream));
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = a.quant;
        g.lda = s.K;
        g.Bp = (const int8_t *)dW + blobB;
        g.M = s.batch;
        g.N = s.N;
        g.K = s.K;
        g.comp = (const int32_t *)((const U8 *)dW + packed_matrix_bytes(s.N, s.K));
        g.ob = g.comp;
        g.C = inter;
        g.epi.mode = EPI_I32;
        HIP_TRY(launch_gemm_u8s8(g, c.stream));
        a.acc_i32 = 1;
        a.scale_w = scale[1];
        HIP_TRY(bg::launch_lstm_gates(a, c.stream));
    } else {
    uint32_t wbits;
    memcpy(&wbits, &scale[1], 4);
    HIP_TRY(bg::launch_fill_u32((uint32_t *)scaleW, s.N, wbits, c.stream));
    HIP_TRY(bg::launch_lstm_xh_quant(a, c.stream));
    e = bolt_gfx950_mvm_int8_strided_batch(s.batch, s.N, s.K, dW, 0, 1, a.quant, inter, a.dscale, scaleW, nullptr);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(bg::launch_lstm_gates(a, c.stream));
    }
    if (projected) {
        HIP_TRY(bg::launch_lstm_project(a, c.stream));  // lstm.cpp:170-178
    }
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(state, dState, stateB, hipMemcpyDeviceToHost, c.stream));
        for (U32 m = 0; m < s.batch; ++m) {
            HIP_TRY(hipMemcpyAsync((float *)output + (size_t)m * batchStrideH, dOut + (size_t)m * s.hDim,
                (size_t)s.hDim * 4, hipMemcpyDeviceToHost, c.stream));
        }
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

// ---- BERT-style int8 encoder layer --------------------------------------------------------------------
namespace {
struct EncoderPlan {
    size_t ws, scales, xq, xq2, qkv, ctx, ao, h1, f, o, total;
};

EncoderPlan encoder_plan(const BoltEncoderLayerInt8 &L)
{
    const size_t T = (size_t)L.batch * L.seq, H = L.hidden, F = L.ffn;
    EncoderPlan p;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += (bytes + 255) / 256 * 256;
        return at;
    };
    p.ws = take(4 * kWsWords * sizeof(uint32_t));
    p.scales = take(64);
    p.xq = take(T * H);   // u8 input of the three FullyConnected layers that read [T, H]
    p.xq2 = take(T * F);  // u8 input of the last one, [T, F] (written while the one before it still reads xq)
    p.qkv = take(T * 3 * H * 4);
    p.ctx = take(T * H * 4);
    p.ao = take(T * H * 4);
    p.h1 = take(T * H * 4);
    p.f = take(T * F * 4);
    p.o = take(T * H * 4);
    p.total = off;
    return p;
}

EE encoder_check(const BoltEncoderLayerInt8 *L)
{
    if (!L) {
        return NULL_POINTER;
    }
    if (!L->wqkv || !L->wo || !L->w1 || !L->w2 || !L->sqkv || !L->so || !L->s1 || !L->s2 || !L->ln1_gamma || !L->ln1_beta ||
        !L->ln2_gamma || !L->ln2_beta) {
        return NULL_POINTER;
    }
    if (L->batch == 0 || L->seq == 0 || L->heads == 0 || L->hidden != L->heads * 64 || L->ffn == 0 || L->ffn % 4 != 0 ||
        L->hidden > 2048) {
        return NOT_SUPPORTED;
    }
    if ((uint64_t)L->batch * L->seq * (L->ffn > 3 * L->hidden ? L->ffn : 3 * L->hidden) > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    return SUCCESS;
}
}  // namespace

EE bolt_gfx950_encoder_layer_int8_workspace_bytes(const BoltEncoderLayerInt8 *layer, size_t *bytes)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    *bytes = encoder_plan(*layer).total;
    return SUCCESS;
}

EE bolt_gfx950_encoder_layer_int8_workspace_layout(const BoltEncoderLayerInt8 *layer, size_t *offsets)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!offsets) {
        return NULL_POINTER;
    }
    const EncoderPlan p = encoder_plan(*layer);
    offsets[0] = p.qkv;
    offsets[1] = p.ctx;
    offsets[2] = p.ao;
    offsets[3] = p.h1;
    offsets[4] = p.f;
    offsets[5] = p.o;
    return SUCCESS;
}

// One layer's launches. input_max_ready: the scratch slots already hold max|hidden| (the LayerNorm that produced
// `hidden` folded it), so no abs-max pass runs; fold_out_max: the last LayerNorm folds max|out| into those slots for
// the layer that follows.
static EE encoder_run(const BoltEncoderLayerInt8 &L, const EncoderPlan &p, const float *hidden, float *out, void *workspace,
    bool input_max_ready, bool fold_out_max)
{
    hipStream_t st = ctx().stream;
    U8 *w = (U8 *)workspace;
    const U32 T = L.batch * L.seq, H = L.hidden, F = L.ffn;
    float *sc = (float *)(w + p.scales);
    uint8_t *xq = w + p.xq, *xq2 = w + p.xq2;
    float *qkv = (float *)(w + p.qkv), *cx = (float *)(w + p.ctx), *ao = (float *)(w + p.ao), *h1 = (float *)(w + p.h1),
          *f = (float *)(w + p.f), *o = (float *)(w + p.o);

    auto gemm = [&](const uint8_t *A, const void *blob, U32 N, U32 K, const float *dsI, const float *sW, const float *bias,
                    float *C) -> hipError_t {
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = A;
        g.lda = K;
        g.Bp = (const int8_t *)blob;
        g.M = T;
        g.N = N;
        g.K = K;
        g.comp = (const int32_t *)((const U8 *)blob + packed_matrix_bytes(N, K));
        g.ob = g.comp;  // no folded bias: the fp32 bias is added in the epilogue
        g.C = C;
        g.epi.mode = EPI_F32_CH;
        g.epi.scaleI = dsI;
        g.epi.scaleW = sW;
        g.epi.bias = bias;
        return launch_gemm_u8s8(g, st);
    };

    // The four running maxima live in slots the library owns and keeps clear between calls: each array is zeroed
    // by the first workgroup of a kernel that runs after the maximum's only reader and before its next producer
    // (one layer call later). A call that fails half way leaves them in an unknown state, so they are refilled
    // before the next one.
    Ctx &c = ctx();
    uint32_t *ws0 = c.enc_ws, *ws1 = ws0 + kWsWords, *ws2 = ws1 + kWsWords, *ws3 = ws2 + kWsWords;
    if (!input_max_ready) {
        if (c.enc_ws_dirty) {
            HIP_TRY(launch_fill_u32(ws0, 4 * kWsWords, 0, st));
        }
        c.enc_ws_dirty = true;
        HIP_TRY(launch_absmax_f32(hidden, T * H, ws0, st, true));
    }
    // x -> u8 (dynamic per-tensor scale), one quantisation shared by Q, K and V
    HIP_TRY(launch_quantize_f32(hidden, T * H, xq, 1, ws0, 0.0f, nullptr, 0, sc + 0, st));
    HIP_TRY(gemm(xq, L.wqkv, 3 * H, H, sc + 0, L.sqkv, L.bqkv, qkv));
    HIP_TRY(launch_attention_f32(qkv, L.batch, L.seq, H, L.heads, cx, ws1, st, ws0));
    HIP_TRY(launch_quantize_f32(cx, T * H, xq, 1, ws1, 0.0f, nullptr, 0, sc + 1, st));
    HIP_TRY(gemm(xq, L.wo, H, H, sc + 1, L.so, L.bo, ao));
    HIP_TRY(launch_add_layernorm(hidden, ao, L.ln1_gamma, L.ln1_beta, T, H, h1, ws2, st, ws1));
    HIP_TRY(launch_quantize_f32(h1, T * H, xq, 1, ws2, 0.0f, nullptr, 0, sc + 2, st));
    // (the fused kernel is one of the tiled ones: it needs what launch_gemm_u8s8 asks of those -- operands on 16-byte
    // boundaries -- and reads the per-column vectors 16 bytes at a time; anything else takes the unfused sequence)
    const bool fused_aligned = ((((uintptr_t)L.w1) | ((uintptr_t)xq) | ((uintptr_t)L.s1) | ((uintptr_t)L.b1)) & 15) == 0;
    if (g_encoder_fused && fused_aligned && gemm_gelu_dyn_fits(T, F, H)) {
        // FullyConnected + GELU + dynamic quantisation in one launch: the accumulators stay in registers across a
        // grid-wide agreement on max|gelu|; the [T, F] fp32 tensor is never written. Should that agreement be abandoned
        // (the CUs were held by other work), the kernel leaves the activated values in f, sets the status word, and
        // its last workgroup quantises them alone.
        uint32_t *status = (uint32_t *)(sc + 8);
        const uint32_t tiles = (T / 256) * (F / 256);
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = xq;
        g.lda = H;
        g.Bp = (const int8_t *)L.w1;
        g.M = T;
        g.N = F;
        g.K = H;
        g.comp = (const int32_t *)((const U8 *)L.w1 + packed_matrix_bytes(F, H));
        g.ob = g.comp;
        g.C = xq2;
        g.epi.mode = EPI_U8_GELU_DYN;
        g.epi.scaleI = sc + 2;
        g.epi.scaleW = L.s1;
        g.epi.bias = L.b1;
        g.sync = c.fsync.next(tiles);
        g.dscale_out = sc + 3;
        g.status = status;
        g.C32 = f;
        g.clear_ws = ws2;  // consumed by the quantiser in front of this product
        hipError_t he = launch_gemm_u8s8(g, st);
        if (he != hipSuccess) {
            return fail(UNKNOWN, "launch_gemm_u8s8 (GELU epilogue)", he);
        }
    } else {
        HIP_TRY(gemm(xq, L.w1, F, H, sc + 2, L.s1, L.b1, f));
        // GELU: one pass takes max|gelu(f)| without writing anything, the quantiser applies the same gelu to what it reads
        HIP_TRY(launch_gelu_f32(f, (size_t)T * F, ws3, st, false, ws2));
        HIP_TRY(launch_quantize_f32(f, T * F, xq2, 1, ws3, 0.0f, nullptr, 0, sc + 3, st, 1));
    }
    HIP_TRY(gemm(xq2, L.w2, H, F, sc + 3, L.s2, L.b2, o));
    // (ws0 was consumed by the first quantiser and cleared by the attention kernel: free for the next layer's maximum)
    HIP_TRY(launch_add_layernorm(h1, o, L.ln2_gamma, L.ln2_beta, T, H, out, fold_out_max ? ws0 : nullptr, st, ws3));
    return SUCCESS;
}

EE bolt_gfx950_encoder_layer_int8(const BoltEncoderLayerInt8 *layer, const float *hidden, float *out, void *workspace,
    size_t workspaceBytes)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!hidden || !out || !workspace) {
        return NULL_POINTER;
    }
    const BoltEncoderLayerInt8 &L = *layer;
    const EncoderPlan p = encoder_plan(L);
    if (workspaceBytes < p.total) {
        return NOT_MATCH;
    }
    if (((uintptr_t)workspace & 255) || ((uintptr_t)hidden & 15) || ((uintptr_t)out & 15)) {
        return fail(NOT_SUPPORTED, "workspace must be 256-byte aligned, hidden / out 16-byte aligned");
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    e = encoder_run(L, p, hidden, out, workspace, false, false);
    if (e != SUCCESS) {
        return e;
    }
    c.enc_ws_dirty = false;
    return SUCCESS;
}

EE bolt_gfx950_encoder_stack_int8(const BoltEncoderLayerInt8 *layers, U32 numLayers, const float *hidden, float *out,
    void *workspace, size_t workspaceBytes)
{
    if (!layers || !hidden || !out || !workspace) {
        return NULL_POINTER;
    }
    if (numLayers == 0) {
        return NOT_SUPPORTED;
    }
    size_t need = 0;
    EE e = bolt_gfx950_encoder_stack_int8_workspace_bytes(layers, numLayers, &need);
    if (e != SUCCESS) {
        return e;
    }
    if (workspaceBytes < need) {
        return NOT_MATCH;
    }
    if (((uintptr_t)workspace & 255) || ((uintptr_t)hidden & 15) || ((uintptr_t)out & 15)) {
        return fail(NOT_SUPPORTED, "workspace must be 256-byte aligned, hidden / out 16-byte aligned");
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    // the layers share one layer's workspace (the largest); behind it two [T, hidden] fp32 buffers take the
    // activations from layer to layer
    size_t one = 0;
    for (U32 i = 0; i < numLayers; ++i) {
        const size_t t = encoder_plan(layers[i]).total;
        one = t > one ? t : one;
    }
    const size_t act = ((size_t)layers[0].batch * layers[0].seq * layers[0].hidden * 4 + 255) / 256 * 256;
    float *pp[2] = {(float *)((U8 *)workspace + one), (float *)((U8 *)workspace + one + act)};
    Ctx &c = ctx();
    const float *in = hidden;
    for (U32 i = 0; i < numLayers; ++i) {
        const bool last = i + 1 == numLayers;
        float *o = last ? out : pp[i & 1];
        e = encoder_run(layers[i], encoder_plan(layers[i]), in, o, workspace, i != 0, !last);
        if (e != SUCCESS) {
            return e;
        }
        in = o;
    }
    c.enc_ws_dirty = false;
    return SUCCESS;
}

EE bolt_gfx950_encoder_stack_int8_workspace_bytes(const BoltEncoderLayerInt8 *layers, U32 numLayers, size_t *bytes)
{
    if (!layers || !bytes) {
        return NULL_POINTER;
    }
    if (numLayers == 0) {
        return NOT_SUPPORTED;
    }
    size_t one = 0;
    for (U32 i = 0; i < numLayers; ++i) {
        EE e = encoder_check(&layers[i]);
        if (e != SUCCESS) {
            return e;
        }
        if (layers[i].batch != layers[0].batch || layers[i].seq != layers[0].seq || layers[i].hidden != layers[0].hidden) {
            return NOT_MATCH;  // the activations keep their shape from layer to layer
        }
        const size_t t = encoder_plan(layers[i]).total;
        one = t > one ? t : one;
    }
    const size_t act = ((size_t)layers[0].batch * layers[0].seq * layers[0].hidden * 4 + 255) / 256 * 256;
    *bytes = one + 2 * act;
    return SUCCESS;
}

EE bolt_gfx950_attention_f32(const float *qkv, U32 batch, U32 seq, U32 hidden, U32 heads, float *context)
{
    if (!qkv || !context) {
        return NULL_POINTER;
    }
    if (heads == 0 || hidden != heads * 64) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_attention_f32(qkv, batch, seq, hidden, heads, context, nullptr, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_add_layernorm_f32(const float *a, const float *b, const float *gamma, const float *beta, U32 rows,
    U32 hidden, float *out)
{
    if (!a || !gamma || !beta || !out) {
        return NULL_POINTER;
    }
    if (hidden % 4 != 0 || hidden > 2048) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_add_layernorm(a, b, gamma, beta, rows, hidden, out, nullptr, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_gelu_f32(float *x, size_t n)
{
    if (!x) {
        return NULL_POINTER;
    }
    if (n % 4 != 0) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_gelu_f32(x, n, nullptr, ctx().stream));
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
