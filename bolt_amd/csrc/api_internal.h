// Shared by the C-ABI source files (api*.hip): the per-thread call context, error plumbing, the host-pointer staging
// pool and the device-pointer cores that more than one operator family builds on. Not part of the public interface.
#pragma once
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <string>
#include <vector>

#include "../../include/bolt_gfx950.h"
#include "kernels.h"
#include "layout.h"

namespace bgapi {

// Everything a call needs besides its arguments. One context per calling thread: its stream, its scratch words, its
// pinned scale word, its quantiser sync area and its staging pool, so that threads calling at the same time (each
// with its own tensors, as CNN::clone() gives them) never share mutable state. Contexts come from a process-wide
// pool: a thread takes one on its first call and returns it when it ends; device memory is never freed, so a
// process that creates and ends threads does not leak one context per thread.
struct Ctx {
    bool ready = false;
    hipStream_t stream = nullptr;
    uint32_t *ws = nullptr;  // device scratch words for the two-pass reductions
    // One pinned host word that kernels write a freshly computed scale into (the interfaces that return a
    // scale through a host pointer read it after the stream has drained: no copy command in between), and
    // the address the device uses for it.
    float *hscale = nullptr, *hscale_dev = nullptr;
    bg::FusedSync fsync;  // sync area of the one-launch dynamic quantiser
    uint32_t *enc_ws = nullptr;  // the encoder layer's four arrays of max slots (behind ws), kept clear between calls
    bool enc_ws_dirty = true;
    // two arrays of max slots (behind enc_ws) that the two-pass u8 convolutions of api_conv_ext.hip alternate between:
    // the second pass of a call clears the array the NEXT call folds into, so no call spends a launch on clearing
    uint32_t *conv_ws[2] = {nullptr, nullptr};
    int conv_ws_next = 0;
    bool conv_ws_dirty = true;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    std::string err;
    bool reused = false;  // taken over from a thread that has ended: its last work may still be running
    struct Buf {
        void *p;
        size_t bytes;
        bool busy;
    };
    std::vector<Buf> pool;
};

Ctx &ctx();  // the calling thread's context (taken from a process-wide pool on its first call)

EE fail(EE code, const char *what, hipError_t he = hipSuccess);  // records the text behind bolt_gfx950_last_error()

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e__ = (expr);                        \
        if (e__ != hipSuccess) {                        \
            return ::bgapi::fail(UNKNOWN, #expr, e__);  \
        }                                               \
    } while (0)

EE ensure_init();  // allocates the context's device state on first use; call before any launch

// A scale that a kernel computes and the interface returns through a host pointer (api.hip)
void arm_scale(Ctx &c);
EE take_scale(Ctx &c, float *dst, bool *gave_up = nullptr);

extern std::atomic<unsigned long long> g_fused_fallbacks;  // behind bolt_gfx950_get_counter("quantize_fused_fallbacks")

// Grow-only device staging pool for the host-pointer mode (per context, so per calling thread).
struct Stage {
    Ctx &c = ctx();
    std::vector<size_t> taken;
    ~Stage()
    {
        for (size_t i : taken) {
            c.pool[i].busy = false;
        }
    }
    void *get(size_t bytes)
    {
        bytes = std::max<size_t>(bytes, 256);
        for (size_t i = 0; i < c.pool.size(); ++i) {
            if (!c.pool[i].busy && c.pool[i].bytes >= bytes) {
                c.pool[i].busy = true;
                taken.push_back(i);
                return c.pool[i].p;
            }
        }
        void *p = nullptr;
        if (hipMalloc(&p, bytes) != hipSuccess) {
            return nullptr;
        }
        c.pool.push_back({p, bytes, true});
        taken.push_back(c.pool.size() - 1);
        return p;
    }
};

// options behind bolt_gfx950_set_option (process-wide; api.hip explains each where it is defined)
extern int g_bnn_mfma, g_conv_direct, g_conv_onepass, g_lstm_gemm_rows, g_quantize_fused, g_encoder_fused;

// descriptor helpers and the device-pointer cores of the two matrix products (api.hip)
EE get2d(TensorDesc d, DataType *dt, DataFormat *df, U32 *rows, U32 *cols);
EE get1d(TensorDesc d, DataType *dt, U32 *len);
EE get4d(TensorDesc d, U32 *n, U32 *c, U32 *h, U32 *w);
uint64_t elements64(TensorDesc d);  // element count in 64 bits (tensorNumElements multiplies in 32 bits and wraps)
constexpr uint64_t kMaxElementwise = 0xf0000000ull;  // element-wise kernels index in 32 bits with grid strides
bool elementwise_count(TensorDesc d, U32 *n);        // false beyond kMaxElementwise
uint32_t f32_bits(float f);
bool aligned4(const void *p);
bg::Epilogue epi_from_scale(const F32 *scale);
void pack_host(bool mmm, const INT8 *src, size_t sk, size_t sn, U32 K, U32 N, INT8 *dst, I32 *comp);
U32 packed_matrix_bytes(U32 N, U32 K);  // bytes of the packed matrix part for an N x K weight
EE mmm_device(U32 M, U32 N, U32 K, DataFormat adf, const void *A, DataFormat bdf, const void *B, void *tmp, DataType cdt, void *C,
    const F32 *scale);
EE mvm_device(U32 N, U32 K, DataType mdt, DataFormat mdf, const void *W, const void *x, void *tmp, void *y, const F32 *scale);
U32 out_elem_bytes(const F32 *scale);

// ---- int8 convolution core (api_conv.hip), also the 1x1 product inside the deconvolution ---------------------------
struct ConvShape {
    U32 n, ic, ih, iw, oc, fh, fw, oh, ow;
    U32 sh, sw, pt, pb, pl, pr, dh, dw;
    U32 Hp, Wp, ICp, Kp, N16;
};

EE conv_shape(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, const ConvolutionParamSpec &p, ConvShape *s);
size_t conv_tmp_layout(const ConvShape &s, size_t *off);  // bytes of tmp the convolution needs; *off = where its bias vector sits
// all pointers device; scale = {input, output (in / out), filter}
EE conv_device(const ConvShape &s, DataFormat idf, const void *input, const void *eltwise, const void *filter, const void *bias,
    void *tmp, DataType odt, DataFormat odf, void *output, F32 *scale, int relu);

}  // namespace bgapi
