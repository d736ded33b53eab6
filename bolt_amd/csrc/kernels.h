// Launchers of the gfx950 kernels. Every pointer is a device pointer; launches are asynchronous on
// the given stream. The C-ABI layer (api*.hip) validates shapes before calling any of these.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "device_common.h"

namespace bg {

// Every field of the argument structs below has a default (null / 0): a caller that leaves one out hands the
// kernel a harmless value, never an indeterminate pointer.

// ---- shared with the C-ABI layer (api*.hip) ---------------------------------------------------------
hipStream_t api_stream();                              // the stream every call is enqueued on (null until set)
void api_set_error(const char *what, hipError_t he);   // text behind bolt_gfx950_last_error()
int noalloc_init_current_device();                     // noalloc.hip: looks up the static scratch array's device address

// ---- GEMV ---------------------------------------------------------------------------------------
struct GemvBatch {
    uint32_t count = 0;      // number of independent products in the launch (0 / 1: a single one)
    uint32_t wcopies = 0;    // slice b reads the weight blob b % wcopies (0: one blob)
    size_t wstride = 0;      // bytes between consecutive weight blobs
    uint32_t xstride = 0;    // bytes between activation vectors
    uint32_t ystride = 0;    // bytes between result vectors
    int ob_in_blob = 0;      // ob points into the blob and moves with it
};

struct GemvArgs {
    const int8_t *W = nullptr;     // packed weight: row-major [ALIGN(N,16)][ldw], rows zero-padded
    uint32_t ldw = 0;        // ALIGN(K, 8)
    const uint8_t *x = nullptr;    // [K]
    uint32_t K = 0, N = 0;
    const int32_t *ob = nullptr;   // caller's offsetC (+ folded bias) [N]
    const int32_t *comp = nullptr; // -128 * sum_k W[n][k], stored behind the packed matrix [N]
    const float *fold_bias = nullptr;  // if set, ob is not read: the offset is (int32)(round(fold_bias[n] * fold_scale) + comp[n])
    float fold_scale = 0;
    void *y = nullptr;
    int add_yin = 0;         // accumulate into the int32 bits already in y
    Epilogue epi;
    GemvBatch batch;
};
hipError_t launch_gemv_s8u8(const GemvArgs &a, hipStream_t st);
hipError_t launch_gemv_u8s8(const uint8_t *A, uint32_t lda, uint32_t sk, const int8_t *x, uint32_t K, uint32_t M,
    void *y, const Epilogue &epi, hipStream_t st);

// ---- GEMM ---------------------------------------------------------------------------------------
// Geometry of an implicit-GEMM convolution (GemmArgs::conv), all in elements / bytes of the padded,
// s8 image in planes of 16 channels, [n][ICp/16][Hp][Wp][16], that conv_pad produces.
struct ConvGeom {
    uint32_t OHW = 0, OW = 0;          // output pixels per image, output width
    uint32_t sh = 0, sw = 0;           // strides
    uint32_t Hp = 0, Wp = 0, ICp = 0;      // padded image height / width, channels rounded up to 16
    uint32_t fh = 0, fw = 0, dh = 0, dw = 0;   // filter taps and dilation: K runs over (kh, kw, c) in 16-channel chunks
    uint32_t out_c = 0;            // channel block of the output layout: 16 (NCHWC16) or 8 (NCHWC8)
    // in_c = 0: A is the padded s8 image in planes of 16 channels (conv_pad's output). in_c = 8 / 16: A is the
    // caller's u8 tensor itself (NCHWC8 / NCHWC16, IC % 16 == 0), gathered in place by the filter-panel kernel:
    // H x W pixels per plane, pt / pl rows / columns of padding above / left of it
    uint32_t in_c = 0, H = 0, W = 0, IC = 0, pt = 0, pl = 0;
    int relu = 0;
    const float *eltwise = nullptr;      // optional fp32 tensor added before the ReLU (fp32 output only)
    uint32_t *absmax = nullptr;          // scratch slots: int32 mode folds max |acc| into them (C may then be null:
                               // nothing is stored); u8 mode reads them for the tensor-wide dynamic scale
    float scaleO = 0;              // u8 mode: scale of the accumulators (input scale * filter scale)
    float *dscale_out = nullptr;         // u8 mode: device word that receives the resulting output scale
    // The input scale may live in device memory (a chain of quantised operators that never waits for the host): then
    // the accumulators' scale is *dscaleI * filter_scale, formed by every consumer inside the kernel with the same
    // single fp32 multiplication the host would do, and scaleO / GemmArgs::fold_scale / the fp32 factor are not used.
    const float *dscaleI = nullptr;
    float filter_scale = 0;
    // EPI_CONV_CH (per-output-channel filter scales in epi.scaleW, fp32 bias in epi.bias): the input scale is *dscaleI
    // when that is set, else scaleI; ch_out is a ConvChOut
    float scaleI = 0;
    int ch_out = 0;
};

// scale of a convolution's accumulators: input scale * filter scale (convolution_direct.cpp:2687)
__device__ __forceinline__ float conv_acc_scale(const ConvGeom &c)
{
    return c.dscaleI ? (*c.dscaleI * c.filter_scale) : c.scaleO;
}

struct GemmArgs {
    const uint8_t *A = nullptr;    // u8 activations
    uint32_t lda = 0;        // bytes between consecutive m (transA = 0) or consecutive k (transA = 1)
    int transA = 0;          // 1: A stored [K][M]
    const int8_t *Bp = nullptr;    // packed right-hand side (fragment layout, see pack.hip)
    uint32_t M = 0, N = 0, K = 0;
    const int32_t *ob = nullptr;   // caller's offsetC (+ folded bias) [N]
    const int32_t *comp = nullptr; // blob's own compensation vector [N]
    const float *fold_bias = nullptr;  // if set, ob is not read: the offset is (int32)(round(fold_bias[n] * fold_scale) + comp[n])
    float fold_scale = 0;
    void *C = nullptr;             // [M][N] row-major
    int add_cin = 0;         // accumulate into the int32 bits already in C
    int stream_c = 0;        // set by the launcher: write C with the non-temporal hint
    int fp4 = 0;             // convolution only: operand bytes are pairs of E2M1 values (1-bit convolution), K counts bytes
    Epilogue epi;
    ConvGeom conv;       // used by launch_conv_u8s8 only
    // EPI_U8_GELU_DYN (256 x 256 tiles, M and N multiples of 256), and the filter-panel convolution with a u8 result in
    // ONE pass (launch_conv_u8s8, conv.absmax null): every workgroup resident at once
    GridSync sync;                 // from FusedSync::next(number of workgroups)
    float *dscale_out = nullptr;   // receives the scale the u8 result was quantised with
    uint32_t *status = nullptr;    // receives 0; or 1 when the grid-wide wait was abandoned: then nothing was quantised and
    float *C32 = nullptr;          //   the activated fp32 values y are in C32 [M][N] for a two-pass quantisation to pick up
    uint32_t *clear_ws = nullptr;  // optional: an array of kWsWords max slots whose maximum has been consumed; zeroed by one workgroup
};
hipError_t launch_gemm_u8s8(const GemmArgs &a, hipStream_t st);
// whether EPI_U8_GELU_DYN can run for an M x N x K product on the current device (grid of that many tiles = M / 256 * N / 256)
bool gemm_gelu_dyn_fits(uint32_t M, uint32_t N, uint32_t K);
// A = padded s8 image, M = n * OH * OW output pixels, N = output channels, K = fh * fw * ICp
hipError_t launch_conv_u8s8(const GemmArgs &a, hipStream_t st);
bool conv_fp4_ok(uint32_t M, uint32_t N);
// whether launch_conv_u8s8 would run the filter-panel kernel for this shape (the one that can gather from the caller's tensor)
bool conv_panel_ok(uint32_t N, uint32_t K);  // whether launch_conv_u8s8 has an fp4 kernel for this shape
uint32_t conv_onepass_max_grid(uint32_t K);  // most workgroups of the filter-panel kernel that a one-pass u8 convolution may span
uint32_t conv_panel_grid(uint32_t M);        // the grid the filter-panel kernel gets for M output pixels
void conv_force_panel(int v);  // 0: shared-pipeline kernel only; 2 / 4: panel kernel with 32 / 64 pixels per wave
// tuning / test hook: -1 = shape heuristic, 0 = general kernel, 1 = 256x256 tiles, 2 = 128x128 tiles
void gemm_force_tile(int tile);

// ---- convolution helpers (conv.hip) -------------------------------------------------------------
// u8 NCHWC8 (cx = 8) / NCHWC16 (cx = 16) -> s8 (x - 128), zero padded, [n][H+pt+pb][W+pl+pr][ALIGN(C,16)]
hipError_t launch_conv_pad(const uint8_t *in, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t cx, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, int8_t *out, hipStream_t st, uint32_t *clear_ws = nullptr);
// s8 NCHW filter -> offsetC[OC] and the fragment-layout matrix over K = (kh, kw, c)
hipError_t launch_conv_pack_filter(const int8_t *src, uint32_t OC, uint32_t IC, uint32_t fh, uint32_t fw, int32_t *offsetC,
    int8_t *dst, hipStream_t st);

// ---- int8 deconvolution (deconv.hip) ------------------------------------------------------------------
// filter s8 [ic][oc][taps] -> offsetC[taps * oc] and the convolution's packed matrix with rows tap * oc + o over K = ic
hipError_t launch_deconv_pack_filter(const int8_t *src, uint32_t IC, uint32_t OC, uint32_t taps, int32_t *offsetC, int8_t *dst,
    hipStream_t st);
hipError_t launch_nchw_to_c8_u8(const uint8_t *in, uint32_t N, uint32_t C, uint32_t HW, uint8_t *out, hipStream_t st);  // C % 8 == 0
hipError_t launch_repeat_f32(const float *src, uint32_t period, uint32_t n, float *out, hipStream_t st);  // out[i] = src[i % period]
hipError_t launch_relu_u8(uint8_t *q, uint32_t n, hipStream_t st);  // in place max(q, 128)
enum DeconvMode {
    DECONV_I32 = 0,          // int32 sums + round(scaleO * bias), optional integer ReLU; stored, max|.| folded into absmax
    DECONV_F32_DEQ = 1,      // the same sums, then cvt(acc) * factor
    DECONV_F32_SUM = 2,      // bias + sum of cvt(col) * factor in ascending (kh, kw) order, optional fp32 ReLU
    DECONV_U8 = 3,           // kernel == stride: the one u8 column byte per output, optional max(q, 128)
    DECONV_F32_FROM_U8 = 4   // kernel == stride: cvt(q - 128) * factor, optional fp32 ReLU
};
struct DeconvArgs {
    const void *col = nullptr;   // [n][fh * fw * oc / 16][ih][iw][16], int32 (u8 for the kernel == stride modes)
    void *out = nullptr;         // [n][oc / 16][oh][ow][16]
    uint32_t n = 0, oc = 0, ih = 0, iw = 0, oh = 0, ow = 0, fh = 0, fw = 0, sh = 0, sw = 0, pt = 0, pl = 0;
    const float *bias = nullptr; // [oc], 16-byte aligned
    float scaleO = 0;            // input scale * filter scale
    float factor = 0;            // 1 / scaleO, or 1 / (scale of the u8 columns)
    int relu = 0;
    int mode = 0;
    uint32_t *absmax = nullptr;  // DECONV_I32: cleared scratch slots
};
hipError_t launch_deconv_gather(const DeconvArgs &a, hipStream_t st);

// ---- int8 depthwise convolution (depthwise.hip) ---------------------------------------------------------
struct DepthwiseArgs {
    const uint8_t *in = nullptr;     // u8 [n][c/16][ih][iw][16]
    const int8_t *filter = nullptr;  // per 16-channel block: [(fh*fw+3)/4][16][4]
    const int32_t *offsetC = nullptr;  // [c], -128 * sum of the channel's taps
    const float *bias = nullptr;     // [c] or null
    float scaleO = 0;                // input scale * filter scale
    int32_t *out = nullptr;          // [n][c/16][oh][ow][16]
    uint32_t n = 0, c = 0, ih = 0, iw = 0, oh = 0, ow = 0, fh = 0, fw = 0, sh = 0, sw = 0;
    int relu = 0;
};
hipError_t launch_depthwise_u8s8_i32(const DepthwiseArgs &a, hipStream_t st);

// ---- weight storage of the post-training quantisation tool (ptq.hip) ---------------------------------------
// ws: kWsWords scratch words (overwritten). floor_: the caller's scale; the scale used, max(127 or 7 / max|w|, floor_),
// goes to *ds_out. n even for the 4-bit form, a multiple of 8 for the 1-bit form.
hipError_t launch_ws_int8(const float *w, uint32_t n, int8_t *q, uint32_t *ws, float floor_, float *ds_out, hipStream_t st);
hipError_t launch_ws_int4(const float *w, uint32_t n, int8_t *q, uint32_t *ws, float floor_, float *ds_out, hipStream_t st);
hipError_t launch_ws_bnn(const float *w, uint32_t n, uint8_t *bits, uint32_t *ws, float *ds_out, hipStream_t st);
// src4: q holds two 4-bit values per byte (value = nibble - 7), else one s8 per byte; dst 0: fp32 = (1 / scale) * value,
// 1: s8 = value, 2: u8 = value + 128 (dst 1 / 2 only from 4-bit storage)
hipError_t launch_ws_expand(const int8_t *q, uint32_t n, int src4, int dst, float scale, void *d, hipStream_t st);

// ---- 1-bit convolution (bnn.hip) ----------------------------------------------------------------
struct BnnArgs {
    const uint32_t *x = nullptr;     // [n][Hp][Wp][IC/32] dwords, zero-bit padded
    const uint32_t *w = nullptr;     // [OC/32][fh*fw][IC/32][32] dwords
    uint32_t M = 0;            // n * OH * OW output pixels
    uint32_t OHW = 0, OW = 0, sh = 0, sw = 0, Hp = 0, Wp = 0, IC = 0, OC = 0, fh = 0, fw = 0;
    int32_t *sums = nullptr;         // optional int32 sums, NCHWC8
    float *out = nullptr;            // optional fma(S, scale[oc], bias[oc]), NCHWC8
    const float *scale = nullptr, *bias = nullptr;
};
hipError_t launch_bnn_pack_input(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, float thr, uint32_t *out, hipStream_t st);
// src_fmt 0: DF_NCHW bit string, 1: DF_NCHWN16C8 bytes
hipError_t launch_bnn_pack_filter(const uint8_t *src, int src_fmt, uint32_t OC, uint32_t IC, uint32_t fhw, uint32_t *dst,
    hipStream_t st);
hipError_t launch_bnn_conv(const BnnArgs &a, int xnor, hipStream_t st);
// matrix-core route: operands expanded to int8 (+1 / -1 or 1 / 0), image in planes of 16 channels like conv_pad's
hipError_t launch_bnn_expand_input(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, float thr, int xnor, int8_t *out, hipStream_t st);
hipError_t launch_bnn_expand_filter(const uint32_t *src, uint32_t OC, uint32_t IC, uint32_t fhw, int xnor, int8_t *dst,
    hipStream_t st);
// the same with two E2M1 values per byte: image in planes of 32 channels [n][ic/32][Hp][Wp][16], K counted in bytes
hipError_t launch_bnn_expand_input_fp4(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
    uint32_t pt, uint32_t pb, uint32_t pl, uint32_t pr, float thr, int xnor, uint8_t *out, hipStream_t st);
hipError_t launch_bnn_expand_filter_fp4(const uint32_t *src, uint32_t OC, uint32_t IC, uint32_t fhw, int xnor, uint8_t *dst,
    hipStream_t st);

// ---- fp32 neighbours of the int8 GEMMs in an encoder layer (encoder.hip) --------------------------
// Each takes an optional `ws` (kWsWords scratch words, zeroed by the caller) into which max|out| is folded, and an
// optional `clear` (another such array, whose maximum has been consumed) that its first workgroup zeroes.
// qkv rows are [Q | K | V] of 3*H floats; head size 64 (H == heads * 64).
hipError_t launch_attention_f32(const float *qkv, uint32_t batch, uint32_t S, uint32_t H, uint32_t heads, float *ctx,
    uint32_t *ws, hipStream_t st, uint32_t *clear = nullptr);
// out = LayerNorm(a + b) (b may be null); H % 4 == 0, H <= 2048
hipError_t launch_add_layernorm(const float *a, const float *b, const float *gamma, const float *beta, uint32_t rows,
    uint32_t H, float *out, uint32_t *ws, hipStream_t st, uint32_t *clear = nullptr);
// store = false: x is left untouched, only max|gelu(x)| is folded into ws (pair it with launch_quantize_f32(..., gelu = 1))
hipError_t launch_gelu_f32(float *x, size_t n, uint32_t *ws, hipStream_t st, bool store = true, uint32_t *clear = nullptr);

// ---- weight pack --------------------------------------------------------------------------------
// src: s8, element (k, n) at src[k * sk + n * sn]. Writes the packed matrix and comp[n].
hipError_t launch_pack_mmm(const int8_t *src, uint32_t sk, uint32_t sn, uint32_t K, uint32_t N, int8_t *dst,
    int32_t *comp, hipStream_t st);
hipError_t launch_pack_mvm(const int8_t *src, uint32_t sk, uint32_t sn, uint32_t K, uint32_t N, int8_t *dst,
    int32_t *comp, hipStream_t st);

// ---- quantize family ----------------------------------------------------------------------------
// Device scratch word layout used by the two-pass kernels: ws[0] = max bits / max int.
// folds max |x| into the scratch slots ws; clears them first unless the caller just did
// only_if (device word, optional): the kernel does nothing unless *only_if != 0
hipError_t launch_absmax_f32(const float *x, uint32_t n, uint32_t *ws, hipStream_t st, bool ws_is_clear = false,
    const uint32_t *only_if = nullptr);
// Caller's scale = *ds_in (device) if given, else s_in. Dynamic when !mode or that scale <= 0:
// the scale used is max(caller's, 127 / max|x|) with max|x| taken from ws[0]. The scale used is
// written to *ds_out (device) when non-null.
hipError_t launch_quantize_f32(const float *x, uint32_t n, void *q, int to_u8, const uint32_t *ws, float s_in,
    const float *ds_in, int mode, float *ds_out, hipStream_t st, int gelu = 0, const uint32_t *only_if = nullptr);
hipError_t launch_absmax_i32(const int32_t *x, uint32_t n, uint32_t *ws, hipStream_t st);
// s0 = output scale (< 0: dynamic from ws[0]), s1 = scale of the int32 data; the resulting output
// scale is written to *ds_out (device) when non-null.
hipError_t launch_requant_i32(const int32_t *x, uint32_t n, void *q, int to_u8, const uint32_t *ws, float s0,
    float s1, float *ds_out, hipStream_t st);
hipError_t launch_u8_to_i8(const uint8_t *x, uint32_t n, int8_t *q, hipStream_t st);
hipError_t launch_dequant_i32(const int32_t *q, uint32_t n, const float *dscale, float scale, float *out,
    hipStream_t st);
hipError_t launch_dequant_u8(const uint8_t *q, uint32_t n, const float *dscale, float scale, float *out,
    hipStream_t st);
// out[n] = (int)round(bias[n] * s) + offsetC[n]; bias / offsetC may be null; s = scale or *dscaleA * scaleB
hipError_t launch_bias_offsetC(const float *bias, uint32_t N, const int32_t *offsetC, const float *dscaleA,
    float scaleB, int32_t *out, hipStream_t st);
hipError_t launch_requantize_i8(const int8_t *in, uint32_t n, float rescale, int8_t *out, hipStream_t st);
hipError_t launch_axpby_f32(uint32_t n, float a, const float *x, float b, float *y, hipStream_t st);  // y = fma(a, x, y * b)
hipError_t launch_fill_u32(uint32_t *p, uint32_t n, uint32_t v, hipStream_t st);
// Host side of a GridSync area (device_common.h): the device words and the running epoch. Every kernel launch that
// synchronises through the area takes the next epoch.
struct FusedSync {
    unsigned long long *slots = nullptr;   // kGridSyncMaxBlocks words, zeroed once when allocated
    unsigned long long *release = nullptr; // 64 release words, 8 words apart, zeroed once when allocated
    uint32_t epoch = 0;
    uint32_t spin_limit = 1u << 19;        // polling rounds (a microsecond or two each) before a waiting workgroup gives up
    // the device-side view for a launch of `grid` workgroups; advances the epoch
    GridSync next(uint32_t grid)
    {
        epoch += 1;
        GridSync g;
        g.slots = slots;
        g.release = release;
        g.epoch = epoch;
        g.blocks = grid;
        g.spin_limit = spin_limit;
        g.done = (unsigned *)(release + 1);  // a spare word beside release word 0
        return g;
    }
};
constexpr uint32_t kFusedSpinDefault = 1u << 19;
constexpr size_t kFusedSyncBytes = kGridSyncMaxBlocks * 8 + 64 * 64;
hipError_t launch_quantize_fused(const void *x, uint32_t n, void *q, int src_i32, int to_u8, FusedSync &fs, float s_in,
    float *ds_out, hipStream_t st, bool *taken);
hipError_t launch_mul_scalars(float *out, const float *a, const float *b, hipStream_t st);  // out[0] = a[0] * b[0]

// ---- u8 pooling and s8 concatenation (pool.hip) ---------------------------------------------------
struct PoolArgs {
    const uint8_t *in = nullptr;   // [planes][IH][IW][16]
    uint8_t *out = nullptr;        // [planes][OH][OW][16]
    uint32_t total = 0;            // planes * OH * OW, one lane each
    uint32_t IH = 0, IW = 0, OH = 0, OW = 0;
    uint32_t kh = 0, kw = 0, sh = 0, sw = 0, pt = 0, pl = 0;
    int mean = 0, count_include_pad = 0;
    uint32_t pool_full = 0;        // 65536 / (kh * kw)
};
// Every window must overlap the image (the caller checks); mean needs kh * kw <= 65536
hipError_t launch_pool_u8_c16(const PoolArgs &a, hipStream_t st);
// rows x len bytes from contiguous rows into rows `ostride` bytes apart; rescale: out = (s8)(r * in)
hipError_t launch_concat_i8(const void *in, void *out, uint32_t rows, uint32_t len, size_t ostride, int rescale,
    float r, hipStream_t st);

// All inputs of a concatenation in one launch (at most 8, everything 16-byte aligned: concat_multi_fits)
struct ConcatMulti {
    const uint8_t *in[8] = {};
    uint32_t len[8] = {};      // bytes per row of input j
    size_t off[8] = {};        // where input j starts inside an output row
    float r[8] = {};
    uint8_t rescale[8] = {};
    uint32_t num = 0, rows = 0;
    size_t ostride = 0;
    uint8_t *out = nullptr;
};
bool concat_multi_fits(const ConcatMulti &a);
hipError_t launch_concat_i8_multi(const ConcatMulti &a, hipStream_t st);

// ---- int8 LSTM cell (lstm.hip) ----------------------------------------------------------------------
struct LstmArgs {
    uint32_t batch = 0, xdim = 0, hdim = 0, column = 0;   // column = hdim when there is no projection
    const float *x = nullptr;      // row m at x + m * x_stride
    uint32_t x_stride = 0;
    float *state = nullptr;        // row m: [C (column) | H (hdim)]
    const float *bias = nullptr;   // row m at bias + m * bias_stride, 4 * column floats: i, g, f, o
    uint32_t bias_stride = 0;
    float scale_in = 0;            // caller's activation scale; <= 0: dynamic per row
    uint8_t *quant = nullptr;      // [batch][xdim + hdim]
    float *dscale = nullptr;       // [batch]
    const float *inter = nullptr;  // [batch][4 * column] products: fp32, or (acc_i32) exact int32 sums still to be
                                   // divided by dscale[m] * scale_w
    int acc_i32 = 0;
    float scale_w = 0;
    float *out = nullptr;          // row m at out + m * out_stride
    uint32_t out_stride = 0;
    float forget_bias = 0, zoneout_cell = 0, zoneout_output = 0;
    // projection (column != hdim): the gates leave their `column` activated values per row in act, and
    // launch_lstm_project forms out / the hidden state from proj, fp32 [hdim / 32][column][32]
    const float *proj = nullptr;
    float *act = nullptr;          // [batch][column]
};
hipError_t launch_lstm_xh_quant(const LstmArgs &a, hipStream_t st);
hipError_t launch_lstm_gates(const LstmArgs &a, hipStream_t st);
hipError_t launch_lstm_project(const LstmArgs &a, hipStream_t st);

}  // namespace bg
