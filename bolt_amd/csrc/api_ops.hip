// C-ABI entry points of the remaining int8 callers of the matrix products: batched matmul, u8 pooling, concatenation
// with a common scale, the int8 LSTM cell and its weight transform. Argument validation, Bolt's tmp / scale
// conventions, host <-> device staging; no arithmetic on tensor data happens on the CPU.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

extern "C" {

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
    const size_t b = 2 * ((size_t)align_up(N, 16) * align_up(K, 8)) + (size_t)N * 4;  // 64-bit: a 32-bit product would wrap
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

}  // extern "C"
