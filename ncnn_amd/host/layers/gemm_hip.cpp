#include <limits.h>

#include <vector>

#include "hip_layers.h"
#include "hip_support.h"

using namespace ncnn;

namespace ncnn_amd {

// quantize_term = bits*100 + has_input_scale*10 + block_code (src/layer/gemm.cpp:11-44)
static bool term_is_block_quant(int term)
{
    const int bits = term / 100, fmt = term % 100 / 10, code = term % 10;
    return (bits == 4 || bits == 6 || bits == 8) && (fmt == 0 || fmt == 1) && code >= 0 && code <= 2;
}
static int term_bits(int term)
{
    return term / 100;
}
static int term_block(int term)
{
    const int code = term % 10;
    return code == 0 ? 32 : code == 1 ? 64 : 128;
}
static bool term_has_input_scale(int term)
{
    return term % 100 / 10 == 1;
}

Gemm_hip::Gemm_hip()
{
    one_blob_only = false;
    support_inplace = false;
    weight_block_quantize = 0;
    B_data_int8_scale = 1.f;
    d_A = d_B = d_B_tiled = d_C = d_A_scales = d_B_scale = d_B_block_scales = d_B_input_scales = d_B_packed = d_B_packed_descales = 0;
    b_ready_int8 = 0;
}

Gemm_hip::~Gemm_hip()
{
    destroy_pipeline(Option());
}

int Gemm_hip::load_param(const ParamDict& pd)
{
    alpha = pd.get(0, 1.f);
    beta = pd.get(1, 1.f);
    transA = pd.get(2, 0);
    transB = pd.get(3, 0);
    constantA = pd.get(4, 0);
    constantB = pd.get(5, 0);
    constantC = pd.get(6, 0);
    constantM = pd.get(7, 0);
    constantN = pd.get(8, 0);
    constantK = pd.get(9, 0);
    constant_broadcast_type_C = pd.get(10, 0);
    output_N1M = pd.get(11, 0);
    output_elempack = pd.get(12, 0);
    output_elemtype = pd.get(13, 0);
    output_transpose = pd.get(14, 0);
    quantize_term = pd.get(18, 0);
    weight_block_quantize = term_is_block_quant(quantize_term);

    if (quantize_term == 0)
    {
        NCNN_LOGE("Gemm %s: no quantize_term; only the quantised paths run on this device runtime", name.c_str());
        return -1;
    }
    if (quantize_term == 4 || quantize_term == 5 || quantize_term == 6 || (quantize_term >= 400 && !weight_block_quantize))
    {
        NCNN_LOGE("Gemm unsupported quantize_term %d", quantize_term);
        return -1;
    }
    if (weight_block_quantize)
    {
        if (constantA != 0 || constantB != 1 || transA != 0 || transB != 1 || output_N1M != 0 || output_elempack != 0
            || (output_elemtype != 0 && output_elemtype != 1) || output_transpose != 0)
        {
            NCNN_LOGE("Gemm unsupported weight block quantize");
            return -1;
        }
    }
    if (constantA == 1 && (constantM == 0 || constantK == 0))
    {
        NCNN_LOGE("constantM and constantK must be non-zero when constantA enabled");
        return -1;
    }
    if (constantB == 1 && (constantN == 0 || constantK == 0))
    {
        NCNN_LOGE("constantN and constantK must be non-zero when constantB enabled");
        return -1;
    }
    if (constantC == 1 && (constant_broadcast_type_C < -1 || constant_broadcast_type_C > 4))
    {
        NCNN_LOGE("constant_broadcast_type_C must be -1 or 0~4 when constantC enabled");
        return -1;
    }
    // one bottom blob is enough when two of the three operands are constants
    if (constantA + constantB + constantC == 2) one_blob_only = true;
    // blobs stay in HBM for the form a network layer has: A is the only input, B (and C, if any) are constants, nothing
    // is transposed on the way in or out.  Every other form takes host Mats as before.
    support_hip = constantA == 0 && constantB == 1 && transA == 0 && output_transpose == 0 && output_N1M == 0 && bottoms.size() == 1
                  && (quantize_term != 0);
    return 0;
}

int Gemm_hip::load_model(const ModelBin& mb)
{
    if (constantA == 1)
    {
        A_data = transA == 0 ? mb.load(constantK, constantM, 0) : mb.load(constantM, constantK, 0);
        if (A_data.empty()) return -100;
    }
    if (constantB == 1)
    {
        if (transB == 0)
            B_data = mb.load(constantN, constantK, 0);
        else if (weight_block_quantize)
        {
            const size_t packed = ((size_t)constantK * term_bits(quantize_term) + 7) / 8;
            if (packed > (size_t)INT_MAX) return -100;
            B_data = mb.load((int)packed, constantN, 0);
        }
        else
            B_data = mb.load(constantK, constantN, 0);
        if (B_data.empty()) return -100;
    }
    if (constantC == 1 && constant_broadcast_type_C != -1)
    {
        switch (constant_broadcast_type_C)
        {
        case 0: C_data = mb.load(1, 0); break;
        case 1: C_data = mb.load(constantM, 0); break;
        case 2: C_data = mb.load(1, constantM, 0); break;
        case 3: C_data = mb.load(constantN, constantM, 0); break;
        case 4: C_data = mb.load(constantN, 1, 0); break;
        }
        if (C_data.empty()) return -100;
    }
    if (weight_block_quantize)
    {
        const int block = term_block(quantize_term);
        B_data_quantize_scales = mb.load((constantK + block - 1) / block, constantN, 1);
        if (B_data_quantize_scales.empty()) return -100;
        if (term_has_input_scale(quantize_term))
        {
            B_data_input_scales = mb.load(constantK, 1);
            if (B_data_input_scales.empty()) return -100;
        }
    }
    else
    {
        if (constantA == 1) A_data_int8_scales = mb.load(constantM, 1);
        if (constantB == 1)
        {
            Mat s = mb.load(1, 1);
            if (s.empty()) return -100;
            B_data_int8_scale = s[0];
        }
    }
    return 0;
}

int Gemm_hip::create_pipeline(const Option&)
{
    int ret = 0;
    if (constantA == 1) ret = upload_constant(A_data.data, A_data.total() * A_data.elemsize, &d_A);
    if (ret == 0 && constantC == 1 && !C_data.empty()) ret = upload_constant(C_data.data, C_data.total() * C_data.elemsize, &d_C);
    if (ret == 0 && constantA == 1 && !A_data_int8_scales.empty()) ret = upload_constant(A_data_int8_scales.data, (size_t)constantM * 4, &d_A_scales);

    if (ret == 0 && weight_block_quantize)
    {
        ret = upload_constant(B_data.data, (size_t)B_data.w * B_data.h, &d_B);
        if (ret == 0) ret = upload_constant(B_data_quantize_scales.data, B_data_quantize_scales.total() * 4, &d_B_block_scales);
        if (ret == 0 && !B_data_input_scales.empty()) ret = upload_constant(B_data_input_scales.data, (size_t)constantK * 4, &d_B_input_scales);
        // second form of B for few activation rows (decoding): matrix-core tiles
        if (ret == 0)
            ret = upload_blockquant_packed(B_data.data, (const float*)B_data_quantize_scales.data, constantN, constantK, term_bits(quantize_term),
                                           term_block(quantize_term), &d_B_packed, &d_B_packed_descales);
    }
    else if (ret == 0 && constantB == 1)
    {
        ret = upload_constant(B_data.data, B_data.total() * B_data.elemsize, &d_B);
        if (ret == 0 && B_data.elemsize == 1u)
        {
            ret = upload_constant(&B_data_int8_scale, 4, &d_B_scale);
            if (ret == 0 && transB == 0)
            {
                // stored [K][N]: bring it to K-contiguous rows once
                void* d_bt = 0;
                int rc = ncnnhip_malloc(&d_bt, (size_t)constantN * constantK);
                if (rc == 0) rc = ncnnhip_transpose_s8((const int8_t*)d_B, (size_t)constantN, constantK, constantN, (int8_t*)d_bt, (size_t)constantK, 0);
                if (rc == 0) rc = ncnnhip_stream_synchronize(0);
                if (rc != 0)
                {
                    if (d_bt) ncnnhip_free(d_bt);
                    ret = to_ncnn_status(rc, "transpose constant B");
                }
                else
                {
                    ncnnhip_free(d_B);
                    d_B = d_bt;
                }
            }
            if (ret == 0) b_ready_int8 = 1;
            if (ret == 0 && constantN % 256 == 0 && constantK % 64 == 0 && constantK <= 8192)
            {
                // second copy of B, laid out once for the 256x256 kernel (used from 128 output tiles up)
                int rc = ncnnhip_malloc(&d_B_tiled, (size_t)constantN * constantK);
                if (rc == 0) rc = ncnnhip_gemm_int8_tile_operand((const int8_t*)d_B, (size_t)constantK, constantN, constantK, 1, (int8_t*)d_B_tiled, 0);
                if (rc == 0) rc = ncnnhip_stream_synchronize(0);
                if (rc != 0) ret = to_ncnn_status(rc, "tile constant B");
            }
        }
    }
    // the device-resident form needs B ready on the device (int8 rows or block-quantised fields)
    support_hip = support_hip && ret == 0 && (weight_block_quantize || b_ready_int8);
    if (ret != 0) destroy_pipeline(Option());
    return ret;
}

int Gemm_hip::destroy_pipeline(const Option&)
{
    void** all[] = {&d_A, &d_B, &d_B_tiled, &d_C, &d_A_scales, &d_B_scale, &d_B_block_scales, &d_B_input_scales, &d_B_packed, &d_B_packed_descales};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++)
    {
        if (*all[i]) ncnnhip_free(*all[i]);
        *all[i] = 0;
    }
    b_ready_int8 = 0;
    return 0;
}

int Gemm_hip::forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const
{
    std::vector<Mat> ins(1, bottom_blob), outs(1);
    int ret = forward(ins, outs, opt);
    top_blob = outs[0];
    return ret;
}

int Gemm_hip::forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
{
    if (weight_block_quantize) return forward_block_quantize(bottom_blobs, top_blobs, opt);
    return forward_int8(bottom_blobs, top_blobs, opt);
}

int Gemm_hip::forward_hip(const HipMat& bottom_blob, HipMat& top_blob, HipCommand& cmd, const Option& opt) const
{
    std::vector<HipMat> ins(1, bottom_blob), outs(1);
    int ret = forward_hip(ins, outs, cmd, opt);
    top_blob = outs[0];
    return ret;
}

int Gemm_hip::forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option&) const
{
    if (bottom_blobs.size() != 1 || top_blobs.empty() || !d_B) return -1;
    const HipMat& A = bottom_blobs[0];
    if (A.elemsize != 4u || (A.dims != 1 && A.dims != 2))
    {
        NCNN_LOGE("Gemm %s: the device-resident form takes a 1-D or 2-D fp32 blob", name.c_str());
        return -1;
    }
    // a batch of 2-D blobs is n*h rows; a 1-D blob is one row per sample
    const int M = A.dims == 2 ? A.n * A.h : A.n, K = A.w, N = constantN;
    if (K != constantK)
    {
        NCNN_LOGE("Gemm %s: K mismatch (%d vs constant %d)", name.c_str(), K, constantK);
        return -1;
    }
    const float* d_c = constantC && !C_data.empty() && constant_broadcast_type_C >= 0 ? (const float*)d_C : 0;
    const int bt = d_c ? constant_broadcast_type_C : -1;
    if (A.n > 1 && (bt == 1 || bt == 2 || bt == 3))
    {
        NCNN_LOGE("Gemm %s: a per-row C does not extend to a batch", name.c_str());
        return -1;
    }
    HipMat& top = top_blobs[0];
    if (A.dims == 2)
        top.create(N, A.h, 4u, A.n, &cmd);
    else
        top.create(N, 4u, A.n, &cmd);
    if (top.empty()) return -100;
    void* st = cmd.stream;
    int rc = 0;
    if (weight_block_quantize)
    {
        ScopedScratch bq_scratch(&cmd);
        rc = blockquant_gemm_with_scratch(bq_scratch, (const float*)A.data, (size_t)K, M, N, K, d_B, term_bits(quantize_term), term_block(quantize_term), d_B_block_scales,
                                    d_B_input_scales, d_B_packed, d_B_packed_descales, d_c, bt, alpha, beta, (float*)top.data, (size_t)N, st);
        return to_ncnn_status(rc, "ncnnhip_gemm_blockquant");
    }
    if (!b_ready_int8)
    {
        NCNN_LOGE("Gemm %s: constant B is not int8 on the device", name.c_str());
        return -1;
    }
    ScopedScratch scratch(&cmd);
    const size_t aq_stride = alignSize((size_t)K, 16);
    void* q = scratch.get((size_t)M * aq_stride);
    void* sa = scratch.get((size_t)M * 4);
    if (!q || !sa) return -100;
    if (d_B_tiled && M % 256 == 0 && (long long)M * N >= 256ll * 256 * 128 && (bt == -1 || bt == 4))
    {
        // both operands in the 256x256 kernel's tiled layout: the quantiser writes A that way (aq_stride == K here)
        rc = ncnnhip_gemm_quantize_rows_tiled((const float*)A.data, (size_t)K, M, K, (int8_t*)q, (float*)sa, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_rows_tiled");
        rc = ncnnhip_gemm_int8_tiled((const int8_t*)q, (const int8_t*)d_B_tiled, M, N, K, (const float*)sa, (const float*)d_B_scale, 1, d_c, bt, alpha, beta,
                                     (float*)top.data, (size_t)N, st);
        return to_ncnn_status(rc, "ncnnhip_gemm_int8_tiled");
    }
    rc = ncnnhip_gemm_quantize_rows((const float*)A.data, (size_t)K, M, K, (int8_t*)q, aq_stride, (float*)sa, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_rows");
    rc = ncnnhip_gemm_int8((const int8_t*)q, aq_stride, (const int8_t*)d_B, (size_t)K, M, N, K, (const float*)sa, (const float*)d_B_scale, 1, d_c, bt, alpha, beta, 0,
                           (float*)top.data, (size_t)N, 0, st);
    return to_ncnn_status(rc, "ncnnhip_gemm_int8");
}

// Layers with equal keys may share a launch: block-quantised constant B in the packed form, the plain network form
// (one dynamic A, no transposes, fp32 out), no per-layer input scales (the shared launch has one activation operand),
// and the same K and field format.  0: this layer runs on its own.
unsigned long long Gemm_hip::hip_sibling_key() const
{
    if (!weight_block_quantize || !d_B_packed || !d_B_packed_descales || d_B_input_scales) return 0;
    if (constantA != 0 || constantB != 1 || transA != 0 || output_transpose != 0 || output_N1M != 0) return 0;
    if (constantC && !C_data.empty() && constant_broadcast_type_C >= 0 && constant_broadcast_type_C != 0 && constant_broadcast_type_C != 4) return 0; // per-row C: not with a batch
    if (!ncnnhip_gemm_blockquant_packed_supported(constantK)) return 0;
    return 1ull | ((unsigned long long)constantK << 1) | ((unsigned long long)term_bits(quantize_term) << 33) | ((unsigned long long)term_block(quantize_term) << 41);
}

// Every member's forward_hip on the one bottom, in one launch of ncnnhip_gemm_blockquant_packed_multi: bit for bit what
// the members give one by one (the same kernel; a workgroup only finds its matrix differently).  Up to four activation
// rows (the one-pass form of fp32 activations) and eight members; anything else: done = false, the layers run on their own.
int Gemm_hip::forward_hip_siblings(const std::vector<const Layer*>& group, const HipMat& A, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option&,
                                   bool& done) const
{
    done = false;
    if (group.size() < 2 || group.size() > 8 || top_blobs.size() != group.size()) return 0;
    if (A.elemsize != 4u || (A.dims != 1 && A.dims != 2)) return 0;
    const int M = A.dims == 2 ? A.n * A.h : A.n, K = A.w;
    if (M > 4 || K != constantK) return 0;
    const unsigned long long key = hip_sibling_key();
    if (!key) return 0;
    int n[8], bt[8];
    const uint8_t* w[8];
    const float* d[8];
    const float* c[8];
    float al[8], be[8];
    float* out[8];
    size_t stride[8];
    for (size_t i = 0; i < group.size(); i++)
    {
        const Gemm_hip* g = static_cast<const Gemm_hip*>(group[i]); // equal keys: the executor only groups layers of this class
        if (g->hip_sibling_key() != key) return 0;
        n[i] = g->constantN;
        w[i] = (const uint8_t*)g->d_B_packed;
        d[i] = (const float*)g->d_B_packed_descales;
        const bool has_c = g->constantC && !g->C_data.empty() && g->constant_broadcast_type_C >= 0;
        c[i] = has_c ? (const float*)g->d_C : 0;
        bt[i] = has_c ? g->constant_broadcast_type_C : -1;
        al[i] = g->alpha;
        be[i] = g->beta;
    }
    for (size_t i = 0; i < group.size(); i++)
    {
        HipMat& top = top_blobs[i];
        if (A.dims == 2)
            top.create(n[i], A.h, 4u, A.n, &cmd);
        else
            top.create(n[i], 4u, A.n, &cmd);
        if (top.empty()) return -100;
        out[i] = (float*)top.data;
        stride[i] = (size_t)n[i];
    }
    const int rc = ncnnhip_gemm_blockquant_packed_multi(A.data, 4, (size_t)K, M, K, (int)group.size(), n, w, d, term_bits(quantize_term), term_block(quantize_term), 0, c,
                                                        bt, al, be, out, stride, cmd.stream);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_blockquant_packed_multi");
    done = true;
    return 0;
}

// rows / row stride of a matrix held in a Mat: 2-D (h rows of w) or 3-D with h == 1 (c rows, cstep apart)
static int mat_rows(const Mat& m)
{
    return m.dims == 3 ? m.c : m.h;
}
static size_t mat_row_stride(const Mat& m)
{
    return m.dims == 3 ? m.cstep : (size_t)m.w;
}

// C operand classification shared by both paths (src/layer/gemm.cpp:887-943)
static int classify_c(const Mat& C, int M, int N)
{
    int bt = -2;
    if (C.dims == 1 && C.w == 1) bt = 0;
    if (C.dims == 1 && C.w == M) bt = 1;
    if (C.dims == 1 && C.w == N) bt = 4;
    if (C.dims == 2 && C.w == 1 && C.h == M) bt = 2;
    if (C.dims == 2 && C.w == N && C.h == M) bt = 3;
    if (C.dims == 2 && C.w == N && C.h == 1) bt = 4;
    return bt;
}

int Gemm_hip::forward_int8(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
{
    if (bottom_blobs.empty() && !(constantA && constantB)) return -1;
    HipContext* ctx = context_for(opt);
    int ret = ctx->ensure_ready();
    if (ret != 0) return ret;
    ScopedLeases leases(ctx);
    void* st = ctx->stream;
    int rc = 0;

    // ---- A: [M][K] K-contiguous int8 + one scale per row
    const Mat& A0 = constantA ? A_data : bottom_blobs[0];
    if (A0.elempack != 1 || (A0.elemsize != 4u && A0.elemsize != 1u)) return -1;
    const int a_rows = mat_rows(A0), a_cols = A0.w;
    const int M = transA ? a_cols : a_rows;
    const int K = transA ? a_rows : a_cols;
    const void* d_a0 = d_A;
    if (!constantA)
    {
        void* p = leases.get(A0.total() * A0.elemsize);
        if (!p) return -100;
        rc = ncnnhip_memcpy_h2d(p, A0.data, A0.total() * A0.elemsize, st);
        if (rc != 0) return to_ncnn_status(rc, "upload A");
        d_a0 = p;
    }
    size_t a_stride = mat_row_stride(A0);
    if (transA)
    {
        void* p = leases.get((size_t)M * K * A0.elemsize);
        if (!p) return -100;
        rc = A0.elemsize == 4u ? ncnnhip_transpose_f32((const float*)d_a0, a_stride, a_rows, a_cols, (float*)p, (size_t)K, st)
                               : ncnnhip_transpose_s8((const int8_t*)d_a0, a_stride, a_rows, a_cols, (int8_t*)p, (size_t)K, st);
        if (rc != 0) return to_ncnn_status(rc, "transpose A");
        d_a0 = p;
        a_stride = (size_t)K;
    }
    const int8_t* d_aq = (const int8_t*)d_a0;
    const float* d_sa = (const float*)d_A_scales;
    size_t aq_stride = a_stride;
    if (A0.elemsize == 4u)
    {
        aq_stride = alignSize((size_t)K, 16);
        void* q = leases.get((size_t)M * aq_stride);
        void* s = leases.get((size_t)M * 4);
        if (!q || !s) return -100;
        rc = ncnnhip_gemm_quantize_rows((const float*)d_a0, a_stride, M, K, (int8_t*)q, aq_stride, (float*)s, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_rows");
        d_aq = (const int8_t*)q;
        d_sa = (const float*)s;
    }
    else if (!d_sa)
    {
        NCNN_LOGE("Gemm %s: int8 A without A_data_int8_scales", name.c_str());
        return -1;
    }

    // ---- B: [N][K] K-contiguous int8 + one scale
    const int8_t* d_bq = 0;
    const float* d_sb = (const float*)d_B_scale;
    size_t bq_stride = 0;
    int N = 0;
    if (b_ready_int8)
    {
        N = constantN;
        if (constantK != K)
        {
            NCNN_LOGE("Gemm %s: K mismatch (%d vs constant %d)", name.c_str(), K, constantK);
            return -1;
        }
        d_bq = (const int8_t*)d_B;
        bq_stride = (size_t)K;
    }
    else
    {
        const Mat& B0 = constantB ? B_data : (constantA ? bottom_blobs[0] : (bottom_blobs.size() > 1 ? bottom_blobs[1] : Mat()));
        if (B0.empty() || B0.elempack != 1 || B0.elemsize != 4u)
        {
            NCNN_LOGE("Gemm %s: B must be an fp32 blob or a constant int8 table", name.c_str());
            return -1;
        }
        const int b_rows = mat_rows(B0), b_cols = B0.w;
        N = transB ? b_rows : b_cols;
        if ((transB ? b_cols : b_rows) != K)
        {
            NCNN_LOGE("Gemm %s: A and B disagree on K", name.c_str());
            return -1;
        }
        const void* d_b0 = constantB ? d_B : 0;
        if (!constantB)
        {
            void* p = leases.get(B0.total() * 4);
            if (!p) return -100;
            rc = ncnnhip_memcpy_h2d(p, B0.data, B0.total() * 4, st);
            if (rc != 0) return to_ncnn_status(rc, "upload B");
            d_b0 = p;
        }
        // whole-tensor dynamic quantisation, then (if stored [K][N]) transpose to K-contiguous rows
        void* q = leases.get((size_t)b_rows * b_cols);
        void* s = leases.get(4);
        if (!q || !s) return -100;
        rc = ncnnhip_gemm_quantize_tensor((const float*)d_b0, mat_row_stride(B0), b_rows, b_cols, (int8_t*)q, (size_t)b_cols, (float*)s, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_tensor");
        d_sb = (const float*)s;
        if (transB)
        {
            d_bq = (const int8_t*)q;
            bq_stride = (size_t)b_cols;
        }
        else
        {
            void* t = leases.get((size_t)N * K);
            if (!t) return -100;
            rc = ncnnhip_transpose_s8((const int8_t*)q, (size_t)b_cols, b_rows, b_cols, (int8_t*)t, (size_t)K, st);
            if (rc != 0) return to_ncnn_status(rc, "transpose B");
            d_bq = (const int8_t*)t;
            bq_stride = (size_t)K;
        }
    }

    // ---- C
    Mat C;
    int bt = 0;
    const float* d_c = 0;
    if (constantC)
    {
        C = C_data;
        bt = constant_broadcast_type_C;
        d_c = (const float*)d_C;
    }
    else
    {
        if (constantA && constantB && bottom_blobs.size() == 1)
            C = bottom_blobs[0];
        else if ((constantA || constantB) && bottom_blobs.size() == 2)
            C = bottom_blobs[1];
        else if (bottom_blobs.size() == 3)
            C = bottom_blobs[2];
        if (!C.empty())
        {
            const int cls = classify_c(C, M, N);
            if (cls >= 0) bt = cls;
            void* p = leases.get(C.total() * 4);
            if (!p) return -100;
            rc = ncnnhip_memcpy_h2d(p, C.data, C.total() * 4, st);
            if (rc != 0) return to_ncnn_status(rc, "upload C");
            d_c = (const float*)p;
        }
    }
    if (C.empty() || bt < 0) d_c = 0;

    // ---- output
    Mat& top = top_blobs[0];
    const int ow = output_transpose ? M : N, oh = output_transpose ? N : M;
    if (output_N1M)
        top.create(ow, 1, oh, 4u, opt.blob_allocator);
    else
        top.create(ow, oh, 4u, opt.blob_allocator);
    if (top.empty()) return -100;
    const size_t out_stride = top.dims == 3 ? top.cstep : (size_t)top.w;
    void* d_out = leases.get(top.total() * 4);
    if (!d_out) return -100;

    rc = ncnnhip_gemm_int8(d_aq, aq_stride, d_bq, bq_stride, M, N, K, d_sa, d_sb, 1, d_c, d_c ? bt : -1, alpha, beta, output_transpose, (float*)d_out,
                           out_stride, 0, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_int8");
    rc = ncnnhip_memcpy_d2h(top.data, d_out, top.total() * 4, st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return to_ncnn_status(rc, "download top blob");
}

int Gemm_hip::forward_block_quantize(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
{
    if (bottom_blobs.empty()) return -1;
    const Mat& A = bottom_blobs[0];
    if (A.elemsize != 4u || A.elempack != 1)
    {
        NCNN_LOGE("Gemm unsupported input");
        return -1;
    }
    const int K = A.w;
    if (K != constantK)
    {
        NCNN_LOGE("Gemm weight block quantize K mismatch");
        return -1;
    }
    const int M = mat_rows(A), N = constantN;

    Mat C;
    int bt = -1;
    if (constantC)
    {
        C = C_data;
        bt = constant_broadcast_type_C;
    }
    else if (bottom_blobs.size() == 2)
    {
        C = bottom_blobs[1];
        if (!C.empty())
        {
            bt = classify_c(C, M, N);
            if (bt < 0 || C.elemsize != 4u || C.elempack != 1)
            {
                NCNN_LOGE("Gemm unsupported C");
                return -1;
            }
        }
    }

    Mat& top = top_blobs[0];
    top.create(N, M, 4u, opt.blob_allocator);
    if (top.empty()) return -100;

    HipContext* ctx = context_for(opt);
    int ret = ctx->ensure_ready();
    if (ret != 0) return ret;
    ScopedLeases leases(ctx);
    void* st = ctx->stream;

    void* d_a = leases.get(A.total() * 4);
    void* d_out = leases.get((size_t)M * N * 4);
    if (!d_a || !d_out) return -100;
    int rc = ncnnhip_memcpy_h2d(d_a, A.data, A.total() * 4, st);
    if (rc != 0) return to_ncnn_status(rc, "upload A");
    const float* d_c = 0;
    if (!C.empty() && bt >= 0)
    {
        if (constantC)
            d_c = (const float*)d_C;
        else
        {
            void* p = leases.get(C.total() * 4);
            if (!p) return -100;
            rc = ncnnhip_memcpy_h2d(p, C.data, C.total() * 4, st);
            if (rc != 0) return to_ncnn_status(rc, "upload C");
            d_c = (const float*)p;
        }
    }
    rc = blockquant_gemm_with_scratch(leases, (const float*)d_a, mat_row_stride(A), M, N, K, d_B, term_bits(quantize_term), term_block(quantize_term), d_B_block_scales,
                                d_B_input_scales, d_B_packed, d_B_packed_descales, d_c, d_c ? bt : -1, alpha, beta, (float*)d_out, (size_t)N, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_blockquant");
    rc = ncnnhip_memcpy_d2h(top.data, d_out, (size_t)M * N * 4, st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return to_ncnn_status(rc, "download top blob");
}

Layer* Gemm_hip_creator(void*)
{
    return new Gemm_hip;
}

} // namespace ncnn_amd
