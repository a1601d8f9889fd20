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

    if (constantM < 0 || constantN < 0 || constantK < 0 || constantM > (1 << 24) || constantN > (1 << 24) || constantK > (1 << 24))
    {
        NCNN_LOGE("Gemm %s: constant sizes out of range (M %d, N %d, K %d)", name.c_str(), constantM, constantN, constantK);
        return -1;
    }
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
    // Blobs stay in HBM for every int8 form: constant or dynamic A, B and C, transposed inputs, transposed and N x 1 x M
    // output (Gemm::forward_int8, src/layer/gemm.cpp:745-966, runs them all in place as well).  A block-quantised B
    // (Gemm::forward_weight_block_quantize, src/layer/gemm.cpp:339-483: A is the first bottom blob, C a constant or the second)
    // stays there too; the reference's function knows no transposes and no other output shape.
    support_hip = quantize_term != 0 && !bottoms.empty()
                  && (!term_is_block_quant(quantize_term) || (constantA == 0 && constantB == 1 && bottoms.size() <= 2 && (bottoms.size() == 1 || constantC == 0)));
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
    // the device-resident forms need a constant B ready on the device (int8 rows, block-quantised fields, or the fp32 table
    // the forward pass quantises as the reference does, src/layer/gemm.cpp:826-860)
    support_hip = support_hip && ret == 0 && (weight_block_quantize || b_ready_int8 || constantB == 0 || (d_B && B_data.elemsize == 4u));
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

// One operand of the general form as it lies in HBM.  A 1-D or 2-D blob is the matrix itself, [rows][cols] with `stride`
// elements from row to row; a 3-D blob of height 1 -- c rows of w values to the reference (src/layer/gemm.cpp:769-785 reads
// A0.channel(j)[i]) -- is channels-last here, i.e. the TRANSPOSE of that matrix, [w][cp].
struct DeviceOperand
{
    const char* data; // sample 0
    size_t sample_bytes;
    int rows, cols;   // of the matrix the reference sees
    size_t stride;    // of the stored matrix, in elements
    bool stored_transposed;
    int n;
};

static bool device_operand(const HipMat& m, DeviceOperand& v)
{
    if (m.empty() || m.elemsize != 4u) return false;
    v.data = (const char*)m.data;
    v.n = m.n;
    if (m.dims == 1 || m.dims == 2)
    {
        v.rows = m.dims == 2 ? m.h : 1;
        v.cols = m.w;
        v.stride = (size_t)m.w;
        v.stored_transposed = false;
        v.sample_bytes = (size_t)v.rows * v.cols * 4;
        return true;
    }
    if (m.dims == 3 && m.h == 1 && !m.narrow())
    {
        v.rows = m.c;
        v.cols = m.w;
        v.stride = (size_t)m.cp;
        v.stored_transposed = true;
        v.sample_bytes = (size_t)m.w * m.cp * 4;
        return true;
    }
    return false;
}

int Gemm_hip::forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option& opt) const
{
    if (bottom_blobs.empty() || top_blobs.empty()) return -1;
    const bool network_form = weight_block_quantize
                              || (constantA == 0 && constantB == 1 && transA == 0 && output_transpose == 0 && output_N1M == 0 && bottom_blobs.size() == 1
                                  && b_ready_int8 && (bottom_blobs[0].dims == 1 || bottom_blobs[0].dims == 2));
    if (!network_form) return forward_hip_general(bottom_blobs, top_blobs[0], cmd, opt);
    if (!d_B) return -1;
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
    int bt = d_c ? constant_broadcast_type_C : -1;
    if (!constantC && bottom_blobs.size() == 2 && !bottom_blobs[1].empty())
    {
        // a block-quantised B with C as its second bottom blob: the shape must be one the reference names (src/layer/gemm.cpp:378-421)
        const HipMat& C = bottom_blobs[1];
        if (C.dims == 1 && C.w == 1) bt = 0;
        if (C.dims == 1 && C.w == M) bt = 1;
        if (C.dims == 1 && C.w == N) bt = 4;
        if (C.dims == 2 && C.w == 1 && C.h == M) bt = 2;
        if (C.dims == 2 && C.w == N && C.h == M) bt = 3;
        if (C.dims == 2 && C.w == N && C.h == 1) bt = 4;
        if (bt < 0 || C.elemsize != 4u || C.n != 1 || A.n != 1)
        {
            NCNN_LOGE("Gemm %s: unsupported C", name.c_str());
            return -1;
        }
        d_c = (const float*)C.data;
    }
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

// Every other int8 form on blobs that lie in HBM, one sample at a time (the reference runs a batch as a per-sample loop,
// src/net.cpp:654-700): the steps of Gemm::forward_int8 (src/layer/gemm.cpp:745-966) in its order -- A to row-major,
// one scale per row of A, one scale for the whole of B, B to K-contiguous rows, C by its shape, the product written plain
// or transposed -- each as the device kernel the host-Mat path uses too.
int Gemm_hip::forward_hip_general(const std::vector<HipMat>& bottom_blobs, HipMat& top, HipCommand& cmd, const Option&) const
{
    if (weight_block_quantize)
    {
        NCNN_LOGE("Gemm %s: a block-quantised B takes one 1-D or 2-D bottom blob on the device", name.c_str());
        return -1;
    }
    // which bottom blob is what (src/layer/gemm.cpp:747-748, 889-902)
    const HipMat* a_blob = constantA ? 0 : &bottom_blobs[0];
    const HipMat* b_blob = constantB ? 0 : (constantA ? &bottom_blobs[0] : (bottom_blobs.size() > 1 ? &bottom_blobs[1] : 0));
    const HipMat* c_blob = 0;
    if (!constantC)
    {
        if (constantA && constantB && bottom_blobs.size() == 1)
            c_blob = &bottom_blobs[0];
        else if ((constantA || constantB) && bottom_blobs.size() == 2)
            c_blob = &bottom_blobs[1];
        else if (bottom_blobs.size() == 3)
            c_blob = &bottom_blobs[2];
    }
    if ((!constantA && !a_blob) || (!constantB && !b_blob))
    {
        NCNN_LOGE("Gemm %s: %d bottom blobs do not cover its dynamic operands", name.c_str(), (int)bottom_blobs.size());
        return -1;
    }

    DeviceOperand a, b;
    int samples = 1;
    if (a_blob)
    {
        if (!device_operand(*a_blob, a))
        {
            NCNN_LOGE("Gemm %s: A must be an fp32 blob of 1 or 2 dimensions, or of 3 with height 1", name.c_str());
            return -1;
        }
        samples = a.n;
    }
    else
    {
        if (!d_A || (A_data.elemsize != 4u && A_data.elemsize != 1u)) return -1;
        a.data = (const char*)d_A;
        a.rows = A_data.dims == 3 ? A_data.c : A_data.h;
        a.cols = A_data.w;
        a.stride = A_data.dims == 3 ? A_data.cstep : (size_t)A_data.w;
        a.stored_transposed = false;
        a.sample_bytes = 0;
        a.n = 1;
        if (A_data.elemsize == 1u && !d_A_scales)
        {
            NCNN_LOGE("Gemm %s: int8 A without A_data_int8_scales", name.c_str());
            return -1;
        }
    }
    const bool a_int8 = !a_blob && A_data.elemsize == 1u;
    const int M = transA ? a.cols : a.rows, K = transA ? a.rows : a.cols;

    int N = 0;
    if (b_ready_int8)
    {
        N = constantN;
        if (constantK != K)
        {
            NCNN_LOGE("Gemm %s: K mismatch (%d vs constant %d)", name.c_str(), K, constantK);
            return -1;
        }
        b.n = 1;
    }
    else
    {
        if (b_blob)
        {
            if (!device_operand(*b_blob, b))
            {
                NCNN_LOGE("Gemm %s: B must be an fp32 blob of 1 or 2 dimensions, or of 3 with height 1", name.c_str());
                return -1;
            }
        }
        else
        {
            if (!d_B || B_data.elemsize != 4u)
            {
                NCNN_LOGE("Gemm %s: B must be an fp32 blob or a constant int8 table", name.c_str());
                return -1;
            }
            b.data = (const char*)d_B;
            b.rows = B_data.dims == 3 ? B_data.c : B_data.h;
            b.cols = B_data.w;
            b.stride = B_data.dims == 3 ? B_data.cstep : (size_t)B_data.w;
            b.stored_transposed = false;
            b.sample_bytes = 0;
            b.n = 1;
        }
        N = transB ? b.rows : b.cols;
        if ((transB ? b.cols : b.rows) != K)
        {
            NCNN_LOGE("Gemm %s: A and B disagree on K", name.c_str());
            return -1;
        }
        if (b_blob)
        {
            if (a_blob && b.n != samples)
            {
                NCNN_LOGE("Gemm %s: A and B disagree on the batch (%d vs %d)", name.c_str(), samples, b.n);
                return -1;
            }
            samples = b.n;
        }
    }

    // C: constant, or a blob classified by its shape (src/layer/gemm.cpp:904-943; a shape that matches nothing is read as a scalar)
    const char* c_data = 0;
    size_t c_sample_bytes = 0;
    int bt = -1;
    if (constantC)
    {
        if (!C_data.empty() && constant_broadcast_type_C >= 0 && d_C)
        {
            c_data = (const char*)d_C;
            bt = constant_broadcast_type_C;
        }
    }
    else if (c_blob && !c_blob->empty())
    {
        if (c_blob->elemsize != 4u || (a_blob || b_blob ? c_blob->n != samples : false))
        {
            NCNN_LOGE("Gemm %s: C must be an fp32 blob with the batch of the other operands", name.c_str());
            return -1;
        }
        if (!a_blob && !b_blob) samples = c_blob->n;
        bt = 0;
        if (c_blob->dims == 1 && c_blob->w == 1) bt = 0;
        if (c_blob->dims == 1 && c_blob->w == M) bt = 1;
        if (c_blob->dims == 1 && c_blob->w == N) bt = 4;
        if (c_blob->dims == 2 && c_blob->w == 1 && c_blob->h == M) bt = 2;
        if (c_blob->dims == 2 && c_blob->w == N && c_blob->h == M) bt = 3;
        if (c_blob->dims == 2 && c_blob->w == N && c_blob->h == 1) bt = 4;
        c_data = (const char*)c_blob->data;
        c_sample_bytes = c_blob->bytes() / (size_t)c_blob->n;
    }

    // the output: oh rows of ow values, or (output_N1M, src/layer/gemm.cpp:945-959) a 3-D blob of oh channels, height 1 and
    // width ow -- channels-last in HBM, so the rows are written to scratch and laid out (pad channels zero) by the converter
    const int ow = output_transpose ? M : N, oh = output_transpose ? N : M;
    if (output_N1M)
        top.create(ow, 1, oh, 4u, samples, &cmd);
    else
        top.create(ow, oh, 4u, samples, &cmd);
    if (top.empty()) return -100;

    ScopedScratch scratch(&cmd);
    void* st = cmd.stream;
    void* rows_out = 0;
    if (output_N1M)
    {
        rows_out = scratch.get((size_t)ow * oh * 4);
        if (!rows_out) return -100;
    }
    const size_t aq_stride = alignSize((size_t)K, 16);
    // scratch of one sample, used again by the next (everything is ordered on the one stream)
    void* a_rm = 0; // A as [M][K] row-major fp32, where the stored matrix is not that already
    void* a_q = 0;
    void* a_s = 0;
    const bool a_needs_transpose = a_int8 ? transA != 0 : (a.stored_transposed != (transA != 0));
    if (a_needs_transpose)
    {
        a_rm = scratch.get((size_t)M * K * (a_int8 ? 1 : 4));
        if (!a_rm) return -100;
    }
    if (!a_int8)
    {
        a_q = scratch.get((size_t)M * aq_stride);
        a_s = scratch.get((size_t)M * 4);
        if (!a_q || !a_s) return -100;
    }
    void* b_q = 0;
    void* b_t = 0;
    void* b_s = 0;
    // the stored matrix has b_srows rows of b_scols values; it is [N][K] already when (stored transposed) == (transB == 0)
    const int b_srows = b_ready_int8 ? 0 : (b.stored_transposed ? b.cols : b.rows), b_scols = b_ready_int8 ? 0 : (b.stored_transposed ? b.rows : b.cols);
    const bool b_needs_transpose = !b_ready_int8 && (b.stored_transposed == (transB != 0));
    if (!b_ready_int8)
    {
        b_q = scratch.get((size_t)b_srows * b_scols);
        b_s = scratch.get(4);
        if (!b_q || !b_s) return -100;
        if (b_needs_transpose)
        {
            b_t = scratch.get((size_t)N * K);
            if (!b_t) return -100;
        }
    }

    for (int s = 0; s < samples; s++)
    {
        int rc = 0;
        // ---- A: [M][K] K-contiguous int8 + one scale per row
        const char* a_src = a.data + (size_t)s * a.sample_bytes;
        const int8_t* d_aq = 0;
        const float* d_sa = 0;
        size_t d_aq_stride = 0;
        if (a_int8)
        {
            d_aq = (const int8_t*)a_src;
            d_aq_stride = a.stride;
            if (transA)
            {
                rc = ncnnhip_transpose_s8((const int8_t*)a_src, a.stride, a.rows, a.cols, (int8_t*)a_rm, (size_t)K, st);
                if (rc != 0) return to_ncnn_status(rc, "transpose A");
                d_aq = (const int8_t*)a_rm;
                d_aq_stride = (size_t)K;
            }
            d_sa = (const float*)d_A_scales;
        }
        else
        {
            const float* rows_src = (const float*)a_src;
            size_t rows_stride = a.stride;
            if (a_needs_transpose)
            {
                // the stored matrix ([cols][rows] when it lies transposed) -> its transpose, dense
                const int srows = a.stored_transposed ? a.cols : a.rows, scols = a.stored_transposed ? a.rows : a.cols;
                rc = ncnnhip_transpose_f32((const float*)a_src, a.stride, srows, scols, (float*)a_rm, (size_t)srows, st);
                if (rc != 0) return to_ncnn_status(rc, "transpose A");
                rows_src = (const float*)a_rm;
                rows_stride = (size_t)K;
            }
            rc = ncnnhip_gemm_quantize_rows(rows_src, rows_stride, M, K, (int8_t*)a_q, aq_stride, (float*)a_s, st);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_rows");
            d_aq = (const int8_t*)a_q;
            d_aq_stride = aq_stride;
            d_sa = (const float*)a_s;
        }

        // ---- B: [N][K] K-contiguous int8 + one scale
        const int8_t* d_bq = (const int8_t*)d_B;
        const float* d_sb = (const float*)d_B_scale;
        size_t d_bq_stride = (size_t)K;
        if (!b_ready_int8)
        {
            const char* b_src = b.data + (size_t)s * b.sample_bytes;
            rc = ncnnhip_gemm_quantize_tensor((const float*)b_src, b.stride, b_srows, b_scols, (int8_t*)b_q, (size_t)b_scols, (float*)b_s, st);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_quantize_tensor");
            d_sb = (const float*)b_s;
            d_bq = (const int8_t*)b_q;
            d_bq_stride = (size_t)b_scols;
            if (b_needs_transpose)
            {
                rc = ncnnhip_transpose_s8((const int8_t*)b_q, (size_t)b_scols, b_srows, b_scols, (int8_t*)b_t, (size_t)b_srows, st);
                if (rc != 0) return to_ncnn_status(rc, "transpose B");
                d_bq = (const int8_t*)b_t;
                d_bq_stride = (size_t)b_srows;
            }
        }

        const float* d_c = c_data ? (const float*)(c_data + (size_t)s * c_sample_bytes) : 0;
        float* d_out = output_N1M ? (float*)rows_out : (float*)top.data + (size_t)s * ow * oh;
        rc = ncnnhip_gemm_int8(d_aq, d_aq_stride, d_bq, d_bq_stride, M, N, K, d_sa, d_sb, 1, d_c, d_c ? bt : -1, alpha, beta, output_transpose, d_out, (size_t)ow, 0, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_gemm_int8");
        if (output_N1M)
        {
            rc = ncnnhip_chw_to_nhwc(rows_out, 4, oh, ow, 1, (size_t)ow, (size_t)ow * oh, (float*)top.data + (size_t)s * ow * top.cp, st);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_chw_to_nhwc");
        }
    }
    return 0;
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
