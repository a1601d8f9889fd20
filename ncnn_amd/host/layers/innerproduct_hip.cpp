#include <vector>

#include "hip_layers.h"
#include "hip_support.h"

using namespace ncnn;

namespace ncnn_amd {

InnerProduct_hip::InnerProduct_hip()
{
    one_blob_only = true;
    support_inplace = false;
    d_weight = d_bias = d_scale_in = d_input_scale = 0;
}

InnerProduct_hip::~InnerProduct_hip()
{
    destroy_pipeline(Option());
}

int InnerProduct_hip::load_param(const ParamDict& pd)
{
    num_output = pd.get(0, 0);
    bias_term = pd.get(1, 0);
    weight_data_size = pd.get(2, 0);
    int8_scale_term = pd.get(8, 0);
    activation_type = pd.get(9, 0);
    activation_params = pd.get(10, Mat());
    if (num_output < 1 || num_output > (1 << 24) || weight_data_size < 1 || weight_data_size % num_output != 0)
    {
        NCNN_LOGE("InnerProduct %s: parameters out of range (num_output %d, weight_data_size %d)", name.c_str(), num_output, weight_data_size);
        return -1;
    }
    if (!int8_scale_term)
    {
        NCNN_LOGE("InnerProduct %s: no int8_scale_term; only the quantised path runs on this device runtime", name.c_str());
        return -1;
    }
    support_int8_storage = true;
    support_hip = true;
    return 0;
}

int InnerProduct_hip::load_model(const ModelBin& mb)
{
    weight_data = mb.load(weight_data_size, 0);
    if (weight_data.empty()) return -100;
    if (bias_term)
    {
        bias_data = mb.load(num_output, 1);
        if (bias_data.empty()) return -100;
    }
    weight_data_int8_scales = mb.load(num_output, 1);
    bottom_blob_int8_scales = mb.load(1, 1);
    if (weight_data_int8_scales.empty() || bottom_blob_int8_scales.empty()) return -100;

    if (weight_data.elemsize == 4u)
    {
        // fp32 weights in the file: quantise per output row now
        Option opt_q;
        opt_q.num_threads = 1;
        Mat rows = weight_data.reshape(weight_data_size / num_output, num_output);
        Mat q;
        quantize_to_int8(rows, q, weight_data_int8_scales, opt_q);
        if (q.empty()) return -100;
        weight_data = q.reshape(weight_data_size);
    }
    return 0;
}

int InnerProduct_hip::create_pipeline(const Option&)
{
    if (weight_data.elemsize != 1u) return -1;
    std::vector<float> scale_in((size_t)num_output);
    int rc = ncnnhip_fold_input_scales(weight_data_int8_scales, num_output, bottom_blob_int8_scales, 1, num_output, scale_in.data());
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_fold_input_scales");
    int ret = upload_constant(weight_data.data, (size_t)weight_data_size, &d_weight);
    if (ret == 0) ret = upload_constant(scale_in.data(), scale_in.size() * 4, &d_scale_in);
    if (ret == 0 && bias_term) ret = upload_constant(bias_data.data, (size_t)num_output * 4, &d_bias);
    if (ret == 0) ret = upload_constant(bottom_blob_int8_scales.data, 4, &d_input_scale);
    if (ret != 0) destroy_pipeline(Option());
    return ret;
}

int InnerProduct_hip::destroy_pipeline(const Option&)
{
    void** all[] = {&d_weight, &d_bias, &d_scale_in, &d_input_scale};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++)
    {
        if (*all[i]) ncnnhip_free(*all[i]);
        *all[i] = 0;
    }
    return 0;
}

int InnerProduct_hip::forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const
{
    if (!opt.use_int8_inference)
    {
        NCNN_LOGE("InnerProduct %s: use_int8_inference is off and there is no fp32 path in this runtime", name.c_str());
        return -1;
    }
    if (!d_weight) return -1;
    if (bottom_blob.elempack != 1 || (bottom_blob.elemsize != 4u && bottom_blob.elemsize != 1u)) return -1;
    const int num_input = weight_data_size / num_output;

    // 2-D blob whose rows are num_input long: one output row per input row; anything else is one
    // flattened vector in channel order (plane padding removed)
    int rows = 1;
    Mat flat;
    if (bottom_blob.dims == 2 && bottom_blob.w == num_input)
    {
        rows = bottom_blob.h;
        flat = bottom_blob;
        top_blob.create(num_output, rows, 4u, opt.blob_allocator);
    }
    else
    {
        const size_t count = (size_t)bottom_blob.w * bottom_blob.h * bottom_blob.d * bottom_blob.c;
        if (count != (size_t)num_input)
        {
            NCNN_LOGE("InnerProduct %s: blob has %zu values, weights expect %d", name.c_str(), count, num_input);
            return -1;
        }
        flat = bottom_blob.reshape(num_input, opt.workspace_allocator);
        top_blob.create(num_output, 4u, opt.blob_allocator);
    }
    if (flat.empty() || top_blob.empty()) return -100;

    HipContext* ctx = context_for(opt);
    int ret = ctx->ensure_ready();
    if (ret != 0) return ret;
    ScopedLeases leases(ctx);
    void* st = ctx->stream;

    const size_t in_bytes = (size_t)rows * num_input * flat.elemsize;
    void* d_in = leases.get(in_bytes);
    void* d_out = leases.get((size_t)rows * num_output * 4);
    if (!d_in || !d_out) return -100;
    int rc = ncnnhip_memcpy_h2d(d_in, flat.data, in_bytes, st);
    if (rc != 0) return to_ncnn_status(rc, "upload bottom blob");

    const int8_t* d_xq = (const int8_t*)d_in;
    if (flat.elemsize == 4u)
    {
        void* d_q = leases.get((size_t)rows * num_input);
        if (!d_q) return -100;
        rc = ncnnhip_quantize((const float*)d_in, (size_t)num_input, 0, (int8_t*)d_q, (size_t)num_input, 0, rows, num_input, 1,
                              (const float*)d_input_scale, 1, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_quantize");
        d_xq = (const int8_t*)d_q;
    }
    rc = ncnnhip_innerproduct_int8(d_xq, (size_t)num_input, rows, num_input, num_output, (const int8_t*)d_weight, (const float*)d_scale_in,
                                   (const float*)d_bias, make_activation(activation_type, activation_params), (float*)d_out,
                                   (size_t)num_output, 0, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_innerproduct_int8");
    rc = ncnnhip_memcpy_d2h(top_blob.data, d_out, (size_t)rows * num_output * 4, st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return to_ncnn_status(rc, "download top blob");
}

// Device-resident form: the blob is already in HBM.  A 1-D blob (or a 3-D one with a single pixel, whose
// channels-last rows are its channels) is one vector per sample; a 2-D blob with rows of num_input is a row-wise
// GEMM; any other 3-D blob is flattened to the planar order first.  The batch folds into the row count.
int InnerProduct_hip::forward_hip(const HipMat& bottom, HipMat& top, HipCommand& cmd, const Option& opt) const
{
    if (!opt.use_int8_inference)
    {
        NCNN_LOGE("InnerProduct %s: use_int8_inference is off and there is no fp32 path in this runtime", name.c_str());
        return -1;
    }
    if (!d_weight) return -1;
    if (bottom.elemsize != 4u && bottom.elemsize != 1u) return -1;
    const int num_input = weight_data_size / num_output;
    ScopedScratch scratch(&cmd);
    void* st = cmd.stream;

    const void* x = bottom.data;
    size_t x_stride = (size_t)num_input;
    int rows = bottom.n;
    if (bottom.dims == 2 && bottom.w == num_input)
    {
        rows = bottom.n * bottom.h;
        top.create(num_output, bottom.h, 4u, bottom.n, &cmd);
    }
    else
    {
        const size_t count = bottom.dims == 3 ? (size_t)bottom.w * bottom.h * bottom.c : (size_t)bottom.w * bottom.h;
        if (count != (size_t)num_input)
        {
            NCNN_LOGE("InnerProduct %s: blob has %zu values, weights expect %d", name.c_str(), count, num_input);
            return -1;
        }
        if (bottom.dims == 3 && bottom.w * bottom.h == 1)
            x_stride = (size_t)bottom.cp;
        else if (bottom.dims == 3)
        {
            const int hw = bottom.w * bottom.h;
            void* flat = scratch.get((size_t)bottom.n * num_input * bottom.elemsize);
            if (!flat) return -100;
            int rc = ncnnhip_nhwc_to_chw(bottom.data, (int)bottom.elemsize, bottom.c, hw, bottom.n, flat, (size_t)hw, (size_t)num_input, st);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_nhwc_to_chw");
            x = flat;
        }
        top.create(num_output, 4u, bottom.n, &cmd);
    }
    if (top.empty()) return -100;

    const int8_t* xq = (const int8_t*)x;
    size_t q_stride = x_stride;
    if (bottom.elemsize == 4u)
    {
        void* q = scratch.get((size_t)rows * num_input);
        if (!q) return -100;
        int rc = ncnnhip_quantize((const float*)x, x_stride, 0, (int8_t*)q, (size_t)num_input, 0, rows, num_input, 1, (const float*)d_input_scale, 1, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_quantize");
        xq = (const int8_t*)q;
        q_stride = (size_t)num_input;
    }
    size_t workspace_bytes = 0;
    int rc = ncnnhip_innerproduct_workspace_bytes(rows, num_input, num_output, &workspace_bytes);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_innerproduct_workspace_bytes");
    void* ws = workspace_bytes ? cmd.zeroed_workspace(workspace_bytes) : 0;
    if (workspace_bytes && !ws) return -100;
    rc = ncnnhip_innerproduct_int8_ws(xq, q_stride, rows, num_input, num_output, (const int8_t*)d_weight, (const float*)d_scale_in, (const float*)d_bias,
                                      make_activation(activation_type, activation_params), (float*)top.data, (size_t)num_output, ws, workspace_bytes, st);
    return to_ncnn_status(rc, "ncnnhip_innerproduct_int8_ws");
}

// The layer quantises an fp32 bottom with this one scale (Quantize with a single scale, as InnerProduct::forward_int8
// does, src/layer/innerproduct.cpp:231-247): a producer that can emit float2int8(value * scale) itself may do so.
float InnerProduct_hip::hip_input_quantise_scale() const
{
    return (support_hip && d_weight && bottom_blob_int8_scales.w > 0) ? bottom_blob_int8_scales[0] : 0.f;
}

Layer* InnerProduct_hip_creator(void*)
{
    return new InnerProduct_hip;
}

} // namespace ncnn_amd
