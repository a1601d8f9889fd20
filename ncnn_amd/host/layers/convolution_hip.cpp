#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include <vector>

#include "hip_layers.h"
#include "hip_support.h"

using namespace ncnn;

namespace ncnn_amd {

Convolution_hip::Convolution_hip(bool depthwise_type) : is_depthwise_type(depthwise_type)
{
    one_blob_only = true;
    support_inplace = false;
    support_batch = true; // Mat.n is folded into the pixel dimension of the implicit GEMM
    d_weight = d_weight_packed = d_weight_stem = d_weight_dw = d_bias = d_scale_in = d_scale_out = d_scale_out_uniform = d_input_scales = 0;
    uniform_scale_out = 0.f;
    output_abs_bound = 0.0;
    input_scale_count = 0;
    group = 1;
}

Convolution_hip::~Convolution_hip()
{
    Option opt;
    destroy_pipeline(opt);
}

int Convolution_hip::load_param(const ParamDict& pd)
{
    num_output = pd.get(0, 0);
    kernel_w = pd.get(1, 0);
    kernel_h = pd.get(11, kernel_w);
    dilation_w = pd.get(2, 1);
    dilation_h = pd.get(12, dilation_w);
    stride_w = pd.get(3, 1);
    stride_h = pd.get(13, stride_w);
    pad_left = pd.get(4, 0);
    pad_right = pd.get(15, pad_left);
    pad_top = pd.get(14, pad_left);
    pad_bottom = pd.get(16, pad_top);
    pad_value = pd.get(18, 0.f);
    bias_term = pd.get(5, 0);
    weight_data_size = pd.get(6, 0);
    group = is_depthwise_type ? pd.get(7, 1) : 1;
    int8_scale_term = pd.get(8, 0);
    activation_type = pd.get(9, 0);
    activation_params = pd.get(10, Mat());
    dynamic_weight = pd.get(19, 0);

    if (dynamic_weight)
    {
        NCNN_LOGE("%s: dynamic weights are not part of the int8 path", type.c_str());
        return -1;
    }
    // values a model file cannot mean (a damaged file): refused here, before any product of them is formed
    const int lim = 32767;
    if (num_output < 1 || num_output > (1 << 24) || kernel_w < 1 || kernel_h < 1 || kernel_w > lim || kernel_h > lim || dilation_w < 1 || dilation_h < 1 ||
        dilation_w > lim || dilation_h > lim || stride_w < 1 || stride_h < 1 || stride_w > lim || stride_h > lim || weight_data_size < 1 ||
        (long long)kernel_w * kernel_h > (1 << 24))
    {
        NCNN_LOGE("%s %s: parameters out of range (num_output %d, kernel %d x %d, dilation %d x %d, stride %d x %d, weight_data_size %d)", type.c_str(),
                  name.c_str(), num_output, kernel_w, kernel_h, dilation_w, dilation_h, stride_w, stride_h, weight_data_size);
        return -1;
    }
    if (group < 1 || num_output % group != 0) return -100; // the reference rejects an invalid group this way
    if (!int8_scale_term)
    {
        NCNN_LOGE("%s %s: no int8_scale_term; only the quantised path runs on this device runtime", type.c_str(), name.c_str());
        return -1;
    }
    support_int8_storage = true;
    // channels-last kernels exist for plain convolutions and for true depthwise ones; a grouped convolution in between
    // stays in HBM as well, through the planar kernel with a layout change on either side (forward_device)
    support_hip = true;
    return 0;
}

bool Convolution_hip::is_depthwise() const
{
    return group > 1 && group == num_output && weight_data_size == num_output * kernel_w * kernel_h;
}

ncnnhip_conv_desc Convolution_hip::describe(int w, int h, int channels, int batch) const
{
    ncnnhip_conv_desc desc;
    desc.w = w;
    desc.h = h;
    desc.c = channels;
    desc.batch = batch;
    desc.num_output = num_output;
    desc.kernel_w = kernel_w;
    desc.kernel_h = kernel_h;
    desc.dilation_w = dilation_w;
    desc.dilation_h = dilation_h;
    desc.stride_w = stride_w;
    desc.stride_h = stride_h;
    desc.pad_left = pad_left;
    desc.pad_right = pad_right;
    desc.pad_top = pad_top;
    desc.pad_bottom = pad_bottom;
    desc.pad_value = pad_value;
    desc.group = group;
    return desc;
}

int Convolution_hip::load_model(const ModelBin& mb)
{
    weight_data = mb.load(weight_data_size, 0);
    if (weight_data.empty()) return -100;
    if (bias_term)
    {
        bias_data = mb.load(num_output, 1);
        if (bias_data.empty()) return -100;
    }

    if (!is_depthwise_type)
    {
        // Convolution: one weight scale per output channel, one input scale (+ one top scale)
        weight_data_int8_scales = mb.load(num_output, 1);
        bottom_blob_int8_scales = mb.load(1, 1);
        if (int8_scale_term > 100) top_blob_int8_scales = mb.load(1, 1);
    }
    else
    {
        // ConvolutionDepthWise: term 1/101 stores one weight scale per group, term 2/102 a single
        // one; every table is then held broadcast to `group` entries
        const bool per_group = int8_scale_term == 1 || int8_scale_term == 101;
        Mat ws = mb.load(per_group ? group : 1, 1);
        Mat is = mb.load(1, 1);
        if (ws.empty() || is.empty()) return -100;
        weight_data_int8_scales.create(group);
        bottom_blob_int8_scales.create(group);
        for (int g = 0; g < group; g++)
        {
            weight_data_int8_scales[g] = per_group ? ws[g] : ws[0];
            bottom_blob_int8_scales[g] = is[0];
        }
        if (int8_scale_term > 100)
        {
            Mat ts = mb.load(1, 1);
            if (ts.empty()) return -100;
            top_blob_int8_scales.create(group);
            top_blob_int8_scales.fill(ts[0]);
        }
    }
    if (weight_data_int8_scales.empty() || bottom_blob_int8_scales.empty()) return -100;
    if (int8_scale_term > 100 && top_blob_int8_scales.empty()) return -100;

    // fp32 weights in the file are quantised here, once: per output channel for Convolution,
    // per group for ConvolutionDepthWise
    if (weight_data.elemsize == 4u)
    {
        Option opt_q;
        opt_q.num_threads = 1;
        const int rows = is_depthwise_type ? group : num_output;
        Mat as_rows = weight_data.reshape(weight_data_size / rows, rows);
        Mat q;
        quantize_to_int8(as_rows, q, weight_data_int8_scales, opt_q);
        if (q.empty()) return -100;
        weight_data = q.reshape(weight_data_size);
    }
    return 0;
}

int Convolution_hip::create_pipeline(const Option& /*opt*/)
{
    if (weight_data.elemsize != 1u)
    {
        NCNN_LOGE("%s %s: weights are not int8 after load_model", type.c_str(), name.c_str());
        return -1;
    }
    std::vector<float> scale_in((size_t)num_output);
    int rc = ncnnhip_fold_input_scales(weight_data_int8_scales, weight_data_int8_scales.w, bottom_blob_int8_scales, bottom_blob_int8_scales.w,
                                       num_output, scale_in.data());
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_fold_input_scales");
    {
        // |output| <= 127 * sum|w| * |scale_in| + |bias| for any input: what hip_prepare_requantise checks
        const size_t per_out = (size_t)weight_data_size / (size_t)num_output;
        const signed char* wq = (const signed char*)weight_data.data;
        double bound = 0.0;
        for (int p = 0; p < num_output; p++)
        {
            double sum = 0.0;
            for (size_t k = 0; k < per_out; k++) sum += abs((int)wq[(size_t)p * per_out + k]);
            double b = 127.0 * sum * fabs((double)scale_in[(size_t)p]) + (bias_term ? fabs((double)bias_data[p]) : 0.0);
            if (!(b <= bound)) bound = b; // a NaN sticks
        }
        output_abs_bound = bound;
    }

    int ret = 0;
    if (group == 1)
    {
        // the channels-last kernel reads weights as [num_output][tap][padded channels]; repack once here
        const int taps = kernel_w * kernel_h;
        if (num_output <= 0 || taps <= 0 || weight_data_size % (num_output * taps) != 0) return -1;
        ncnnhip_conv_desc desc;
        memset(&desc, 0, sizeof(desc));
        desc.c = weight_data_size / (num_output * taps);
        desc.w = kernel_w; // any extent the kernel fits in: only c, num_output and the kernel size matter for packing
        desc.h = kernel_h;
        desc.batch = 1;
        desc.num_output = num_output;
        desc.kernel_w = kernel_w;
        desc.kernel_h = kernel_h;
        desc.dilation_w = desc.dilation_h = desc.stride_w = desc.stride_h = 1;
        desc.group = 1;
        size_t packed_bytes = 0;
        rc = ncnnhip_conv_nhwc_sizes(&desc, 0, &packed_bytes, 0);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_nhwc_sizes");
        std::vector<int8_t> packed(packed_bytes);
        rc = ncnnhip_conv_pack_weights(&desc, (const int8_t*)weight_data.data, packed.data());
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_pack_weights");
        ret = upload_constant(packed.data(), packed_bytes, &d_weight_packed);
        // a layer with at most 4 input channels (the first layer of an image net) also gets the narrow-input packing
        desc.dilation_w = dilation_w;
        desc.dilation_h = dilation_h;
        desc.pad_value = pad_value;
        if (ret == 0 && ncnnhip_conv_stem_supported(&desc))
        {
            size_t stem_bytes = 0;
            rc = ncnnhip_conv_stem_sizes(&desc, 0, &stem_bytes, 0);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_stem_sizes");
            std::vector<int8_t> stem(stem_bytes);
            rc = ncnnhip_conv_stem_pack_weights(&desc, (const int8_t*)weight_data.data, stem.data());
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_stem_pack_weights");
            ret = upload_constant(stem.data(), stem_bytes, &d_weight_stem);
        }
    }
    else
        ret = upload_constant(weight_data.data, (size_t)weight_data_size, &d_weight);
    if (ret == 0 && is_depthwise())
    {
        // device-resident form of the depthwise kernel: weights as [tap][padded channels]
        size_t packed_bytes = 0;
        rc = ncnnhip_dwconv_packed_bytes(num_output, kernel_w, kernel_h, &packed_bytes);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_dwconv_packed_bytes");
        std::vector<int8_t> packed(packed_bytes);
        rc = ncnnhip_dwconv_pack_weights(num_output, kernel_w, kernel_h, (const int8_t*)weight_data.data, packed.data());
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_dwconv_pack_weights");
        ret = upload_constant(packed.data(), packed.size(), &d_weight_dw);
    }
    if (ret == 0) ret = upload_constant(scale_in.data(), scale_in.size() * 4, &d_scale_in);
    if (ret == 0 && bias_term) ret = upload_constant(bias_data.data, (size_t)num_output * 4, &d_bias);
    if (ret == 0 && int8_scale_term > 100)
    {
        std::vector<float> so((size_t)num_output);
        const int per = num_output / top_blob_int8_scales.w;
        for (int p = 0; p < num_output; p++) so[(size_t)p] = top_blob_int8_scales[p / per];
        ret = upload_constant(so.data(), so.size() * 4, &d_scale_out);
    }
    // input quantisation scales: the single value for Convolution; depthwise expands its per-group
    // table to channels once the channel count is known, which is at forward time for the first
    // blob -- the group table itself is what gets uploaded and indexed by channel/(channels/group)
    if (ret == 0) ret = upload_constant(bottom_blob_int8_scales.data, (size_t)bottom_blob_int8_scales.w * 4, &d_input_scales);
    input_scale_count = bottom_blob_int8_scales.w;
    if (ret != 0) destroy_pipeline(Option());
    return ret;
}

int Convolution_hip::destroy_pipeline(const Option& /*opt*/)
{
    void** all[] = {&d_weight, &d_weight_packed, &d_weight_stem, &d_weight_dw, &d_bias, &d_scale_in, &d_scale_out, &d_scale_out_uniform, &d_input_scales};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++)
    {
        if (*all[i]) ncnnhip_free(*all[i]);
        *all[i] = 0;
    }
    uniform_scale_out = 0.f;
    return 0;
}

int Convolution_hip::forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const
{
    if (!opt.use_int8_inference)
    {
        NCNN_LOGE("%s %s: use_int8_inference is off and there is no fp32 path in this runtime", type.c_str(), name.c_str());
        return -1;
    }
    if (!d_weight && !d_weight_packed)
    {
        NCNN_LOGE("%s %s: forward before create_pipeline", type.c_str(), name.c_str());
        return -1;
    }
    if (bottom_blob.dims != 3 || bottom_blob.elempack != 1 || (bottom_blob.elemsize != 4u && bottom_blob.elemsize != 1u))
    {
        NCNN_LOGE("%s %s: needs a pack-1 fp32 or int8 3-D blob", type.c_str(), name.c_str());
        return -1;
    }
    const int channels = bottom_blob.c, batch = bottom_blob.n;
    if (channels % group != 0 || num_output % group != 0) return -100;
    if (weight_data_size != (num_output / group) * (channels / group) * kernel_w * kernel_h * group)
    {
        NCNN_LOGE("%s %s: weight_data_size %d does not match %d input channels", type.c_str(), name.c_str(), weight_data_size, channels);
        return -1;
    }

    ncnnhip_conv_desc desc = describe(bottom_blob.w, bottom_blob.h, channels, batch);
    int outw = 0, outh = 0;
    int rc = ncnnhip_conv_out_shape(&desc, &outw, &outh);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_out_shape");

    const bool requant = int8_scale_term > 100;
    top_blob.create(outw, outh, num_output, requant ? (size_t)1u : (size_t)4u, 1, batch, opt.blob_allocator);
    if (top_blob.empty()) return -100;

    HipContext* ctx = context_for(opt);
    int ret = ctx->ensure_ready();
    if (ret != 0) return ret;
    ScopedLeases leases(ctx);
    void* st = ctx->stream;

    void* d_in = leases.get(mat_bytes(bottom_blob));
    void* d_out = leases.get(mat_bytes(top_blob));
    if (!d_in || !d_out) return -100;
    rc = ncnnhip_memcpy_h2d(d_in, bottom_blob.data, mat_bytes(bottom_blob), st);
    if (rc != 0) return to_ncnn_status(rc, "upload bottom blob");

    if (group == 1)
    {
        // channels-last path: quantise (or copy) into [n][h][w][Cp] int8, then the implicit GEMM
        size_t nhwc_bytes = 0, packed_bytes = 0, workspace_bytes = 0;
        rc = ncnnhip_conv_nhwc_sizes(&desc, &nhwc_bytes, &packed_bytes, &workspace_bytes);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_nhwc_sizes");
        void* d_nhwc = leases.get(nhwc_bytes);
        void* d_ws = workspace_bytes ? ctx->zeroed_workspace(workspace_bytes) : 0;
        if (!d_nhwc || (workspace_bytes && !d_ws)) return -100;
        rc = ncnnhip_to_nhwc_int8(&desc, d_in, (int)bottom_blob.elemsize, bottom_blob.cstep, bottom_blob.nstep, (const float*)d_input_scales, 1,
                                  (int8_t*)d_nhwc, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_to_nhwc_int8");
        rc = ncnnhip_conv_int8_nhwc(&desc, (const int8_t*)d_nhwc, (const int8_t*)d_weight_packed, (const float*)d_scale_in, (const float*)d_bias,
                                    (const float*)d_scale_out, make_activation(activation_type, activation_params), d_out, NCNNHIP_PLANAR,
                                    top_blob.cstep, top_blob.nstep, d_ws, workspace_bytes, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_int8_nhwc");
        rc = ncnnhip_memcpy_d2h(top_blob.data, d_out, mat_bytes(top_blob), st);
        if (rc == 0) rc = ncnnhip_stream_synchronize(st);
        return to_ncnn_status(rc, "download top blob");
    }

    const int8_t* d_xq = (const int8_t*)d_in;
    size_t q_cstep = bottom_blob.cstep, q_nstep = bottom_blob.nstep;
    if (bottom_blob.elemsize == 4u)
    {
        // Quantize: one scale for Convolution, the group's scale for every channel of a group
        q_cstep = alignSize((size_t)bottom_blob.w * bottom_blob.h, 16);
        q_nstep = q_cstep * channels;
        void* d_q = leases.get(q_nstep * batch);
        if (!d_q) return -100;
        const float* scales = (const float*)d_input_scales;
        void* d_expanded = 0;
        int nscales = 1;
        if (input_scale_count > 1)
        {
            std::vector<float> per_channel((size_t)channels);
            const int cg = channels / group;
            for (int q = 0; q < channels; q++) per_channel[(size_t)q] = bottom_blob_int8_scales[q / cg];
            d_expanded = leases.get((size_t)channels * 4);
            if (!d_expanded) return -100;
            rc = ncnnhip_memcpy_h2d(d_expanded, per_channel.data(), (size_t)channels * 4, st);
            if (rc == 0) rc = ncnnhip_stream_synchronize(st); // per_channel dies with this scope
            if (rc != 0) return to_ncnn_status(rc, "upload channel scales");
            scales = (const float*)d_expanded;
            nscales = channels;
        }
        rc = ncnnhip_quantize((const float*)d_in, bottom_blob.cstep, bottom_blob.nstep, (int8_t*)d_q, q_cstep, q_nstep, channels,
                              bottom_blob.w * bottom_blob.h, batch, scales, nscales, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_quantize");
        d_xq = (const int8_t*)d_q;
    }

    rc = ncnnhip_conv_int8(&desc, d_xq, q_cstep, q_nstep, (const int8_t*)d_weight, (const float*)d_scale_in, (const float*)d_bias,
                           (const float*)d_scale_out, make_activation(activation_type, activation_params), d_out, top_blob.cstep,
                           top_blob.nstep, 0, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_int8");
    rc = ncnnhip_memcpy_d2h(top_blob.data, d_out, mat_bytes(top_blob), st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return to_ncnn_status(rc, "download top blob");
}

// Device-resident form: bottom and top are channels-last blobs in HBM.  An fp32 bottom is quantised into scratch
// (one coalesced pass), an int8 bottom -- written by the previous layer's requantising epilogue -- feeds the kernel
// as it is.  Nothing is copied to or from the host and nothing waits.
int Convolution_hip::forward_hip(const HipMat& bottom, HipMat& top, HipCommand& cmd, const Option& opt) const
{
    return forward_hip_fused(bottom, 0, false, 0.f, top, cmd, opt);
}

float Convolution_hip::hip_input_quantise_scale() const
{
    return (support_hip && bottom_blob_int8_scales.w > 0) ? bottom_blob_int8_scales[0] : 0.f;
}

bool Convolution_hip::hip_can_fuse_tail() const
{
    // the folded tail lives in the fp32 epilogue of the pipelined kernel: plain convolution, zero border value
    return support_hip && group == 1 && int8_scale_term <= 100 && (int)(signed char)pad_value == 0;
}

int Convolution_hip::forward_hip_fused(const HipMat& bottom, const HipMat* residual, bool relu, float q8_scale, HipMat& top, HipCommand& cmd,
                                       const Option& opt) const
{
    return forward_device(bottom, residual, relu, q8_scale, 0.f, top, cmd, opt);
}

bool Convolution_hip::hip_accepts_narrow_input() const
{
    return support_hip; // the narrow-input kernel quantises straight from it; any other form widens it itself
}

int Convolution_hip::hip_prepare_requantise(float scale)
{
    // fp32-output layers only: the reference's own requantising epilogue (convolution.cpp:489-496) then runs with
    // the consumers' input scale in every channel, which is what their Quantize passes would compute
    if (!support_hip || int8_scale_term > 100 || !(scale > 0.f) || !d_scale_in) return -1;
    // Quantize is monotonic (so that it commutes with max pooling) only while value * scale stays inside the int32
    // range: beyond it the reference's float2int8 wraps to -127.  The weights bound the output, so this is known now.
    double gain = 1.0;
    if (activation_type == 2 && activation_params.w >= 1) gain = std::max(1.0, fabs((double)activation_params[0]));
    if (activation_type < 0 || activation_type > 3) return -1;
    if (!(output_abs_bound * gain * (double)scale < 1073741824.0)) return -1;
    if (uniform_scale_out == scale) return 0;
    if (d_scale_out_uniform)
    {
        ncnnhip_free(d_scale_out_uniform);
        d_scale_out_uniform = 0;
        uniform_scale_out = 0.f;
    }
    std::vector<float> so((size_t)num_output, scale);
    if (upload_constant(so.data(), so.size() * 4, &d_scale_out_uniform) != 0) return -1;
    uniform_scale_out = scale;
    return 0;
}

int Convolution_hip::forward_hip_requantised(const HipMat& bottom, float scale, HipMat& top, HipCommand& cmd, const Option& opt) const
{
    if (uniform_scale_out == 0.f || scale != uniform_scale_out) return -1;
    return forward_device(bottom, 0, false, 0.f, scale, top, cmd, opt);
}

// The one-launch form is taken where it measured faster than Quantize + convolution: every layer it accepts whose K
// stays in one workgroup, and of those that split K over workgroups (few output tiles, long K) only the 1x1 stride-1
// ones -- a 3x3 layer split nine ways quantises the same input pixels in nine workgroups (512 -> 512 on 7x7: 15.6 us
// against 14.6 in two launches; 1024 -> 256 1x1 on 14x14: 10.1 against 10.9).
static bool one_launch_from_float_pays(const ncnnhip_conv_desc& desc)
{
    if (!ncnnhip_conv_from_float_supported(&desc)) return false;
    size_t workspace_bytes = 0;
    if (ncnnhip_conv_from_float_workspace_bytes(&desc, &workspace_bytes) != 0) return false;
    const bool pointwise = desc.kernel_w == 1 && desc.kernel_h == 1 && desc.stride_w == 1 && desc.stride_h == 1;
    return workspace_bytes == 0 || pointwise;
}

int Convolution_hip::forward_device(const HipMat& bottom_in, const HipMat* residual, bool relu, float q8_scale, float only_scale, HipMat& top, HipCommand& cmd,
                                    const Option& opt) const
{
    HipMat bottom = bottom_in;
    if (bottom.narrow() && !(group == 1 && d_weight_stem))
    {
        int wret = cmd.widen(bottom_in, bottom);
        if (wret != 0) return wret;
    }
    const bool fused = residual || relu || q8_scale != 0.f;
    if (fused && !hip_can_fuse_tail()) return -1;
    if (!opt.use_int8_inference)
    {
        NCNN_LOGE("%s %s: use_int8_inference is off and there is no fp32 path in this runtime", type.c_str(), name.c_str());
        return -1;
    }
    if (!d_scale_in || (group == 1 ? !d_weight_packed : (is_depthwise() ? !d_weight_dw : !d_weight)))
    {
        NCNN_LOGE("%s %s: forward before create_pipeline", type.c_str(), name.c_str());
        return -1;
    }
    if (bottom.dims != 3 || (bottom.elemsize != 4u && bottom.elemsize != 1u))
    {
        NCNN_LOGE("%s %s: needs a 3-D fp32 or int8 blob", type.c_str(), name.c_str());
        return -1;
    }
    const int channels = bottom.c;
    if (channels % group != 0) return -100;
    if (weight_data_size != (num_output / group) * (channels / group) * kernel_w * kernel_h * group)
    {
        NCNN_LOGE("%s %s: weight_data_size %d does not match %d input channels", type.c_str(), name.c_str(), weight_data_size, channels);
        return -1;
    }
    ncnnhip_conv_desc desc = describe(bottom.w, bottom.h, channels, bottom.n);
    int outw = 0, outh = 0;
    int rc = ncnnhip_conv_out_shape(&desc, &outw, &outh);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_out_shape");

    if (bottom.elemsize == 1u && bottom.q8_scale != 0.f && bottom.q8_scale != bottom_blob_int8_scales[0])
    {
        NCNN_LOGE("%s %s: the int8 blob was quantised with scale %g, this layer expects %g", type.c_str(), name.c_str(), bottom.q8_scale, bottom_blob_int8_scales[0]);
        return -1;
    }
    const bool requant = int8_scale_term > 100 || only_scale != 0.f;
    const float* scale_out_table = (const float*)(only_scale != 0.f ? d_scale_out_uniform : d_scale_out);
    top.create(outw, outh, num_output, requant ? (size_t)1u : (size_t)4u, bottom.n, &cmd);
    if (top.empty()) return -100;
    if (only_scale != 0.f) top.q8_scale = only_scale;
    ScopedScratch scratch(&cmd);
    void* st = cmd.stream;

    if (residual && (residual->elemsize != 4u || residual->dims != 3 || residual->count() != top.count()))
    {
        NCNN_LOGE("%s %s: the residual blob does not have the output's shape", type.c_str(), name.c_str());
        return -1;
    }
    if (group == 1 && d_weight_stem && ncnnhip_conv_stem_supported(&desc))
    {
        // narrow input: quantise into the bordered 4-byte-per-pixel image, 4 neighbouring pixels per K chunk
        size_t image_bytes = 0, workspace_bytes = 0;
        rc = ncnnhip_conv_stem_sizes(&desc, &image_bytes, 0, &workspace_bytes);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_stem_sizes");
        void* image = scratch.get(image_bytes);
        if (!image) return -100;
        rc = ncnnhip_quantize_stem(&desc, bottom.data, (int)bottom.elemsize, bottom.cp, (const float*)d_input_scales, (int8_t*)image, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_quantize_stem");
        void* ws = workspace_bytes ? cmd.zeroed_workspace(workspace_bytes) : 0;
        if (workspace_bytes && !ws) return -100;
        ncnnhip_conv_fusion fu;
        fu.residual_dev = residual ? (const float*)residual->data : 0;
        fu.relu_after = relu ? 1 : 0;
        fu.quantised_out_dev = 0;
        fu.quantise_scale = q8_scale;
        if (q8_scale != 0.f)
        {
            top.q8.reset(new HipMat);
            top.q8->create(outw, outh, num_output, 1u, bottom.n, &cmd);
            if (top.q8->empty()) return -100;
            top.q8_scale = q8_scale;
            fu.quantised_out_dev = (int8_t*)top.q8->data;
        }
        rc = ncnnhip_conv_int8_stem(&desc, (const int8_t*)image, (const int8_t*)d_weight_stem, (const float*)d_scale_in, (const float*)d_bias,
                                    requant ? scale_out_table : 0, make_activation(activation_type, activation_params), top.data, fused ? &fu : 0, ws,
                                    workspace_bytes, st);
        return to_ncnn_status(rc, "ncnnhip_conv_int8_stem");
    }
    const int8_t* xq = (const int8_t*)bottom.data;
    if (bottom.elemsize == 4u && bottom.q8 && !bottom.q8->empty() && bottom.q8_scale == bottom_blob_int8_scales[0] && bottom.q8->count() == bottom.count())
        xq = (const int8_t*)bottom.q8->data; // the producer's epilogue already quantised this blob with our scale
    else if (bottom.elemsize == 4u && group == 1 && one_launch_from_float_pays(desc))
    {
        // one launch: the kernel's loader quantises the fp32 blob on its way into LDS
        ncnnhip_conv_fusion fu;
        fu.residual_dev = residual ? (const float*)residual->data : 0;
        fu.relu_after = relu ? 1 : 0;
        fu.quantised_out_dev = 0;
        fu.quantise_scale = q8_scale;
        if (q8_scale != 0.f)
        {
            top.q8.reset(new HipMat);
            top.q8->create(outw, outh, num_output, 1u, bottom.n, &cmd);
            if (top.q8->empty()) return -100;
            top.q8_scale = q8_scale;
            fu.quantised_out_dev = (int8_t*)top.q8->data;
        }
        size_t workspace_bytes = 0;
        rc = ncnnhip_conv_from_float_workspace_bytes(&desc, &workspace_bytes);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_from_float_workspace_bytes");
        void* ws = workspace_bytes ? cmd.zeroed_workspace(workspace_bytes) : 0;
        if (workspace_bytes && !ws) return -100;
        rc = ncnnhip_conv_int8_nhwc_from_float(&desc, bottom.data, 4, (const float*)d_input_scales, (const int8_t*)d_weight_packed, (const float*)d_scale_in,
                                               (const float*)d_bias, requant ? scale_out_table : 0, make_activation(activation_type, activation_params), top.data,
                                               fused ? &fu : 0, ws, workspace_bytes, st);
        return to_ncnn_status(rc, "ncnnhip_conv_int8_nhwc_from_float");
    }
    else if (bottom.elemsize == 4u)
    {
        void* q = scratch.get(bottom.count());
        if (!q) return -100;
        // every entry of a depthwise layer's input scale table holds the same value (load_model broadcasts the
        // single stored scale), so one scale serves all channels
        rc = ncnnhip_quantize_nhwc((const float*)bottom.data, (int8_t*)q, (size_t)bottom.n * bottom.h * bottom.w, channels, (const float*)d_input_scales, 1, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_quantize_nhwc");
        xq = (const int8_t*)q;
    }

    const ncnnhip_activation act = make_activation(activation_type, activation_params);
    if (group == 1)
    {
        size_t workspace_bytes = 0;
        rc = ncnnhip_conv_nhwc_sizes(&desc, 0, 0, &workspace_bytes);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_nhwc_sizes");
        void* ws = workspace_bytes ? cmd.zeroed_workspace(workspace_bytes) : 0;
        if (workspace_bytes && !ws) return -100;
        if (fused)
        {
            ncnnhip_conv_fusion fu;
            fu.residual_dev = residual ? (const float*)residual->data : 0;
            fu.relu_after = relu ? 1 : 0;
            fu.quantised_out_dev = 0;
            fu.quantise_scale = q8_scale;
            if (q8_scale != 0.f)
            {
                top.q8.reset(new HipMat);
                top.q8->create(outw, outh, num_output, 1u, bottom.n, &cmd);
                if (top.q8->empty()) return -100;
                top.q8_scale = q8_scale;
                fu.quantised_out_dev = (int8_t*)top.q8->data;
            }
            rc = ncnnhip_conv_int8_nhwc_fused(&desc, xq, (const int8_t*)d_weight_packed, (const float*)d_scale_in, (const float*)d_bias, act, (float*)top.data,
                                              &fu, ws, workspace_bytes, st);
            return to_ncnn_status(rc, "ncnnhip_conv_int8_nhwc_fused");
        }
        rc = ncnnhip_conv_int8_nhwc(&desc, xq, (const int8_t*)d_weight_packed, (const float*)d_scale_in, (const float*)d_bias, scale_out_table, act,
                                    top.data, NCNNHIP_CHANNELS_LAST, 0, 0, ws, workspace_bytes, st);
        return to_ncnn_status(rc, "ncnnhip_conv_int8_nhwc");
    }
    if (!is_depthwise())
    {
        // A grouped convolution that is not depthwise (ConvolutionDepthWise::forward_int8, src/layer/convolutiondepthwise.cpp:
        // 515-636, group by group): the planar kernel of the host-Mat path, on planar copies made and undone in HBM.
        const size_t hw = (size_t)bottom.w * bottom.h, ohw = (size_t)outw * outh;
        const size_t x_cstep = alignSize(hw, 16), x_nstep = x_cstep * channels;
        const size_t out_es = requant ? 1u : 4u;
        const size_t o_cstep = alignSize(ohw * out_es, 16) / out_es, o_nstep = o_cstep * num_output;
        void* x_planar = scratch.get(x_nstep * bottom.n);
        void* o_planar = scratch.get(o_nstep * out_es * bottom.n);
        if (!x_planar || !o_planar) return -100;
        rc = ncnnhip_nhwc_to_chw(xq, 1, channels, (int)hw, bottom.n, x_planar, x_cstep, x_nstep, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_nhwc_to_chw");
        rc = ncnnhip_conv_int8(&desc, (const int8_t*)x_planar, x_cstep, x_nstep, (const int8_t*)d_weight, (const float*)d_scale_in, (const float*)d_bias,
                               scale_out_table, act, o_planar, o_cstep, o_nstep, 0, st);
        if (rc != 0) return to_ncnn_status(rc, "ncnnhip_conv_int8");
        rc = ncnnhip_chw_to_nhwc(o_planar, (int)out_es, num_output, (int)ohw, bottom.n, o_cstep, o_nstep, top.data, st);
        return to_ncnn_status(rc, "ncnnhip_chw_to_nhwc");
    }
    rc = ncnnhip_dwconv_int8_nhwc(&desc, xq, (const int8_t*)d_weight_dw, (const float*)d_scale_in, (const float*)d_bias, scale_out_table, act, top.data, st);
    return to_ncnn_status(rc, "ncnnhip_dwconv_int8_nhwc");
}

Layer* Convolution_hip_creator(void*)
{
    return new Convolution_hip(false);
}
Layer* ConvolutionDepthWise_hip_creator(void*)
{
    return new Convolution_hip(true);
}
void hip_layer_destroyer(Layer* layer, void*)
{
    delete layer;
}

} // namespace ncnn_amd
