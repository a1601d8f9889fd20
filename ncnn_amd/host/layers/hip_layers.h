// The four ncnn::Layer implementations whose forward() runs on the MI355X.  They read the same
// param ids and the same .bin order as the reference layers they replace and are installed with
// Net::register_custom_layer under the built-in type names (see ncnnhip_register_int8_layers).
#ifndef NCNN_AMD_HIP_LAYERS_H
#define NCNN_AMD_HIP_LAYERS_H

#include "../ncnn/layer.h"
#include "ncnnhip.h"

namespace ncnn_amd {

// Convolution (src/layer/convolution.{h,cpp}) and ConvolutionDepthWise
// (src/layer/convolutiondepthwise.{h,cpp}) share everything except the group count and how
// the scale tables are indexed, so one class serves both type names.
class Convolution_hip : public ncnn::Layer
{
public:
    explicit Convolution_hip(bool depthwise_type);
    virtual ~Convolution_hip();
    virtual int load_param(const ncnn::ParamDict& pd);
    virtual int load_model(const ncnn::ModelBin& mb);
    virtual int create_pipeline(const ncnn::Option& opt);
    virtual int destroy_pipeline(const ncnn::Option& opt);
    virtual int forward(const ncnn::Mat& bottom_blob, ncnn::Mat& top_blob, const ncnn::Option& opt) const;
    virtual int forward_hip(const ncnn::HipMat& bottom_blob, ncnn::HipMat& top_blob, ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    virtual float hip_input_quantise_scale() const;
    virtual bool hip_can_fuse_tail() const;
    virtual int forward_hip_fused(const ncnn::HipMat& bottom_blob, const ncnn::HipMat* residual, bool relu, float q8_scale, ncnn::HipMat& top_blob,
                                  ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    virtual int hip_prepare_requantise(float scale);
    virtual bool hip_accepts_narrow_input() const;
    virtual int forward_hip_requantised(const ncnn::HipMat& bottom_blob, float scale, ncnn::HipMat& top_blob, ncnn::HipCommand& cmd,
                                        const ncnn::Option& opt) const;

public:
    // same member names as the reference layers
    int num_output, kernel_w, kernel_h, dilation_w, dilation_h, stride_w, stride_h;
    int pad_left, pad_right, pad_top, pad_bottom;
    float pad_value;
    int bias_term, weight_data_size, group, int8_scale_term, activation_type, dynamic_weight;
    ncnn::Mat activation_params;
    ncnn::Mat weight_data, bias_data;
    ncnn::Mat weight_data_int8_scales, bottom_blob_int8_scales, top_blob_int8_scales;

private:
    const bool is_depthwise_type;
    // device copies made at create_pipeline
    void* d_weight;        // group > 1: [num_output][c/group][kh][kw] as stored in the model
    void* d_weight_packed; // group == 1: [num_output][kh*kw][16*ceil(c/16)] for the channels-last kernel
    void* d_weight_stem;   // group == 1 and at most 4 input channels: [num_output][kh][ceil(kw/4)][4 pixels][4 channels]
    void* d_bias;
    void* d_scale_in;      // one per output channel: 1/(in_scale*w_scale), 0 when w_scale is 0
    void* d_scale_out;     // one per output channel, only when requantising
    void* d_scale_out_uniform; // num_output copies of uniform_scale_out: the consumers' common input scale
    float uniform_scale_out;   // 0: hip_prepare_requantise was not called
    double output_abs_bound;   // no input makes an output (before the activation) larger in magnitude
    int forward_device(const ncnn::HipMat& bottom_blob, const ncnn::HipMat* residual, bool relu, float q8_scale, float only_scale, ncnn::HipMat& top_blob,
                       ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    void* d_input_scales;  // the layer's input scale table (1 entry, or `group` entries for depthwise types)
    int input_scale_count; // 1 or group
    void* d_weight_dw;     // depthwise (channels == group == num_output): [kh*kw][16*ceil(c/16)]
    bool is_depthwise() const;
    ncnnhip_conv_desc describe(int w, int h, int channels, int batch) const;
};

// InnerProduct (src/layer/innerproduct.{h,cpp})
class InnerProduct_hip : public ncnn::Layer
{
public:
    InnerProduct_hip();
    virtual ~InnerProduct_hip();
    virtual int load_param(const ncnn::ParamDict& pd);
    virtual int load_model(const ncnn::ModelBin& mb);
    virtual int create_pipeline(const ncnn::Option& opt);
    virtual int destroy_pipeline(const ncnn::Option& opt);
    virtual int forward(const ncnn::Mat& bottom_blob, ncnn::Mat& top_blob, const ncnn::Option& opt) const;
    virtual int forward_hip(const ncnn::HipMat& bottom_blob, ncnn::HipMat& top_blob, ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    virtual float hip_input_quantise_scale() const;

public:
    int num_output, bias_term, weight_data_size, int8_scale_term, activation_type;
    ncnn::Mat activation_params;
    ncnn::Mat weight_data, bias_data, weight_data_int8_scales, bottom_blob_int8_scales;

private:
    void* d_weight;
    void* d_bias;
    void* d_scale_in;
    void* d_input_scale;
};

// Gemm with quantize_term (src/layer/gemm.{h,cpp}): int8 (per-row A, per-tensor B) and the
// weight-only block-quantised form
class Gemm_hip : public ncnn::Layer
{
public:
    Gemm_hip();
    virtual ~Gemm_hip();
    virtual int load_param(const ncnn::ParamDict& pd);
    virtual int load_model(const ncnn::ModelBin& mb);
    virtual int create_pipeline(const ncnn::Option& opt);
    virtual int destroy_pipeline(const ncnn::Option& opt);
    virtual int forward(const std::vector<ncnn::Mat>& bottom_blobs, std::vector<ncnn::Mat>& top_blobs, const ncnn::Option& opt) const;
    virtual int forward(const ncnn::Mat& bottom_blob, ncnn::Mat& top_blob, const ncnn::Option& opt) const;
    // device-resident forms: the shape a network layer has (one dynamic A, constant B, constant or no C: rows of a batch
    // folded into one product) and, sample by sample, every other int8 form
    virtual int forward_hip(const std::vector<ncnn::HipMat>& bottom_blobs, std::vector<ncnn::HipMat>& top_blobs, ncnn::HipCommand& cmd,
                            const ncnn::Option& opt) const;
    virtual int forward_hip(const ncnn::HipMat& bottom_blob, ncnn::HipMat& top_blob, ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    // block-quantised Gemms on the same activation rows (gate + up of a decoder layer behind one Split) as one launch
    virtual unsigned long long hip_sibling_key() const;
    virtual int forward_hip_siblings(const std::vector<const ncnn::Layer*>& group, const ncnn::HipMat& bottom_blob, std::vector<ncnn::HipMat>& top_blobs,
                                     ncnn::HipCommand& cmd, const ncnn::Option& opt, bool& done) const;

public:
    float alpha, beta;
    int transA, transB, constantA, constantB, constantC, constantM, constantN, constantK;
    int constant_broadcast_type_C, output_N1M, output_elempack, output_elemtype, output_transpose;
    int quantize_term, weight_block_quantize;
    ncnn::Mat A_data, B_data, C_data, A_data_int8_scales, B_data_quantize_scales, B_data_input_scales;
    float B_data_int8_scale;

private:
    int forward_int8(const std::vector<ncnn::Mat>& bottom_blobs, std::vector<ncnn::Mat>& top_blobs, const ncnn::Option& opt) const;
    int forward_block_quantize(const std::vector<ncnn::Mat>& bottom_blobs, std::vector<ncnn::Mat>& top_blobs, const ncnn::Option& opt) const;
    int forward_hip_general(const std::vector<ncnn::HipMat>& bottom_blobs, ncnn::HipMat& top_blob, ncnn::HipCommand& cmd, const ncnn::Option& opt) const;
    void* d_A;        // constant A as loaded (fp32 or int8), row-major as stored
    void* d_B;        // constant B: int8 [N][K] for the int8 path (already K-contiguous), packed bytes for block quant
    void* d_B_tiled;  // the same int8 B in the 256x256 Gemm kernel's tiled operand layout (N % 256 == 0, K % 64 == 0), else null
    void* d_C;
    void* d_A_scales; // [M] when A is constant int8
    void* d_B_scale;  // [1]
    void* d_B_block_scales;
    void* d_B_input_scales;
    void* d_B_packed;          // block-quantised B as matrix-core tiles + its descales (null when K has no kernel for them)
    void* d_B_packed_descales;
    int b_ready_int8; // constant B sits on the device quantised and transposed
};

// MultiHeadAttention with block-quantised weights (src/layer/multiheadattention.{h,cpp})
class MultiHeadAttention_hip : public ncnn::Layer
{
public:
    MultiHeadAttention_hip();
    virtual ~MultiHeadAttention_hip();
    virtual int load_param(const ncnn::ParamDict& pd);
    virtual int load_model(const ncnn::ModelBin& mb);
    virtual int create_pipeline(const ncnn::Option& opt);
    virtual int destroy_pipeline(const ncnn::Option& opt);
    virtual int forward(const std::vector<ncnn::Mat>& bottom_blobs, std::vector<ncnn::Mat>& top_blobs, const ncnn::Option& opt) const;
    // the same on blobs that already lie in HBM (2-D blobs are dense there; a per-head mask arrives channels-last)
    virtual int forward_hip(const std::vector<ncnn::HipMat>& bottom_blobs, std::vector<ncnn::HipMat>& top_blobs, ncnn::HipCommand& cmd, const ncnn::Option& opt) const;

public:
    int embed_dim, num_heads, weight_data_size, kdim, vdim, attn_mask, kv_cache, quantize_term, weight_block_quantize;
    float scale;
    // index 0..3 = the q, k, v and out projections
    ncnn::Mat weight_data[4], bias_data[4], weight_data_quantize_scales[4], weight_data_input_scales[4];

private:
    void* dev[4][6]; // per projection: weight fields, block scales, input scales (or 0), bias, matrix-core tiles and their descales (or 0)
    void* dev_qkv[6]; // the same six for the q, k and v matrices as one (self-attention with equal input widths and no input scales), or all 0
};

ncnn::Layer* MultiHeadAttention_hip_creator(void* userdata);
ncnn::Layer* Convolution_hip_creator(void* userdata);
ncnn::Layer* ConvolutionDepthWise_hip_creator(void* userdata);
ncnn::Layer* InnerProduct_hip_creator(void* userdata);
ncnn::Layer* Gemm_hip_creator(void* userdata);
void hip_layer_destroyer(ncnn::Layer* layer, void* userdata);

} // namespace ncnn_amd

#endif // NCNN_AMD_HIP_LAYERS_H
