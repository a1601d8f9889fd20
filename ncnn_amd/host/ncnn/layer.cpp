#include "layer.h"

#include <string.h>

namespace ncnn {

Layer::Layer()
{
    one_blob_only = false;
    support_inplace = false;
    support_vulkan = false;
    support_packing = false;
    support_bf16_storage = false;
    support_fp16_storage = false;
    support_int8_storage = false;
    support_tensor_storage = false;
    support_vulkan_packing = false;
    support_any_packing = false;
    support_vulkan_any_packing = false;
    support_batch = false;
    support_hip = false;
    featmask = 0;
    userdata = 0;
    typeindex = -1;
}

Layer::~Layer() {}

int Layer::load_param(const ParamDict&)
{
    return 0;
}
int Layer::load_model(const ModelBin&)
{
    return 0;
}
int Layer::create_pipeline(const Option&)
{
    return 0;
}
int Layer::destroy_pipeline(const Option&)
{
    return 0;
}

// default bridges between the out-of-place and in-place entry points
int Layer::forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
{
    if (!support_inplace) return -1;
    top_blobs = bottom_blobs;
    for (size_t i = 0; i < top_blobs.size(); i++)
    {
        top_blobs[i] = bottom_blobs[i].clone(opt.blob_allocator);
        if (top_blobs[i].empty()) return -100;
    }
    return forward_inplace(top_blobs, opt);
}

int Layer::forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const
{
    if (!support_inplace) return -1;
    top_blob = bottom_blob.clone(opt.blob_allocator);
    if (top_blob.empty()) return -100;
    return forward_inplace(top_blob, opt);
}

int Layer::forward_inplace(std::vector<Mat>&, const Option&) const
{
    return -1;
}
int Layer::forward_inplace(Mat&, const Option&) const
{
    return -1;
}

int Layer::forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option& opt) const
{
    // one-blob layers reached through the list form
    if (!one_blob_only || bottom_blobs.size() != 1) return -1;
    top_blobs.resize(1);
    return forward_hip(bottom_blobs[0], top_blobs[0], cmd, opt);
}
int Layer::forward_hip(const HipMat&, HipMat&, HipCommand&, const Option&) const
{
    return -1;
}
int Layer::forward_inplace_hip(HipMat&, HipCommand&, const Option&) const
{
    return -1;
}
bool Layer::hip_plain_sum() const
{
    return false;
}
bool Layer::hip_plain_relu() const
{
    return false;
}
float Layer::hip_input_quantise_scale() const
{
    return 0.f;
}
bool Layer::hip_can_fuse_tail() const
{
    return false;
}
unsigned long long Layer::hip_sibling_key() const
{
    return 0;
}
int Layer::forward_hip_siblings(const std::vector<const Layer*>&, const HipMat&, std::vector<HipMat>&, HipCommand&, const Option&, bool& done) const
{
    done = false;
    return 0;
}
int Layer::forward_hip_fused(const HipMat&, const HipMat*, bool, float, HipMat&, HipCommand&, const Option&) const
{
    return -1;
}
int Layer::hip_prepare_requantise(float)
{
    return -1;
}
int Layer::forward_hip_requantised(const HipMat&, float, HipMat&, HipCommand&, const Option&) const
{
    return -1;
}
bool Layer::hip_quantise_transparent() const
{
    return false;
}
bool Layer::hip_accepts_narrow_input() const
{
    return false;
}

// ---- built-in type table ------------------------------------------------------------------

Layer* Input_layer_creator(void*);
Layer* Split_layer_creator(void*);
Layer* ReLU_layer_creator(void*);
Layer* Pooling_layer_creator(void*);
Layer* Eltwise_layer_creator(void*);
Layer* Flatten_layer_creator(void*);
Layer* Softmax_layer_creator(void*);
Layer* Dropout_layer_creator(void*);

static const layer_registry_entry g_builtin[] = {
    {"Input", Input_layer_creator},
    {"Convolution", 0},
    {"ConvolutionDepthWise", 0},
    {"InnerProduct", 0},
    {"Gemm", 0},
    {"Split", Split_layer_creator},
    {"ReLU", ReLU_layer_creator},
    {"Pooling", Pooling_layer_creator},
    {"Eltwise", Eltwise_layer_creator},
    {"Flatten", Flatten_layer_creator},
    {"Softmax", Softmax_layer_creator},
    {"Dropout", Dropout_layer_creator},
};
static const int g_builtin_count = (int)(sizeof(g_builtin) / sizeof(g_builtin[0]));

int layer_to_index(const char* type)
{
    for (int i = 0; i < g_builtin_count; i++)
        if (strcmp(type, g_builtin[i].name) == 0) return i;
    return -1;
}

Layer* create_layer(int index)
{
    if (index < 0 || index >= g_builtin_count || !g_builtin[index].creator) return 0;
    Layer* layer = g_builtin[index].creator(0);
    layer->typeindex = index;
    return layer;
}

Layer* create_layer(const char* type)
{
    return create_layer(layer_to_index(type));
}
Layer* create_layer_cpu(const char* type)
{
    return create_layer(type);
}
Layer* create_layer_cpu(int index)
{
    return create_layer(index);
}

} // namespace ncnn
