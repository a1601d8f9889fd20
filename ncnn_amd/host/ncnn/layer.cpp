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

// The index of a type is its place in the reference's list of layers (the ncnn_add_layer calls of src/CMakeLists.txt:66-176,
// numbered from 0 by cmake/ncnn_add_layer.cmake into layer_type_enum.h): a .param.bin file names its layers by these numbers.
static const layer_registry_entry g_builtin[] = {
    {"Input", Input_layer_creator, 16},
    {"Convolution", 0, 6},
    {"ConvolutionDepthWise", 0, 42},
    {"InnerProduct", 0, 15},
    {"Gemm", 0, 74},
    {"MultiHeadAttention", 0, 79},
    {"Split", Split_layer_creator, 33},
    {"ReLU", ReLU_layer_creator, 26},
    {"Pooling", Pooling_layer_creator, 21},
    {"Eltwise", Eltwise_layer_creator, 10},
    {"Flatten", Flatten_layer_creator, 14},
    {"Softmax", Softmax_layer_creator, 32},
    {"Dropout", Dropout_layer_creator, 9},
};
static const int g_builtin_count = (int)(sizeof(g_builtin) / sizeof(g_builtin[0]));

static const layer_registry_entry* builtin_of(int index)
{
    for (int i = 0; i < g_builtin_count; i++)
        if (g_builtin[i].typeindex == index) return &g_builtin[i];
    return 0;
}

int layer_to_index(const char* type)
{
    for (int i = 0; i < g_builtin_count; i++)
        if (strcmp(type, g_builtin[i].name) == 0) return g_builtin[i].typeindex;
    return -1;
}

const char* layer_index_to_type(int index)
{
    const layer_registry_entry* e = builtin_of(index);
    return e ? e->name : 0;
}

Layer* create_layer(int index)
{
    const layer_registry_entry* e = builtin_of(index);
    if (!e || !e->creator) return 0;
    Layer* layer = e->creator(0);
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
