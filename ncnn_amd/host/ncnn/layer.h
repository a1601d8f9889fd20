// ncnn::Layer, the operator plug-in interface (src/layer.h:20-142), and the layer factories.
#ifndef NCNN_LAYER_H
#define NCNN_LAYER_H

#include <string>
#include <vector>

#include "hipmat.h"
#include "mat.h"
#include "modelbin.h"
#include "option.h"
#include "paramdict.h"
#include "platform.h"

namespace ncnn {

class NCNN_EXPORT Layer
{
public:
    Layer();
    virtual ~Layer();

    // all return 0 on success, -100 on allocation failure, -1 otherwise
    virtual int load_param(const ParamDict& pd);
    virtual int load_model(const ModelBin& mb);
    virtual int create_pipeline(const Option& opt);
    virtual int destroy_pipeline(const Option& opt);

    bool one_blob_only;
    bool support_inplace;
    bool support_vulkan;
    bool support_packing;
    bool support_bf16_storage;
    bool support_fp16_storage;
    bool support_int8_storage;
    bool support_tensor_storage;
    bool support_vulkan_packing;
    bool support_any_packing;
    bool support_vulkan_any_packing;
    bool support_batch; // takes a Mat with n > 1 whole; otherwise the net loops over samples
    // forward_hip is implemented: blobs stay in HBM between such layers (the part support_vulkan, src/layer.h:51-52,
    // plays for the reference's GPU path).  A layer that sets it handles batches (HipMat::n) itself.
    bool support_hip;
    int featmask;

    virtual int forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const;
    virtual int forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const;
    virtual int forward_inplace(std::vector<Mat>& bottom_top_blobs, const Option& opt) const;
    virtual int forward_inplace(Mat& bottom_top_blob, const Option& opt) const;

    // device-resident overloads, same contract as the VkMat overloads of src/layer.h:111-117: inputs and outputs
    // are blobs in HBM, all work is enqueued on cmd.stream, nothing is synchronised
    virtual int forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option& opt) const;
    virtual int forward_hip(const HipMat& bottom_blob, HipMat& top_blob, HipCommand& cmd, const Option& opt) const;
    virtual int forward_inplace_hip(HipMat& bottom_top_blob, HipCommand& cmd, const Option& opt) const;

    // Hooks with which the device-resident executor folds elementwise neighbours into a producer's epilogue
    // (conv -> Eltwise sum -> ReLU -> the next convolution's Quantize becomes one kernel).  Every statement of the
    // folded layers is applied per element in the original order, so results do not change.
    virtual bool hip_plain_sum() const;             // Eltwise: sum of exactly two inputs, no coefficients
    virtual bool hip_plain_relu() const;            // ReLU with slope 0
    virtual float hip_input_quantise_scale() const; // scale of this layer's own Quantize of an fp32 3-D bottom; 0: none
    virtual bool hip_can_fuse_tail() const;         // forward_hip_fused works for this layer as configured
    // top = [relu](forward(bottom) + *residual);  q8_scale != 0: top.q8 = Quantize(top, q8_scale) as well
    virtual int forward_hip_fused(const HipMat& bottom_blob, const HipMat* residual, bool relu, float q8_scale, HipMat& top_blob, HipCommand& cmd,
                                  const Option& opt) const;
    // When every consumer of a layer's fp32 output quantises it with one positive scale, the executor asks the layer
    // (once, after load_model) whether it can emit the quantised values alone; 0 = yes, and from then on
    // forward_hip_requantised(bottom, scale) gives the int8 blob float2int8(forward(bottom) * scale).
    virtual int hip_prepare_requantise(float scale);
    virtual int forward_hip_requantised(const HipMat& bottom_blob, float scale, HipMat& top_blob, HipCommand& cmd, const Option& opt) const;
    // Sibling layers that read the same blob (through a Split) and can run as ONE launch: a layer that can take part
    // describes itself with a key (layers with equal non-zero keys may share a launch); forward_hip_siblings is called on
    // the first layer of such a group with the whole group (itself included, all of its own class) and the one bottom,
    // and fills one top per layer, each identical to what that layer's forward_hip gives on its own.
    virtual unsigned long long hip_sibling_key() const;
    virtual int forward_hip_siblings(const std::vector<const Layer*>& group, const HipMat& bottom_blob, std::vector<HipMat>& top_blobs, HipCommand& cmd,
                                     const Option& opt, bool& done) const;
    // takes a narrow fp32 image (HipMat::narrow) as it is; everyone else gets it widened to the ordinary layout first
    virtual bool hip_accepts_narrow_input() const;
    // forward_hip of an int8 blob holding Quantize(x, s), s > 0, gives Quantize(forward_hip(x), s) (windowed max pooling)
    virtual bool hip_quantise_transparent() const;

    void* userdata;
    int typeindex;
    std::string type;
    std::string name;
    std::vector<int> bottoms;
    std::vector<int> tops;
    std::vector<Mat> bottom_shapes;
    std::vector<Mat> top_shapes;
};

typedef Layer* (*layer_creator_func)(void*);
typedef void (*layer_destroyer_func)(Layer*, void*);

struct layer_registry_entry
{
    const char* name;
    layer_creator_func creator; // NULL: the type is known but has no host implementation
    int typeindex;              // the reference's number for the type
};

// built-in type table.  The four int8 hot-path types are listed (so that registering them
// through Net::register_custom_layer takes the overwrite-builtin route) but deliberately have
// no host implementation: without the HIP layers registered, loading a net that uses them fails.
NCNN_EXPORT int layer_to_index(const char* type);
NCNN_EXPORT const char* layer_index_to_type(int index); // NULL for a number no built-in type has
NCNN_EXPORT Layer* create_layer(const char* type);
NCNN_EXPORT Layer* create_layer(int index);
NCNN_EXPORT Layer* create_layer_cpu(const char* type);
NCNN_EXPORT Layer* create_layer_cpu(int index);

#define DEFINE_LAYER_CREATOR(name)                          \
    ::ncnn::Layer* name##_layer_creator(void* /*userdata*/) \
    {                                                       \
        return new name;                                    \
    }

#define DEFINE_LAYER_DESTROYER(name)                                      \
    void name##_layer_destroyer(::ncnn::Layer* layer, void* /*userdata*/) \
    {                                                                     \
        delete layer;                                                     \
    }

} // namespace ncnn

#endif // NCNN_LAYER_H
