// Per-net / per-call switches (field set of src/option.h; defaults of src/option.cpp:10-76).
// Only the fields the int8 path and the executor read are acted on; the rest are carried so
// that code written against ncnn::Option compiles unchanged.
#ifndef NCNN_OPTION_H
#define NCNN_OPTION_H

#include "platform.h"

namespace ncnn {

class Allocator;
class NCNN_EXPORT Option
{
public:
    Option();

    bool lightmode;        // release a bottom blob as soon as its last consumer ran
    int num_threads;       // OpenMP width for host-side work
    Allocator* blob_allocator;
    Allocator* workspace_allocator;
    int openmp_blocktime;
    bool use_winograd_convolution;
    bool use_sgemm_convolution;
    bool use_int8_inference; // gate of the int8 path in Convolution / ConvolutionDepthWise / InnerProduct
    bool use_vulkan_compute;
    // run layers that implement forward_hip with device-resident blobs (what use_vulkan_compute, src/option.h:84,
    // switches for the reference's GPU path); off: every layer sees host Mats
    bool use_hip_compute;
    bool use_bf16_storage;
    bool use_fp16_packed;
    bool use_fp16_storage;
    bool use_fp16_arithmetic;
    bool use_int8_packed;
    bool use_int8_storage;
    bool use_int8_arithmetic;
    bool use_packing_layout;
    int flush_denormals;
    bool use_local_pool_allocator;
};

} // namespace ncnn

#endif // NCNN_OPTION_H
