#include "option.h"

#include <thread>

namespace ncnn {

Option::Option()
{
    lightmode = true;
    const unsigned hc = std::thread::hardware_concurrency();
    num_threads = hc ? (int)hc : 1;
    blob_allocator = 0;
    workspace_allocator = 0;
    openmp_blocktime = 20;
    use_winograd_convolution = true;
    use_sgemm_convolution = true;
    use_int8_inference = true;
    use_vulkan_compute = false;
    use_hip_compute = false;
    use_bf16_storage = false;
    use_fp16_packed = true;
    use_fp16_storage = true;
    use_fp16_arithmetic = true;
    use_int8_packed = true;
    use_int8_storage = true;
    use_int8_arithmetic = true;
    use_packing_layout = true;
    flush_denormals = 3;
    use_local_pool_allocator = true;
}

} // namespace ncnn
