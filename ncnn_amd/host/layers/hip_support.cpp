#include "hip_support.h"

#include "../ncnn/platform.h"

namespace ncnn_amd {

HipBlobAllocator::HipBlobAllocator()
{
    pool.set_size_compare_ratio(0.f);
}
HipBlobAllocator::~HipBlobAllocator() {}
void* HipBlobAllocator::fastMalloc(size_t size)
{
    return pool.fastMalloc(size);
}
void HipBlobAllocator::fastFree(void* ptr)
{
    pool.fastFree(ptr);
}

HipContext* context_for(const ncnn::Option& opt)
{
    if (HipBlobAllocator* a = dynamic_cast<HipBlobAllocator*>(opt.blob_allocator)) return &a->context;
    static thread_local HipContext per_thread;
    return &per_thread;
}

int to_ncnn_status(int rc, const char* where)
{
    if (rc == 0) return 0;
    NCNN_LOGE("%s failed: %s", where, ncnnhip_last_error());
    return rc == NCNNHIP_OOM ? -100 : -1;
}

int upload_constant(const void* host, size_t bytes, void** dev)
{
    *dev = 0;
    if (bytes == 0) return 0;
    int rc = ncnnhip_init(0);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_init");
    rc = ncnnhip_malloc(dev, bytes);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_malloc");
    rc = ncnnhip_memcpy_h2d(*dev, host, bytes, 0);
    if (rc == 0) rc = ncnnhip_stream_synchronize(0);
    return to_ncnn_status(rc, "upload_constant");
}

} // namespace ncnn_amd
