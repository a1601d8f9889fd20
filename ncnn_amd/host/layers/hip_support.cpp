#include "hip_support.h"

#include "../ncnn/platform.h"

namespace ncnn_amd {

HipContext::HipContext() : stream(0), ready(false) {}

HipContext::~HipContext()
{
    for (size_t i = 0; i < pool.size(); i++) ncnnhip_free(pool[i].ptr);
    if (stream) ncnnhip_stream_destroy(stream);
}

int HipContext::ensure_ready()
{
    if (ready) return 0;
    int rc = ncnnhip_init(0);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_init");
    rc = ncnnhip_stream_create(&stream);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_stream_create");
    ready = true;
    return 0;
}

void* HipContext::borrow(size_t bytes)
{
    if (bytes == 0) bytes = 4;
    // smallest idle buffer that fits
    int best = -1;
    for (size_t i = 0; i < pool.size(); i++)
        if (!pool[i].busy && pool[i].bytes >= bytes && (best < 0 || pool[i].bytes < pool[(size_t)best].bytes)) best = (int)i;
    if (best >= 0)
    {
        pool[(size_t)best].busy = true;
        return pool[(size_t)best].ptr;
    }
    Lease l;
    l.bytes = (bytes + 0xffff) & ~(size_t)0xffff;
    l.busy = true;
    l.ptr = 0;
    if (ncnnhip_malloc(&l.ptr, l.bytes) != 0 || !l.ptr) return 0;
    pool.push_back(l);
    return l.ptr;
}

void HipContext::give_back_all()
{
    for (size_t i = 0; i < pool.size(); i++) pool[i].busy = false;
}

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
