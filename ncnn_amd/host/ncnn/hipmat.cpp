#include "hipmat.h"

#include "ncnnhip.h"

namespace ncnn {

static int hip_status(int rc, const char* where)
{
    if (rc == 0) return 0;
    NCNN_LOGE("%s failed: %s", where, ncnnhip_last_error());
    return rc == NCNNHIP_OOM ? -100 : -1;
}

// ---- HipMat -----------------------------------------------------------------------------------

HipMat::HipMat() : data(0), refcount(0), dims(0), w(0), h(0), c(0), n(0), cp(0), elemsize(0), q8_scale(0.f) {}

HipMat::HipMat(const HipMat& m) : data(m.data), refcount(m.refcount), pool(m.pool), dims(m.dims), w(m.w), h(m.h), c(m.c), n(m.n), cp(m.cp), elemsize(m.elemsize), q8(m.q8), q8_scale(m.q8_scale)
{
    if (refcount) __sync_fetch_and_add(refcount, 1);
}

HipMat::~HipMat()
{
    release();
}

HipMat& HipMat::operator=(const HipMat& m)
{
    if (this == &m) return *this;
    if (m.refcount) __sync_fetch_and_add(m.refcount, 1);
    release();
    data = m.data;
    refcount = m.refcount;
    pool = m.pool;
    dims = m.dims;
    w = m.w;
    h = m.h;
    c = m.c;
    n = m.n;
    cp = m.cp;
    elemsize = m.elemsize;
    q8 = m.q8;
    q8_scale = m.q8_scale;
    return *this;
}

void HipMat::release()
{
    if (refcount && __sync_fetch_and_add(refcount, -1) == 1)
    {
        if (pool && data) pool->give_back(data);
        delete refcount;
    }
    data = 0;
    refcount = 0;
    pool.reset();
    dims = w = h = c = n = cp = 0;
    elemsize = 0;
    q8.reset();
    q8_scale = 0.f;
}

void HipMat::allocate(HipCommand* command)
{
    size_t need = bytes();
    if (need == 0) need = 4;
    void* p = command->alloc(need);
    if (!p)
    {
        dims = w = h = c = n = cp = 0;
        elemsize = 0;
        return;
    }
    data = p;
    pool = command->pool;
    refcount = new int(1);
}

void HipMat::create(int _w, size_t _elemsize, int _n, HipCommand* command)
{
    release();
    dims = 1;
    w = _w;
    h = 1;
    c = 1;
    n = _n < 1 ? 1 : _n;
    cp = 0;
    elemsize = _elemsize;
    allocate(command);
}

void HipMat::create(int _w, int _h, size_t _elemsize, int _n, HipCommand* command)
{
    release();
    dims = 2;
    w = _w;
    h = _h;
    c = 1;
    n = _n < 1 ? 1 : _n;
    cp = 0;
    elemsize = _elemsize;
    allocate(command);
}

void HipMat::create(int _w, int _h, int _c, size_t _elemsize, int _n, HipCommand* command)
{
    release();
    dims = 3;
    w = _w;
    h = _h;
    c = _c;
    n = _n < 1 ? 1 : _n;
    cp = ncnnhip_padded_channels(_c);
    elemsize = _elemsize;
    allocate(command);
}

void HipMat::create_narrow(int _w, int _h, int _c, int _n, HipCommand* command)
{
    release();
    dims = 3;
    w = _w;
    h = _h;
    c = _c;
    n = _n < 1 ? 1 : _n;
    cp = 4;
    elemsize = 4u;
    allocate(command);
}

void HipMat::create_like(const HipMat& m, HipCommand* command)
{
    if (m.dims == 1)
        create(m.w, m.elemsize, m.n, command);
    else if (m.dims == 2)
        create(m.w, m.h, m.elemsize, m.n, command);
    else
        create(m.w, m.h, m.c, m.elemsize, m.n, command);
}

// ---- HipCommand ---------------------------------------------------------------------------------

// ---- HipPool ------------------------------------------------------------------------------------

HipPool::HipPool(bool defer) : returns(0), defer_reuse(defer) {}

HipPool::~HipPool()
{
    // the last owner: the command (which synchronised its stream when it went) and every blob are gone
    for (size_t i = 0; i < slots.size(); i++) ncnnhip_free(slots[i].ptr);
}

void* HipPool::take(size_t bytes, int state)
{
    if (bytes == 0) bytes = 4;
    {
        std::unique_lock<std::mutex> g(lock);
        for (int pass = 0; pass < 2; pass++)
        {
            // smallest idle buffer that fits without wasting more than half of it
            int best = -1;
            bool retired_fits = false;
            for (size_t i = 0; i < slots.size(); i++)
            {
                const bool fits = slots[i].bytes >= bytes && slots[i].bytes <= 2 * bytes + 0x10000;
                if (slots[i].state == 0 && fits && (best < 0 || slots[i].bytes < slots[(size_t)best].bytes)) best = (int)i;
                if (slots[i].state == 3 && fits) retired_fits = true;
            }
            if (best >= 0)
            {
                slots[(size_t)best].state = state;
                return slots[(size_t)best].ptr;
            }
            if (pass == 1 || !retired_fits) break;
            // A returned buffer would do, but a kernel on some other stream may still read it: wait for the device once,
            // after which every buffer that had come back BEFORE the wait began is free to go out again.  The wait runs
            // without the lock (other threads keep taking and returning buffers meanwhile; what they return during the wait
            // stays retired), and fails under another thread's stream capture: a new allocation then serves the request.
            const unsigned long long seen = returns;
            g.unlock();
            const bool waited = ncnnhip_device_synchronize() == 0;
            g.lock();
            if (!waited) break;
            for (size_t i = 0; i < slots.size(); i++)
                if (slots[i].state == 3 && slots[i].retired <= seen) slots[i].state = 0;
        }
    }
    // nothing idle fits: a new buffer, allocated without the lock
    Slot s;
    s.bytes = (bytes + 0xffff) & ~(size_t)0xffff;
    s.state = state;
    s.ptr = 0;
    s.retired = 0;
    if (ncnnhip_malloc(&s.ptr, s.bytes) != 0 || !s.ptr) return 0;
    std::lock_guard<std::mutex> g(lock);
    slots.push_back(s);
    return s.ptr;
}

void HipPool::give_back(void* ptr)
{
    std::lock_guard<std::mutex> g(lock);
    for (size_t i = 0; i < slots.size(); i++)
        if (slots[i].ptr == ptr)
        {
            slots[i].state = defer_reuse ? 3 : 0;
            slots[i].retired = ++returns;
            return;
        }
}

void HipPool::give_back_all_borrowed()
{
    std::lock_guard<std::mutex> g(lock);
    for (size_t i = 0; i < slots.size(); i++)
        if (slots[i].state == 2) slots[i].state = 0; // scratch is only ever used on the command's own stream
}

size_t HipPool::pooled_bytes() const
{
    std::lock_guard<std::mutex> g(lock);
    size_t s = 0;
    for (size_t i = 0; i < slots.size(); i++) s += slots[i].bytes;
    return s;
}

HipCommand::HipCommand(bool blobs_cross_streams) : stream(0), ready(false), pool(new HipPool(blobs_cross_streams)), zero_ws(0), zero_ws_bytes(0) {}

HipCommand::~HipCommand()
{
    // whatever was enqueued on this stream has finished before the stream goes; the buffers go with the pool's last owner
    if (ready) ncnnhip_stream_synchronize(stream);
    if (zero_ws) ncnnhip_free(zero_ws);
    if (stream) ncnnhip_stream_destroy(stream);
}

void* HipCommand::zeroed_workspace(size_t bytes)
{
    if (bytes <= zero_ws_bytes) return zero_ws;
    // grow: whatever still uses the old buffer was enqueued on this stream, so wait before freeing it
    if (ncnnhip_stream_synchronize(stream) != 0) return 0;
    if (zero_ws) ncnnhip_free(zero_ws);
    zero_ws = 0;
    zero_ws_bytes = 0;
    const size_t rounded = (bytes + 0xfffff) & ~(size_t)0xfffff;
    void* p = 0;
    if (ncnnhip_malloc(&p, rounded) != 0 || !p) return 0;
    if (ncnnhip_memset(p, 0, rounded, stream) != 0 || ncnnhip_stream_synchronize(stream) != 0)
    {
        ncnnhip_free(p);
        return 0;
    }
    zero_ws = p;
    zero_ws_bytes = rounded;
    return zero_ws;
}

int HipCommand::ensure_ready()
{
    if (ready) return 0;
    int rc = ncnnhip_init(0);
    if (rc != 0) return hip_status(rc, "ncnnhip_init");
    rc = ncnnhip_stream_create(&stream);
    if (rc != 0) return hip_status(rc, "ncnnhip_stream_create");
    ready = true;
    return 0;
}

void* HipCommand::alloc(size_t bytes)
{
    return pool->take(bytes, 1);
}

void HipCommand::free(void* ptr)
{
    pool->give_back(ptr);
}

void* HipCommand::borrow(size_t bytes)
{
    return pool->take(bytes, 2);
}

void HipCommand::give_back_all()
{
    pool->give_back_all_borrowed();
}

size_t HipCommand::pooled_bytes() const
{
    return pool->pooled_bytes();
}

int HipCommand::synchronize()
{
    return hip_status(ncnnhip_stream_synchronize(stream), "ncnnhip_stream_synchronize");
}

static size_t host_bytes(const Mat& m)
{
    return (m.n > 1 ? m.nstep * m.n : m.total()) * m.elemsize;
}

int HipCommand::upload(const Mat& src, HipMat& dst)
{
    int ret = ensure_ready();
    if (ret != 0) return ret;
    if (src.empty() || src.elempack != 1 || (src.elemsize != 4u && src.elemsize != 1u) || src.dims < 1 || src.dims > 3)
    {
        NCNN_LOGE("HipCommand::upload: needs a pack-1 fp32 or int8 blob of 1 to 3 dimensions");
        return -1;
    }
    if (src.dims == 3 && src.elemsize == 4u && src.c <= 4)
        dst.create_narrow(src.w, src.h, src.c, src.n, this); // an image: a quarter of the padded blob's bytes
    else if (src.dims == 3)
        dst.create(src.w, src.h, src.c, src.elemsize, src.n, this);
    else if (src.dims == 1)
        dst.create(src.w, src.elemsize, src.n, this);
    else
        dst.create(src.w, src.h, src.elemsize, src.n, this);
    if (dst.empty()) return -100;
    return upload_into(src, dst);
}

int HipCommand::upload_into(const Mat& src, HipMat& dst)
{
    int ret = ensure_ready();
    if (ret != 0) return ret;
    if (src.empty() || dst.empty() || src.elempack != 1 || src.dims != dst.dims || src.elemsize != dst.elemsize || src.w != dst.w || src.n != dst.n
        || (src.dims >= 2 && src.h != dst.h) || (src.dims == 3 && src.c != dst.c) || src.dims < 1 || src.dims > 3)
    {
        NCNN_LOGE("HipCommand::upload_into: the host blob does not have the device blob's shape and type");
        return -1;
    }
    if (src.dims == 3)
    {
        // planar bytes as they lie on the host, then one layout kernel
        ScopedScratch scratch(this);
        void* staging = scratch.get(host_bytes(src));
        if (!staging) return -100;
        int rc = ncnnhip_memcpy_h2d(staging, src.data, host_bytes(src), stream);
        if (rc == 0 && dst.narrow())
            rc = ncnnhip_chw_to_nhwc4_f32((const float*)staging, src.c, src.w * src.h, src.n, src.cstep, src.nstep, (float*)dst.data, stream);
        else if (rc == 0)
            rc = ncnnhip_chw_to_nhwc(staging, (int)src.elemsize, src.c, src.w * src.h, src.n, src.cstep, src.nstep, dst.data, stream);
        // the copy out of pageable host memory must have left the caller's buffer before we return
        if (rc == 0) rc = ncnnhip_stream_synchronize(stream);
        return hip_status(rc, "upload");
    }
    const size_t sample = (size_t)src.w * src.h * src.elemsize;
    int rc = 0;
    for (int b = 0; b < src.n && rc == 0; b++)
        rc = ncnnhip_memcpy_h2d((unsigned char*)dst.data + sample * b, (const unsigned char*)src.data + src.nstep * b * src.elemsize, sample, stream);
    if (rc == 0) rc = ncnnhip_stream_synchronize(stream);
    return hip_status(rc, "upload");
}

int HipCommand::widen(const HipMat& src, HipMat& dst)
{
    if (src.empty() || !src.narrow() || src.elemsize != 4u) return -1;
    HipMat wide;
    wide.create(src.w, src.h, src.c, 4u, src.n, this);
    if (wide.empty()) return -100;
    int rc = ncnnhip_widen_nhwc4_f32((const float*)src.data, (float*)wide.data, (size_t)src.n * src.h * src.w, stream);
    if (rc != 0) return hip_status(rc, "ncnnhip_widen_nhwc4_f32");
    dst = wide;
    return 0;
}

int HipCommand::download(const HipMat& blob, Mat& dst, Allocator* allocator)
{
    if (blob.empty()) return -1;
    int ready_ret = ensure_ready();
    if (ready_ret != 0) return ready_ret;
    HipMat src = blob;
    if (src.narrow())
    {
        int ret = widen(blob, src);
        if (ret != 0) return ret;
    }
    if (src.dims == 3)
    {
        dst.create(src.w, src.h, src.c, src.elemsize, 1, src.n, allocator);
        if (dst.empty()) return -100;
        ScopedScratch scratch(this);
        void* staging = scratch.get(host_bytes(dst));
        if (!staging) return -100;
        int rc = ncnnhip_nhwc_to_chw(src.data, (int)src.elemsize, src.c, src.w * src.h, src.n, staging, dst.cstep, dst.nstep, stream);
        if (rc == 0) rc = ncnnhip_memcpy_d2h(dst.data, staging, host_bytes(dst), stream);
        if (rc == 0) rc = ncnnhip_stream_synchronize(stream);
        return hip_status(rc, "download");
    }
    if (src.dims == 1)
        dst.create(src.w, src.elemsize, 1, src.n, allocator);
    else
        dst.create(src.w, src.h, src.elemsize, 1, src.n, allocator);
    if (dst.empty()) return -100;
    const size_t sample = (size_t)src.w * src.h * src.elemsize;
    int rc = 0;
    for (int b = 0; b < src.n && rc == 0; b++)
        rc = ncnnhip_memcpy_d2h((unsigned char*)dst.data + dst.nstep * b * dst.elemsize, (const unsigned char*)src.data + sample * b, sample, stream);
    if (rc == 0) rc = ncnnhip_stream_synchronize(stream);
    return hip_status(rc, "download");
}

} // namespace ncnn
