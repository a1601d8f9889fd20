#include "allocator.h"

#include <mutex>
#include <vector>

namespace ncnn {

Allocator::~Allocator() {}

struct PoolBlock
{
    size_t size;
    void* ptr;
};

class PoolAllocatorState
{
public:
    explicit PoolAllocatorState(bool locked) : use_lock(locked), ratio(0.f), drop_threshold(10) {}

    void* take(size_t size)
    {
        std::unique_lock<std::mutex> guard(mu, std::defer_lock);
        if (use_lock) guard.lock();
        // a kept block qualifies when it is big enough and not wastefully bigger
        size_t best = (size_t)-1;
        for (size_t i = 0; i < idle.size(); i++)
        {
            const size_t bs = idle[i].size;
            if (bs >= size && (float)size >= (float)bs * ratio)
            {
                if (best == (size_t)-1 || bs < idle[best].size) best = i;
            }
        }
        if (best != (size_t)-1)
        {
            PoolBlock b = idle[best];
            idle.erase(idle.begin() + best);
            busy.push_back(b);
            return b.ptr;
        }
        // keep the idle list bounded: drop the block that is furthest from being useful
        if (idle.size() >= drop_threshold && !idle.empty())
        {
            size_t victim = 0;
            for (size_t i = 1; i < idle.size(); i++)
                if (idle[i].size < idle[victim].size) victim = i;
            ncnn::fastFree(idle[victim].ptr);
            idle.erase(idle.begin() + victim);
        }
        PoolBlock b;
        b.size = size;
        b.ptr = ncnn::fastMalloc(size);
        if (!b.ptr) return 0;
        busy.push_back(b);
        return b.ptr;
    }

    void give(void* ptr)
    {
        if (!ptr) return;
        std::unique_lock<std::mutex> guard(mu, std::defer_lock);
        if (use_lock) guard.lock();
        for (size_t i = 0; i < busy.size(); i++)
        {
            if (busy[i].ptr == ptr)
            {
                idle.push_back(busy[i]);
                busy.erase(busy.begin() + i);
                return;
            }
        }
        NCNN_LOGE("FATAL ERROR! pool allocator get wild %p", ptr);
        ncnn::fastFree(ptr);
    }

    void drop_idle()
    {
        std::unique_lock<std::mutex> guard(mu, std::defer_lock);
        if (use_lock) guard.lock();
        for (size_t i = 0; i < idle.size(); i++) ncnn::fastFree(idle[i].ptr);
        idle.clear();
    }

    ~PoolAllocatorState()
    {
        drop_idle();
        if (!busy.empty()) NCNN_LOGE("FATAL ERROR! pool allocator destroyed too early");
    }

    bool use_lock;
    float ratio;
    size_t drop_threshold;
    std::mutex mu;
    std::vector<PoolBlock> idle, busy;
};

static float clamp01(float v)
{
    if (v < 0.f || v > 1.f)
    {
        NCNN_LOGE("invalid size compare ratio %f", v);
        return v < 0.f ? 0.f : 1.f;
    }
    return v;
}

PoolAllocator::PoolAllocator() : d(new PoolAllocatorState(true)) {}
PoolAllocator::~PoolAllocator()
{
    delete d;
}
void PoolAllocator::set_size_compare_ratio(float scr)
{
    d->ratio = clamp01(scr);
}
void PoolAllocator::set_size_drop_threshold(size_t threshold)
{
    d->drop_threshold = threshold;
}
void PoolAllocator::clear()
{
    d->drop_idle();
}
void* PoolAllocator::fastMalloc(size_t size)
{
    return d->take(size);
}
void PoolAllocator::fastFree(void* ptr)
{
    d->give(ptr);
}

UnlockedPoolAllocator::UnlockedPoolAllocator() : d(new PoolAllocatorState(false)) {}
UnlockedPoolAllocator::~UnlockedPoolAllocator()
{
    delete d;
}
void UnlockedPoolAllocator::set_size_compare_ratio(float scr)
{
    d->ratio = clamp01(scr);
}
void UnlockedPoolAllocator::set_size_drop_threshold(size_t threshold)
{
    d->drop_threshold = threshold;
}
void UnlockedPoolAllocator::clear()
{
    d->drop_idle();
}
void* UnlockedPoolAllocator::fastMalloc(size_t size)
{
    return d->take(size);
}
void UnlockedPoolAllocator::fastFree(void* ptr)
{
    d->give(ptr);
}

} // namespace ncnn
