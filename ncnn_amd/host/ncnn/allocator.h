// Host allocators behind ncnn::Mat (interface of src/allocator.h:142-205).
#ifndef NCNN_ALLOCATOR_H
#define NCNN_ALLOCATOR_H

#include <stddef.h>
#include <stdlib.h>

#include "platform.h"

namespace ncnn {

static inline size_t alignSize(size_t sz, int n)
{
    return (sz + n - 1) & -(size_t)n;
}

// 64-byte aligned block with 64 bytes of slack after it, so vector code may read past the end
static inline void* fastMalloc(size_t size)
{
    void* p = 0;
    if (posix_memalign(&p, NCNN_MALLOC_ALIGN, size + NCNN_MALLOC_OVERREAD)) p = 0;
    return p;
}

static inline void fastFree(void* p)
{
    free(p);
}

class NCNN_EXPORT Allocator
{
public:
    virtual ~Allocator();
    virtual void* fastMalloc(size_t size) = 0;
    virtual void fastFree(void* ptr) = 0;
};

// Size-bucketed recycling allocator: a freed block is kept and handed out again to a request
// of similar size (within the compare ratio).  PoolAllocator locks, the Unlocked flavour is
// for per-Extractor use.
class PoolAllocatorState;
class NCNN_EXPORT PoolAllocator : public Allocator
{
public:
    PoolAllocator();
    ~PoolAllocator();
    void set_size_compare_ratio(float scr); // 0 ~ 1
    void set_size_drop_threshold(size_t threshold);
    void clear();
    virtual void* fastMalloc(size_t size);
    virtual void fastFree(void* ptr);

private:
    PoolAllocator(const PoolAllocator&);
    PoolAllocator& operator=(const PoolAllocator&);
    PoolAllocatorState* const d;
};

class NCNN_EXPORT UnlockedPoolAllocator : public Allocator
{
public:
    UnlockedPoolAllocator();
    ~UnlockedPoolAllocator();
    void set_size_compare_ratio(float scr);
    void set_size_drop_threshold(size_t threshold);
    void clear();
    virtual void* fastMalloc(size_t size);
    virtual void fastFree(void* ptr);

private:
    UnlockedPoolAllocator(const UnlockedPoolAllocator&);
    UnlockedPoolAllocator& operator=(const UnlockedPoolAllocator&);
    PoolAllocatorState* const d;
};

} // namespace ncnn

#endif // NCNN_ALLOCATOR_H
