// ncnn::Mat: the refcounted tensor handle at the layer boundary (data members and layout rules
// of src/mat.h:341-381 and src/mat.cpp:300-830).
//
//   dims 1: w                      dims 2: h rows of w            dims 3: c planes of h*w
//   dims 4: c planes of d*h*w      every plane starts on a 16-byte boundary (cstep)
//   batch:  n samples, nstep elements apart (4096-byte aligned when n > 1)
//
// The reference counter lives in the same allocation, directly behind the (4-byte aligned)
// payload, so a Mat's `data` must always be host memory the CPU can write.
#ifndef NCNN_MAT_H
#define NCNN_MAT_H

#include <stddef.h>
#include <string.h>

#include "allocator.h"
#include "platform.h"

namespace ncnn {

class Option;

class NCNN_EXPORT Mat
{
public:
    Mat();
    // owning constructors
    Mat(int w, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, int c, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, int d, int c, size_t elemsize = 4u, Allocator* allocator = 0);
    // views over caller-owned memory (no refcount)
    Mat(int w, void* data, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, void* data, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, int c, void* data, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(int w, int h, int d, int c, void* data, size_t elemsize = 4u, Allocator* allocator = 0);
    Mat(const Mat& m);
    ~Mat();
    Mat& operator=(const Mat& m);

    // (re)allocate; an identical existing shape is kept as is
    void create(int w, size_t elemsize = 4u, Allocator* allocator = 0);
    void create(int w, int h, size_t elemsize = 4u, Allocator* allocator = 0);
    void create(int w, int h, int c, size_t elemsize = 4u, Allocator* allocator = 0);
    void create(int w, int h, int d, int c, size_t elemsize = 4u, Allocator* allocator = 0);
    void create(int w, size_t elemsize, int elempack, Allocator* allocator);
    void create(int w, int h, size_t elemsize, int elempack, Allocator* allocator);
    void create(int w, int h, int c, size_t elemsize, int elempack, Allocator* allocator);
    void create(int w, int h, int d, int c, size_t elemsize, int elempack, Allocator* allocator);
    // batched
    void create(int w, size_t elemsize, int elempack, int n, Allocator* allocator);
    void create(int w, int h, size_t elemsize, int elempack, int n, Allocator* allocator);
    void create(int w, int h, int c, size_t elemsize, int elempack, int n, Allocator* allocator);
    void create(int w, int h, int d, int c, size_t elemsize, int elempack, int n, Allocator* allocator);
    void create_like(const Mat& m, Allocator* allocator = 0);
    void create_like(const Mat& m, int n, Allocator* allocator);

    void fill(float v);
    void fill(int v);
    template<typename T>
    void fill(T v);

    Mat clone(Allocator* allocator = 0) const;
    // same memory, new shape (copies only when plane padding forces it)
    Mat reshape(int w, Allocator* allocator = 0) const;
    Mat reshape(int w, int h, Allocator* allocator = 0) const;
    Mat reshape(int w, int h, int c, Allocator* allocator = 0) const;

    void addref();
    void release();

    bool empty() const
    {
        return data == 0 || total() == 0;
    }
    size_t total() const
    {
        return cstep * c;
    }
    int elembits() const
    {
        return elempack ? (int)(elemsize * 8) / elempack : 0;
    }
    Mat shape() const;

    Mat channel(int q);
    const Mat channel(int q) const;
    Mat channel_range(int q, int channels);
    const Mat channel_range(int q, int channels) const;
    Mat row_range(int y, int rows);
    const Mat row_range(int y, int rows) const;
    Mat range(int x, int count);
    const Mat range(int x, int count) const;
    Mat batch(int b);
    const Mat batch(int b) const;

    float* row(int y)
    {
        return (float*)((unsigned char*)data + (size_t)w * y * elemsize);
    }
    const float* row(int y) const
    {
        return (const float*)((const unsigned char*)data + (size_t)w * y * elemsize);
    }
    template<typename T>
    T* row(int y)
    {
        return (T*)((unsigned char*)data + (size_t)w * y * elemsize);
    }
    template<typename T>
    const T* row(int y) const
    {
        return (const T*)((const unsigned char*)data + (size_t)w * y * elemsize);
    }

    template<typename T>
    operator T*()
    {
        return (T*)data;
    }
    template<typename T>
    operator const T*() const
    {
        return (const T*)data;
    }
    float& operator[](size_t i)
    {
        return ((float*)data)[i];
    }
    const float& operator[](size_t i) const
    {
        return ((const float*)data)[i];
    }

    static Mat from_float16(const unsigned short* data, int size);

    void* data;
    int* refcount; // NULL for views over caller-owned memory
    size_t elemsize;
    int elempack;
    Allocator* allocator;
    int dims;
    int w;
    int h;
    int d;
    int c;
    size_t cstep;
    int n;        // batch count, default 1
    size_t nstep; // elements from one sample to the next; total() for a non-batch Mat

private:
    void set_shape(int dims, int w, int h, int d, int c, size_t elemsize, int elempack, int n);
    void allocate(Allocator* allocator);
    bool same_as(int dims, int w, int h, int d, int c, size_t elemsize, int elempack, int n, Allocator* allocator) const;
    void create_any(int dims, int w, int h, int d, int c, size_t elemsize, int elempack, int n, Allocator* allocator);
    Mat reshape_samples(int dims, int w, int h, int c, Allocator* allocator) const;
    void view(int dims, int w, int h, int d, int c, void* data, size_t elemsize, Allocator* allocator);
};

template<typename T>
void Mat::fill(T v)
{
    const size_t count = (n > 1 ? nstep * n : total()) * elempack;
    T* p = (T*)data;
    for (size_t i = 0; i < count; i++) p[i] = v;
}

// fp32 -> int8 with one scale or one scale per row/channel (the Quantize layer's arithmetic);
// used at load time to quantise fp32 weights exactly as the reference does
NCNN_EXPORT void quantize_to_int8(const Mat& src, Mat& dst, const Mat& scale_data, const Option& opt);

NCNN_EXPORT unsigned short float32_to_float16(float value);
NCNN_EXPORT float float16_to_float32(unsigned short value);

} // namespace ncnn

#endif // NCNN_MAT_H
