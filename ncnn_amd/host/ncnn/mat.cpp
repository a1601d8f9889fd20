#include "mat.h"

#include <math.h>
#include <stdint.h>

#include "option.h"

namespace ncnn {

Mat::Mat() : data(0), refcount(0), elemsize(0), elempack(0), allocator(0), dims(0), w(0), h(0), d(0), c(0), cstep(0), n(1), nstep(0) {}

// ---- shape bookkeeping ------------------------------------------------------------------

void Mat::set_shape(int _dims, int _w, int _h, int _d, int _c, size_t _elemsize, int _elempack, int _n)
{
    dims = _dims;
    w = _w;
    h = _h;
    d = _d;
    c = _c;
    elemsize = _elemsize;
    elempack = _elempack;
    n = _n < 1 ? 1 : _n;
    const size_t plane = (size_t)w * h * d;
    // planes of 3-D / 4-D blobs are padded to 16 bytes, vectors and images are dense
    cstep = dims >= 3 ? alignSize(plane * elemsize, 16) / elemsize : plane;
    nstep = n > 1 ? alignSize(cstep * c * elemsize, 4096) / elemsize : cstep * c;
}

void Mat::allocate(Allocator* _allocator)
{
    allocator = _allocator;
    const size_t payload = alignSize((n > 1 ? nstep * n : cstep * c) * elemsize, 4);
    if (payload == 0) return;
    data = allocator ? allocator->fastMalloc(payload + sizeof(int)) : ncnn::fastMalloc(payload + sizeof(int));
    if (!data) return;
    refcount = (int*)((unsigned char*)data + payload);
    *refcount = 1;
}

bool Mat::same_as(int _dims, int _w, int _h, int _d, int _c, size_t _elemsize, int _elempack, int _n, Allocator* _allocator) const
{
    return dims == _dims && w == _w && h == _h && d == _d && c == _c && elemsize == _elemsize && elempack == _elempack && n == (_n < 1 ? 1 : _n)
           && allocator == _allocator;
}

void Mat::create_any(int _dims, int _w, int _h, int _d, int _c, size_t _elemsize, int _elempack, int _n, Allocator* _allocator)
{
    if (same_as(_dims, _w, _h, _d, _c, _elemsize, _elempack, _n, _allocator)) return;
    release();
    if (_w < 0 || _h < 0 || _d < 0 || _c < 0) return; // a negative extent (a damaged model file): the Mat stays empty, callers test empty()
    set_shape(_dims, _w, _h, _d, _c, _elemsize, _elempack, _n);
    allocate(_allocator);
}

void Mat::view(int _dims, int _w, int _h, int _d, int _c, void* _data, size_t _elemsize, Allocator* _allocator)
{
    set_shape(_dims, _w, _h, _d, _c, _elemsize, 1, 1);
    data = _data;
    refcount = 0;
    allocator = _allocator;
}

// ---- constructors -----------------------------------------------------------------------

Mat::Mat(int _w, size_t _elemsize, Allocator* _allocator) : Mat()
{
    create(_w, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, size_t _elemsize, Allocator* _allocator) : Mat()
{
    create(_w, _h, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, int _c, size_t _elemsize, Allocator* _allocator) : Mat()
{
    create(_w, _h, _c, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, int _d, int _c, size_t _elemsize, Allocator* _allocator) : Mat()
{
    create(_w, _h, _d, _c, _elemsize, _allocator);
}
Mat::Mat(int _w, void* _data, size_t _elemsize, Allocator* _allocator) : Mat()
{
    view(1, _w, 1, 1, 1, _data, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, void* _data, size_t _elemsize, Allocator* _allocator) : Mat()
{
    view(2, _w, _h, 1, 1, _data, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, int _c, void* _data, size_t _elemsize, Allocator* _allocator) : Mat()
{
    view(3, _w, _h, 1, _c, _data, _elemsize, _allocator);
}
Mat::Mat(int _w, int _h, int _d, int _c, void* _data, size_t _elemsize, Allocator* _allocator) : Mat()
{
    view(4, _w, _h, _d, _c, _data, _elemsize, _allocator);
}

Mat::Mat(const Mat& m)
    : data(m.data), refcount(m.refcount), elemsize(m.elemsize), elempack(m.elempack), allocator(m.allocator), dims(m.dims), w(m.w), h(m.h), d(m.d), c(m.c), cstep(m.cstep), n(m.n), nstep(m.nstep)
{
    addref();
}

Mat::~Mat()
{
    release();
}

Mat& Mat::operator=(const Mat& m)
{
    if (this == &m) return *this;
    if (m.refcount) __sync_fetch_and_add(m.refcount, 1);
    release();
    data = m.data;
    refcount = m.refcount;
    elemsize = m.elemsize;
    elempack = m.elempack;
    allocator = m.allocator;
    dims = m.dims;
    w = m.w;
    h = m.h;
    d = m.d;
    c = m.c;
    cstep = m.cstep;
    n = m.n;
    nstep = m.nstep;
    return *this;
}

void Mat::addref()
{
    if (refcount) __sync_fetch_and_add(refcount, 1);
}

void Mat::release()
{
    if (refcount && __sync_fetch_and_add(refcount, -1) == 1)
    {
        if (allocator)
            allocator->fastFree(data);
        else
            ncnn::fastFree(data);
    }
    data = 0;
    refcount = 0;
    elemsize = 0;
    elempack = 0;
    dims = 0;
    w = h = d = c = 0;
    cstep = 0;
    n = 1;
    nstep = 0;
}

// ---- create family ----------------------------------------------------------------------

void Mat::create(int _w, size_t _elemsize, Allocator* _allocator)
{
    create_any(1, _w, 1, 1, 1, _elemsize, 1, 1, _allocator);
}
void Mat::create(int _w, int _h, size_t _elemsize, Allocator* _allocator)
{
    create_any(2, _w, _h, 1, 1, _elemsize, 1, 1, _allocator);
}
void Mat::create(int _w, int _h, int _c, size_t _elemsize, Allocator* _allocator)
{
    create_any(3, _w, _h, 1, _c, _elemsize, 1, 1, _allocator);
}
void Mat::create(int _w, int _h, int _d, int _c, size_t _elemsize, Allocator* _allocator)
{
    create_any(4, _w, _h, _d, _c, _elemsize, 1, 1, _allocator);
}
void Mat::create(int _w, size_t _elemsize, int _elempack, Allocator* _allocator)
{
    create_any(1, _w, 1, 1, 1, _elemsize, _elempack, 1, _allocator);
}
void Mat::create(int _w, int _h, size_t _elemsize, int _elempack, Allocator* _allocator)
{
    create_any(2, _w, _h, 1, 1, _elemsize, _elempack, 1, _allocator);
}
void Mat::create(int _w, int _h, int _c, size_t _elemsize, int _elempack, Allocator* _allocator)
{
    create_any(3, _w, _h, 1, _c, _elemsize, _elempack, 1, _allocator);
}
void Mat::create(int _w, int _h, int _d, int _c, size_t _elemsize, int _elempack, Allocator* _allocator)
{
    create_any(4, _w, _h, _d, _c, _elemsize, _elempack, 1, _allocator);
}
void Mat::create(int _w, size_t _elemsize, int _elempack, int _n, Allocator* _allocator)
{
    create_any(1, _w, 1, 1, 1, _elemsize, _elempack, _n, _allocator);
}
void Mat::create(int _w, int _h, size_t _elemsize, int _elempack, int _n, Allocator* _allocator)
{
    create_any(2, _w, _h, 1, 1, _elemsize, _elempack, _n, _allocator);
}
void Mat::create(int _w, int _h, int _c, size_t _elemsize, int _elempack, int _n, Allocator* _allocator)
{
    create_any(3, _w, _h, 1, _c, _elemsize, _elempack, _n, _allocator);
}
void Mat::create(int _w, int _h, int _d, int _c, size_t _elemsize, int _elempack, int _n, Allocator* _allocator)
{
    create_any(4, _w, _h, _d, _c, _elemsize, _elempack, _n, _allocator);
}

void Mat::create_like(const Mat& m, Allocator* _allocator)
{
    create_any(m.dims, m.w, m.h, m.d, m.c, m.elemsize, m.elempack, m.n, _allocator);
}
void Mat::create_like(const Mat& m, int _n, Allocator* _allocator)
{
    create_any(m.dims, m.w, m.h, m.d, m.c, m.elemsize, m.elempack, _n, _allocator);
}

void Mat::fill(float v)
{
    fill<float>(v);
}
void Mat::fill(int v)
{
    fill<int>(v);
}

// ---- copies and reshapes ----------------------------------------------------------------

Mat Mat::clone(Allocator* _allocator) const
{
    if (empty()) return Mat();
    Mat m;
    m.create_any(dims, w, h, d, c, elemsize, elempack, n, _allocator);
    if (m.empty()) return m;
    if (n > 1)
    {
        for (int b = 0; b < n; b++)
            memcpy((unsigned char*)m.data + m.nstep * b * elemsize, (const unsigned char*)data + nstep * b * elemsize, cstep * c * elemsize);
    }
    else
    {
        memcpy(m.data, data, total() * elemsize);
    }
    return m;
}

Mat Mat::shape() const
{
    Mat s;
    s.set_shape(dims, w, h, d, c, elemsize, elempack, n);
    s.elemsize = 0; // shape only: carries extents, no storage
    s.elemsize = elemsize;
    s.data = 0;
    return s;
}

static bool planes_are_dense(const Mat& m)
{
    return m.dims < 3 || m.cstep == (size_t)m.w * m.h * m.d;
}

// gather a blob with padded planes into dense order
static Mat densify(const Mat& m, Allocator* allocator)
{
    const size_t plane = (size_t)m.w * m.h * m.d;
    Mat flat;
    flat.create((int)(plane * m.c), m.elemsize, m.elempack, allocator);
    if (flat.empty()) return flat;
    for (int q = 0; q < m.c; q++)
        memcpy((unsigned char*)flat.data + plane * q * m.elemsize, (const unsigned char*)m.data + m.cstep * q * m.elemsize, plane * m.elemsize);
    return flat;
}

// A batched blob under a new shape (src/mat.cpp:113-250 hands these to its reshape_batch): every sample is reshaped by
// itself and the samples stay nstep apart.  Dense planes on both sides share the storage; otherwise each sample is copied.
Mat Mat::reshape_samples(int _dims, int _w, int _h, int _c, Allocator* _allocator) const
{
    const size_t plane = _dims == 3 ? (size_t)_w * _h : _dims == 2 ? (size_t)_w * _h : (size_t)_w;
    const size_t padded = _dims == 3 ? alignSize(plane * elemsize, 16) / elemsize : plane;
    if (planes_are_dense(*this) && padded == plane)
    {
        Mat m = *this; // n and nstep stay as they are
        m.dims = _dims;
        m.w = _w;
        m.h = _dims >= 2 ? _h : 1;
        m.d = 1;
        m.c = _dims == 3 ? _c : 1;
        m.cstep = plane;
        return m;
    }
    Mat out;
    out.create_any(_dims, _w, _dims >= 2 ? _h : 1, 1, _dims == 3 ? _c : 1, elemsize, elempack, n, _allocator);
    if (out.empty()) return out;
    for (int b = 0; b < n; b++)
    {
        const Mat sample = batch(b);
        const Mat r = _dims == 3 ? sample.reshape(_w, _h, _c, _allocator) : _dims == 2 ? sample.reshape(_w, _h, _allocator) : sample.reshape(_w, _allocator);
        if (r.empty()) return Mat();
        unsigned char* to = (unsigned char*)out.data + out.nstep * b * elemsize;
        for (int q = 0; q < out.c; q++)
            memcpy(to + out.cstep * q * elemsize, (const unsigned char*)r.data + r.cstep * q * elemsize, plane * elemsize);
    }
    return out;
}

Mat Mat::reshape(int _w, Allocator* _allocator) const
{
    if ((size_t)w * h * d * c != (size_t)_w) return Mat();
    if (n > 1) return reshape_samples(1, _w, 1, 1, _allocator);
    if (!planes_are_dense(*this)) return densify(*this, _allocator);
    Mat m = *this;
    m.dims = 1;
    m.w = _w;
    m.h = m.d = m.c = 1;
    m.cstep = (size_t)_w;
    m.nstep = m.cstep;
    return m;
}

Mat Mat::reshape(int _w, int _h, Allocator* _allocator) const
{
    if ((size_t)w * h * d * c != (size_t)_w * _h) return Mat();
    if (n > 1) return reshape_samples(2, _w, _h, 1, _allocator);
    if (!planes_are_dense(*this))
    {
        Mat flat = densify(*this, _allocator);
        if (flat.empty()) return flat;
        return flat.reshape(_w, _h, _allocator);
    }
    Mat m = *this;
    m.dims = 2;
    m.w = _w;
    m.h = _h;
    m.d = m.c = 1;
    m.cstep = (size_t)_w * _h;
    m.nstep = m.cstep;
    return m;
}

Mat Mat::reshape(int _w, int _h, int _c, Allocator* _allocator) const
{
    if ((size_t)w * h * d * c != (size_t)_w * _h * _c) return Mat();
    if (n > 1) return reshape_samples(3, _w, _h, _c, _allocator);
    const size_t plane = (size_t)_w * _h;
    const size_t padded = alignSize(plane * elemsize, 16) / elemsize;
    const bool src_dense = planes_are_dense(*this);
    if (src_dense && padded == plane)
    {
        Mat m = *this;
        m.dims = 3;
        m.w = _w;
        m.h = _h;
        m.d = 1;
        m.c = _c;
        m.cstep = plane;
        m.nstep = m.cstep * _c;
        return m;
    }
    // plane padding differs between the two shapes: copy plane by plane
    Mat src = src_dense ? *this : densify(*this, _allocator);
    if (src.empty()) return src;
    Mat m;
    m.create(_w, _h, _c, elemsize, elempack, _allocator);
    if (m.empty()) return m;
    for (int q = 0; q < _c; q++)
        memcpy((unsigned char*)m.data + m.cstep * q * elemsize, (const unsigned char*)src.data + plane * q * elemsize, plane * elemsize);
    return m;
}

// ---- views ------------------------------------------------------------------------------

Mat Mat::channel(int q)
{
    unsigned char* p = (unsigned char*)data + cstep * q * elemsize;
    Mat m = dims == 4 ? Mat(w, h, d, p, elemsize, allocator) : Mat(w, h, p, elemsize, allocator);
    if (dims == 4)
    {
        // one plane of a 4-D blob is a dense 3-D block
        m.dims = 3;
        m.c = d;
        m.d = 1;
        m.cstep = (size_t)w * h;
    }
    m.elempack = elempack;
    m.nstep = m.total();
    return m;
}

const Mat Mat::channel(int q) const
{
    return const_cast<Mat*>(this)->channel(q);
}

Mat Mat::channel_range(int q, int channels)
{
    Mat m = *this; // shares the refcount
    m.data = (unsigned char*)data + cstep * q * elemsize;
    m.c = channels;
    m.n = 1;
    m.nstep = m.cstep * channels;
    return m;
}

const Mat Mat::channel_range(int q, int channels) const
{
    return const_cast<Mat*>(this)->channel_range(q, channels);
}

Mat Mat::row_range(int y, int rows)
{
    Mat m(w, rows, (unsigned char*)data + (size_t)w * y * elemsize, elemsize, allocator);
    m.elempack = elempack;
    return m;
}

const Mat Mat::row_range(int y, int rows) const
{
    return const_cast<Mat*>(this)->row_range(y, rows);
}

Mat Mat::range(int x, int count)
{
    Mat m(count, (unsigned char*)data + (size_t)x * elemsize, elemsize, allocator);
    m.elempack = elempack;
    return m;
}

const Mat Mat::range(int x, int count) const
{
    return const_cast<Mat*>(this)->range(x, count);
}

Mat Mat::batch(int b)
{
    Mat m;
    m.set_shape(dims, w, h, d, c, elemsize, elempack, 1);
    m.cstep = cstep; // a reshaped blob may hold dense planes where a created one pads them
    m.nstep = cstep * c;
    m.data = (unsigned char*)data + nstep * b * elemsize;
    m.refcount = 0;
    m.allocator = allocator;
    return m;
}

const Mat Mat::batch(int b) const
{
    return const_cast<Mat*>(this)->batch(b);
}

// ---- fp16 helpers -----------------------------------------------------------------------

float float16_to_float32(unsigned short h)
{
    const unsigned sign = (h >> 15) & 1u, expo = (h >> 10) & 0x1fu, frac = h & 0x3ffu;
    union
    {
        unsigned u;
        float f;
    } v;
    if (expo == 0)
    {
        if (frac == 0)
            v.u = sign << 31;
        else
        {
            // subnormal half: renormalise
            int e = -1;
            unsigned m = frac;
            do
            {
                e++;
                m <<= 1;
            } while ((m & 0x400u) == 0);
            v.u = (sign << 31) | ((unsigned)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
        }
    }
    else if (expo == 31)
        v.u = (sign << 31) | 0x7f800000u | (frac << 13);
    else
        v.u = (sign << 31) | ((expo + 112u) << 23) | (frac << 13);
    return v.f;
}

unsigned short float32_to_float16(float value)
{
    union
    {
        unsigned u;
        float f;
    } v;
    v.f = value;
    const unsigned sign = (v.u >> 16) & 0x8000u;
    const int expo = (int)((v.u >> 23) & 0xffu);
    unsigned frac = v.u & 0x7fffffu;
    if (expo == 255) return (unsigned short)(sign | 0x7c00u | (frac ? 0x200u : 0u));
    int e = expo - 127 + 15;
    if (e >= 31) return (unsigned short)(sign | 0x7c00u);
    if (e <= 0)
    {
        if (e < -10) return (unsigned short)sign;
        frac |= 0x800000u;
        const int shift = 14 - e;
        unsigned half = frac >> shift;
        const unsigned rem = frac & ((1u << shift) - 1u), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        return (unsigned short)(sign | half);
    }
    unsigned half = ((unsigned)e << 10) | (frac >> 13);
    const unsigned rem = frac & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (unsigned short)(sign | half);
}

Mat Mat::from_float16(const unsigned short* src, int size)
{
    Mat m(size);
    if (m.empty()) return m;
    float* p = m;
    for (int i = 0; i < size; i++) p[i] = float16_to_float32(src[i]);
    return m;
}

// ---- load-time quantisation -------------------------------------------------------------

static inline signed char float2int8(float v)
{
    // round half away from zero, saturate to [-127, 127] (src/layer/quantize.cpp:30-36)
    int q = static_cast<int>(round(v));
    if (q > 127) return 127;
    if (q < -127) return -127;
    return (signed char)q;
}

void quantize_to_int8(const Mat& src, Mat& dst, const Mat& scale_data, const Option& opt)
{
    const float* scales = scale_data;
    const int nscales = scale_data.w;
    if (src.dims == 1)
    {
        dst.create(src.w, (size_t)1u, opt.blob_allocator);
        if (dst.empty()) return;
        const float* p = src;
        signed char* q = dst;
        for (int i = 0; i < src.w; i++) q[i] = float2int8(p[i] * scales[0]);
        return;
    }
    if (src.dims == 2)
    {
        dst.create(src.w, src.h, (size_t)1u, opt.blob_allocator);
        if (dst.empty()) return;
        for (int y = 0; y < src.h; y++)
        {
            const float s = nscales == 1 ? scales[0] : scales[y];
            const float* p = src.row(y);
            signed char* q = dst.row<signed char>(y);
            for (int i = 0; i < src.w; i++) q[i] = float2int8(p[i] * s);
        }
        return;
    }
    if (src.dims == 3)
        dst.create(src.w, src.h, src.c, (size_t)1u, opt.blob_allocator);
    else
        dst.create(src.w, src.h, src.d, src.c, (size_t)1u, opt.blob_allocator);
    if (dst.empty()) return;
    const size_t plane = (size_t)src.w * src.h * src.d;
    for (int ch = 0; ch < src.c; ch++)
    {
        const float s = nscales == 1 ? scales[0] : scales[ch];
        const float* p = (const float*)src.data + src.cstep * ch;
        signed char* q = (signed char*)dst.data + dst.cstep * ch;
        for (size_t i = 0; i < plane; i++) q[i] = float2int8(p[i] * s);
    }
}

} // namespace ncnn
