// Host fp32 implementations of the few non-quantised layers that sit between the int8 layers
// in the two benchmark nets (pack-1 semantics of the reference's naive layers):
//   Input    src/layer/input.cpp:19-22          Split    src/layer/split.cpp
//   ReLU     src/layer/relu.cpp                 Pooling  src/layer/pooling.cpp:18-415
//   Eltwise  src/layer/eltwise.cpp:14-178       Flatten  src/layer/flatten.cpp
//   Softmax  src/layer/softmax.cpp              Dropout  src/layer/dropout.cpp
// They keep the same summation order as the reference loops, so fp32 results match it.
#include <float.h>
#include <math.h>

#include <algorithm>

#include "../ncnn/layer.h"
#include "ncnnhip.h"

namespace ncnn {

// C-ABI status -> ncnn's 0 / -100 / -1
static int dev_status(int rc, const char* where)
{
    if (rc == 0) return 0;
    NCNN_LOGE("%s failed: %s", where, ncnnhip_last_error());
    return rc == NCNNHIP_OOM ? -100 : -1;
}

// ---------------------------------------------------------------------------------- Input
class Input : public Layer
{
public:
    Input()
    {
        one_blob_only = true;
        support_inplace = true;
        support_batch = true;
        support_hip = true;
    }
    virtual int forward_inplace_hip(HipMat&, HipCommand&, const Option&) const
    {
        return 0;
    }
    virtual int load_param(const ParamDict& pd)
    {
        w = pd.get(0, 0);
        h = pd.get(1, 0);
        d = pd.get(11, 0);
        c = pd.get(2, 0);
        return 0;
    }
    virtual int forward_inplace(Mat&, const Option&) const
    {
        return 0;
    }
    int w, h, d, c;
};

// ---------------------------------------------------------------------------------- Split
class Split : public Layer
{
public:
    Split()
    {
        support_batch = true;
        support_int8_storage = true; // int8 blobs pass through untouched
        support_hip = true;
    }
    virtual bool hip_accepts_narrow_input() const
    {
        return true; // handles are passed on, the data is not touched
    }
    virtual int forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand&, const Option&) const
    {
        for (size_t i = 0; i < top_blobs.size(); i++) top_blobs[i] = bottom_blobs[0]; // shared, refcounted
        return 0;
    }
    virtual int forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option&) const
    {
        for (size_t i = 0; i < top_blobs.size(); i++) top_blobs[i] = bottom_blobs[0]; // shared, refcounted
        return 0;
    }
};

// ---------------------------------------------------------------------------------- ReLU
class ReLU : public Layer
{
public:
    ReLU()
    {
        one_blob_only = true;
        support_inplace = true;
        support_int8_storage = true;
        support_hip = true;
    }
    virtual int load_param(const ParamDict& pd)
    {
        slope = pd.get(0, 0.f);
        return 0;
    }
    virtual bool hip_plain_relu() const
    {
        return slope == 0.f;
    }
    virtual int forward_inplace_hip(HipMat& m, HipCommand& cmd, const Option&) const
    {
        m.q8.reset(); // a quantised copy travelling with the blob describes the values before this layer
        // flat over the blob, pad channels included (zero stays zero)
        if (m.elemsize == 4u && m.count() % 4 != 0)
        {
            // dense 1-D / 2-D blobs of odd size: the pool rounds allocations up to 64 KiB, so the tail is ours
            return dev_status(ncnnhip_relu(m.data, m.data, 4, (m.count() + 3) / 4 * 4, slope, cmd.stream), "ncnnhip_relu");
        }
        return dev_status(ncnnhip_relu(m.data, m.data, (int)m.elemsize, m.count(), slope, cmd.stream), "ncnnhip_relu");
    }
    virtual int forward_inplace(Mat& m, const Option& opt) const
    {
        const size_t plane = (size_t)m.w * m.h * m.d;
        if (m.elemsize == 1)
        {
            #pragma omp parallel for num_threads(opt.num_threads)
            for (int q = 0; q < m.c; q++)
            {
                signed char* p = (signed char*)m.data + m.cstep * q;
                for (size_t i = 0; i < plane; i++)
                    if (p[i] < 0) p[i] = 0;
            }
            return 0;
        }
        #pragma omp parallel for num_threads(opt.num_threads)
        for (int q = 0; q < m.c; q++)
        {
            float* p = (float*)m.data + m.cstep * q;
            if (slope == 0.f)
            {
                for (size_t i = 0; i < plane; i++)
                    if (p[i] < 0.f) p[i] = 0.f;
            }
            else
            {
                for (size_t i = 0; i < plane; i++)
                    if (p[i] < 0.f) p[i] *= slope;
            }
        }
        return 0;
    }
    float slope;
};

// ---------------------------------------------------------------------------------- Pooling
class Pooling : public Layer
{
public:
    Pooling()
    {
        one_blob_only = true;
    }
    virtual int load_param(const ParamDict& pd)
    {
        pooling_type = pd.get(0, 0);
        kernel_w = pd.get(1, 0);
        kernel_h = pd.get(11, kernel_w);
        stride_w = pd.get(2, 1);
        stride_h = pd.get(12, stride_w);
        pad_left = pd.get(3, 0);
        pad_right = pd.get(14, pad_left);
        pad_top = pd.get(13, pad_left);
        pad_bottom = pd.get(15, pad_top);
        global_pooling = pd.get(4, 0);
        pad_mode = pd.get(5, 0);
        avgpool_count_include_pad = pd.get(6, 0);
        adaptive_pooling = pd.get(7, 0);
        if (adaptive_pooling)
        {
            NCNN_LOGE("Pooling: adaptive pooling is not part of this runtime");
            return -1;
        }
        support_hip = true;
        return 0;
    }

    // head pads and output extent of the border the reference would materialise (pad_mode 0 keeps the last
    // partial window, 1 drops it, 2/3 are the SAME splits)
    void resolve(int w, int h, int& pt, int& pl, int& outw, int& outh) const
    {
        int pb = pad_bottom, pr = pad_right;
        pt = pad_top;
        pl = pad_left;
        if (pad_mode == 0)
        {
            const int wtail = (w + pad_left + pad_right - kernel_w) % stride_w;
            const int htail = (h + pad_top + pad_bottom - kernel_h) % stride_h;
            if (wtail != 0) pr += stride_w - wtail;
            if (htail != 0) pb += stride_h - htail;
        }
        else if (pad_mode == 2 || pad_mode == 3)
        {
            const int wpad = kernel_w + (w - 1) / stride_w * stride_w - w;
            const int hpad = kernel_h + (h - 1) / stride_h * stride_h - h;
            pt = pb = pl = pr = 0;
            if (wpad > 0 || hpad > 0)
            {
                const int hs = hpad / 2, hl = hpad - hpad / 2, ws = wpad / 2, wl = wpad - wpad / 2;
                pt = pad_mode == 2 ? hs : hl;
                pb = pad_mode == 2 ? hl : hs;
                pl = pad_mode == 2 ? ws : wl;
                pr = pad_mode == 2 ? wl : ws;
            }
        }
        outw = (w + pl + pr - kernel_w) / stride_w + 1;
        outh = (h + pt + pb - kernel_h) / stride_h + 1;
    }

    // A SAME mode gives a negative border where the window is below the stride in one dimension while the other dimension
    // needs a border; the reference's border copy then writes every source row into a blob with fewer rows
    // (src/layer/padding.cpp:62-87), out of bounds and with no defined result: such a layer is refused.
    bool negative_same_border(int w, int h) const
    {
        if (pad_mode != 2 && pad_mode != 3) return false;
        const int wpad = kernel_w + (w - 1) / stride_w * stride_w - w;
        const int hpad = kernel_h + (h - 1) / stride_h * stride_h - h;
        if (!((wpad > 0 || hpad > 0) && (wpad < 0 || hpad < 0))) return false;
        NCNN_LOGE("Pooling: the padding mode resolves to a negative border (wpad %d hpad %d); the reference's border copy runs out of bounds for such a layer", wpad, hpad);
        return true;
    }

    // The rectangle (image coordinates) whose taps make up the divisor of an average without count_include_pad.  The
    // reference tests taps against the layer's own pad parameters in the bordered image -- rows [pad_top, hb - pad_bottom -
    // htailpad), tail pad only in pad_mode 0 (src/layer/pooling.cpp:255-305) -- so in pad_mode 2 / 3 the SAME border counts.
    void count_rect(int w, int h, int& x0, int& x1, int& y0, int& y1) const
    {
        int pt, pl, outw, outh;
        resolve(w, h, pt, pl, outw, outh);
        int wb = w + pad_left + pad_right, hb = h + pad_top + pad_bottom; // bordered extent without the tail pad of mode 0
        if (pad_mode == 2 || pad_mode == 3)
        {
            const int wpad = kernel_w + (w - 1) / stride_w * stride_w - w;
            const int hpad = kernel_h + (h - 1) / stride_h * stride_h - h;
            wb = w + ((wpad > 0 || hpad > 0) ? wpad : 0);
            hb = h + ((wpad > 0 || hpad > 0) ? hpad : 0);
        }
        x0 = pad_left - pl;
        x1 = wb - pad_right - pl;
        y0 = pad_top - pt;
        y1 = hb - pad_bottom - pt;
        if (x1 <= x0 || y1 <= y0)
        {
            // pad parameters that leave no tap to count (the reference divides 0 by 0): an empty rectangle that is not the
            // all-zero one, which the kernel's interface reads as "the image itself"
            x0 = y0 = 1;
            x1 = y1 = 0;
        }
    }

    virtual bool hip_quantise_transparent() const
    {
        return support_hip && pooling_type == 0 && !global_pooling;
    }

    // Global pooling can hand its consumers the quantised vector directly: float2int8(pool(x) * scale), the value
    // their own Quantize would compute from the fp32 result.
    virtual int hip_prepare_requantise(float scale)
    {
        return (support_hip && global_pooling && scale > 0.f) ? 0 : -1;
    }
    virtual int forward_hip_requantised(const HipMat& bottom, float scale, HipMat& top, HipCommand& cmd, const Option&) const
    {
        if (!global_pooling || bottom.dims != 3 || bottom.elemsize != 4u)
        {
            NCNN_LOGE("Pooling: the quantised form needs global pooling of a 3-D fp32 blob");
            return -1;
        }
        ncnnhip_pool_desc d;
        memset(&d, 0, sizeof(d));
        d.w = bottom.w;
        d.h = bottom.h;
        d.c = bottom.c;
        d.batch = bottom.n;
        d.pooling_type = pooling_type;
        d.global_pooling = 1;
        top.create(bottom.c, 1u, bottom.n, &cmd);
        if (top.empty()) return -100;
        top.q8_scale = scale;
        return dev_status(ncnnhip_global_pooling_nhwc_quantised(&d, (const float*)bottom.data, scale, (int8_t*)top.data, cmd.stream),
                          "ncnnhip_global_pooling_nhwc_quantised");
    }

    virtual int forward_hip(const HipMat& bottom, HipMat& top, HipCommand& cmd, const Option&) const
    {
        // an int8 blob only arrives here when the executor routed quantised values through this layer
        const bool quantised = bottom.elemsize == 1u && bottom.q8_scale > 0.f && hip_quantise_transparent();
        if (bottom.dims != 3 || (bottom.elemsize != 4u && !quantised))
        {
            NCNN_LOGE("Pooling: needs a 3-D fp32 blob");
            return -1;
        }
        ncnnhip_pool_desc d;
        memset(&d, 0, sizeof(d));
        d.w = bottom.w;
        d.h = bottom.h;
        d.c = bottom.c;
        d.batch = bottom.n;
        d.pooling_type = pooling_type;
        d.global_pooling = global_pooling;
        d.avgpool_count_include_pad = avgpool_count_include_pad;
        if (global_pooling)
        {
            top.create(bottom.c, 4u, bottom.n, &cmd);
            if (top.empty()) return -100;
            return dev_status(ncnnhip_pooling_nhwc(&d, (const float*)bottom.data, (float*)top.data, cmd.stream), "ncnnhip_pooling_nhwc");
        }
        d.kernel_w = kernel_w;
        d.kernel_h = kernel_h;
        d.stride_w = stride_w;
        d.stride_h = stride_h;
        if (negative_same_border(bottom.w, bottom.h)) return -1;
        resolve(bottom.w, bottom.h, d.pad_top, d.pad_left, d.outw, d.outh);
        count_rect(bottom.w, bottom.h, d.count_x0, d.count_x1, d.count_y0, d.count_y1);
        top.create(d.outw, d.outh, bottom.c, quantised ? (size_t)1u : (size_t)4u, bottom.n, &cmd);
        if (top.empty()) return -100;
        if (quantised)
        {
            top.q8_scale = bottom.q8_scale;
            return dev_status(ncnnhip_maxpool_nhwc_int8(&d, (const int8_t*)bottom.data, (int8_t*)top.data, cmd.stream), "ncnnhip_maxpool_nhwc_int8");
        }
        return dev_status(ncnnhip_pooling_nhwc(&d, (const float*)bottom.data, (float*)top.data, cmd.stream), "ncnnhip_pooling_nhwc");
    }

    virtual int forward(const Mat& bottom, Mat& top, const Option& opt) const
    {
        if (bottom.elemsize != 4u)
        {
            NCNN_LOGE("Pooling: only fp32 blobs are handled by this runtime");
            return -1;
        }
        const int w = bottom.w, h = bottom.h, channels = bottom.c;
        if (global_pooling)
        {
            top.create(channels, 4u, opt.blob_allocator);
            if (top.empty()) return -100;
            const int size = w * h;
            #pragma omp parallel for num_threads(opt.num_threads)
            for (int q = 0; q < channels; q++)
            {
                const float* p = (const float*)bottom.data + bottom.cstep * q;
                if (pooling_type == 0)
                {
                    float m = p[0];
                    for (int i = 0; i < size; i++) m = std::max(m, p[i]);
                    top[q] = m;
                }
                else
                {
                    float s = 0.f;
                    for (int i = 0; i < size; i++) s += p[i];
                    top[q] = s / size;
                }
            }
            return 0;
        }

        int pt, pl, outw, outh;
        if (negative_same_border(w, h)) return -1;
        resolve(w, h, pt, pl, outw, outh);
        top.create(outw, outh, channels, 4u, opt.blob_allocator);
        if (top.empty()) return -100;

        int cx0, cx1, cy0, cy1;
        count_rect(w, h, cx0, cx1, cy0, cy1);
        #pragma omp parallel for num_threads(opt.num_threads)
        for (int q = 0; q < channels; q++)
        {
            const float* in = (const float*)bottom.data + bottom.cstep * q;
            float* out = (float*)top.data + top.cstep * q;
            for (int i = 0; i < outh; i++)
            {
                for (int j = 0; j < outw; j++)
                {
                    const int y0 = i * stride_h - pt, x0 = j * stride_w - pl;
                    if (pooling_type == 0)
                    {
                        float m = -FLT_MAX;
                        bool first = true;
                        for (int ky = 0; ky < kernel_h; ky++)
                            for (int kx = 0; kx < kernel_w; kx++)
                            {
                                const int y = y0 + ky, x = x0 + kx;
                                const float v = (y >= 0 && y < h && x >= 0 && x < w) ? in[y * w + x] : -FLT_MAX;
                                m = first ? v : std::max(m, v);
                                first = false;
                            }
                        out[i * outw + j] = m;
                    }
                    else if (avgpool_count_include_pad == 0)
                    {
                        float s = 0.f;
                        int area = 0;
                        for (int ky = 0; ky < kernel_h; ky++)
                        {
                            const int y = y0 + ky;
                            if (y < cy0) continue;
                            if (y >= cy1) break;
                            for (int kx = 0; kx < kernel_w; kx++)
                            {
                                const int x = x0 + kx;
                                if (x < cx0) continue;
                                if (x >= cx1) break;
                                s += (y >= 0 && y < h && x >= 0 && x < w) ? in[y * w + x] : 0.f; // a counted border tap is the border's zero
                                area++;
                            }
                        }
                        out[i * outw + j] = s / area;
                    }
                    else
                    {
                        float s = 0.f;
                        for (int ky = 0; ky < kernel_h; ky++)
                            for (int kx = 0; kx < kernel_w; kx++)
                            {
                                const int y = y0 + ky, x = x0 + kx;
                                s += (y >= 0 && y < h && x >= 0 && x < w) ? in[y * w + x] : 0.f;
                            }
                        out[i * outw + j] = s / (kernel_w * kernel_h);
                    }
                }
            }
        }
        return 0;
    }

    int pooling_type, kernel_w, kernel_h, stride_w, stride_h, pad_left, pad_right, pad_top, pad_bottom;
    int global_pooling, pad_mode, avgpool_count_include_pad, adaptive_pooling;
};

// ---------------------------------------------------------------------------------- Eltwise
class Eltwise : public Layer
{
public:
    virtual int load_param(const ParamDict& pd)
    {
        op_type = pd.get(0, 0);
        coeffs = pd.get(1, Mat());
        support_hip = true;
        return 0;
    }
    virtual bool hip_plain_sum() const
    {
        return op_type == 1 && coeffs.w == 0;
    }
    virtual int forward_hip(const std::vector<HipMat>& bottoms, std::vector<HipMat>& tops, HipCommand& cmd, const Option&) const
    {
        if (bottoms.size() < 2) return -1;
        std::vector<const float*> srcs(bottoms.size());
        for (size_t i = 0; i < bottoms.size(); i++)
        {
            if (bottoms[i].elemsize != 4u || bottoms[i].count() != bottoms[0].count())
            {
                NCNN_LOGE("Eltwise: inputs must be fp32 blobs of one shape");
                return -1;
            }
            srcs[i] = (const float*)bottoms[i].data;
        }
        tops[0].create_like(bottoms[0], &cmd);
        if (tops[0].empty()) return -100;
        const size_t count = (bottoms[0].count() + 3) / 4 * 4; // allocations are rounded up, the tail is ours
        return dev_status(ncnnhip_eltwise(srcs.data(), (int)srcs.size(), op_type, coeffs.w ? (const float*)coeffs.data : 0, coeffs.w, (float*)tops[0].data, count, cmd.stream),
                          "ncnnhip_eltwise");
    }
    virtual int forward(const std::vector<Mat>& bottoms, std::vector<Mat>& tops, const Option& opt) const
    {
        const Mat& a = bottoms[0];
        if (bottoms.size() < 2 || a.elemsize != 4u) return -1;
        Mat& top = tops[0];
        top.create_like(a, opt.blob_allocator);
        if (top.empty()) return -100;
        const size_t plane = (size_t)a.w * a.h * a.d;
        const bool weighted = op_type == 1 && coeffs.w != 0;
        #pragma omp parallel for num_threads(opt.num_threads)
        for (int q = 0; q < a.c; q++)
        {
            float* out = (float*)top.data + top.cstep * q;
            const float* p0 = (const float*)a.data + a.cstep * q;
            const float* p1 = (const float*)bottoms[1].data + bottoms[1].cstep * q;
            if (op_type == 0)
                for (size_t i = 0; i < plane; i++) out[i] = p0[i] * p1[i];
            else if (op_type == 2)
                for (size_t i = 0; i < plane; i++) out[i] = std::max(p0[i], p1[i]);
            else if (weighted)
                for (size_t i = 0; i < plane; i++) out[i] = p0[i] * coeffs[0] + p1[i] * coeffs[1];
            else
                for (size_t i = 0; i < plane; i++) out[i] = p0[i] + p1[i];
            for (size_t b = 2; b < bottoms.size(); b++)
            {
                const float* pb = (const float*)bottoms[b].data + bottoms[b].cstep * q;
                if (op_type == 0)
                    for (size_t i = 0; i < plane; i++) out[i] *= pb[i];
                else if (op_type == 2)
                    for (size_t i = 0; i < plane; i++) out[i] = std::max(out[i], pb[i]);
                else if (weighted)
                    for (size_t i = 0; i < plane; i++) out[i] += pb[i] * coeffs[b];
                else
                    for (size_t i = 0; i < plane; i++) out[i] += pb[i];
            }
        }
        return 0;
    }
    int op_type;
    Mat coeffs;
};

// ---------------------------------------------------------------------------------- Flatten
class Flatten : public Layer
{
public:
    Flatten()
    {
        one_blob_only = true;
        support_hip = true;
        support_int8_storage = true;
    }
    virtual int forward_hip(const HipMat& bottom, HipMat& top, HipCommand& cmd, const Option&) const
    {
        if (bottom.dims != 3)
        {
            // dense blobs are already flat: same memory, new shape
            top = bottom;
            top.dims = 1;
            top.w = bottom.w * bottom.h;
            top.h = 1;
            return 0;
        }
        // the flattened order is the planar one: channel-major
        const int hw = bottom.w * bottom.h;
        top.create(hw * bottom.c, bottom.elemsize, bottom.n, &cmd);
        if (top.empty()) return -100;
        return dev_status(ncnnhip_nhwc_to_chw(bottom.data, (int)bottom.elemsize, bottom.c, hw, bottom.n, top.data, (size_t)hw, (size_t)hw * bottom.c, cmd.stream),
                          "ncnnhip_nhwc_to_chw");
    }
    virtual int forward(const Mat& bottom, Mat& top, const Option& opt) const
    {
        const size_t plane = (size_t)bottom.w * bottom.h * bottom.d;
        top.create((int)(plane * bottom.c), bottom.elemsize, opt.blob_allocator);
        if (top.empty()) return -100;
        for (int q = 0; q < bottom.c; q++)
            memcpy((unsigned char*)top.data + plane * q * bottom.elemsize, (const unsigned char*)bottom.data + bottom.cstep * q * bottom.elemsize, plane * bottom.elemsize);
        return 0;
    }
};

// ---------------------------------------------------------------------------------- Softmax
class Softmax : public Layer
{
public:
    Softmax()
    {
        one_blob_only = true;
        support_inplace = true;
    }
    virtual int load_param(const ParamDict& pd)
    {
        axis = pd.get(0, 0);
        support_hip = axis == 0;
        return 0;
    }
    virtual int forward_inplace_hip(HipMat& m, HipCommand& cmd, const Option&) const
    {
        if (m.dims != 1 || m.elemsize != 4u)
        {
            NCNN_LOGE("Softmax: the device overload handles 1-D fp32 blobs");
            return -1;
        }
        m.q8.reset();
        return dev_status(ncnnhip_softmax((const float*)m.data, (float*)m.data, m.w, m.n, cmd.stream), "ncnnhip_softmax");
    }
    virtual int forward_inplace(Mat& m, const Option&) const
    {
        // softmax over the outermost axis (axis 0), which is what classification heads use
        if (axis != 0 || m.elemsize != 4u)
        {
            NCNN_LOGE("Softmax: only axis 0 on fp32 blobs is handled by this runtime");
            return -1;
        }
        const int count = m.dims == 1 ? m.w : m.dims == 2 ? m.h : m.c;
        const size_t inner = m.dims == 1 ? 1 : m.dims == 2 ? (size_t)m.w : (size_t)m.w * m.h * m.d;
        const size_t step = m.dims == 1 ? 1 : m.dims == 2 ? (size_t)m.w : m.cstep;
        float* base = m;
        for (size_t i = 0; i < inner; i++)
        {
            float mx = -FLT_MAX;
            for (int q = 0; q < count; q++) mx = std::max(mx, base[q * step + i]);
            float sum = 0.f;
            for (int q = 0; q < count; q++)
            {
                float& v = base[q * step + i];
                v = expf(v - mx);
                sum += v;
            }
            for (int q = 0; q < count; q++) base[q * step + i] /= sum;
        }
        return 0;
    }
    int axis;
};

// ---------------------------------------------------------------------------------- Dropout
class Dropout : public Layer
{
public:
    Dropout()
    {
        one_blob_only = true;
        support_inplace = true;
    }
    virtual int load_param(const ParamDict& pd)
    {
        scale = pd.get(0, 1.f);
        support_hip = true;
        return 0;
    }
    virtual int forward_inplace_hip(HipMat& m, HipCommand& cmd, const Option&) const
    {
        if (scale == 1.f) return 0;
        if (m.elemsize != 4u) return -1;
        m.q8.reset();
        return dev_status(ncnnhip_scale((const float*)m.data, (float*)m.data, m.count(), scale, cmd.stream), "ncnnhip_scale");
    }
    virtual int forward_inplace(Mat& m, const Option&) const
    {
        if (scale == 1.f) return 0;
        const size_t plane = (size_t)m.w * m.h * m.d;
        for (int q = 0; q < m.c; q++)
        {
            float* p = (float*)m.data + m.cstep * q;
            for (size_t i = 0; i < plane; i++) p[i] *= scale;
        }
        return 0;
    }
    float scale;
};

DEFINE_LAYER_CREATOR(Input)
DEFINE_LAYER_CREATOR(Split)
DEFINE_LAYER_CREATOR(ReLU)
DEFINE_LAYER_CREATOR(Pooling)
DEFINE_LAYER_CREATOR(Eltwise)
DEFINE_LAYER_CREATOR(Flatten)
DEFINE_LAYER_CREATOR(Softmax)
DEFINE_LAYER_CREATOR(Dropout)

} // namespace ncnn
