// MultiHeadAttention with block-quantised projection weights on the MI355X kernels
// (src/layer/multiheadattention.{h,cpp}: load_param :64-117, load_model :119-200, forward_weight_block_quantize :561-912,
// which bottom blob is what :914-1028).  The four projections are block-quantised Gemms with the bias as the per-column
// C term (sum starts at the bias, as in the reference loops); keys and values live on the device as [embed_dim][time],
// the layout of the layer's cache blobs, so a cache goes in and comes out without a transpose on the host.
#include <limits.h>
#include <math.h>
#include <string.h>

#include <vector>

#include "hip_layers.h"
#include "hip_support.h"

using namespace ncnn;

namespace ncnn_amd {

// quantize_term = bits*100 + has_input_scale*10 + block_code (src/layer/multiheadattention.cpp:11-44)
static bool att_is_block_quant(int term)
{
    const int bits = term / 100, fmt = term % 100 / 10, code = term % 10;
    return (bits == 4 || bits == 6 || bits == 8) && (fmt == 0 || fmt == 1) && code >= 0 && code <= 2;
}
static int att_bits(int term)
{
    return term / 100;
}
static int att_block(int term)
{
    const int code = term % 10;
    return code == 0 ? 32 : code == 1 ? 64 : 128;
}
static bool att_has_input_scale(int term)
{
    return term % 100 / 10 == 1;
}
static int att_packed_bytes(int k, int bits)
{
    if (k <= 0 || bits <= 0) return -1;
    const size_t b = ((size_t)k * bits + 7) / 8;
    return b > (size_t)INT_MAX ? -1 : (int)b;
}

MultiHeadAttention_hip::MultiHeadAttention_hip()
{
    one_blob_only = false;
    support_inplace = false;
    support_hip = true;
    weight_block_quantize = 0;
    memset(dev, 0, sizeof(dev));
    memset(dev_qkv, 0, sizeof(dev_qkv));
}

MultiHeadAttention_hip::~MultiHeadAttention_hip()
{
    destroy_pipeline(Option());
}

int MultiHeadAttention_hip::load_param(const ParamDict& pd)
{
    embed_dim = pd.get(0, 0);
    num_heads = pd.get(1, 1);
    weight_data_size = pd.get(2, 0);
    kdim = pd.get(3, embed_dim);
    vdim = pd.get(4, embed_dim);
    attn_mask = pd.get(5, 0);
    scale = pd.get(6, (embed_dim > 0 && num_heads > 0 && embed_dim / num_heads > 0) ? 1.f / sqrtf((float)(embed_dim / num_heads)) : 1.f);
    kv_cache = pd.get(7, 0);
    quantize_term = pd.get(18, 0);
    weight_block_quantize = att_is_block_quant(quantize_term) ? 1 : 0;
    if (!weight_block_quantize)
    {
        NCNN_LOGE("MultiHeadAttention %s: quantize_term %d; only block-quantised weights (4xx/6xx/8xx) run on this device path", name.c_str(), quantize_term);
        return -1;
    }
    if (embed_dim <= 0 || num_heads <= 0 || embed_dim % num_heads != 0 || weight_data_size <= 0 || weight_data_size % embed_dim != 0 || kdim <= 0 || vdim <= 0)
    {
        NCNN_LOGE("MultiHeadAttention unsupported weight block quantize");
        return -1;
    }
    return 0;
}

int MultiHeadAttention_hip::load_model(const ModelBin& mb)
{
    const int qdim = weight_data_size / embed_dim;
    const int bits = att_bits(quantize_term), block = att_block(quantize_term);
    // in, out of the four projections, in file order q, k, v, out
    const int in_dim[4] = {qdim, kdim, vdim, embed_dim};
    const int out_dim[4] = {embed_dim, embed_dim, embed_dim, qdim};
    for (int i = 0; i < 4; i++)
    {
        const int packed = att_packed_bytes(in_dim[i], bits);
        if (packed < 0) return -100;
        weight_data[i] = mb.load(packed, out_dim[i], 0);
        if (weight_data[i].empty()) return -100;
        bias_data[i] = mb.load(out_dim[i], 1);
        if (bias_data[i].empty()) return -100;
    }
    for (int i = 0; i < 4; i++)
    {
        weight_data_quantize_scales[i] = mb.load((in_dim[i] + block - 1) / block, out_dim[i], 1);
        if (weight_data_quantize_scales[i].empty()) return -100;
    }
    if (att_has_input_scale(quantize_term))
        for (int i = 0; i < 4; i++)
        {
            weight_data_input_scales[i] = mb.load(in_dim[i], 1);
            if (weight_data_input_scales[i].empty()) return -100;
        }
    return 0;
}

int MultiHeadAttention_hip::create_pipeline(const Option&)
{
    int ret = 0;
    for (int i = 0; i < 4 && ret == 0; i++)
    {
        if (weight_data[i].elemsize != 1u)
        {
            NCNN_LOGE("MultiHeadAttention %s: packed weights must be stored as bytes", name.c_str());
            return -1;
        }
        ret = upload_constant(weight_data[i].data, (size_t)weight_data[i].w * weight_data[i].h, &dev[i][0]);
        if (ret == 0) ret = upload_constant(weight_data_quantize_scales[i].data, (size_t)weight_data_quantize_scales[i].w * weight_data_quantize_scales[i].h * 4, &dev[i][1]);
        if (ret == 0 && !weight_data_input_scales[i].empty()) ret = upload_constant(weight_data_input_scales[i].data, (size_t)weight_data_input_scales[i].w * 4, &dev[i][2]);
        if (ret == 0) ret = upload_constant(bias_data[i].data, (size_t)bias_data[i].w * 4, &dev[i][3]);
        // second form of the weights for few rows (decoding): matrix-core tiles
        if (ret == 0)
        {
            const int in_dim[4] = {weight_data_size / embed_dim, kdim, vdim, embed_dim};
            ret = upload_blockquant_packed(weight_data[i].data, (const float*)weight_data_quantize_scales[i].data, weight_data[i].h, in_dim[i],
                                           att_bits(quantize_term), att_block(quantize_term), &dev[i][4], &dev[i][5]);
        }
    }
    // Self-attention reads one blob three times: with equal input widths and no per-projection input scales the three
    // weight matrices are also kept as one of 3 * embed_dim rows (q rows, k rows, v rows), so that q, k and v come out of
    // one Gemm.  The query's scale is applied where the attention kernel reads it.
    const int qdim = embed_dim > 0 ? weight_data_size / embed_dim : 0;
    if (ret == 0 && qdim == kdim && qdim == vdim && !att_has_input_scale(quantize_term))
    {
        const size_t wbytes = (size_t)weight_data[0].w * weight_data[0].h, sfloats = (size_t)weight_data_quantize_scales[0].w * weight_data_quantize_scales[0].h;
        bool same = true;
        for (int i = 1; i < 3; i++)
            same = same && (size_t)weight_data[i].w * weight_data[i].h == wbytes && (size_t)weight_data_quantize_scales[i].w * weight_data_quantize_scales[i].h == sfloats && weight_data[i].h == embed_dim;
        if (same && weight_data[0].h == embed_dim)
        {
            std::vector<unsigned char> fields(3 * wbytes);
            std::vector<float> scales(3 * sfloats), bias(3 * (size_t)embed_dim);
            for (int i = 0; i < 3; i++)
            {
                memcpy(fields.data() + i * wbytes, weight_data[i].data, wbytes);
                memcpy(scales.data() + i * sfloats, weight_data_quantize_scales[i].data, sfloats * 4);
                memcpy(bias.data() + (size_t)i * embed_dim, bias_data[i].data, (size_t)embed_dim * 4);
            }
            ret = upload_constant(fields.data(), fields.size(), &dev_qkv[0]);
            if (ret == 0) ret = upload_constant(scales.data(), scales.size() * 4, &dev_qkv[1]);
            if (ret == 0) ret = upload_constant(bias.data(), bias.size() * 4, &dev_qkv[3]);
            if (ret == 0)
                ret = upload_blockquant_packed(fields.data(), scales.data(), 3 * embed_dim, qdim, att_bits(quantize_term), att_block(quantize_term), &dev_qkv[4], &dev_qkv[5]);
        }
    }
    if (ret != 0) destroy_pipeline(Option());
    return ret;
}

int MultiHeadAttention_hip::destroy_pipeline(const Option&)
{
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 6; j++)
        {
            if (dev[i][j]) ncnnhip_free(dev[i][j]);
            dev[i][j] = 0;
        }
    for (int j = 0; j < 6; j++)
    {
        if (dev_qkv[j]) ncnnhip_free(dev_qkv[j]);
        dev_qkv[j] = 0;
    }
    return 0;
}

// dense 2-D fp32 blob [h][w]?  (rows of a 2-D Mat are contiguous)
static bool dense_2d(const Mat& m)
{
    return m.dims == 2 && m.elemsize == 4u && m.elempack == 1;
}

int MultiHeadAttention_hip::forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
{
    if (!dev[0][0])
    {
        NCNN_LOGE("MultiHeadAttention %s: forward before create_pipeline", name.c_str());
        return -1;
    }
    // q [, k [, v]] [, mask] [, cached k, cached v]
    const int extra = (attn_mask ? 1 : 0) + (kv_cache ? 2 : 0);
    const int n_qkv = (int)bottom_blobs.size() - extra;
    if (n_qkv < 1 || n_qkv > 3 || (int)top_blobs.size() < (kv_cache ? 3 : 1))
    {
        NCNN_LOGE("MultiHeadAttention %s: %d bottom blobs do not fit attn_mask=%d kv_cache=%d", name.c_str(), (int)bottom_blobs.size(), attn_mask, kv_cache);
        return -1;
    }
    const int k_i = n_qkv >= 2 ? 1 : 0, v_i = n_qkv == 3 ? 2 : k_i;
    const Mat& q_blob = bottom_blobs[0];
    const Mat& k_blob = bottom_blobs[(size_t)k_i];
    const Mat& v_blob = bottom_blobs[(size_t)v_i];
    const Mat mask_blob = attn_mask ? bottom_blobs[(size_t)n_qkv] : Mat();
    const Mat cached_k = kv_cache ? bottom_blobs[(size_t)(n_qkv + (attn_mask ? 1 : 0))] : Mat();
    const Mat cached_v = kv_cache ? bottom_blobs[(size_t)(n_qkv + (attn_mask ? 1 : 0) + 1)] : Mat();
    const bool self_attention = k_i == 0;

    const int qdim = weight_data_size / embed_dim;
    const int bits = att_bits(quantize_term), block = att_block(quantize_term);
    const int head_dim = embed_dim / num_heads;
    if (!dense_2d(q_blob) || !dense_2d(k_blob) || !dense_2d(v_blob) || q_blob.w != qdim || k_blob.w != kdim || v_blob.w != vdim || k_blob.h != v_blob.h)
    {
        NCNN_LOGE("MultiHeadAttention %s: q/k/v must be 2-D fp32 blobs of widths %d/%d/%d", name.c_str(), qdim, kdim, vdim);
        return -1;
    }
    const int src = q_blob.h, cur = k_blob.h;
    const int past = (kv_cache && !cached_k.empty()) ? cached_k.w : 0;
    const int dst = past > 0 ? (self_attention ? past + cur : past) : cur;
    const bool reuse_cache = past > 0 && !self_attention; // keys and values are the cache as it is
    if (past > 0 && (!dense_2d(cached_k) || !dense_2d(cached_v) || cached_k.h != embed_dim || cached_v.h != embed_dim || cached_v.w != past))
    {
        NCNN_LOGE("MultiHeadAttention %s: the cache blobs must be [%d][past] fp32", name.c_str(), embed_dim);
        return -1;
    }
    int mask_heads = 0;
    if (attn_mask)
    {
        const bool ok2 = mask_blob.dims == 2 && mask_blob.w == dst && mask_blob.h == src;
        const bool ok3 = mask_blob.dims == 3 && mask_blob.w == dst && mask_blob.h == src && mask_blob.c == num_heads;
        if ((!ok2 && !ok3) || mask_blob.elemsize != 4u || mask_blob.elempack != 1)
        {
            NCNN_LOGE("MultiHeadAttention %s: the mask must be [%d][%d] or [%d][%d][%d] fp32", name.c_str(), src, dst, num_heads, src, dst);
            return -1;
        }
        mask_heads = ok3 ? num_heads : 1;
    }

    Mat& top = top_blobs[0];
    top.create(qdim, src, 4u, opt.blob_allocator);
    if (top.empty()) return -100;
    Mat k_out, v_out;
    if (kv_cache)
    {
        if (reuse_cache)
        {
            k_out = cached_k;
            v_out = cached_v;
        }
        else
        {
            k_out.create(dst, embed_dim, 4u, opt.blob_allocator);
            v_out.create(dst, embed_dim, 4u, opt.blob_allocator);
            if (k_out.empty() || v_out.empty()) return -100;
        }
    }

    HipContext* ctx = context_for(opt);
    int ret = ctx->ensure_ready();
    if (ret != 0) return ret;
    ScopedLeases leases(ctx);
    void* st = ctx->stream;
    const size_t E = (size_t)embed_dim;

    const bool fused_qkv = dev_qkv[0] && self_attention; // one blob in, q / k / v out of one Gemm
    const size_t q_stride = fused_qkv ? 3 * E : E;
    float* d_q = (float*)leases.get((size_t)src * qdim * 4);
    float* d_qa = (float*)leases.get((size_t)src * q_stride * 4);
    float* d_kt = (float*)leases.get(E * dst * 4);
    float* d_vt = (float*)leases.get(E * dst * 4);
    float* d_ctx = (float*)leases.get((size_t)src * E * 4);
    float* d_out = (float*)leases.get((size_t)src * qdim * 4);
    if (!d_q || !d_qa || !d_kt || !d_vt || !d_ctx || !d_out) return -100;

    int rc = ncnnhip_memcpy_h2d(d_q, q_blob.data, (size_t)src * qdim * 4, st);
    if (rc == 0 && fused_qkv)
        rc = blockquant_gemm_with_scratch(leases, d_q, (size_t)qdim, src, 3 * embed_dim, qdim, dev_qkv[0], bits, block, dev_qkv[1], dev_qkv[2], dev_qkv[4], dev_qkv[5],
                                    (const float*)dev_qkv[3], 4, 1.f, 1.f, d_qa, q_stride, st);
    else if (rc == 0)
        rc = blockquant_gemm_with_scratch(leases, d_q, (size_t)qdim, src, embed_dim, qdim, dev[0][0], bits, block, dev[0][1], dev[0][2], dev[0][4], dev[0][5],
                                    (const float*)dev[0][3], 4, scale, 1.f, d_qa, E, st);
    if (rc != 0) return to_ncnn_status(rc, "q projection");

    if (reuse_cache)
    {
        rc = ncnnhip_memcpy_h2d(d_kt, cached_k.data, E * dst * 4, st);
        if (rc == 0) rc = ncnnhip_memcpy_h2d(d_vt, cached_v.data, E * dst * 4, st);
        if (rc != 0) return to_ncnn_status(rc, "upload cache");
    }
    else
    {
        if (past > 0)
        {
            float* d_ck = (float*)leases.get(E * past * 4);
            float* d_cv = (float*)leases.get(E * past * 4);
            if (!d_ck || !d_cv) return -100;
            rc = ncnnhip_memcpy_h2d(d_ck, cached_k.data, E * past * 4, st);
            if (rc == 0) rc = ncnnhip_memcpy_h2d(d_cv, cached_v.data, E * past * 4, st);
            if (rc == 0) rc = ncnnhip_copy2d(d_kt, (size_t)dst * 4, d_ck, (size_t)past * 4, (size_t)past * 4, E, st);
            if (rc == 0) rc = ncnnhip_copy2d(d_vt, (size_t)dst * 4, d_cv, (size_t)past * 4, (size_t)past * 4, E, st);
            if (rc != 0) return to_ncnn_status(rc, "cache into keys/values");
        }
        // k and v projections as [cur][embed_dim], then transposed into columns past.. of the [embed_dim][dst] blobs
        const Mat* in[2] = {&k_blob, &v_blob};
        float* outT[2] = {d_kt, d_vt};
        const int in_dim[2] = {kdim, vdim};
        float* d_kv_in = 0;
        for (int t = 0; t < 2 && !fused_qkv; t++)
        {
            const float* d_in = d_q;
            if (!(in[t]->data == q_blob.data && in_dim[t] == qdim))
            {
                if (t == 1 && v_blob.data == k_blob.data && d_kv_in)
                    d_in = d_kv_in;
                else
                {
                    d_kv_in = (float*)leases.get((size_t)cur * in_dim[t] * 4);
                    if (!d_kv_in) return -100;
                    rc = ncnnhip_memcpy_h2d(d_kv_in, in[t]->data, (size_t)cur * in_dim[t] * 4, st);
                    if (rc != 0) return to_ncnn_status(rc, "upload k/v");
                    d_in = d_kv_in;
                }
            }
            float* d_aff = (float*)leases.get((size_t)cur * E * 4);
            if (!d_aff) return -100;
            rc = blockquant_gemm_with_scratch(leases, d_in, (size_t)in_dim[t], cur, embed_dim, in_dim[t], dev[1 + t][0], bits, block, dev[1 + t][1], dev[1 + t][2], dev[1 + t][4], dev[1 + t][5],
                                    (const float*)dev[1 + t][3], 4, 1.f, 1.f, d_aff, E, st);
            if (rc == 0) rc = ncnnhip_transpose_f32(d_aff, E, cur, embed_dim, outT[t] + past, (size_t)dst, st);
            if (rc != 0) return to_ncnn_status(rc, "k/v projection");
        }
    }

    const float* d_mask = 0;
    if (attn_mask)
    {
        const size_t plane = (size_t)src * dst;
        float* m = (float*)leases.get(plane * mask_heads * 4);
        if (!m) return -100;
        for (int h = 0; h < mask_heads && rc == 0; h++) // channels of a 3-D Mat are cstep apart
            rc = ncnnhip_memcpy_h2d(m + plane * h, (const float*)mask_blob.data + (mask_blob.dims == 3 ? mask_blob.cstep * h : 0), plane * 4, st);
        if (rc != 0) return to_ncnn_status(rc, "upload mask");
        d_mask = m;
    }
    size_t att_ws_bytes = 0;
    rc = ncnnhip_attention_workspace_bytes(num_heads, head_dim, src, dst, &att_ws_bytes);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_attention_workspace_bytes");
    void* att_ws = att_ws_bytes ? leases.get(att_ws_bytes) : 0;
    if (att_ws_bytes && !att_ws) return -100;
    if (fused_qkv) // the new key and value columns are written behind the cache by the same call
        rc = ncnnhip_attention_f32_append(d_qa, q_stride, scale, d_kt, d_vt, (size_t)dst, past, d_mask, mask_heads, num_heads, head_dim, src, d_ctx, att_ws, att_ws_bytes, st);
    else
        rc = ncnnhip_attention_f32(d_qa, d_kt, d_vt, (size_t)dst, d_mask, mask_heads, num_heads, head_dim, src, dst, d_ctx, att_ws, att_ws_bytes, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_attention_f32");
    rc = blockquant_gemm_with_scratch(leases, d_ctx, E, src, qdim, embed_dim, dev[3][0], bits, block, dev[3][1], dev[3][2], dev[3][4], dev[3][5],
                                    (const float*)dev[3][3], 4, 1.f, 1.f, d_out, (size_t)qdim, st);
    if (rc != 0) return to_ncnn_status(rc, "out projection");
    rc = ncnnhip_memcpy_d2h(top.data, d_out, (size_t)src * qdim * 4, st);
    if (rc == 0 && kv_cache && !reuse_cache)
    {
        rc = ncnnhip_memcpy_d2h(k_out.data, d_kt, E * dst * 4, st);
        if (rc == 0) rc = ncnnhip_memcpy_d2h(v_out.data, d_vt, E * dst * 4, st);
    }
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    if (rc != 0) return to_ncnn_status(rc, "download");
    if (kv_cache)
    {
        top_blobs[1] = k_out;
        top_blobs[2] = v_out;
    }
    return 0;
}

// dense 2-D fp32 device blob of one sample
static bool dense_2d_dev(const HipMat& m)
{
    return m.dims == 2 && m.elemsize == 4u && m.n == 1;
}

int MultiHeadAttention_hip::forward_hip(const std::vector<HipMat>& bottom_blobs, std::vector<HipMat>& top_blobs, HipCommand& cmd, const Option& /*opt*/) const
{
    if (!dev[0][0])
    {
        NCNN_LOGE("MultiHeadAttention %s: forward before create_pipeline", name.c_str());
        return -1;
    }
    const int extra = (attn_mask ? 1 : 0) + (kv_cache ? 2 : 0);
    const int n_qkv = (int)bottom_blobs.size() - extra;
    if (n_qkv < 1 || n_qkv > 3 || (int)top_blobs.size() < (kv_cache ? 3 : 1))
    {
        NCNN_LOGE("MultiHeadAttention %s: %d bottom blobs do not fit attn_mask=%d kv_cache=%d", name.c_str(), (int)bottom_blobs.size(), attn_mask, kv_cache);
        return -1;
    }
    const int k_i = n_qkv >= 2 ? 1 : 0, v_i = n_qkv == 3 ? 2 : k_i;
    const HipMat& q_blob = bottom_blobs[0];
    const HipMat& k_blob = bottom_blobs[(size_t)k_i];
    const HipMat& v_blob = bottom_blobs[(size_t)v_i];
    const HipMat mask_blob = attn_mask ? bottom_blobs[(size_t)n_qkv] : HipMat();
    const HipMat cached_k = kv_cache ? bottom_blobs[(size_t)(n_qkv + (attn_mask ? 1 : 0))] : HipMat();
    const HipMat cached_v = kv_cache ? bottom_blobs[(size_t)(n_qkv + (attn_mask ? 1 : 0) + 1)] : HipMat();
    const bool self_attention = k_i == 0;

    const int qdim = weight_data_size / embed_dim;
    const int bits = att_bits(quantize_term), block = att_block(quantize_term);
    const int head_dim = embed_dim / num_heads;
    if (!dense_2d_dev(q_blob) || !dense_2d_dev(k_blob) || !dense_2d_dev(v_blob) || q_blob.w != qdim || k_blob.w != kdim || v_blob.w != vdim || k_blob.h != v_blob.h)
    {
        NCNN_LOGE("MultiHeadAttention %s: q/k/v must be 2-D fp32 blobs of widths %d/%d/%d", name.c_str(), qdim, kdim, vdim);
        return -1;
    }
    const int src = q_blob.h, cur = k_blob.h;
    const int past = (kv_cache && !cached_k.empty()) ? cached_k.w : 0;
    const int dst = past > 0 ? (self_attention ? past + cur : past) : cur;
    const bool reuse_cache = past > 0 && !self_attention; // keys and values are the cache as it is
    if (past > 0 && (!dense_2d_dev(cached_k) || !dense_2d_dev(cached_v) || cached_k.h != embed_dim || cached_v.h != embed_dim || cached_v.w != past))
    {
        NCNN_LOGE("MultiHeadAttention %s: the cache blobs must be [%d][past] fp32", name.c_str(), embed_dim);
        return -1;
    }
    ScopedScratch scratch(&cmd);
    void* st = cmd.stream;
    const size_t E = (size_t)embed_dim;
    int rc = 0;

    int mask_heads = 0;
    const float* d_mask = 0;
    if (attn_mask)
    {
        const bool ok2 = mask_blob.dims == 2 && mask_blob.w == dst && mask_blob.h == src;
        const bool ok3 = mask_blob.dims == 3 && mask_blob.w == dst && mask_blob.h == src && mask_blob.c == num_heads;
        if ((!ok2 && !ok3) || mask_blob.elemsize != 4u || mask_blob.n != 1)
        {
            NCNN_LOGE("MultiHeadAttention %s: the mask must be [%d][%d] or [%d][%d][%d] fp32", name.c_str(), src, dst, num_heads, src, dst);
            return -1;
        }
        mask_heads = ok3 ? num_heads : 1;
        d_mask = (const float*)mask_blob.data;
        if (ok3)
        {
            // a 3-D blob lies channels-last in HBM; the attention kernel reads one [src][dst] plane per head
            const size_t plane = (size_t)src * dst;
            float* planar = (float*)scratch.get(plane * num_heads * 4);
            if (!planar) return -100;
            rc = ncnnhip_nhwc_to_chw(mask_blob.data, 4, num_heads, (int)plane, 1, planar, plane, plane * num_heads, st);
            if (rc != 0) return to_ncnn_status(rc, "ncnnhip_nhwc_to_chw");
            d_mask = planar;
        }
    }

    HipMat& top = top_blobs[0];
    top.create(qdim, src, 4u, 1, &cmd);
    if (top.empty()) return -100;
    HipMat k_out, v_out;
    float* d_kt = 0;
    float* d_vt = 0;
    if (reuse_cache)
    {
        k_out = cached_k;
        v_out = cached_v;
        d_kt = (float*)cached_k.data;
        d_vt = (float*)cached_v.data;
    }
    else if (kv_cache)
    {
        k_out.create(dst, embed_dim, 4u, 1, &cmd);
        v_out.create(dst, embed_dim, 4u, 1, &cmd);
        if (k_out.empty() || v_out.empty()) return -100;
        d_kt = (float*)k_out.data;
        d_vt = (float*)v_out.data;
    }
    else
    {
        d_kt = (float*)scratch.get(E * dst * 4);
        d_vt = (float*)scratch.get(E * dst * 4);
        if (!d_kt || !d_vt) return -100;
    }
    const bool fused_qkv = dev_qkv[0] && self_attention; // one blob in, q / k / v out of one Gemm
    const size_t q_stride = fused_qkv ? 3 * E : E;
    float* d_qa = (float*)scratch.get((size_t)src * q_stride * 4);
    float* d_ctx = (float*)scratch.get((size_t)src * E * 4);
    if (!d_qa || !d_ctx) return -100;

    if (fused_qkv)
        rc = blockquant_gemm_with_scratch(scratch, (const float*)q_blob.data, (size_t)qdim, src, 3 * embed_dim, qdim, dev_qkv[0], bits, block, dev_qkv[1], dev_qkv[2], dev_qkv[4],
                                    dev_qkv[5], (const float*)dev_qkv[3], 4, 1.f, 1.f, d_qa, q_stride, st);
    else
        rc = blockquant_gemm_with_scratch(scratch, (const float*)q_blob.data, (size_t)qdim, src, embed_dim, qdim, dev[0][0], bits, block, dev[0][1], dev[0][2], dev[0][4], dev[0][5],
                                    (const float*)dev[0][3], 4, scale, 1.f, d_qa, E, st);
    if (rc != 0) return to_ncnn_status(rc, "q projection");
    if (!reuse_cache)
    {
        if (past > 0)
        {
            rc = ncnnhip_copy2d(d_kt, (size_t)dst * 4, cached_k.data, (size_t)past * 4, (size_t)past * 4, E, st);
            if (rc == 0) rc = ncnnhip_copy2d(d_vt, (size_t)dst * 4, cached_v.data, (size_t)past * 4, (size_t)past * 4, E, st);
            if (rc != 0) return to_ncnn_status(rc, "cache into keys/values");
        }
        const HipMat* in[2] = {&k_blob, &v_blob};
        float* outT[2] = {d_kt, d_vt};
        const int in_dim[2] = {kdim, vdim};
        for (int t = 0; t < 2 && !fused_qkv; t++)
        {
            float* d_aff = (float*)scratch.get((size_t)cur * E * 4);
            if (!d_aff) return -100;
            rc = blockquant_gemm_with_scratch(scratch, (const float*)in[t]->data, (size_t)in_dim[t], cur, embed_dim, in_dim[t], dev[1 + t][0], bits, block, dev[1 + t][1], dev[1 + t][2], dev[1 + t][4], dev[1 + t][5],
                                    (const float*)dev[1 + t][3], 4, 1.f, 1.f, d_aff, E, st);
            if (rc == 0) rc = ncnnhip_transpose_f32(d_aff, E, cur, embed_dim, outT[t] + past, (size_t)dst, st);
            if (rc != 0) return to_ncnn_status(rc, "k/v projection");
        }
    }
    size_t att_ws_bytes = 0;
    rc = ncnnhip_attention_workspace_bytes(num_heads, head_dim, src, dst, &att_ws_bytes);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_attention_workspace_bytes");
    void* att_ws = att_ws_bytes ? scratch.get(att_ws_bytes) : 0;
    if (att_ws_bytes && !att_ws) return -100;
    if (fused_qkv) // the new key and value columns are written behind the cache by the same call
        rc = ncnnhip_attention_f32_append(d_qa, q_stride, scale, d_kt, d_vt, (size_t)dst, past, d_mask, mask_heads, num_heads, head_dim, src, d_ctx, att_ws, att_ws_bytes, st);
    else
        rc = ncnnhip_attention_f32(d_qa, d_kt, d_vt, (size_t)dst, d_mask, mask_heads, num_heads, head_dim, src, dst, d_ctx, att_ws, att_ws_bytes, st);
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_attention_f32");
    rc = blockquant_gemm_with_scratch(scratch, d_ctx, E, src, qdim, embed_dim, dev[3][0], bits, block, dev[3][1], dev[3][2], dev[3][4], dev[3][5],
                                    (const float*)dev[3][3], 4, 1.f, 1.f, (float*)top.data, (size_t)qdim, st);
    if (rc != 0) return to_ncnn_status(rc, "out projection");
    if (kv_cache)
    {
        top_blobs[1] = k_out;
        top_blobs[2] = v_out;
    }
    return 0;
}

Layer* MultiHeadAttention_hip_creator(void*)
{
    return new MultiHeadAttention_hip;
}

} // namespace ncnn_amd
