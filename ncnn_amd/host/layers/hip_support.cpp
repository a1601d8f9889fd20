#include "hip_support.h"

#include "../ncnn/platform.h"

#include <stdint.h>
#include <vector>

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

int upload_blockquant_packed(const void* fields_host, const float* scales_host, int n, int k, int bits, int block, void** d_packed, void** d_descales)
{
    *d_packed = 0;
    *d_descales = 0;
    if (k % 16 != 0) return 0;
    const bool halves = bits != 8 || block == 32; // those layouts stop at K = 16384; 8-bit fields in blocks of 64 / 128 serve the tiled kernel beyond it
    if (halves && k > 16384) return 0;
    size_t wb = 0, db = 0;
    if (ncnnhip_blockquant_packed_size(n, k, bits, block, &wb, &db) != 0) return 0;
    std::vector<uint8_t> pw(wb);
    std::vector<float> pd(db / sizeof(float));
    int rc = ncnnhip_blockquant_pack((const uint8_t*)fields_host, scales_host, n, k, bits, block, pw.data(), pd.data());
    if (rc != 0) return to_ncnn_status(rc, "ncnnhip_blockquant_pack");
    int ret = upload_constant(pw.data(), wb, d_packed);
    if (ret == 0) ret = upload_constant(pd.data(), db, d_descales);
    if (ret != 0)
    {
        if (*d_packed) ncnnhip_free(*d_packed);
        if (*d_descales) ncnnhip_free(*d_descales);
        *d_packed = 0;
        *d_descales = 0;
    }
    return ret;
}

size_t blockquant_gemm_workspace_bytes(int M, int K, const void* d_packed)
{
    // 5 rows and more: the kernels that split the activations in a pass of their own (the weight-streaming one on pre-split
    // operands, 16 rows per pass, while that is cheaper than a tiled pass; else the tiled one: the entry point picks).
    // 3 and 4 rows of a K beyond 4096 too: the few-row kernel holds three planes per row in LDS and takes such rows one at
    // a time, a pass over the weights each (4096 x 11008, 4 rows: 48 us against 26 us this way).
    if (!d_packed || K % 16 != 0 || M < 3 || (M < 5 && K <= 4096)) return 0;
    size_t bytes = 0;
    if (ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(M, K, &bytes) != 0) return 0;
    return bytes;
}

int blockquant_gemm_device(const float* a_dev, size_t a_stride, int M, int N, int K, const void* d_fields, int bits, int block, const void* d_scales,
                           const void* d_in_scales, const void* d_packed, const void* d_descales, const float* c_dev, int bt, float alpha, float beta,
                           float* out_dev, size_t out_stride, void* workspace, size_t workspace_bytes, void* stream)
{
    // five rows and more: the kernels that split the activations in a pass of their own, when the caller brought the workspace for it
    const size_t need = blockquant_gemm_workspace_bytes(M, K, d_packed);
    if (need && d_descales && workspace && workspace_bytes >= need)
        return ncnnhip_gemm_blockquant_packed_rows(a_dev, a_stride, M, N, K, (const uint8_t*)d_packed, (const float*)d_descales, bits, block,
                                                   (const float*)d_in_scales, c_dev, bt, alpha, beta, out_dev, out_stride, workspace, workspace_bytes, stream);
    // few rows: the packed tiles, one pass over the weights per four rows at most
    if (d_packed && d_descales && M < 32 && ncnnhip_gemm_blockquant_packed_supported(K) && a_stride % 4 == 0 && ((uintptr_t)a_dev & 15) == 0
        && (!d_in_scales || ((uintptr_t)d_in_scales & 15) == 0))
        return ncnnhip_gemm_blockquant_packed(a_dev, a_stride, M, N, K, (const uint8_t*)d_packed, (const float*)d_descales, bits, block,
                                              (const float*)d_in_scales, c_dev, bt, alpha, beta, out_dev, out_stride, stream);
    return ncnnhip_gemm_blockquant(a_dev, a_stride, M, N, K, (const uint8_t*)d_fields, bits, block, (const float*)d_scales, (const float*)d_in_scales, c_dev, bt,
                                   alpha, beta, out_dev, out_stride, stream);
}

} // namespace ncnn_amd
