// Glue between the ncnn::Layer implementations and the C ABI in include/ncnnhip.h:
// per-Extractor device context (one stream + a pool of device buffers), uploads of constant
// tables at create_pipeline, and the mapping of C-ABI return codes to ncnn's 0 / -100 / -1.
#ifndef NCNN_AMD_HIP_SUPPORT_H
#define NCNN_AMD_HIP_SUPPORT_H

#include <stddef.h>

#include <vector>

#include "../ncnn/allocator.h"
#include "../ncnn/hipmat.h"
#include "../ncnn/mat.h"
#include "../ncnn/option.h"
#include "ncnnhip.h"

namespace ncnn_amd {

// One stream and a pool of device buffers: the same object that carries device-resident blobs.  forward() of a
// HIP layer on host Mats borrows scratch for the duration of the call; everything it launched has completed
// (stream synchronised) before the scratch goes back.
typedef ncnn::HipCommand HipContext;

// Host allocator to install with Extractor::set_blob_allocator(): it hands out ordinary host
// memory (ncnn keeps a Mat's refcount inside the allocation and touches results on the host) and
// carries the Extractor's device context -- "one hipStream per Extractor".  Layers find it through
// opt.blob_allocator; without it a per-thread context is used.
class HipBlobAllocator : public ncnn::Allocator
{
public:
    HipBlobAllocator();
    virtual ~HipBlobAllocator();
    virtual void* fastMalloc(size_t size);
    virtual void fastFree(void* ptr);
    HipContext context;

private:
    ncnn::UnlockedPoolAllocator pool;
};

HipContext* context_for(const ncnn::Option& opt);

// RAII: buffers borrowed during one forward() return to the pool when it goes out of scope
class ScopedLeases
{
public:
    explicit ScopedLeases(HipContext* c) : ctx(c) {}
    ~ScopedLeases()
    {
        ctx->give_back_all();
    }
    void* get(size_t bytes)
    {
        return ctx->borrow(bytes);
    }

private:
    HipContext* ctx;
};

// 0 stays 0, -100 stays -100 (out of memory), anything else becomes -1 and is logged
int to_ncnn_status(int rc, const char* where);

// constant table -> device (create_pipeline); *dev is freed with ncnnhip_free at destroy_pipeline
int upload_constant(const void* host, size_t bytes, void** dev);

// Block-quantised weights (fields [n][ceil(k*bits/8)] and scales [n][ceil(k/block)] as the .bin holds them) repacked into
// matrix-core tiles and uploaded; both pointers stay null (and 0 is returned) when K has no kernel for that form.
int upload_blockquant_packed(const void* fields_host, const float* scales_host, int n, int k, int bits, int block, void** d_packed, void** d_descales);

// Gemm::forward_weight_block_quantize (src/layer/gemm.cpp:338-483) on device operands: for fewer than 32 activation rows the
// packed tiles when they exist and the rows are 16-byte aligned; from 32 rows up the tiled bf16 kernel on the packed tiles
// when the caller passes the scratch blockquant_gemm_workspace_bytes asks for (0: not applicable); else the .bin layout.
// Returns an ncnnhip status.
size_t blockquant_gemm_workspace_bytes(int M, int K, const void* d_packed);
int blockquant_gemm_device(const float* a_dev, size_t a_stride, int M, int N, int K, const void* d_fields, int bits, int block, const void* d_scales,
                           const void* d_in_scales, const void* d_packed, const void* d_descales, const float* c_dev, int bt, float alpha, float beta,
                           float* out_dev, size_t out_stride, void* workspace, size_t workspace_bytes, void* stream);

// blockquant_gemm_device with the scratch its many-row form wants, borrowed from the call's own allocator (leases / scratch: both
// hand the buffer back when the call's scope ends, after everything was enqueued on the one stream)
template<typename Alloc>
static inline int blockquant_gemm_with_scratch(Alloc& alloc, const float* a_dev, size_t a_stride, int M, int N, int K, const void* d_fields, int bits, int block,
                                        const void* d_scales, const void* d_in_scales, const void* d_packed, const void* d_descales, const float* c_dev, int bt,
                                        float alpha, float beta, float* out_dev, size_t out_stride, void* stream)
{
    const size_t bytes = blockquant_gemm_workspace_bytes(M, K, d_packed);
    void* ws = bytes ? alloc.get(bytes) : 0; // no room: the call falls back to the kernels that need none
    return blockquant_gemm_device(a_dev, a_stride, M, N, K, d_fields, bits, block, d_scales, d_in_scales, d_packed, d_descales, c_dev, bt, alpha, beta, out_dev,
                                  out_stride, ws, ws ? bytes : 0, stream);
}


// payload bytes of a Mat as it lies in memory (whole batch, including plane padding)
static inline size_t mat_bytes(const ncnn::Mat& m)
{
    return (m.n > 1 ? m.nstep * m.n : m.total()) * m.elemsize;
}

static inline ncnnhip_activation make_activation(int type, const ncnn::Mat& params)
{
    ncnnhip_activation a;
    a.type = type;
    a.p0 = params.w > 0 ? params[0] : 0.f;
    a.p1 = params.w > 1 ? params[1] : 0.f;
    return a;
}

} // namespace ncnn_amd

#endif // NCNN_AMD_HIP_SUPPORT_H
