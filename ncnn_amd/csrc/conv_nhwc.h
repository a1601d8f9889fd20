// Shared between the two channels-last convolution kernels (conv_nhwc.hip: any border value, planar or
// channels-last output; conv_nhwc_pipelined.hip: zero border, channels-last output, direct-to-LDS pipeline).
#ifndef NCNNHIP_CONV_NHWC_H
#define NCNNHIP_CONV_NHWC_H

#include "epilogues.h"

namespace ncnnhip {

struct NhwcGeom
{
    int H, W, Cp; // Cp: bytes from one pixel to the next
    int tapK;     // bytes of K one tap contributes (a multiple of 16).  Cp for an ordinary blob; 16 with Cp = 4 for the
                  // narrow-input image, where one "tap" is 4 neighbouring pixels x 4 channels and kw counts such groups
    int kw, kh, dw, dh, sw, sh;
    int pad_top, pad_left;
    int outw, outh;
    int npix;   // batch * outh * outw
    int ntaps;  // kh * kw
    int K;      // ntaps * Cp rounded up to 64
    int cout;
    int pad_word; // border byte replicated 4x
};

// Optional tail of the pipelined kernel's fp32 epilogue: out = [relu](act(acc*scale_in + bias) + residual), and a
// second, quantised copy of the result for the convolution that consumes it.
struct ConvFusion
{
    const float* residual; // channels-last fp32, the output's shape; 0: none
    int relu_after;
    int8_t* q8_out;        // channels-last int8 copy: float2int8(result * q8_scale); 0: none
    float q8_scale;
};

// The same kernel as a plain Gemm (a 1x1 convolution whose "pixels" are the rows of A): Gemm's dequantising epilogue
//   out = alpha * ((float)acc * (1/(sA_i*sB)) + beta*C)     or, one B scale per column,  ((float)acc * (1/sA_i)) * (1/sB_j)
// (Gemm::forward_int8, src/layer/gemm.cpp:509-555) replaces the convolution's.
struct GemmTail
{
    const float* a_scales; // [M]
    const float* b_scales; // [1] or [N]
    int per_col;
    const float* c;
    int bt; // -1 none, 0 scalar, 1/2 per row, 4 per column
    float alpha, beta;
};

// Workspace contract of the channels-last convolutions: the first SPLIT_COUNTER_BYTES hold one arrival counter per
// output tile of a K-split launch.  They must be zero when a call starts (the caller clears the workspace once, after
// allocating it) and are zero again when it has finished; the rest is scratch without a contract.
constexpr int SPLIT_MAX_TILES = 1024;
constexpr size_t SPLIT_COUNTER_BYTES = SPLIT_MAX_TILES * sizeof(unsigned);

// int32 words of workspace (counters included) the pipelined kernel wants for this problem (0: it does not split)
size_t conv_nhwc_pipelined_workspace_words(int cout, long long npix, int steps);

// Launches the pipelined kernel; the caller has checked: zero border byte, channels-last output.
int launch_conv_nhwc_pipelined(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp,
                               void* workspace, size_t workspace_bytes, hipStream_t stream);

// The 1x1 small-K int8-output kernel (conv_pointwise.hip): does this problem fit it, and its launch.  The pipelined
// launch asks first.
// One launch for a layer whose input is still fp32 (x_elemsize 4) or fp16 (2): quantised with x_scale[0] inside the kernel.
// Layers with few tiles split K over workgroups and need the workspace of conv_nhwc_staged_workspace_bytes (same contract
// as the other channels-last convolutions: zero when handed over, left zero).
bool conv_nhwc_staged_supported(const NhwcGeom& g);
size_t conv_nhwc_staged_workspace_bytes(const NhwcGeom& g);
int launch_conv_nhwc_staged(const NhwcGeom& g, const int8_t* wpk, const void* x, int x_elemsize, const float* x_scale, const ConvEpilogue& epi,
                            const ConvFusion& fusion, int out_cp, void* workspace, size_t workspace_bytes, hipStream_t stream);
// The small-tile kernel (conv_patch.hip: 2-D tiles of 32 output pixels, the input patch quantised into LDS, no
// workspace) for layers with few output pixels; x_elemsize 1 (int8 blob), 4 or 2 (fp32 / fp16 blob + x_scale).
// conv_patch_pays: the layer fits AND is of the kind that measured faster there than on the pipelined kernel.
bool conv_patch_supported(const NhwcGeom& g, int batch);
bool conv_patch_pays(const NhwcGeom& g, int batch, int x_elemsize);
int launch_conv_patch(const NhwcGeom& g, const int8_t* wpk, const void* x, int x_elemsize, const float* x_scale, const ConvEpilogue& epi, const ConvFusion& fusion,
                      int out_cp, hipStream_t stream);
bool conv_pointwise_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp);
bool conv_pointwise_stem_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp); // the narrow-input first layer on the same kernel
// The weights-resident kernel for layers with many output pixels (conv_resident.hip): does this problem fit it, and its
// launch.  The pipelined launch asks first.
bool conv_resident_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp);
int launch_conv_resident(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp, hipStream_t stream);
int launch_conv_pointwise(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, int out_cp, hipStream_t stream);

// D[M][N] = A[M][K] * B[N][K]^T through the pipelined kernel; handled = false when the shape does not fit it
// (K % 64, N % 4, strides, alignment) and the caller should take another kernel.
int launch_gemm_via_conv_pipelined(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmTail& tail,
                                   float* out, size_t out_stride, hipStream_t stream, bool* handled);

// InnerProduct as a 1x1 convolution over the activation rows (rows = pixels, K = channels): same epilogue as the
// convolution (scale_in, bias, activation), dense fp32 output with row stride out_stride.  handled = false when the
// shape does not fit (K % 64, num_output % 4, strides, alignment, workspace) and the caller should take another kernel.
int launch_fc_via_conv_pipelined(const int8_t* x, size_t x_stride, int rows, int K, int num_output, const int8_t* weight, const ConvEpilogue& epi,
                                 size_t out_stride, void* workspace, size_t workspace_bytes, hipStream_t stream, bool* handled);

// InnerProduct shapes the few-row kernel (gemm_int8.hip) serves without any workspace, given aligned operands
bool fc_skinny_takes(int rows, int num_input, int num_output);

// Device address, on the current device, of the scratch array the library holds for ncnnhip_innerproduct_int8_noalloc
// (looked up once per device; ncnnhip_init calls it so that the first real call finds it ready).
int static_scratch_for_current_device(void** ptr);

} // namespace ncnnhip

#endif // NCNNHIP_CONV_NHWC_H
