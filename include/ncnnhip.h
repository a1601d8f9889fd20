/*
 * ncnnhip -- C ABI of the MI355X (gfx950) implementation of ncnn's int8 / block-quant hot path.
 *
 * Plain pointers and sizes only.  Every `*_dev` / device pointer is memory obtained from
 * ncnnhip_malloc (or any hipMalloc'd buffer); `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  All launch functions are asynchronous on `stream`, allocate
 * nothing and never synchronise; temporaries are passed in by the caller.
 *
 * Return values follow ncnn's layer convention (src/layer/convolution.cpp:402-403,
 * src/layer.cpp:69): 0 success, -100 out of memory, -1 any other failure;
 * ncnnhip_last_error() gives the text of the last failure on the calling thread.
 *
 * Layouts are ncnn::Mat layouts (src/mat.h:341-381): a 3-D blob is [c][h][w] with `cstep`
 * elements between channels, a batch adds `nstep` elements between samples, a 2-D blob is
 * [h][w] rows.  Strides are in ELEMENTS of the pointed-to type.
 */
#ifndef NCNNHIP_H
#define NCNNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* every declaration below is exported from libncnnhip.so (the library is built with hidden default visibility) */
#pragma GCC visibility push(default)

#define NCNNHIP_OK 0
#define NCNNHIP_ERROR (-1)
#define NCNNHIP_OOM (-100)

/* ------------------------------------------------------------------ runtime plumbing
 * Replaces what ncnn's only device back-end does through VkAllocator / VkCompute
 * (src/net.cpp:2906-2930): buffers, one stream per Extractor, uploads and downloads. */
int ncnnhip_init(int device);
const char* ncnnhip_last_error(void);
int ncnnhip_device_info(char* name, size_t name_len, int* compute_units, size_t* total_mem);
int ncnnhip_stream_create(void** stream);
int ncnnhip_stream_destroy(void* stream);
int ncnnhip_stream_synchronize(void* stream);
int ncnnhip_device_synchronize(void);
/* Record once, replay with one call: what the reference's GPU path does with a recorded VkCompute command buffer
 * (src/command.h:22-67, record_* then submit_and_wait).  Between begin and end every launch on `stream` is recorded
 * instead of run; nothing may allocate, copy from pageable memory or synchronise on the capturing thread.  The
 * executable graph replays the same kernels on the same buffers. */
int ncnnhip_stream_begin_capture(void* stream);
int ncnnhip_stream_end_capture(void* stream, void** graph_exec);
int ncnnhip_graph_launch(void* graph_exec, void* stream);
int ncnnhip_graph_destroy(void* graph_exec);
int ncnnhip_malloc(void** dev, size_t bytes);
int ncnnhip_free(void* dev);
/* The device allocator behind ncnnhip_malloc / ncnnhip_free, and so behind every device buffer the host library cuts its
 * blobs and workspaces from: the role ncnn::VkAllocator plays for the reference's GPU path (src/allocator.h:267-300,
 * Option::blob_vkallocator, src/option.h:48).  A caller that already runs a device pool installs its own pair; malloc_fn returns 0 and a
 * device pointer, or anything else to refuse (ncnnhip_malloc then reports -100, as the reference's layers do when an
 * allocator returns NULL: tests/testutil.cpp:2111-2156 forces that condition the same way).  Passing two null functions
 * restores hipMalloc / hipFree, which ncnnhip_default_device_malloc / _free expose for allocators that wrap them.  Install
 * before the first buffer is allocated or make free_fn accept pointers of the previous allocator. */
typedef int (*ncnnhip_device_malloc_fn)(void** dev, size_t bytes, void* user);
typedef int (*ncnnhip_device_free_fn)(void* dev, void* user);
int ncnnhip_set_device_allocator(ncnnhip_device_malloc_fn malloc_fn, ncnnhip_device_free_fn free_fn, void* user);
int ncnnhip_default_device_malloc(void** dev, size_t bytes);
int ncnnhip_default_device_free(void* dev);
int ncnnhip_memcpy_h2d(void* dev, const void* host, size_t bytes, void* stream);
int ncnnhip_memcpy_d2h(void* host, const void* dev, size_t bytes, void* stream);
int ncnnhip_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
int ncnnhip_memset(void* dev, int byte, size_t bytes, void* stream);
/* rows x row_bytes between two pitched device buffers (appending to a key/value cache whose rows grow) */
int ncnnhip_copy2d(void* dst_dev, size_t dst_pitch, const void* src_dev, size_t src_pitch, size_t row_bytes, size_t rows, void* stream);
int ncnnhip_event_create(void** event);
int ncnnhip_event_destroy(void* event);
int ncnnhip_event_record(void* event, void* stream);
int ncnnhip_event_synchronize(void* event);
int ncnnhip_event_elapsed_ms(void* start, void* stop, float* ms);

/* ------------------------------------------------------------------ fused activation
 * ncnn activation_type / activation_params (src/layer/fused_activation.h:10-64):
 * 0 none, 1 relu, 2 leaky(p0), 3 clip[p0,p1], 4 sigmoid, 5 mish, 6 hardswish(p0,p1). */
typedef struct ncnnhip_activation
{
    int type;
    float p0;
    float p1;
} ncnnhip_activation;

/* ------------------------------------------------------------------ Quantize
 * Quantize::forward, src/layer/quantize.cpp:48-111 (reached through quantize_to_int8,
 * src/mat.cpp:2406-2427): y = float2int8(x * scale), one scale or one per row.
 * rows = h of a 2-D blob or c of a 3-D blob (cols = w*h of a channel); `batch` samples. */
int ncnnhip_quantize(const float* x_dev, size_t x_stride, size_t x_nstep, int8_t* y_dev, size_t y_stride, size_t y_nstep,
                     int rows, int cols, int batch, const float* scales_dev, int nscales, void* stream);

/* ------------------------------------------------------------------ Convolution / ConvolutionDepthWise
 * Geometry of Convolution::load_param ids 0,1,11,2,12,3,13,4,15,14,16,18 (src/layer/convolution.cpp:18-38)
 * plus ConvolutionDepthWise id 7 (src/layer/convolutiondepthwise.cpp:34). */
typedef struct ncnnhip_conv_desc
{
    int w, h, c;    /* input blob */
    int batch;      /* Mat.n; folded into the pixel dimension */
    int num_output;
    int kernel_w, kernel_h;
    int dilation_w, dilation_h;
    int stride_w, stride_h;
    int pad_left, pad_right, pad_top, pad_bottom; /* raw param values incl. -233 / -234 */
    float pad_value;                              /* border byte = (signed char)pad_value */
    int group;                                    /* 1 for Convolution */
} ncnnhip_conv_desc;

/* Output extent after make_padding (src/layer/convolution.cpp:328-372, 412-413).  NCNNHIP_ERROR for an empty output and
 * for a SAME mode (-233 / -234) that resolves to a negative border (kernel extent below the stride in one dimension while
 * the other needs a border): the reference's border copy (src/layer/padding.cpp:62-87) writes out of bounds there and has
 * no defined result.  Every convolution entry point sizes its output through this call and refuses the same layers. */
int ncnnhip_conv_out_shape(const ncnnhip_conv_desc* desc, int* outw, int* outh);
/* Head pads make_padding resolves to (literal values, or the SAME_UPPER / SAME_LOWER split, :348-371). */
int ncnnhip_conv_resolved_pads(const ncnnhip_conv_desc* desc, int* pad_top, int* pad_left);

/* Host helper used at create_pipeline: expands ncnn's scale tables to one value per output
 * channel with the reference's own expression
 *   scale_in[p] = w_scale == 0 ? 0 : 1.f / (in_scale * w_scale)
 * (src/layer/convolution.cpp:476-480; per-group indexing src/layer/convolutiondepthwise.cpp:529-533).
 * n_w_scales is num_output (Convolution, InnerProduct) or group (depthwise); n_in_scales 1 or group. */
int ncnnhip_fold_input_scales(const float* w_scales, int n_w_scales, const float* in_scales, int n_in_scales,
                              int num_output, float* scale_in_out);

/* Convolution::forward_int8 (src/layer/convolution.cpp:383-508) and
 * ConvolutionDepthWise::forward_int8 (src/layer/convolutiondepthwise.cpp:418-636) after input
 * quantisation.  x is int8 [batch][c][h][w]; weight int8 [num_output][c/group][kh][kw];
 * scale_in / bias / scale_out hold one float per OUTPUT CHANNEL (bias, scale_out may be NULL).
 * scale_out != NULL selects the requantising epilogue (int8 output), otherwise fp32 output.
 * acc_out (optional, may be NULL) receives the raw int32 accumulators [batch][num_output][outh*outw]. */
int ncnnhip_conv_int8(const ncnnhip_conv_desc* desc, const int8_t* x_dev, size_t x_cstep, size_t x_nstep,
                      const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                      const float* scale_out_dev, ncnnhip_activation act, void* out_dev, size_t out_cstep,
                      size_t out_nstep, int32_t* acc_out_dev, void* stream);

/* Channels-last fast path of Convolution::forward_int8 (group 1).  The activations are first copied to
 * [batch][h][w][Cp] int8, Cp = 16*ceil(c/16) -- from fp32 with the Quantize arithmetic (one scale or one per
 * channel) or from int8 as is -- and the weights are repacked once (host side, at create_pipeline) to
 * [num_output][kh*kw][Cp] with K padded to a multiple of 64.  Results are identical to ncnnhip_conv_int8.
 * workspace: scratch for layers whose K loop is split across workgroups (size from ncnnhip_conv_nhwc_sizes, may be 0).
 * Zero-fill it ONCE after allocating it (ncnnhip_memset); every call leaves it fit for the next call, so one workspace of
 * the largest size serves all layers of a net, one call at a time (calls that overlap on one workspace race).
 * out_layout NCNNHIP_PLANAR: out is ncnn's [batch][num_output][out_cstep] (out_nstep between samples);
 * NCNNHIP_CHANNELS_LAST: out is [batch][outh*outw][16*ceil(num_output/16)], pad channels written as zero
 * (out_cstep / out_nstep ignored) -- the form the next layer's kernel consumes without a conversion pass. */
#define NCNNHIP_PLANAR 0
#define NCNNHIP_CHANNELS_LAST 1
int ncnnhip_conv_nhwc_sizes(const ncnnhip_conv_desc* desc, size_t* nhwc_bytes, size_t* packed_weight_bytes, size_t* workspace_bytes);
int ncnnhip_conv_pack_weights(const ncnnhip_conv_desc* desc, const int8_t* weight_host, int8_t* packed_host);
int ncnnhip_to_nhwc_int8(const ncnnhip_conv_desc* desc, const void* x_dev, int x_elemsize, size_t x_cstep, size_t x_nstep,
                         const float* scales_dev, int nscales, int8_t* nhwc_dev, void* stream);
int ncnnhip_conv_int8_nhwc(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev,
                           const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act,
                           void* out_dev, int out_layout, size_t out_cstep, size_t out_nstep, void* workspace_dev,
                           size_t workspace_bytes, void* stream);

/* The same convolution (fp32 channels-last output, zero border value) with the layers that follow it folded into its
 * epilogue, element by element in the reference's order:
 *   f = act(acc*scale_in + bias)                      Convolution::forward_int8, src/layer/convolution.cpp:476-502
 *   f = f + residual                                  Eltwise sum of two inputs, src/layer/eltwise.cpp:95-118
 *   f = max(f, 0)                  (relu_after)       ReLU slope 0, src/layer/relu.cpp:30-45
 *   out = f;  quantised_out = float2int8(f * scale)   Quantize of the next convolution's input, src/layer/quantize.cpp:48-111
 * Every step is optional (NULL / 0).  ncnnhip_conv_fusion_supported says whether a geometry can take this path. */
typedef struct ncnnhip_conv_fusion
{
    const float* residual_dev;  /* channels-last fp32 blob of the output's shape */
    int relu_after;
    int8_t* quantised_out_dev;  /* channels-last int8 blob of the output's shape */
    float quantise_scale;
} ncnnhip_conv_fusion;
int ncnnhip_conv_fusion_supported(const ncnnhip_conv_desc* desc);
int ncnnhip_conv_int8_nhwc_fused(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev,
                                 const float* scale_in_dev, const float* bias_dev, ncnnhip_activation act, float* out_dev,
                                 const ncnnhip_conv_fusion* fusion, void* workspace_dev, size_t workspace_bytes, void* stream);

/* The same convolution in ONE launch for an input blob that is still fp32 (elemsize 4) or fp16 (2), channels-last: the
 * layer's own Quantize pass (Quantize::forward, src/layer/quantize.cpp:48-111 as Convolution::forward_int8 calls it at
 * src/layer/convolution.cpp:392-405: q = float2int8(x * in_scale[0])) runs inside the kernel's loader, so the int8 copy of
 * the blob is never written.  Group 1, zero border value, channels-last output (fp32, or int8 when scale_out_dev is
 * given); fusion (may be NULL) as in ncnnhip_conv_int8_nhwc_fused.  A workgroup holds its share of both operands in LDS
 * (64 pixels and up to 128 channels times its K steps, at most 96 KiB); layers beyond that are refused: ask
 * ncnnhip_conv_from_float_supported first and keep the separate ncnnhip_quantize_nhwc + ncnnhip_conv_int8_nhwc for those.
 * Layers with few output tiles split K over workgroups and need a workspace of ncnnhip_conv_from_float_workspace_bytes
 * (0 for the others), under the contract of ncnnhip_conv_int8_nhwc's workspace: zero-filled once by the caller, left
 * zero by every launch, used by one launch at a time. */
int ncnnhip_conv_from_float_supported(const ncnnhip_conv_desc* desc);
int ncnnhip_conv_from_float_workspace_bytes(const ncnnhip_conv_desc* desc, size_t* workspace_bytes);
int ncnnhip_conv_int8_nhwc_from_float(const ncnnhip_conv_desc* desc, const void* nhwc_dev, int elemsize, const float* in_scale_dev,
                                      const int8_t* packed_weight_dev, const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev,
                                      ncnnhip_activation act, void* out_nhwc_dev, const ncnnhip_conv_fusion* fusion, void* workspace_dev,
                                      size_t workspace_bytes, void* stream);

/* Which kernel a channels-last layer gets: 1 when ncnnhip_conv_int8_nhwc / _fused (elemsize 1) or
 * ncnnhip_conv_int8_nhwc_from_float (elemsize 4 or 2) would run this layer on the small-tile kernel -- two-dimensional
 * tiles of 32 output pixels x 64 channels whose input patch is quantised into LDS, for layers with too few output pixels
 * to fill the chip with 64-pixel tiles; it needs no workspace -- and 0 otherwise.  The same arithmetic either way
 * (Convolution::forward_int8, src/layer/convolution.cpp:383-508); the answer depends on the shape and on the environment
 * variable NCNNHIP_PATCH (0: never, 1: whenever the layer fits).  No counterpart in the reference: a query for tests
 * and for callers that size workspaces. */
int ncnnhip_conv_small_tile_selected(const ncnnhip_conv_desc* desc, int elemsize);


/* Convolution::forward_int8 (src/layer/convolution.cpp:383-508) for layers with at most 4 input channels (the 3-channel
 * first layer of an image net), group 1, dilation_w 1, zero border value.  The input is quantised into an image of 4 bytes
 * per pixel with a physical zero border (ncnnhip_quantize_stem; source: channels-last fp32 blob with pixel stride src_cp, or
 * int8), and one 16-byte K chunk of the contraction is 4 neighbouring pixels x 4 channels, so a 7x7x3 kernel costs K = 256
 * instead of 832.  Output, epilogue, fused tail (may be NULL) and workspace contract as in ncnnhip_conv_int8_nhwc[_fused]
 * with channels-last output; scale_out_dev non-NULL selects the requantised int8 output. */
int ncnnhip_conv_stem_supported(const ncnnhip_conv_desc* desc);
int ncnnhip_conv_stem_sizes(const ncnnhip_conv_desc* desc, size_t* image_bytes, size_t* packed_weight_bytes, size_t* workspace_bytes);
int ncnnhip_conv_stem_pack_weights(const ncnnhip_conv_desc* desc, const int8_t* weight_host, int8_t* packed_host);
int ncnnhip_quantize_stem(const ncnnhip_conv_desc* desc, const void* nhwc_dev, int elemsize, int src_cp, const float* scale_dev,
                          int8_t* image_dev, void* stream);
int ncnnhip_conv_int8_stem(const ncnnhip_conv_desc* desc, const int8_t* image_dev, const int8_t* packed_weight_dev,
                           const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act,
                           void* out_dev, const ncnnhip_conv_fusion* fusion, void* workspace_dev, size_t workspace_bytes,
                           void* stream);

/* ------------------------------------------------------------------ device-resident blobs (channels-last)
 * Between layers a 3-D blob stays in HBM as [batch][h*w][Cp] (Cp = ncnnhip_padded_channels(c), fp32 or int8, pad
 * channels zero); 1-D / 2-D blobs are dense.  ncnn's planar Mat layout (src/mat.h:341-381) exists only at the host
 * boundary.  This plays the part of the reference's VkMat upload / download and packing conversion
 * (src/net.cpp:2107-2230, src/layer/vulkan/packing_vulkan.cpp) for this device. */
int ncnnhip_padded_channels(int c);
int ncnnhip_chw_to_nhwc(const void* src_dev, int elemsize, int c, int hw, int batch, size_t cstep, size_t nstep, void* dst_dev, void* stream);
int ncnnhip_nhwc_to_chw(const void* src_dev, int elemsize, int c, int hw, int batch, void* dst_dev, size_t cstep, size_t nstep, void* stream);
/* An fp32 image of at most 4 channels may stay at 4 floats per pixel, [n][h*w][4] (a quarter of the padded blob): the
 * narrow-input convolution quantises straight from it (ncnnhip_quantize_stem with src_cp = 4); ncnnhip_widen_nhwc4_f32 turns
 * it into the ordinary [n][h*w][16] blob for anything else. */
int ncnnhip_chw_to_nhwc4_f32(const float* src_dev, int c, int hw, int batch, size_t cstep, size_t nstep, float* dst_dev, void* stream);
int ncnnhip_widen_nhwc4_f32(const float* src_dev, float* dst_dev, size_t pixels, void* stream);
/* Quantize::forward (src/layer/quantize.cpp:48-111) on a channels-last fp32 blob of npix pixels: one scale or one per channel. */
int ncnnhip_quantize_nhwc(const float* src_dev, int8_t* dst_dev, size_t npix, int c, const float* scales_dev, int nscales, void* stream);
/* The executor's int8 -> fp32 value cast for layers without int8 storage support (src/net.cpp:3007-3012 does the same at extract). */
int ncnnhip_int8_to_f32(const int8_t* src_dev, float* dst_dev, size_t count, void* stream);

/* ConvolutionDepthWise::forward_int8, depthwise branch (channels == group == num_output,
 * src/layer/convolutiondepthwise.cpp:505-559), channels-last int8 in, channels-last int8 (scale_out != NULL) or fp32 out.
 * Weights repacked once (ncnnhip_dwconv_packed_bytes of host memory): [kh*kw][Cp] bytes, for 3x3 kernels followed by each
 * kernel row as (w0, w1, w2, 0) per channel, the form the v_dot4 kernel multiplies.  scale_in / bias / scale_out: one float
 * per channel. */
int ncnnhip_dwconv_packed_bytes(int channels, int kernel_w, int kernel_h, size_t* bytes);
int ncnnhip_dwconv_pack_weights(int channels, int kernel_w, int kernel_h, const int8_t* weight_host, int8_t* packed_host);
int ncnnhip_dwconv_int8_nhwc(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev,
                             const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act,
                             void* out_nhwc_dev, void* stream);

/* ------------------------------------------------------------------ fp32 layers between the int8 layers
 * ReLU::forward_inplace (src/layer/relu.cpp): x < 0 ? x*slope : x; int8 blobs clamp at zero.  Flat over `count` elements.
 * fp32: count is a multiple of 4 and the blobs are 16-byte aligned, as device blobs are (channels padded to 16); anything
 * else is NCNNHIP_ERROR.  The same holds for ncnnhip_eltwise. */
int ncnnhip_relu(const void* src_dev, void* dst_dev, int elemsize, size_t count, float slope, void* stream);
/* Dropout::forward_inplace (src/layer/dropout.cpp): x * scale. */
int ncnnhip_scale(const float* src_dev, float* dst_dev, size_t count, float scale, void* stream);
/* Eltwise::forward (src/layer/eltwise.cpp:14-178): op_type 0 product, 1 sum (with coefficients when ncoeffs != 0), 2 max,
 * folded left to right over nsrc inputs.  srcs_dev is a HOST array of device pointers, coeffs_host a host array. */
int ncnnhip_eltwise(const float* const* srcs_dev, int nsrc, int op_type, const float* coeffs_host, int ncoeffs, float* dst_dev, size_t count, void* stream);
/* Pooling::forward (src/layer/pooling.cpp:18-415) on a channels-last fp32 blob.  pad_top / pad_left are the resolved head pads,
 * outw / outh the resolved output extent (pad_mode is the caller's business); global_pooling writes dense [batch][c]. */
typedef struct ncnnhip_pool_desc
{
    int w, h, c, batch;
    int pooling_type; /* 0 max, 1 average */
    int kernel_w, kernel_h, stride_w, stride_h;
    int pad_top, pad_left;
    int outw, outh;
    int global_pooling;
    int avgpool_count_include_pad;
    /* Average pooling with avgpool_count_include_pad == 0 divides by the number of taps inside this rectangle of IMAGE
     * coordinates, [count_x0, count_x1) x [count_y0, count_y1); taps inside it but outside the image add zero and still
     * count.  The reference excludes taps by the layer's own pad parameters (and the tail pad only in pad_mode 0,
     * src/layer/pooling.cpp:255-305), so with SAME padding (pad_mode 2 / 3, pad parameters 0) the rectangle is the whole
     * bordered image.  All four zero means the image itself; any other rectangle is taken as given, an empty one too (pad
     * parameters that leave no tap to count: the reference then divides 0 by 0 and so does this). */
    int count_x0, count_x1, count_y0, count_y1;
} ncnnhip_pool_desc;
int ncnnhip_pooling_nhwc(const ncnnhip_pool_desc* desc, const float* src_dev, float* dst_dev, void* stream);
/* Windowed max pooling (src/layer/pooling.cpp:105-222) of an int8 blob that holds Quantize(x, s), s > 0: the result is
 * Quantize(maxpool(x), s), because rounding and clamping are monotonic (for |x*s| < 2^31; the caller knows a bound).  Lets a requantising convolution feed the
 * quantising consumers of its pooled output without an fp32 blob in between. */
int ncnnhip_maxpool_nhwc_int8(const ncnnhip_pool_desc* desc, const int8_t* src_dev, int8_t* dst_dev, void* stream);
/* Global pooling (src/layer/pooling.cpp:60-103) followed by the consumer's Quantize (src/layer/quantize.cpp:29-60, one
 * scale for the tensor): dst[n][c] = float2int8(pool(x) * scale), dense int8.  Lets the pooled vector reach an int8
 * InnerProduct without an fp32 blob and a Quantize launch in between. */
int ncnnhip_global_pooling_nhwc_quantised(const ncnnhip_pool_desc* desc, const float* src_dev, float scale, int8_t* dst_dev, void* stream);
/* Softmax::forward_inplace (src/layer/softmax.cpp) over a dense vector of `count` values per sample. */
int ncnnhip_softmax(const float* src_dev, float* dst_dev, int count, int batch, void* stream);

/* ------------------------------------------------------------------ InnerProduct
 * InnerProduct::forward_int8 (src/layer/innerproduct.cpp:168-273) after input quantisation:
 * x int8 [rows][num_input] -> fp32 [rows][num_output];  scale_in / bias per output channel. */
int ncnnhip_innerproduct_int8(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output,
                              const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                              ncnnhip_activation act, float* out_dev, size_t out_stride, int32_t* acc_out_dev,
                              void* stream);
/* The same with a workspace (zero-filled once after allocation, like the convolution's): from 8 activation rows up the layer
 * then runs on the matrix cores as a 1x1 convolution over the rows, its K loop split across workgroups. */
int ncnnhip_innerproduct_workspace_bytes(int rows, int num_input, int num_output, size_t* workspace_bytes);
int ncnnhip_innerproduct_int8_ws(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output,
                                 const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                                 ncnnhip_activation act, float* out_dev, size_t out_stride, void* workspace_dev,
                                 size_t workspace_bytes, void* stream);

/* The same again for callers that cannot allocate device memory or pass a workspace (code under stream capture, serving
 * loops and harnesses that forbid hipMalloc).  No counterpart in the reference.  The K-split scratch is an array of
 * 4 MiB + 4 KiB that the library itself holds on every device it runs on (its address is looked up at ncnnhip_init, or at
 * the first call on a device); the call allocates and frees nothing.  Shapes whose split needs more scratch than that are
 * refused with -1 and a message naming ncnnhip_innerproduct_int8_ws.  All calls on one device share the one array: calls
 * that overlap on a device (two streams, two threads) race; calls in stream order on one stream do not.  Results are
 * those of ncnnhip_innerproduct_int8_ws bit for bit. */
int ncnnhip_innerproduct_int8_noalloc(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output,
                                      const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                                      ncnnhip_activation act, float* out_dev, size_t out_stride, void* stream);

/* ------------------------------------------------------------------ Gemm int8
 * Dynamic per-row quantisation of A (src/layer/gemm.cpp:791-823): scales[i] = 127/absmax_i (1 for a
 * zero row), aq = float2int8(a*scale). */
int ncnnhip_gemm_quantize_rows(const float* a_dev, size_t a_stride, int rows, int cols, int8_t* aq_dev, size_t aq_stride,
                               float* scales_dev, void* stream);
/* Dynamic whole-tensor quantisation of a non-constant B (src/layer/gemm.cpp:826-860). scale_dev[0]
 * receives 127/absmax. */
int ncnnhip_gemm_quantize_tensor(const float* b_dev, size_t b_stride, int rows, int cols, int8_t* bq_dev,
                                 size_t bq_stride, float* scale_dev, void* stream);
/* Transposes used for transA=1 / transB=0 / output_transpose (src/layer/gemm.cpp:751-788, 862-882). */
int ncnnhip_transpose_f32(const float* src_dev, size_t src_stride, int rows, int cols, float* dst_dev, size_t dst_stride,
                          void* stream);
int ncnnhip_transpose_s8(const int8_t* src_dev, size_t src_stride, int rows, int cols, int8_t* dst_dev, size_t dst_stride,
                         void* stream);
/* Two fp32 transposes of one shape and one pair of strides in a single launch: the new key and value rows of
 * MultiHeadAttention written as columns past.. of the [embed_dim][time] blobs (src/layer/multiheadattention.cpp:662-692,
 * 716-746 write k_affine / v_affine column by column). */
int ncnnhip_transpose_pair_f32(const float* src_a_dev, const float* src_b_dev, size_t src_stride, int rows, int cols,
                               float* dst_a_dev, float* dst_b_dev, size_t dst_stride, void* stream);

/* gemm_transB_int8 (src/layer/gemm.cpp:495-567): out = alpha*((float)acc / (sA_i*sB) + beta*C).
 * aq [M][K], bq [N][K] (K contiguous).  n_b_scales == 1 is ncnn's per-tensor B scale;
 * n_b_scales == N is a per-column generalisation that ncnn cannot express:
 * out = alpha*(((float)acc * (1/sA_i)) * (1/sB_j) + beta*C).
 * broadcast_type_c: -1 no C, 0 scalar, 1/2 per row, 3 [M][N] (row stride N), 4 per column. */
int ncnnhip_gemm_int8(const int8_t* aq_dev, size_t aq_stride, const int8_t* bq_dev, size_t bq_stride, int M, int N, int K,
                      const float* a_scales_dev, const float* b_scales_dev, int n_b_scales, const float* c_dev,
                      int broadcast_type_c, float alpha, float beta, int output_transpose, float* out_dev,
                      size_t out_stride, int32_t* acc_out_dev, void* stream);

/* The same Gemm on operands in the 256x256 kernel's own layout, for the form a network layer has (dynamic A, constant B;
 * gemm.cpp:745-966 with constantB=1, transB=1): element (r, k) of a tiled operand lies at
 * ((r / 256 * (K / 64) + k / 64) * 256 + r % 256) * 64 + k % 64 (the B operand with its rows interleaved inside a tile, which
 * ncnnhip_gemm_int8_tile_operand does), rows * K bytes, rows % 256 == 0, K % 64 == 0.  One K step of a tile is then 16 KB
 * of consecutive memory instead of 256 pieces of 64 bytes.  B is tiled once where the weights are uploaded
 * (create_pipeline), A is written tiled by the quantiser.  Results are those of ncnnhip_gemm_int8 bit for bit.
 * operand: 0 = A, 1 = B.  C: none or per column (broadcast_type_c 4). */
int ncnnhip_gemm_int8_tile_operand(const int8_t* src_dev, size_t src_stride, int rows, int K, int operand, int8_t* dst_dev,
                                   void* stream);
int ncnnhip_gemm_quantize_rows_tiled(const float* a_dev, size_t a_stride, int rows, int cols, int8_t* aq_tiled_dev,
                                     float* scales_dev, void* stream);
int ncnnhip_gemm_int8_tiled(const int8_t* aq_tiled_dev, const int8_t* bq_tiled_dev, int M, int N, int K,
                            const float* a_scales_dev, const float* b_scales_dev, int n_b_scales, const float* c_dev,
                            int broadcast_type_c, float alpha, float beta, float* out_dev, size_t out_stride, void* stream);

/* ------------------------------------------------------------------ block-quantised Gemm
 * Gemm::forward_weight_block_quantize (src/layer/gemm.cpp:338-483): a fp32 [M][K];
 * b packed [N][ceil(K*bits/8)] LSB-first `bits`-wide signed fields (bits 4/6/8);
 * scales fp32 [N][ceil(K/block)] exactly as stored in the .bin (value = qmax/absmax, the kernel
 * multiplies by 1.f/scale); in_scales optional fp32 [K]; out fp32 [M][N]. */
int ncnnhip_gemm_blockquant(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* b_dev, int bits,
                            int block, const float* scales_dev, const float* in_scales_dev, const float* c_dev,
                            int broadcast_type_c, float alpha, float beta, float* out_dev, size_t out_stride,
                            void* stream);

/* Benchmark-only variant of the same contraction taking IEEE half activations (the block-quant
 * LLM-decode configuration feeds fp16 activations; ncnn's layer itself rejects non-fp32 input,
 * src/layer/gemm.cpp:341-345).  a is fp16 [M][K]. */
int ncnnhip_gemm_blockquant_f16a(const uint16_t* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* b_dev,
                                 int bits, int block, const float* scales_dev, float* out_dev, size_t out_stride,
                                 void* stream);

/* Packed form of the block-quantised weights, made once at create_pipeline (the repacking of
 * constant weights into matrix-core tiles).  ncnn keeps B_data [N][ceil(K*bits/8)] and
 * B_data_quantize_scales [N][ceil(K/block)] as loaded (src/layer/gemm.cpp:182-221); here they become
 * tiles of 16 weight rows by 64 K, [ceil(N/16)][ceil(K/64)], each holding what the 64 lanes of a
 * wavefront load for it, every field stored as q + 2^(bits-1):
 *   8-bit fields in blocks of 64 or 128:  [64 lanes][16 bytes], lane l = row l%16, K (l/16)*16..+15;
 *     descales [tile][step][16 rows] fp32 = 1.f/scale (the reference's per-block division);
 *   every other combination (bits 4/6/8, block 32/64/128; K <= 16384):  lane l = row l%16 and the
 *     eight K (l/16)*8..+7 of each 32-wide half of the step; 8-bit 16 bytes per lane, 4-bit 8 bytes
 *     (a dword per half, fields 2p and 2p+1 in nibbles p and p+4), 6-bit [64 lanes][8 bytes] then
 *     [64 lanes][4 bytes]; descales as above, for blocks of 32 [tile][step][2 halves][16 rows].
 * Both functions run on the host. */
int ncnnhip_blockquant_packed_size(int N, int K, int bits, int block, size_t* weight_bytes, size_t* descale_bytes);
int ncnnhip_blockquant_pack(const uint8_t* b_host, const float* scales_host, int N, int K, int bits, int block,
                            uint8_t* packed_w_host, float* packed_descale_host);
/* Gemm::forward_weight_block_quantize (src/layer/gemm.cpp:338-483) on the packed weights with fp16
 * activations a [M][K] (K % 16 == 0), any M; out fp32 [M][N].  bits / block as given to the packer.
 * Same C / alpha / beta meaning as ncnnhip_gemm_blockquant. */
int ncnnhip_gemm_blockquant_packed_f16a(const uint16_t* a_dev, size_t a_stride, int M, int N, int K,
                                        const uint8_t* packed_w_dev, const float* packed_descale_dev, int bits, int block,
                                        const float* c_dev, int broadcast_type_c, float alpha, float beta, float* out_dev,
                                        size_t out_stride, void* stream);

/* The layer's own contract on the packed weights: fp32 activations a [M][K] (16-byte aligned rows, K % 16 == 0,
 * K <= 16384: ncnnhip_gemm_blockquant_packed_supported says whether a K qualifies), optional in_scales [K], any M (rows
 * go four at a time, fewer where K is long).  Each activation (times its input scale) is split exactly into three bf16
 * numbers, so every product is the reference's q * a and the result differs from ncnnhip_gemm_blockquant's only by the
 * order of the fp32 additions.  From 32 rows up ncnnhip_gemm_blockquant (fp32 matrix cores, one pass) is the faster call. */
int ncnnhip_gemm_blockquant_packed_supported(int K);
int ncnnhip_gemm_blockquant_packed(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev,
                                   const float* packed_descale_dev, int bits, int block, const float* in_scales_dev,
                                   const float* c_dev, int broadcast_type_c, float alpha, float beta, float* out_dev,
                                   size_t out_stride, void* stream);

/* Several packed weight matrices on the SAME activation rows in one launch: the gate and up projections of a decoder layer, the
 * q / k / v projections of an attention layer -- in the reference one Gemm / MultiHeadAttention projection after the other
 * (src/layer/gemm.cpp:425-483 per matrix); the results are those of `count` calls of ncnnhip_gemm_blockquant_packed(_f16a), bit
 * for bit.  a_elemsize 2: fp16 activations (up to 16 rows in one pass); 4: fp32 (up to 4 rows, with optional in_scales [K]).
 * All matrices share K, bits and block; N, the packed weights and descales, C (c_dev or its entries may be null), its broadcast
 * type, alpha, beta (null: 1) and the outputs are per matrix, count <= 8.  A decode-sized launch is paced by its ramp and tail,
 * not by bandwidth: one launch over 2 x 45.8 MB reaches what two launches of 45.8 MB cannot.  Shapes the one-pass kernel does
 * not take run matrix by matrix. */
int ncnnhip_gemm_blockquant_packed_multi(const void* a_dev, int a_elemsize, size_t a_stride, int M, int K, int count, const int* N,
                                         const uint8_t* const* packed_w_dev, const float* const* packed_descale_dev, int bits,
                                         int block, const float* in_scales_dev, const float* const* c_dev, const int* broadcast_type_c,
                                         const float* alpha, const float* beta, float* const* out_dev, const size_t* out_stride,
                                         void* stream);

/* The same contract from five activation rows up, with a workspace: the three-way split is made once, by a pass of its own,
 * into the workspace (ncnnhip_gemm_blockquant_packed_rows_workspace_bytes: 6 bytes per activation, rows and K rounded up to 64).
 * Up to 128 rows, while streaming the weights once per 16 rows is cheaper than a tiled pass (small weight matrices, or few
 * rows), the weights are streamed once per 16 rows in the few-row kernel's shape, all passes in one launch, the activations
 * pre-arranged as the lanes load them; otherwise a tiled Gemm runs on the bf16 matrix cores, 128 weight rows x 64 activation
 * rows per workgroup (prefill, attention projections).  K % 16 == 0; the workspace is scratch
 * (overwritten by every call). */
int ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(int M, int K, size_t* bytes);
int ncnnhip_gemm_blockquant_packed_rows(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev,
                                        const float* packed_descale_dev, int bits, int block, const float* in_scales_dev,
                                        const float* c_dev, int broadcast_type_c, float alpha, float beta, float* out_dev,
                                        size_t out_stride, void* workspace_dev, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ attention
 * The core of MultiHeadAttention::forward_weight_block_quantize (src/layer/multiheadattention.cpp:776-866):
 * per head, scores = q k^T (+ mask), softmax over the keys, times v.  q (already scaled) and out are
 * [seq][num_heads*head_dim]; kt / vt are [num_heads*head_dim][dst_seqlen] with row stride kv_stride, the layout of
 * the layer's cache blobs; mask is additive, [src][dst] (mask_heads 1) or [num_heads][src][dst], or NULL.
 * Head dimensions 32/64/96/128 run on the fp32 matrix cores with any dst_seqlen; others need head_dim + dst_seqlen <= 4096.
 * With few queries and many keys (decoding against a cache) the keys are split over workgroups if the caller passes
 * the scratch ncnnhip_attention_workspace_bytes asks for (may be 0 / NULL: then one workgroup per head and 32 queries);
 * one to four queries on 256 to 32768 keys then run on a streaming kernel of their own (64 keys per workgroup, any
 * head_dim up to 256) followed by a merge. */
int ncnnhip_attention_workspace_bytes(int num_heads, int head_dim, int src_seqlen, int dst_seqlen, size_t* workspace_bytes);
int ncnnhip_attention_f32(const float* q_dev, const float* kt_dev, const float* vt_dev, size_t kv_stride, const float* mask_dev,
                          int mask_heads, int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev,
                          void* workspace_dev, size_t workspace_bytes, void* stream);
/* The same with the queries taken as they come out of one Gemm that makes q, k and v together: row stride q_stride
 * (>= num_heads*head_dim) and every query value multiplied by q_scale on load - the (sum + bias) * scale of
 * src/layer/multiheadattention.cpp:618-634 with the same roundings, made where the query is read. */
int ncnnhip_attention_f32_strided(const float* q_dev, size_t q_stride, float q_scale, const float* kt_dev, const float* vt_dev,
                                  size_t kv_stride, const float* mask_dev, int mask_heads, int num_heads, int head_dim, int src_seqlen,
                                  int dst_seqlen, float* out_dev, void* workspace_dev, size_t workspace_bytes, void* stream);
/* Self-attention on rows that hold q, k and v side by side ([src_seqlen][>= 3*embed_dim]: q at column 0, k at embed_dim, v at
 * 2*embed_dim): the new keys and values are first written as columns past_seqlen.. of kt / vt (rows of kv_stride >=
 * past_seqlen + src_seqlen; columns 0..past_seqlen-1 hold the cache), then the attention runs over all past_seqlen +
 * src_seqlen keys - what src/layer/multiheadattention.cpp:640-746 does by writing k_affine / v_affine behind the cached
 * columns.  One to four queries on 256 keys and more write the columns inside the attention kernel (no launch of their
 * own); other shapes run ncnnhip_transpose_pair_f32 first.  Workspace as for ncnnhip_attention_f32 with dst_seqlen =
 * past_seqlen + src_seqlen. */
int ncnnhip_attention_f32_append(const float* qkv_dev, size_t qkv_stride, float q_scale, float* kt_dev, float* vt_dev, size_t kv_stride,
                                 int past_seqlen, const float* mask_dev, int mask_heads, int num_heads, int head_dim, int src_seqlen,
                                 float* out_dev, void* workspace_dev, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ measured ceilings (benchmark support)
 * No counterpart in the reference.  What this chip sustains, to set beside the published peaks in a roofline line:
 * ncnnhip_peak_mfma_i8 spins v_mfma_i32_32x32x32_i8 from registers on every SIMD (one workgroup of four wavefronts per
 * compute unit, eight independent accumulator chains, `iters` rounds of 8 instructions = iters * 8 * 65536 operations per
 * wavefront) on all-zero or pseudo-random operands; scratch_dev (>= 64 bytes) receives two int64: the shader cycles and
 * the 100 MHz wall ticks workgroup 0 spent in the loop.  ncnnhip_peak_hbm_read reads `bytes` (a multiple of 16) once with
 * 16-byte non-temporal loads, `loads_per_lane` (4, 8, 16, 32) of them in flight per lane, and writes nothing; time it with
 * events over buffers larger than the last-level cache to get the read bandwidth a kernel of that size can reach.
 * ncnnhip_peak_launch_chain enqueues `launches` one-wavefront kernels, each adding 1 to the int at scratch_dev (so each
 * depends on the one before, as the layers of a net do): timed with events, or captured into a graph and replayed, it
 * gives what one dependent launch costs on this chip whatever the kernel does. */
int ncnnhip_peak_launch_chain(int launches, void* scratch_dev, void* stream);
int ncnnhip_peak_mfma_i8(int iters, int random_operands, void* scratch_dev, void* stream);
int ncnnhip_peak_hbm_read(const void* src_dev, size_t bytes, int loads_per_lane, void* scratch_dev, void* stream);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif

#endif /* NCNNHIP_H */
