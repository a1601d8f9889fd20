/*
 * CPU restatement of ncnn's naive int8 / block-quant arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP path: only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg may load it.
 * Nothing shipped in the product library links or calls it.
 *
 * Every float operation below is one IEEE-754 binary32 operation (build with
 * -O2 -fno-fast-math -ffp-contract=off); integer accumulation is exact int32.
 * All tensors are dense C arrays described by explicit strides (in elements):
 *   3-D activations  x[c][h][w]   with a channel stride `cstep`
 *   2-D matrices     a[rows][cols] with a row stride
 *
 * Reference statements followed (paths relative to the ncnn source root):
 *   float2int8          src/layer/convolution.cpp:375-381 (same text in quantize.cpp:30-36,
 *                       requantize.cpp:10-16, gemm.cpp:487-493, convolutiondepthwise.cpp:410-416)
 *   quantize            src/layer/quantize.cpp:39-111
 *   activation          src/layer/fused_activation.h:10-64
 *   constant padding    src/layer/padding.cpp:297-432, src/layer/convolution.cpp:328-372
 *   convolution int8    src/layer/convolution.cpp:383-508
 *   depthwise / group   src/layer/convolutiondepthwise.cpp:418-636
 *   inner product int8  src/layer/innerproduct.cpp:168-273
 *   gemm int8           src/layer/gemm.cpp:495-567, 745-966
 *   gemm block quant    src/layer/gemm.cpp:318-483
 *   attention with block-quantised weights  src/layer/multiheadattention.cpp:541-912 (which blob is
 *                       q / k / v / mask / cache: :914-1028)
 *   load-time weight quantisation  convolution.cpp:89-107, convolutiondepthwise.cpp:118-140,
 *                       innerproduct.cpp:62-79
 *
 * Parity pins (tests/test_oracle_*.py): float2int8 against hand-listed special cases; every
 * integer accumulator against an independent numpy int64 im2col/matmul; every epilogue against
 * a numpy float32 op-by-op evaluation; block-quant against a float64 dot product and against the
 * packing inverse that ncnn's tests/test_gemm_block_quant.cpp:11-25,80-129 defines; structural
 * identities (1x1 conv == gemm rows, depthwise == group conv with group=C, zero weight scale
 * => act(bias)).
 * the attention layer against a float64 evaluation of softmax(q k^T * scale + mask) v on the
 * dequantised weights, against torch.nn.functional.multi_head_attention_forward, and through the
 * cache identity (a pass over n tokens == n passes of one token that feed their cache back).
 * Activation types 4 (sigmoid) and 5 (mish) call expf / logf / tanhf of the host libm, so they are pinned to a
 * tolerance instead of a bit pattern: against the float64 closed forms 1/(1+exp(-v)) (4 ulp) and
 * v*tanh(log1p(exp(v))) (1e-6*|v|), with exact known answers at 0, at the +-88.376 clamp and where tanh saturates.
 * The out-of-range / NaN branch of float2int8 follows what x86 cvttss2si produces ("integer indefinite", INT_MIN,
 * which then saturates to -127); the pin executes that conversion on the x86 host and compares.
 * Parity unpinned: nothing in this file.  (The per-column-B Gemm epilogue of the standalone Gemm configuration is a
 * generalisation ncnn cannot express -- one B scale only, src/layer/gemm.h:69 -- so the reference fixes no value for
 * it: "parity unpinned by the reference"; oracle_gemm_int8 evaluates ((float)acc * (1/sA_i)) * (1/sB_j) for it.)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ scalars */

ORACLE_API int8_t oracle_float2int8(float v)
{
    /* round half away from zero, then saturate to [-127, 127].  For NaN and for magnitudes
     * beyond int range the C conversion is undefined; ncnn's x86 builds get INT_MIN from
     * cvttsd2si, which then saturates to -127.  State that explicitly. */
    double r = round((double)v);
    int q;
    if (!(r >= -2147483648.0 && r <= 2147483647.0))
        q = INT32_MIN;
    else
        q = (int)r;
    if (q > 127) return 127;
    if (q < -127) return -127;
    return (int8_t)q;
}

ORACLE_API float oracle_activation(float v, int type, const float* p)
{
    if (type == 1)
        return fmaxf(v, 0.f);
    if (type == 2)
        return v > 0.f ? v : v * p[0];
    if (type == 3)
    {
        if (v < p[0]) v = p[0];
        if (v > p[1]) v = p[1];
        return v;
    }
    if (type == 4)
    {
        if (v > 88.3762626647949f) v = 88.3762626647949f;
        if (v < -88.3762626647949f) v = -88.3762626647949f;
        return 1.f / (1.f + expf(-v));
    }
    if (type == 5)
        return v * tanhf(logf(expf(v) + 1.f));
    if (type == 6)
    {
        float lower = -p[1] / p[0];
        float upper = (1.f / p[0]) + lower;
        if (v < lower) return 0.f;
        if (v > upper) return v;
        return v * (v * p[0] + p[1]);
    }
    return v;
}

/* ------------------------------------------------------------------ quantize */

/* y[r][i] = float2int8(x[r][i] * s_r), s_r = scales[0] if nscales == 1 else scales[r].
 * rows = h for a 2-D blob, c for a 3-D blob (cols = w*h*d of one channel). */
ORACLE_API void oracle_quantize(const float* x, size_t x_stride, int8_t* y, size_t y_stride,
                                int rows, int cols, const float* scales, int nscales)
{
    for (int r = 0; r < rows; r++)
    {
        const float s = nscales == 1 ? scales[0] : scales[r];
        const float* xr = x + (size_t)r * x_stride;
        int8_t* yr = y + (size_t)r * y_stride;
        for (int i = 0; i < cols; i++)
            yr[i] = oracle_float2int8(xr[i] * s);
    }
}

/* ------------------------------------------------------------------ padding */

/* ncnn resolves the four pad fields into explicit borders before the integer loop:
 * positive pads are taken literally, -233 is SAME_UPPER and -234 SAME_LOWER. */
ORACLE_API void oracle_resolve_padding(int w, int h, int kernel_w, int kernel_h, int dilation_w, int dilation_h,
                                       int stride_w, int stride_h, int pad_left, int pad_right, int pad_top,
                                       int pad_bottom, int* out4 /* top, bottom, left, right */)
{
    const int kext_w = dilation_w * (kernel_w - 1) + 1;
    const int kext_h = dilation_h * (kernel_h - 1) + 1;
    int t = 0, b = 0, l = 0, r = 0;
    if (pad_left > 0 || pad_right > 0 || pad_top > 0 || pad_bottom > 0)
    {
        t = pad_top;
        b = pad_bottom;
        l = pad_left;
        r = pad_right;
    }
    else if (pad_left == -233 && pad_right == -233 && pad_top == -233 && pad_bottom == -233)
    {
        int wpad = kext_w + (w - 1) / stride_w * stride_w - w;
        int hpad = kext_h + (h - 1) / stride_h * stride_h - h;
        if (wpad > 0 || hpad > 0)
        {
            t = hpad / 2;
            b = hpad - hpad / 2;
            l = wpad / 2;
            r = wpad - wpad / 2;
        }
    }
    else if (pad_left == -234 && pad_right == -234 && pad_top == -234 && pad_bottom == -234)
    {
        int wpad = kext_w + (w - 1) / stride_w * stride_w - w;
        int hpad = kext_h + (h - 1) / stride_h * stride_h - h;
        if (wpad > 0 || hpad > 0)
        {
            t = hpad - hpad / 2;
            b = hpad / 2;
            l = wpad - wpad / 2;
            r = wpad / 2;
        }
    }
    out4[0] = t;
    out4[1] = b;
    out4[2] = l;
    out4[3] = r;
}

/* Builds the bordered int8 tensor (dense, channel stride = ph*pw). Border byte is the C cast
 * of the float pad value to signed char.
 * A SAME mode resolves to a NEGATIVE border in one dimension when the kernel's extent is below the
 * stride there while the other dimension needs a border (e.g. a 3 x 1 kernel at stride 3 on 37 x 20:
 * wpad 2, hpad -1, so bottom = -1).  The reference then makes a bordered blob smaller than the source
 * and still copies every source row and column into it (src/layer/padding.cpp:62-87: the centre loop
 * runs to top + src.h whatever dst.h is), i.e. it writes past the rows it allocated, and which values
 * end up inside the blob depends on the order its threads write the channels in.  There is no result
 * to restate: conv_core returns -1 for such a layer and never comes here with a negative border. */
static int8_t* make_bordered(const int8_t* x, size_t cstep, int c, int h, int w, const int pads[4], float pad_value,
                             int* ph, int* pw)
{
    const int H = h + pads[0] + pads[1];
    const int W = w + pads[2] + pads[3];
    int8_t* out = (int8_t*)malloc((size_t)c * H * W + 1);
    if (!out) return 0;
    const int8_t border = (int8_t)pad_value;
    memset(out, border, (size_t)c * H * W);
    for (int q = 0; q < c; q++)
        for (int y = 0; y < h; y++)
            memcpy(out + ((size_t)q * H + y + pads[0]) * W + pads[2], x + q * cstep + (size_t)y * w, (size_t)w);
    *ph = H;
    *pw = W;
    return out;
}

/* ------------------------------------------------------------------ conv family core */

typedef struct
{
    int w, h, c;          /* input (unpadded) */
    int num_output;
    int kernel_w, kernel_h, dilation_w, dilation_h, stride_w, stride_h;
    int pad_left, pad_right, pad_top, pad_bottom;
    float pad_value;
    int bias_term;
    int group;            /* 1 for Convolution */
    int int8_scale_term;
    int activation_type;
    float activation_params[2];
} oracle_conv_desc;

ORACLE_API void oracle_conv_out_shape(const oracle_conv_desc* d, int* outw, int* outh)
{
    int pads[4];
    oracle_resolve_padding(d->w, d->h, d->kernel_w, d->kernel_h, d->dilation_w, d->dilation_h, d->stride_w, d->stride_h,
                           d->pad_left, d->pad_right, d->pad_top, d->pad_bottom, pads);
    const int W = d->w + pads[2] + pads[3];
    const int H = d->h + pads[0] + pads[1];
    *outw = (W - (d->dilation_w * (d->kernel_w - 1) + 1)) / d->stride_w + 1;
    *outh = (H - (d->dilation_h * (d->kernel_h - 1) + 1)) / d->stride_h + 1;
}

/*
 * Shared integer loop + epilogue.
 *   x_q          int8 input, [c][h][w] with channel stride x_cstep (already quantised)
 *   weight       int8, [num_output][c/group][kh][kw]
 *   scale_by_group  0: weight scale / bias index = output channel, input & top scale index 0
 *                      (Convolution)
 *                   1: weight, input and top scales indexed by group (ConvolutionDepthWise;
 *                      caller passes arrays already broadcast to `group` entries)
 *   out          int8 if int8_scale_term > 100 else float, [num_output][outh][outw], stride out_cstep
 *   acc_out      optional int32 accumulators, dense [num_output][outh*outw]
 */
static int conv_core(const oracle_conv_desc* d, const int8_t* x_q, size_t x_cstep, const int8_t* weight,
                     const float* bias, const float* w_scales, const float* in_scales, const float* top_scales,
                     int scale_by_group, void* out, size_t out_cstep, int32_t* acc_out)
{
    if (d->group < 1 || d->c % d->group != 0 || d->num_output % d->group != 0) return -100;

    int pads[4];
    oracle_resolve_padding(d->w, d->h, d->kernel_w, d->kernel_h, d->dilation_w, d->dilation_h, d->stride_w, d->stride_h,
                           d->pad_left, d->pad_right, d->pad_top, d->pad_bottom, pads);
    if (pads[0] < 0 || pads[1] < 0 || pads[2] < 0 || pads[3] < 0) return -1; /* see make_bordered */
    int H, W;
    int8_t* xb = make_bordered(x_q, x_cstep, d->c, d->h, d->w, pads, d->pad_value, &H, &W);
    if (!xb) return -100;

    const int outw = (W - (d->dilation_w * (d->kernel_w - 1) + 1)) / d->stride_w + 1;
    const int outh = (H - (d->dilation_h * (d->kernel_h - 1) + 1)) / d->stride_h + 1;
    const int taps = d->kernel_w * d->kernel_h;
    const int cin_g = d->c / d->group;
    const int cout_g = d->num_output / d->group;
    const int requant = d->int8_scale_term > 100;

#pragma omp parallel for schedule(static)
    for (int p = 0; p < d->num_output; p++)
    {
        const int g = p / cout_g;
        const int8_t* wp = weight + (size_t)p * cin_g * taps;
        const int si = scale_by_group ? g : p;  /* weight-scale index */
        const int ai = scale_by_group ? g : 0;  /* activation-scale index */

        for (int oy = 0; oy < outh; oy++)
        {
            for (int ox = 0; ox < outw; ox++)
            {
                int32_t acc = 0;
                for (int q = 0; q < cin_g; q++)
                {
                    const int8_t* xc = xb + ((size_t)(g * cin_g + q) * H + (size_t)oy * d->stride_h) * W + (size_t)ox * d->stride_w;
                    const int8_t* wq = wp + (size_t)q * taps;
                    for (int ky = 0; ky < d->kernel_h; ky++)
                        for (int kx = 0; kx < d->kernel_w; kx++)
                            acc += (int32_t)xc[(size_t)ky * d->dilation_h * W + kx * d->dilation_w] * (int32_t)wq[ky * d->kernel_w + kx];
                }
                if (acc_out) acc_out[((size_t)p * outh + oy) * outw + ox] = acc;

                float scale_in;
                if (w_scales[si] == 0.f)
                    scale_in = 0.f;
                else
                    scale_in = 1.f / (in_scales[ai] * w_scales[si]);

                float f = (float)acc * scale_in;
                if (d->bias_term) f = f + bias[p];
                f = oracle_activation(f, d->activation_type, d->activation_params);

                const size_t o = (size_t)p * out_cstep + (size_t)oy * outw + ox;
                if (requant)
                    ((int8_t*)out)[o] = oracle_float2int8(f * top_scales[ai]);
                else
                    ((float*)out)[o] = f;
            }
        }
    }
    free(xb);
    return 0;
}

/* Quantise an fp32 activation tensor per channel with scales chosen by `scale_of_channel`. */
static int8_t* quantize_input(const float* x, size_t x_cstep, int c, int hw, const float* scales, int group, int by_group)
{
    int8_t* q = (int8_t*)malloc((size_t)c * hw + 1);
    if (!q) return 0;
    const int cg = c / group;
    for (int ch = 0; ch < c; ch++)
    {
        const float s = by_group ? scales[ch / cg] : scales[0];
        for (int i = 0; i < hw; i++) q[(size_t)ch * hw + i] = oracle_float2int8(x[ch * x_cstep + i] * s);
    }
    return q;
}

/* Convolution::forward_int8.  x_elemsize 4: fp32 input quantised with in_scale[0]; 1: int8. */
ORACLE_API int oracle_convolution_int8(const oracle_conv_desc* d, const void* x, int x_elemsize, size_t x_cstep,
                                       const int8_t* weight, const float* bias, const float* w_scales /*[num_output]*/,
                                       const float* in_scale /*[1]*/, const float* top_scale /*[1] or NULL*/, void* out,
                                       size_t out_cstep, int32_t* acc_out)
{
    oracle_conv_desc dd = *d;
    dd.group = 1;
    if (x_elemsize == 1)
        return conv_core(&dd, (const int8_t*)x, x_cstep, weight, bias, w_scales, in_scale, top_scale, 0, out, out_cstep, acc_out);
    int8_t* xq = quantize_input((const float*)x, x_cstep, d->c, d->w * d->h, in_scale, 1, 0);
    if (!xq) return -100;
    int ret = conv_core(&dd, xq, (size_t)d->w * d->h, weight, bias, w_scales, in_scale, top_scale, 0, out, out_cstep, acc_out);
    free(xq);
    return ret;
}

/* ConvolutionDepthWise::forward_int8, depthwise and grouped branches alike.  Scale arrays have
 * `group` entries (the layer broadcasts single values to that length when it loads the model). */
ORACLE_API int oracle_convolutiondepthwise_int8(const oracle_conv_desc* d, const void* x, int x_elemsize, size_t x_cstep,
                                                const int8_t* weight, const float* bias, const float* w_scales /*[group]*/,
                                                const float* in_scales /*[group]*/, const float* top_scales /*[group] or NULL*/,
                                                void* out, size_t out_cstep, int32_t* acc_out)
{
    if (d->group < 1 || d->c % d->group != 0 || d->num_output % d->group != 0) return -100;
    if (x_elemsize == 1)
        return conv_core(d, (const int8_t*)x, x_cstep, weight, bias, w_scales, in_scales, top_scales, 1, out, out_cstep, acc_out);
    int8_t* xq = quantize_input((const float*)x, x_cstep, d->c, d->w * d->h, in_scales, d->group, 1);
    if (!xq) return -100;
    int ret = conv_core(d, xq, (size_t)d->w * d->h, weight, bias, w_scales, in_scales, top_scales, 1, out, out_cstep, acc_out);
    free(xq);
    return ret;
}

/* Load-time quantisation of fp32 weights: rows = output channels (conv / fc) or groups
 * (depthwise), one scale per row. */
ORACLE_API void oracle_quantize_weights(const float* w, int8_t* wq, int rows, int row_size, const float* scales)
{
    oracle_quantize(w, (size_t)row_size, wq, (size_t)row_size, rows, row_size, scales, rows == 1 ? 1 : rows);
}

/* ------------------------------------------------------------------ inner product */

/* InnerProduct::forward_int8.  The input is `rows` vectors of num_input values (rows > 1 is
 * the 2-D "gemm" mode; a 1/3/4-D blob is one flattened vector in channel-major order with the
 * channel padding already removed by the caller).  Output fp32 [rows][num_output]. */
ORACLE_API int oracle_innerproduct_int8(const void* x, int x_elemsize, size_t x_stride, int rows, int num_input,
                                        int num_output, const int8_t* weight, const float* bias /*or NULL*/,
                                        const float* w_scales, const float* in_scale, int activation_type,
                                        const float* activation_params, float* out, size_t out_stride, int32_t* acc_out)
{
    int8_t* xq = (int8_t*)malloc((size_t)rows * num_input + 1);
    if (!xq) return -100;
    for (int r = 0; r < rows; r++)
        for (int i = 0; i < num_input; i++)
            xq[(size_t)r * num_input + i] = x_elemsize == 1 ? ((const int8_t*)x)[r * x_stride + i]
                                                            : oracle_float2int8(((const float*)x)[r * x_stride + i] * in_scale[0]);

#pragma omp parallel for schedule(static)
    for (int p = 0; p < num_output; p++)
    {
        for (int r = 0; r < rows; r++)
        {
            int32_t acc = 0;
            for (int i = 0; i < num_input; i++) acc += (int32_t)xq[(size_t)r * num_input + i] * (int32_t)weight[(size_t)p * num_input + i];
            if (acc_out) acc_out[(size_t)r * num_output + p] = acc;

            float scale_in = w_scales[p] == 0.f ? 0.f : 1.f / (in_scale[0] * w_scales[p]);
            float f = (float)acc * scale_in;
            if (bias) f = f + bias[p];
            out[r * out_stride + p] = oracle_activation(f, activation_type, activation_params);
        }
    }
    free(xq);
    return 0;
}

/* ------------------------------------------------------------------ gemm int8 */

/* Per-row dynamic quantisation of A (gemm.cpp:791-823): scale = 127/absmax, 1 when the row is 0. */
ORACLE_API void oracle_gemm_quantize_rows(const float* a, size_t a_stride, int rows, int cols, int8_t* aq,
                                          size_t aq_stride, float* scales)
{
#pragma omp parallel for schedule(static)
    for (int i = 0; i < rows; i++)
    {
        const float* ar = a + (size_t)i * a_stride;
        float absmax = 0.f;
        for (int k = 0; k < cols; k++)
        {
            float t = (float)fabs(ar[k]);
            absmax = absmax > t ? absmax : t; /* std::max(absmax, t) */
        }
        const float s = absmax == 0.f ? 1.f : 127.f / absmax;
        scales[i] = s;
        for (int k = 0; k < cols; k++) aq[(size_t)i * aq_stride + k] = oracle_float2int8(ar[k] * s);
    }
}

/* Whole-tensor dynamic quantisation of B (gemm.cpp:826-860). */
ORACLE_API float oracle_gemm_quantize_tensor(const float* b, size_t b_stride, int rows, int cols, int8_t* bq,
                                             size_t bq_stride)
{
    float absmax = 0.f;
    for (int i = 0; i < rows; i++)
        for (int k = 0; k < cols; k++)
        {
            float t = (float)fabs(b[(size_t)i * b_stride + k]);
            absmax = absmax > t ? absmax : t;
        }
    const float s = absmax == 0.f ? 1.f : 127.f / absmax;
    for (int i = 0; i < rows; i++)
        for (int k = 0; k < cols; k++) bq[(size_t)i * bq_stride + k] = oracle_float2int8(b[(size_t)i * b_stride + k] * s);
    return s;
}

/*
 * gemm_transB_int8 (gemm.cpp:495-567): aq [M][K], bq [N][K] (B already transposed to
 * K-contiguous rows).
 *   b_scales: one value (ncnn's per-tensor B scale) when n_b_scales == 1.  n_b_scales == N is
 *   this repository's per-column generalisation, f = ((float)acc * (1/sA_i)) * (1/sB_j);
 *   ncnn itself cannot express it, so that branch is pinned only by the numpy restatement.
 *   broadcast_type_c: -1 none, 0 scalar, 1/2 per row, 3 full [M][N], 4 per column.
 *   out: [M][N] (or [N][M] when output_transpose) with row stride out_stride.
 */
ORACLE_API void oracle_gemm_int8(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N,
                                 int K, const float* a_scales, const float* b_scales, int n_b_scales, const float* c,
                                 int broadcast_type_c, float alpha, float beta, int output_transpose, float* out,
                                 size_t out_stride, int32_t* acc_out)
{
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; i++)
    {
        const int8_t* ar = aq + (size_t)i * aq_stride;
        for (int j = 0; j < N; j++)
        {
            const int8_t* br = bq + (size_t)j * bq_stride;
            int32_t acc = 0;
            for (int k = 0; k < K; k++) acc += (int32_t)ar[k] * (int32_t)br[k];
            if (acc_out) acc_out[(size_t)i * N + j] = acc;

            float f;
            if (n_b_scales == 1)
            {
                const float descale = 1.f / (a_scales[i] * b_scales[0]);
                f = (float)acc * descale;
            }
            else
            {
                const float da = 1.f / a_scales[i];
                const float db = 1.f / b_scales[j];
                f = (float)acc * da;
                f = f * db;
            }
            if (c && broadcast_type_c >= 0)
            {
                float cv = 0.f;
                if (broadcast_type_c == 0) cv = c[0];
                if (broadcast_type_c == 1 || broadcast_type_c == 2) cv = c[i];
                if (broadcast_type_c == 3) cv = c[(size_t)i * N + j];
                if (broadcast_type_c == 4) cv = c[j];
                f = f + cv * beta;
            }
            f = f * alpha;
            if (output_transpose)
                out[(size_t)j * out_stride + i] = f;
            else
                out[(size_t)i * out_stride + j] = f;
        }
    }
}

/* ------------------------------------------------------------------ block-quantised gemm */

ORACLE_API int oracle_blockquant_unpack(const uint8_t* row, int k, int bits, int packed_k_bytes)
{
    /* LSB-first bit stream of `bits`-wide two's-complement fields (gemm.cpp:318-336) */
    const int bit = k * bits;
    const int byte = bit >> 3;
    unsigned v = row[byte];
    if (byte + 1 < packed_k_bytes) v |= (unsigned)row[byte + 1] << 8;
    const int field = (int)((v >> (bit & 7)) & ((1u << bits) - 1u));
    const int sign = 1 << (bits - 1);
    return (field ^ sign) - sign;
}

/*
 * Gemm::forward_weight_block_quantize (gemm.cpp:338-483).
 *   a        fp32 [M][K], row stride a_stride
 *   b        packed rows [N][packed_k_bytes], packed_k_bytes = ceil(K*bits/8)
 *   scales   fp32 quantisation scales [N][ceil(K/block)] (value = qmax/absmax; the kernel
 *            multiplies by 1/scale)
 *   in_scales  optional fp32 [K]
 * Sequential fp32 accumulation in ascending k, starting from c*beta.
 */
ORACLE_API void oracle_gemm_blockquant(const float* a, size_t a_stride, int M, int N, int K, const uint8_t* b, int bits,
                                       int block, const float* scales, const float* in_scales, const float* c,
                                       int broadcast_type_c, float alpha, float beta, float* out, size_t out_stride)
{
    const int packed = (int)(((size_t)K * bits + 7) / 8);
    const int nblk = (K + block - 1) / block;
#pragma omp parallel for schedule(static) collapse(2)
    for (int i = 0; i < M; i++)
    {
        for (int j = 0; j < N; j++)
        {
            const float* ar = a + (size_t)i * a_stride;
            float sum = 0.f;
            if (c && broadcast_type_c >= 0)
            {
                if (broadcast_type_c == 0) sum = c[0];
                if (broadcast_type_c == 1 || broadcast_type_c == 2) sum = c[i];
                if (broadcast_type_c == 3) sum = c[(size_t)i * N + j];
                if (broadcast_type_c == 4) sum = c[j];
                sum = sum * beta;
            }
            const uint8_t* br = b + (size_t)j * packed;
            const float* sr = scales + (size_t)j * nblk;
            for (int k0 = 0; k0 < K; k0 += block)
            {
                const int kend = k0 + block < K ? k0 + block : K;
                const float descale = 1.f / sr[k0 / block];
                for (int k = k0; k < kend; k++)
                {
                    const int q = oracle_blockquant_unpack(br, k, bits, packed);
                    float v = ar[k];
                    if (in_scales) v = v * in_scales[k];
                    const float wv = (float)q * descale;
                    const float prod = v * wv;
                    sum = sum + prod;
                }
            }
            out[(size_t)i * out_stride + j] = sum * alpha;
        }
    }
}

/* Block quantiser that ncnn's own test defines (tests/test_gemm_block_quant.cpp:80-129) and its
 * tools use: per block scale = qmax/absmax (1 when the block is all zero), q = clamp(round(v*scale)),
 * fields packed LSB-first.  Used to make fixtures; it is the inverse the unpacker is pinned by. */
ORACLE_API void oracle_blockquant_pack(const float* w, int N, int K, int bits, int block, uint8_t* packed_out, float* scales_out)
{
    const int packed = (int)(((size_t)K * bits + 7) / 8);
    const int nblk = (K + block - 1) / block;
    const int qmax = (1 << (bits - 1)) - 1;
    memset(packed_out, 0, (size_t)N * packed);
    for (int j = 0; j < N; j++)
    {
        for (int bidx = 0; bidx < nblk; bidx++)
        {
            const int k0 = bidx * block;
            const int kend = k0 + block < K ? k0 + block : K;
            float absmax = 0.f;
            for (int k = k0; k < kend; k++)
            {
                float t = fabsf(w[(size_t)j * K + k]);
                if (t > absmax) absmax = t;
            }
            const float s = absmax == 0.f ? 1.f : (float)qmax / absmax;
            scales_out[(size_t)j * nblk + bidx] = s;
            for (int k = k0; k < kend; k++)
            {
                int q = (int)roundf(w[(size_t)j * K + k] * s);
                if (q > qmax) q = qmax;
                if (q < -qmax) q = -qmax;
                const unsigned field = (unsigned)q & ((1u << bits) - 1u);
                const int bit = k * bits;
                const int byte = bit >> 3;
                const int sh = bit & 7;
                packed_out[(size_t)j * packed + byte] |= (uint8_t)(field << sh);
                if (sh + bits > 8) packed_out[(size_t)j * packed + byte + 1] |= (uint8_t)(field >> (8 - sh));
            }
        }
    }
}

ORACLE_API int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}


/* ------------------------------------------------------------------ attention, block-quantised weights
 * MultiHeadAttention::forward_weight_block_quantize (src/layer/multiheadattention.cpp:561-912).
 * Inputs as the layer sees them: q [src_seqlen][qdim], k [cur_seqlen][kdim], v [cur_seqlen][vdim] fp32;
 * mask [src][dst] (mask_heads 1) or [num_heads][src][dst]; cached_k / cached_v [embed_dim][past_seqlen].
 * self_attention != 0: k and v are computed from their inputs and appended to the cache (dst = past + cur);
 * self_attention == 0 with a cache: k and v ARE the cache (dst = past), their inputs are not read.
 * Weight matrices in the .bin layout of the block-quantised Gemm; w[0..3] = q, k, v, out.
 * out [src][qdim]; k_out / v_out (optional) [embed_dim][dst], the layout the layer hands back as its cache. */
typedef struct
{
    const uint8_t* packed;   /* [rows][ceil(K*bits/8)] */
    const float* scales;     /* [rows][ceil(K/block)] */
    const float* in_scales;  /* [K] or NULL */
    const float* bias;       /* [rows] */
} oracle_mha_weight;

typedef struct
{
    int embed_dim, num_heads, qdim, kdim, vdim;
    int src_seqlen, cur_seqlen, past_seqlen;
    int self_attention;
    int mask_heads; /* 0: none */
    float scale;
    int bits, block;
} oracle_mha_desc;

/* one projection, result transposed: dst[j][col0 + i] = bias[j] + sum_k x[i][k] * w[j][k]  (times post) */
static void mha_affine(const float* x, int rows, int K, const oracle_mha_weight* w, int out_rows, int bits, int block, float post, int use_post,
                       float* dst, int dst_stride, int col0)
{
    const int packed = (int)(((size_t)K * bits + 7) / 8);
    const int nblk = (K + block - 1) / block;
#pragma omp parallel for schedule(static) collapse(2)
    for (int i = 0; i < rows; i++)
    {
        for (int j = 0; j < out_rows; j++)
        {
            const float* ptr = x + (size_t)i * K;
            const uint8_t* kptr = w->packed + (size_t)j * packed;
            const float* sr = w->scales + (size_t)j * nblk;
            float sum = w->bias[j];
            for (int k0 = 0; k0 < K; k0 += block)
            {
                const int kend = k0 + block < K ? k0 + block : K;
                const float descale = 1.f / sr[k0 / block];
                for (int k = k0; k < kend; k++)
                {
                    const int q = oracle_blockquant_unpack(kptr, k, bits, packed);
                    float v = ptr[k];
                    if (w->in_scales) v = v * w->in_scales[k];
                    const float wv = (float)q * descale;
                    const float prod = v * wv;
                    sum = sum + prod;
                }
            }
            dst[(size_t)j * dst_stride + col0 + i] = use_post ? sum * post : sum;
        }
    }
}

ORACLE_API int oracle_mha_blockquant(const oracle_mha_desc* d, const float* q, const float* k, const float* v, const float* mask, const float* cached_k,
                                     const float* cached_v, const oracle_mha_weight* w, float* out, float* k_out, float* v_out)
{
    const int E = d->embed_dim, H = d->num_heads, src = d->src_seqlen, cur = d->cur_seqlen, past = d->past_seqlen;
    if (E <= 0 || H <= 0 || E % H != 0) return -1;
    const int hd = E / H;
    const int dst = past > 0 ? (d->self_attention ? past + cur : past) : cur;
    float* qa = (float*)malloc((size_t)E * src * sizeof(float));   /* [E][src] */
    float* ka = (float*)malloc((size_t)E * dst * sizeof(float));   /* [E][dst] */
    float* va = (float*)malloc((size_t)E * dst * sizeof(float));
    float* att = (float*)malloc((size_t)H * src * dst * sizeof(float));
    float* ctx = (float*)malloc((size_t)src * E * sizeof(float));  /* [src][E]: the out projection reads rows */
    if (!qa || !ka || !va || !att || !ctx)
    {
        free(qa); free(ka); free(va); free(att); free(ctx);
        return -100;
    }
    mha_affine(q, src, d->qdim, &w[0], E, d->bits, d->block, d->scale, 1, qa, src, 0);
    if (past > 0 && !d->self_attention)
    {
        memcpy(ka, cached_k, (size_t)E * dst * sizeof(float));
        memcpy(va, cached_v, (size_t)E * dst * sizeof(float));
    }
    else
    {
        for (int e = 0; e < E && past > 0; e++)
        {
            memcpy(ka + (size_t)e * dst, cached_k + (size_t)e * past, (size_t)past * sizeof(float));
            memcpy(va + (size_t)e * dst, cached_v + (size_t)e * past, (size_t)past * sizeof(float));
        }
        mha_affine(k, cur, d->kdim, &w[1], E, d->bits, d->block, 0.f, 0, ka, dst, past);
        mha_affine(v, cur, d->vdim, &w[2], E, d->bits, d->block, 0.f, 0, va, dst, past);
    }
#pragma omp parallel for schedule(static) collapse(2)
    for (int h = 0; h < H; h++)
    {
        for (int i = 0; i < src; i++)
        {
            float* row = att + ((size_t)h * src + i) * dst;
            for (int j = 0; j < dst; j++)
            {
                float sum = 0.f;
                for (int l = 0; l < hd; l++)
                {
                    const float prod = qa[(size_t)(h * hd + l) * src + i] * ka[(size_t)(h * hd + l) * dst + j];
                    sum = sum + prod;
                }
                row[j] = sum;
            }
            if (d->mask_heads)
            {
                const float* m = mask + ((size_t)(d->mask_heads > 1 ? h : 0) * src + i) * dst;
                for (int j = 0; j < dst; j++) row[j] = row[j] + m[j];
            }
            float mx = -3.402823466e+38f;
            for (int j = 0; j < dst; j++) mx = row[j] > mx ? row[j] : mx;
            float total = 0.f;
            for (int j = 0; j < dst; j++)
            {
                row[j] = expf(row[j] - mx);
                total = total + row[j];
            }
            for (int j = 0; j < dst; j++) row[j] = row[j] / total;
            for (int l = 0; l < hd; l++)
            {
                const float* vr = va + (size_t)(h * hd + l) * dst;
                float sum = 0.f;
                for (int j = 0; j < dst; j++)
                {
                    const float prod = row[j] * vr[j];
                    sum = sum + prod;
                }
                ctx[(size_t)i * E + h * hd + l] = sum;
            }
        }
    }
    /* out[i][j] = bias[j] + sum_k ctx[i][k] * w_out[j][k] */
    {
        float* tmp = (float*)malloc((size_t)d->qdim * src * sizeof(float));
        if (!tmp)
        {
            free(qa); free(ka); free(va); free(att); free(ctx);
            return -100;
        }
        mha_affine(ctx, src, E, &w[3], d->qdim, d->bits, d->block, 0.f, 0, tmp, src, 0);
        for (int i = 0; i < src; i++)
            for (int j = 0; j < d->qdim; j++) out[(size_t)i * d->qdim + j] = tmp[(size_t)j * src + i];
        free(tmp);
    }
    if (k_out) memcpy(k_out, ka, (size_t)E * dst * sizeof(float));
    if (v_out) memcpy(v_out, va, (size_t)E * dst * sizeof(float));
    free(qa); free(ka); free(va); free(att); free(ctx);
    return 0;
}
