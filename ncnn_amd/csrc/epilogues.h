// Fused epilogues applied to the int32 accumulators of the contraction kernels.
// Each one reproduces the reference's scalar statement order with single rounded fp32 ops.
#ifndef NCNNHIP_EPILOGUES_H
#define NCNNHIP_EPILOGUES_H

#include "common.h"

namespace ncnnhip {

// out = alpha * ((float)acc * (1/(sA_i*sB)) + beta*C)   -- every step one rounded fp32 op.
// With one B scale per column the dequantisation is ((float)acc * (1/sA_i)) * (1/sB_j).
struct GemmEpilogue
{
    const float* a_scales;
    const float* b_scales;
    int per_col;
    const float* c;
    int bt;
    float alpha, beta;
    int transpose;
    float* out;
    size_t out_stride;
    int N;
    int32_t* acc_out;

    __device__ __forceinline__ void operator()(int i, int j, int acc) const
    {
        if (acc_out) acc_out[(size_t)i * N + j] = acc;
        float f;
        if (per_col)
            f = mul_rn(mul_rn((float)acc, div_rn(1.f, a_scales[i])), div_rn(1.f, b_scales[j]));
        else
            f = mul_rn((float)acc, div_rn(1.f, mul_rn(a_scales[i], b_scales[0])));
        if (bt >= 0)
        {
            float cv;
            if (bt == 0)
                cv = c[0];
            else if (bt == 1 || bt == 2)
                cv = c[i];
            else if (bt == 3)
                cv = c[(size_t)i * N + j];
            else
                cv = c[j];
            f = add_rn(f, mul_rn(cv, beta));
        }
        f = mul_rn(f, alpha);
        if (transpose)
            out[(size_t)j * out_stride + i] = f;
        else
            out[(size_t)i * out_stride + j] = f;
    }
};

// InnerProduct: rows of the A operand are output channels p, columns are input rows
struct FcEpilogue
{
    const float* scale_in;
    const float* bias;
    ncnnhip_activation act;
    float* out;
    size_t out_stride;
    int num_output;
    int32_t* acc_out;

    __device__ __forceinline__ void operator()(int p, int row, int acc) const
    {
        if (acc_out) acc_out[(size_t)row * num_output + p] = acc;
        float f = mul_rn((float)acc, scale_in[p]);
        if (bias) f = add_rn(f, bias[p]);
        out[(size_t)row * out_stride + p] = apply_activation(f, act);
    }
};

// Convolution / grouped convolution: row i is output channel (group_channel0 + i), column n is
// output pixel n = img*pix_per_img + pix.  scale_out selects the requantising (int8) store.
struct ConvEpilogue
{
    const float* scale_in;
    const float* bias;
    const float* scale_out;
    ncnnhip_activation act;
    void* out;
    size_t out_cstep, out_nstep;
    int pix_per_img;
    int batch;
    int out_channel0;
    int num_output;
    int32_t* acc_out;

    __device__ __forceinline__ void operator()(int i, int n, int acc) const
    {
        const int p = out_channel0 + i;
        int img = 0, pix = n;
        if (batch > 1)
        {
            img = n / pix_per_img;
            pix = n - img * pix_per_img;
        }
        if (acc_out) acc_out[((size_t)img * num_output + p) * pix_per_img + pix] = acc;
        float f = mul_rn((float)acc, scale_in[p]);
        if (bias) f = add_rn(f, bias[p]);
        f = apply_activation(f, act);
        const size_t o = (size_t)img * out_nstep + (size_t)p * out_cstep + pix;
        if (scale_out)
            static_cast<int8_t*>(out)[o] = (int8_t)float2int8(mul_rn(f, scale_out[p]));
        else
            static_cast<float*>(out)[o] = f;
    }
};

} // namespace ncnnhip

#endif // NCNNHIP_EPILOGUES_H
