/*
 * The MI355X int8 layers as a plug-in for an UNMODIFIED ncnn: a C file that knows ncnn only through its public C API
 * (src/c_api.h) and the kernels only through libncnnhip.so's C ABI (ncnnhip.h).  It builds layers the way src/c_api.h means
 * a C program to build them -- ncnn_layer_create() and then the table of function pointers overwritten entry by entry
 * (src/c_api.h:254-269) -- and registers them on a net under the built-in type names, which replaces the built-in layers
 * for that net (ncnn_net_register_custom_layer_by_type, src/c_api.h:349; src/net.cpp:1214-1237):
 *
 *     ncnn_net_t net = ncnn_net_create();
 *     ncnnhip_plugin_register(net);            // before ncnn_net_load_param
 *     ncnn_net_load_param(net, "model.param"); ncnn_net_load_model(net, "model.bin"); ...
 *
 * Every blob crosses PCIe on its way in and out of each layer (host Mat -> device -> host Mat): ncnn's C API has no
 * device blob, so this is the compatibility route, bit-identical to the reference's CPU layers but not the fast one.
 *
 * What each table follows in the reference:
 *   Convolution            src/layer/convolution.cpp:18-119 (load_param, load_model), :383-508 (forward_int8)
 *   ConvolutionDepthWise   src/layer/convolutiondepthwise.cpp:28-124, :418-636
 *   InnerProduct           src/layer/innerproduct.cpp:18-98, :168-273
 *   Gemm                   src/layer/gemm.cpp:25-90, :108-221, :338-483 (block-quantised weights), :745-966 (int8)
 * Layers of these types without an int8 / quantize term are refused at load_param (-1): there is no fp32 path here.
 *
 * Build: cc -shared -fPIC -I<dir of c_api.h and its generated platform.h / ncnn_export.h> -I<dir of ncnnhip.h>
 *        ncnnhip_plugin.c -lncnnhip -lpthread.
 */
#ifdef NCNNHIP_PLUGIN_AGAINST_NCNN_AMD
#include "ncnn_amd_c_api.h" /* this repository's own copy of the same declarations */
#else
#include "c_api.h"
#endif
#include "ncnnhip.h"

#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

enum
{
    KIND_CONVOLUTION = 0,
    KIND_DEPTHWISE = 1,
    KIND_INNERPRODUCT = 2,
    KIND_GEMM = 3
};

/* device scratch of one layer, one slot per purpose, grown on demand and kept between calls */
enum
{
    SLOT_IN = 0,
    SLOT_OUT,
    SLOT_NHWC,
    SLOT_WORKSPACE,
    SLOT_QUANT,
    SLOT_SCALES,
    SLOT_B,
    SLOT_BQ,
    SLOT_BT,
    SLOT_BSCALE,
    SLOT_C,
    SLOT_AT,
    SLOT_COUNT
};

typedef struct plugin_state
{
    struct plugin_state* next;
    ncnn_layer_t layer;
    int kind;
    pthread_mutex_t lock; /* one forward at a time per layer: the scratch slots are the layer's */
    void* stream;
    void* slot[SLOT_COUNT];
    size_t slot_bytes[SLOT_COUNT];

    /* Convolution / ConvolutionDepthWise / InnerProduct */
    int num_output, kernel_w, kernel_h, dilation_w, dilation_h, stride_w, stride_h;
    int pad_left, pad_right, pad_top, pad_bottom;
    float pad_value;
    int bias_term, weight_data_size, group, int8_scale_term, activation_type;
    float activation_params[2];
    int8_t* weight_q;      /* int8 weights, host */
    float* bias;           /* [num_output] or NULL */
    float* weight_scales;  /* Convolution / InnerProduct: [num_output]; depthwise: [group] */
    float* bottom_scales;  /* Convolution / InnerProduct: [1]; depthwise: [group] */
    float* top_scales;     /* [1] / [group], int8_scale_term > 100 */
    int n_weight_scales, n_bottom_scales, n_top_scales;
    void *d_weight, *d_weight_packed, *d_bias, *d_scale_in, *d_scale_out, *d_input_scales;

    /* Gemm */
    float alpha, beta;
    int transA, transB, constantA, constantB, constantC, constantM, constantN, constantK, constant_broadcast_type_C;
    int output_N1M, output_elempack, output_elemtype, output_transpose, quantize_term, block_quant;
    void* A_host; size_t A_bytes; int A_elemsize, A_w, A_h;
    void* B_host; size_t B_bytes; int B_elemsize, B_w, B_h;
    float* C_host; size_t C_count;
    float* A_scales_host;  /* [constantM] */
    float B_scale;
    float* B_block_scales; size_t B_block_scales_count;
    float* B_input_scales;
    void *d_A, *d_B, *d_C, *d_A_scales, *d_B_scale, *d_B_block_scales, *d_B_input_scales, *d_B_packed, *d_B_packed_descales;
    int b_ready_int8;
} plugin_state;

/* ncnn_layer_create() owns the table and its pthis (src/c_api.cpp:1352-1365), so a layer's own state lives beside it, found
 * by the table's address */
static plugin_state* g_states = 0;
static pthread_mutex_t g_states_lock = PTHREAD_MUTEX_INITIALIZER;

static plugin_state* state_of(const ncnn_layer_t layer)
{
    plugin_state* s;
    pthread_mutex_lock(&g_states_lock);
    for (s = g_states; s; s = s->next)
        if (s->layer == layer) break;
    pthread_mutex_unlock(&g_states_lock);
    return s;
}

static int fail(const plugin_state* s, const char* what)
{
    static const char* const names[] = {"Convolution", "ConvolutionDepthWise", "InnerProduct", "Gemm"};
    fprintf(stderr, "ncnnhip plugin %s: %s: %s\n", s ? names[s->kind] : "", what, ncnnhip_last_error());
    return -1;
}
static int refuse(const plugin_state* s, const char* why)
{
    static const char* const names[] = {"Convolution", "ConvolutionDepthWise", "InnerProduct", "Gemm"};
    fprintf(stderr, "ncnnhip plugin %s: %s\n", s ? names[s->kind] : "", why);
    return -1;
}

/* the device is chosen once per thread (HIP's current device is a per-thread setting) */
static int device_ready(void)
{
    static __thread int ready = 0;
    if (!ready)
    {
        const char* e = getenv("NCNNHIP_PLUGIN_DEVICE");
        if (ncnnhip_init(e ? atoi(e) : 0) != 0) return -1;
        ready = 1;
    }
    return 0;
}

static void* scratch(plugin_state* s, int slot, size_t bytes)
{
    if (bytes == 0) bytes = 16;
    if (s->slot_bytes[slot] < bytes)
    {
        if (s->slot[slot])
        {
            ncnnhip_stream_synchronize(s->stream);
            ncnnhip_free(s->slot[slot]);
        }
        s->slot[slot] = 0;
        s->slot_bytes[slot] = 0;
        if (ncnnhip_malloc(&s->slot[slot], bytes) != 0) return 0;
        s->slot_bytes[slot] = bytes;
        /* the K-split workspace starts from zero and every call leaves it so */
        if (slot == SLOT_WORKSPACE && ncnnhip_memset(s->slot[slot], 0, bytes, s->stream) != 0) return 0;
    }
    return s->slot[slot];
}

static int upload_constant(const void* host, size_t bytes, void** dev)
{
    int rc;
    *dev = 0;
    if (bytes == 0) return 0;
    rc = ncnnhip_malloc(dev, bytes);
    if (rc == 0) rc = ncnnhip_memcpy_h2d(*dev, host, bytes, 0);
    if (rc == 0) rc = ncnnhip_stream_synchronize(0);
    if (rc != 0 && *dev)
    {
        ncnnhip_free(*dev);
        *dev = 0;
    }
    return rc;
}

static void free_device(void** p)
{
    if (*p) ncnnhip_free(*p);
    *p = 0;
}

/* bytes a Mat's buffer holds: c planes of cstep elements (src/mat.h:total) */
static size_t mat_bytes(const ncnn_mat_t m)
{
    return ncnn_mat_get_cstep(m) * (size_t)ncnn_mat_get_c(m) * ncnn_mat_get_elemsize(m);
}
static size_t mat_count(const ncnn_mat_t m)
{
    return (size_t)ncnn_mat_get_w(m) * (size_t)ncnn_mat_get_h(m) * (size_t)ncnn_mat_get_d(m) * (size_t)ncnn_mat_get_c(m);
}

/* copies a model blob out of its Mat (which is destroyed) into malloc'ed memory; 1-D and 2-D blobs are dense */
static void* take_blob(ncnn_mat_t m, size_t* bytes, int* elemsize)
{
    void* p = 0;
    if (!m) return 0;
    if (ncnn_mat_get_data(m) && mat_count(m) > 0)
    {
        const size_t n = mat_count(m) * ncnn_mat_get_elemsize(m);
        p = malloc(n);
        if (p) memcpy(p, ncnn_mat_get_data(m), n);
        if (bytes) *bytes = n;
        if (elemsize) *elemsize = (int)ncnn_mat_get_elemsize(m);
    }
    ncnn_mat_destroy(m);
    return p;
}
static float* take_floats(ncnn_mat_t m, int expect)
{
    size_t bytes = 0;
    int elemsize = 0;
    float* p = (float*)take_blob(m, &bytes, &elemsize);
    if (p && (elemsize != 4 || bytes != (size_t)expect * 4))
    {
        free(p);
        p = 0;
    }
    return p;
}

/* float2int8 (src/layer/quantize.cpp:18-24): round half away from zero, clamp to [-127, 127] */
static int8_t float2int8(float v)
{
    int i = (int)roundf(v);
    if (i > 127) return 127;
    if (i < -127) return -127;
    return (int8_t)i;
}

static ncnnhip_activation make_activation(const plugin_state* s)
{
    ncnnhip_activation a;
    a.type = s->activation_type;
    a.p0 = s->activation_params[0];
    a.p1 = s->activation_params[1];
    return a;
}

static void read_activation(plugin_state* s, const ncnn_paramdict_t pd)
{
    ncnn_mat_t none = ncnn_mat_create();
    ncnn_mat_t arr = ncnn_paramdict_get_array(pd, 10, none);
    s->activation_type = ncnn_paramdict_get_int(pd, 9, 0);
    s->activation_params[0] = s->activation_params[1] = 0.f;
    if (arr)
    {
        const float* v = (const float*)ncnn_mat_get_data(arr);
        const int n = v ? ncnn_mat_get_w(arr) : 0;
        if (n > 0) s->activation_params[0] = v[0];
        if (n > 1) s->activation_params[1] = v[1];
        ncnn_mat_destroy(arr);
    }
    ncnn_mat_destroy(none);
}

/* ------------------------------------------------------------------ Convolution / ConvolutionDepthWise */

static int conv_load_param(ncnn_layer_t layer, const ncnn_paramdict_t pd)
{
    plugin_state* s = state_of(layer);
    if (!s) return -1;
    s->num_output = ncnn_paramdict_get_int(pd, 0, 0);
    s->kernel_w = ncnn_paramdict_get_int(pd, 1, 0);
    s->kernel_h = ncnn_paramdict_get_int(pd, 11, s->kernel_w);
    s->dilation_w = ncnn_paramdict_get_int(pd, 2, 1);
    s->dilation_h = ncnn_paramdict_get_int(pd, 12, s->dilation_w);
    s->stride_w = ncnn_paramdict_get_int(pd, 3, 1);
    s->stride_h = ncnn_paramdict_get_int(pd, 13, s->stride_w);
    s->pad_left = ncnn_paramdict_get_int(pd, 4, 0);
    s->pad_right = ncnn_paramdict_get_int(pd, 15, s->pad_left);
    s->pad_top = ncnn_paramdict_get_int(pd, 14, s->pad_left);
    s->pad_bottom = ncnn_paramdict_get_int(pd, 16, s->pad_top);
    s->pad_value = ncnn_paramdict_get_float(pd, 18, 0.f);
    s->bias_term = ncnn_paramdict_get_int(pd, 5, 0);
    s->weight_data_size = ncnn_paramdict_get_int(pd, 6, 0);
    s->group = s->kind == KIND_DEPTHWISE ? ncnn_paramdict_get_int(pd, 7, 1) : 1;
    s->int8_scale_term = ncnn_paramdict_get_int(pd, 8, 0);
    read_activation(s, pd);
    if (ncnn_paramdict_get_int(pd, 19, 0)) return refuse(s, "dynamic_weight layers take their weights as blobs; not an int8 layer");
    if (s->group < 1 || s->num_output <= 0 || s->num_output % s->group != 0) return -100;
    if (!s->int8_scale_term) return refuse(s, "no int8_scale_term; only the quantised path runs on this device");
    return 0;
}

static int conv_load_model(ncnn_layer_t layer, const ncnn_modelbin_t mb)
{
    plugin_state* s = state_of(layer);
    size_t bytes = 0;
    int elemsize = 0, g;
    void* w;
    if (!s) return -1;
    w = take_blob(mb->load_1d(mb, s->weight_data_size, 0), &bytes, &elemsize);
    if (!w) return -100;
    if (s->bias_term)
    {
        s->bias = take_floats(mb->load_1d(mb, s->num_output, 1), s->num_output);
        if (!s->bias)
        {
            free(w);
            return -100;
        }
    }
    if (s->kind == KIND_CONVOLUTION)
    {
        s->n_weight_scales = s->num_output;
        s->n_bottom_scales = 1;
        s->weight_scales = take_floats(mb->load_1d(mb, s->num_output, 1), s->num_output);
        s->bottom_scales = take_floats(mb->load_1d(mb, 1, 1), 1);
        if (s->int8_scale_term > 100)
        {
            s->n_top_scales = 1;
            s->top_scales = take_floats(mb->load_1d(mb, 1, 1), 1);
        }
    }
    else
    {
        /* term 1 / 101 stores one weight scale per group, 2 / 102 a single one; every table is then held per group
         * (src/layer/convolutiondepthwise.cpp:92-117) */
        const int per_group = s->int8_scale_term == 1 || s->int8_scale_term == 101;
        const int stored = per_group ? s->group : 1;
        float* ws = take_floats(mb->load_1d(mb, stored, 1), stored);
        float* is = take_floats(mb->load_1d(mb, 1, 1), 1);
        float* ts = s->int8_scale_term > 100 ? take_floats(mb->load_1d(mb, 1, 1), 1) : 0;
        s->n_weight_scales = s->n_bottom_scales = s->group;
        s->weight_scales = (float*)malloc((size_t)s->group * 4);
        s->bottom_scales = (float*)malloc((size_t)s->group * 4);
        if (ts)
        {
            s->n_top_scales = s->group;
            s->top_scales = (float*)malloc((size_t)s->group * 4);
        }
        if (ws && is && s->weight_scales && s->bottom_scales && (!ts || s->top_scales))
        {
            for (g = 0; g < s->group; g++)
            {
                s->weight_scales[g] = per_group ? ws[g] : ws[0];
                s->bottom_scales[g] = is[0];
                if (ts) s->top_scales[g] = ts[0];
            }
        }
        else
        {
            free(s->weight_scales);
            s->weight_scales = 0;
        }
        free(ws);
        free(is);
        free(ts);
    }
    if (!s->weight_scales || !s->bottom_scales || (s->int8_scale_term > 100 && !s->top_scales))
    {
        free(w);
        return -100;
    }

    if (elemsize == 1 && bytes == (size_t)s->weight_data_size)
        s->weight_q = (int8_t*)w;
    else if (elemsize == 4 && bytes == (size_t)s->weight_data_size * 4)
    {
        /* fp32 weights in the file: quantised here, once, per output channel (per group for depthwise) */
        const int rows = s->kind == KIND_DEPTHWISE ? s->group : s->num_output;
        const size_t per_row = (size_t)s->weight_data_size / (size_t)rows;
        size_t i;
        s->weight_q = (int8_t*)malloc((size_t)s->weight_data_size);
        if (!s->weight_q)
        {
            free(w);
            return -100;
        }
        for (i = 0; i < (size_t)s->weight_data_size; i++) s->weight_q[i] = float2int8(((const float*)w)[i] * s->weight_scales[i / per_row]);
        free(w);
    }
    else
    {
        free(w);
        return refuse(s, "weights are neither int8 nor fp32");
    }
    return 0;
}

static int conv_destroy_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    int i;
    (void)opt;
    if (!s) return -1;
    if (s->stream) ncnnhip_stream_synchronize(s->stream);
    free_device(&s->d_weight);
    free_device(&s->d_weight_packed);
    free_device(&s->d_bias);
    free_device(&s->d_scale_in);
    free_device(&s->d_scale_out);
    free_device(&s->d_input_scales);
    for (i = 0; i < SLOT_COUNT; i++)
    {
        free_device(&s->slot[i]);
        s->slot_bytes[i] = 0;
    }
    if (s->stream) ncnnhip_stream_destroy(s->stream);
    s->stream = 0;
    return 0;
}

static int conv_create_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    float *scale_in = 0, *scale_out = 0;
    int rc, p;
    (void)opt;
    if (!s || !s->weight_q) return -1;
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    if (ncnnhip_stream_create(&s->stream) != 0) return fail(s, "ncnnhip_stream_create");
    scale_in = (float*)malloc((size_t)s->num_output * 4);
    if (!scale_in) return -100;
    rc = ncnnhip_fold_input_scales(s->weight_scales, s->n_weight_scales, s->bottom_scales, s->n_bottom_scales, s->num_output, scale_in);
    if (rc == 0 && s->group == 1)
    {
        /* the channels-last kernel reads weights as [num_output][tap][padded channels]: repacked once here */
        const int taps = s->kernel_w * s->kernel_h;
        ncnnhip_conv_desc desc;
        size_t packed_bytes = 0;
        int8_t* packed;
        if (taps <= 0 || s->weight_data_size % (s->num_output * taps) != 0)
        {
            free(scale_in);
            return refuse(s, "weight_data_size does not divide into num_output x taps");
        }
        memset(&desc, 0, sizeof(desc));
        desc.c = s->weight_data_size / (s->num_output * taps);
        desc.w = s->kernel_w;
        desc.h = s->kernel_h;
        desc.batch = 1;
        desc.num_output = s->num_output;
        desc.kernel_w = s->kernel_w;
        desc.kernel_h = s->kernel_h;
        desc.dilation_w = desc.dilation_h = desc.stride_w = desc.stride_h = 1;
        desc.group = 1;
        rc = ncnnhip_conv_nhwc_sizes(&desc, 0, &packed_bytes, 0);
        packed = rc == 0 ? (int8_t*)malloc(packed_bytes ? packed_bytes : 1) : 0;
        if (rc == 0 && !packed) rc = -1;
        if (rc == 0) rc = ncnnhip_conv_pack_weights(&desc, s->weight_q, packed);
        if (rc == 0) rc = upload_constant(packed, packed_bytes, &s->d_weight_packed);
        free(packed);
    }
    else if (rc == 0)
        rc = upload_constant(s->weight_q, (size_t)s->weight_data_size, &s->d_weight);
    if (rc == 0) rc = upload_constant(scale_in, (size_t)s->num_output * 4, &s->d_scale_in);
    if (rc == 0 && s->bias_term) rc = upload_constant(s->bias, (size_t)s->num_output * 4, &s->d_bias);
    if (rc == 0 && s->int8_scale_term > 100)
    {
        const int per = s->num_output / s->n_top_scales;
        scale_out = (float*)malloc((size_t)s->num_output * 4);
        if (!scale_out)
            rc = -1;
        else
        {
            for (p = 0; p < s->num_output; p++) scale_out[p] = s->top_scales[p / per];
            rc = upload_constant(scale_out, (size_t)s->num_output * 4, &s->d_scale_out);
        }
    }
    if (rc == 0) rc = upload_constant(s->bottom_scales, (size_t)s->n_bottom_scales * 4, &s->d_input_scales);
    free(scale_in);
    free(scale_out);
    if (rc != 0)
    {
        fail(s, "create_pipeline");
        conv_destroy_pipeline(layer, opt);
        return -1;
    }
    return 0;
}

static int conv_forward_locked(plugin_state* s, const ncnn_mat_t bottom, ncnn_mat_t* top_blob)
{
    const int w = ncnn_mat_get_w(bottom), h = ncnn_mat_get_h(bottom), channels = ncnn_mat_get_c(bottom);
    const size_t elemsize = ncnn_mat_get_elemsize(bottom), cstep = ncnn_mat_get_cstep(bottom);
    const int requant = s->int8_scale_term > 100;
    ncnnhip_conv_desc desc;
    int outw = 0, outh = 0, rc;
    size_t out_cstep;
    ncnn_mat_t top;
    void *d_in, *d_out, *st = s->stream;

    if (channels % s->group != 0) return -100;
    if (s->weight_data_size != (s->num_output / s->group) * (channels / s->group) * s->kernel_w * s->kernel_h * s->group)
        return refuse(s, "weight_data_size does not match the blob's channels");

    desc.w = w;
    desc.h = h;
    desc.c = channels;
    desc.batch = 1;
    desc.num_output = s->num_output;
    desc.kernel_w = s->kernel_w;
    desc.kernel_h = s->kernel_h;
    desc.dilation_w = s->dilation_w;
    desc.dilation_h = s->dilation_h;
    desc.stride_w = s->stride_w;
    desc.stride_h = s->stride_h;
    desc.pad_left = s->pad_left;
    desc.pad_right = s->pad_right;
    desc.pad_top = s->pad_top;
    desc.pad_bottom = s->pad_bottom;
    desc.pad_value = s->pad_value;
    desc.group = s->group;
    if (ncnnhip_conv_out_shape(&desc, &outw, &outh) != 0) return fail(s, "ncnnhip_conv_out_shape");

    top = ncnn_mat_create_3d_elem(outw, outh, s->num_output, requant ? (size_t)1u : (size_t)4u, 1, NULL);
    if (!top || !ncnn_mat_get_data(top))
    {
        if (top) ncnn_mat_destroy(top);
        return -100;
    }
    *top_blob = top;
    out_cstep = ncnn_mat_get_cstep(top);

    d_in = scratch(s, SLOT_IN, mat_bytes(bottom));
    d_out = scratch(s, SLOT_OUT, mat_bytes(top));
    if (!d_in || !d_out) return fail(s, "device scratch");
    if (ncnnhip_memcpy_h2d(d_in, ncnn_mat_get_data(bottom), mat_bytes(bottom), st) != 0) return fail(s, "upload bottom blob");

    if (s->group == 1)
    {
        /* quantise (or copy) into [h][w][padded channels] int8, then the implicit GEMM on the matrix cores */
        size_t nhwc_bytes = 0, packed_bytes = 0, workspace_bytes = 0;
        void *d_nhwc, *d_ws = 0;
        if (ncnnhip_conv_nhwc_sizes(&desc, &nhwc_bytes, &packed_bytes, &workspace_bytes) != 0) return fail(s, "ncnnhip_conv_nhwc_sizes");
        d_nhwc = scratch(s, SLOT_NHWC, nhwc_bytes);
        if (workspace_bytes) d_ws = scratch(s, SLOT_WORKSPACE, workspace_bytes);
        if (!d_nhwc || (workspace_bytes && !d_ws)) return fail(s, "device scratch");
        rc = ncnnhip_to_nhwc_int8(&desc, d_in, (int)elemsize, cstep, 0, (const float*)s->d_input_scales, 1, (int8_t*)d_nhwc, st);
        if (rc != 0) return fail(s, "ncnnhip_to_nhwc_int8");
        rc = ncnnhip_conv_int8_nhwc(&desc, (const int8_t*)d_nhwc, (const int8_t*)s->d_weight_packed, (const float*)s->d_scale_in,
                                    (const float*)s->d_bias, (const float*)s->d_scale_out, make_activation(s), d_out, NCNNHIP_PLANAR,
                                    out_cstep, 0, d_ws, workspace_bytes, st);
        if (rc != 0) return fail(s, "ncnnhip_conv_int8_nhwc");
    }
    else
    {
        const int8_t* d_xq = (const int8_t*)d_in;
        size_t q_cstep = cstep;
        if (elemsize == 4u)
        {
            /* Quantize with the group's scale for every channel of a group */
            const int cg = channels / s->group;
            float* per_channel = (float*)malloc((size_t)channels * 4);
            void *d_q, *d_scales;
            int q;
            if (!per_channel) return -100;
            for (q = 0; q < channels; q++) per_channel[q] = s->bottom_scales[q / cg];
            q_cstep = ((size_t)w * h + 15) / 16 * 16;
            d_q = scratch(s, SLOT_QUANT, q_cstep * (size_t)channels);
            d_scales = scratch(s, SLOT_SCALES, (size_t)channels * 4);
            rc = (d_q && d_scales) ? ncnnhip_memcpy_h2d(d_scales, per_channel, (size_t)channels * 4, st) : -1;
            if (rc == 0) rc = ncnnhip_stream_synchronize(st); /* per_channel is freed below */
            free(per_channel);
            if (rc != 0) return fail(s, "upload channel scales");
            rc = ncnnhip_quantize((const float*)d_in, cstep, 0, (int8_t*)d_q, q_cstep, 0, channels, w * h, 1, (const float*)d_scales, channels, st);
            if (rc != 0) return fail(s, "ncnnhip_quantize");
            d_xq = (const int8_t*)d_q;
        }
        rc = ncnnhip_conv_int8(&desc, d_xq, q_cstep, 0, (const int8_t*)s->d_weight, (const float*)s->d_scale_in, (const float*)s->d_bias,
                               (const float*)s->d_scale_out, make_activation(s), d_out, out_cstep, 0, 0, st);
        if (rc != 0) return fail(s, "ncnnhip_conv_int8");
    }
    rc = ncnnhip_memcpy_d2h(ncnn_mat_get_data(top), d_out, mat_bytes(top), st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return rc == 0 ? 0 : fail(s, "download top blob");
}

static int conv_forward_1(const ncnn_layer_t layer, const ncnn_mat_t bottom, ncnn_mat_t* top_blob, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    int ret;
    (void)opt;
    if (!s || (!s->d_weight && !s->d_weight_packed)) return refuse(s, "forward before create_pipeline");
    if (ncnn_mat_get_dims(bottom) != 3 || ncnn_mat_get_elempack(bottom) != 1 || (ncnn_mat_get_elemsize(bottom) != 4u && ncnn_mat_get_elemsize(bottom) != 1u))
        return refuse(s, "needs a pack-1 fp32 or int8 3-D blob");
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    pthread_mutex_lock(&s->lock);
    ret = conv_forward_locked(s, bottom, top_blob);
    pthread_mutex_unlock(&s->lock);
    return ret;
}

/* ------------------------------------------------------------------ InnerProduct */

static int ip_load_param(ncnn_layer_t layer, const ncnn_paramdict_t pd)
{
    plugin_state* s = state_of(layer);
    if (!s) return -1;
    s->num_output = ncnn_paramdict_get_int(pd, 0, 0);
    s->bias_term = ncnn_paramdict_get_int(pd, 1, 0);
    s->weight_data_size = ncnn_paramdict_get_int(pd, 2, 0);
    s->int8_scale_term = ncnn_paramdict_get_int(pd, 8, 0);
    s->group = 1;
    read_activation(s, pd);
    if (s->num_output <= 0 || s->weight_data_size % s->num_output != 0) return -100;
    if (!s->int8_scale_term) return refuse(s, "no int8_scale_term; only the quantised path runs on this device");
    return 0;
}

static int ip_load_model(ncnn_layer_t layer, const ncnn_modelbin_t mb)
{
    plugin_state* s = state_of(layer);
    size_t bytes = 0;
    int elemsize = 0;
    void* w;
    if (!s) return -1;
    w = take_blob(mb->load_1d(mb, s->weight_data_size, 0), &bytes, &elemsize);
    if (!w) return -100;
    if (s->bias_term) s->bias = take_floats(mb->load_1d(mb, s->num_output, 1), s->num_output);
    s->n_weight_scales = s->num_output;
    s->n_bottom_scales = 1;
    s->weight_scales = take_floats(mb->load_1d(mb, s->num_output, 1), s->num_output);
    s->bottom_scales = take_floats(mb->load_1d(mb, 1, 1), 1);
    if ((s->bias_term && !s->bias) || !s->weight_scales || !s->bottom_scales)
    {
        free(w);
        return -100;
    }
    if (elemsize == 1 && bytes == (size_t)s->weight_data_size)
        s->weight_q = (int8_t*)w;
    else if (elemsize == 4 && bytes == (size_t)s->weight_data_size * 4)
    {
        const size_t per_row = (size_t)s->weight_data_size / (size_t)s->num_output;
        size_t i;
        s->weight_q = (int8_t*)malloc((size_t)s->weight_data_size);
        if (!s->weight_q)
        {
            free(w);
            return -100;
        }
        for (i = 0; i < (size_t)s->weight_data_size; i++) s->weight_q[i] = float2int8(((const float*)w)[i] * s->weight_scales[i / per_row]);
        free(w);
    }
    else
    {
        free(w);
        return refuse(s, "weights are neither int8 nor fp32");
    }
    return 0;
}

static int ip_create_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    float* scale_in;
    int rc;
    if (!s || !s->weight_q) return -1;
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    if (ncnnhip_stream_create(&s->stream) != 0) return fail(s, "ncnnhip_stream_create");
    scale_in = (float*)malloc((size_t)s->num_output * 4);
    if (!scale_in) return -100;
    rc = ncnnhip_fold_input_scales(s->weight_scales, s->num_output, s->bottom_scales, 1, s->num_output, scale_in);
    if (rc == 0) rc = upload_constant(s->weight_q, (size_t)s->weight_data_size, &s->d_weight);
    if (rc == 0) rc = upload_constant(scale_in, (size_t)s->num_output * 4, &s->d_scale_in);
    if (rc == 0 && s->bias_term) rc = upload_constant(s->bias, (size_t)s->num_output * 4, &s->d_bias);
    if (rc == 0) rc = upload_constant(s->bottom_scales, 4, &s->d_input_scales);
    free(scale_in);
    if (rc != 0)
    {
        fail(s, "create_pipeline");
        conv_destroy_pipeline(layer, opt);
        return -1;
    }
    return 0;
}

static int ip_forward_locked(plugin_state* s, const ncnn_mat_t bottom, ncnn_mat_t* top_blob)
{
    const int num_input = s->weight_data_size / s->num_output;
    const size_t elemsize = ncnn_mat_get_elemsize(bottom);
    const int dims = ncnn_mat_get_dims(bottom), w = ncnn_mat_get_w(bottom), h = ncnn_mat_get_h(bottom), c = ncnn_mat_get_c(bottom);
    const size_t cstep = ncnn_mat_get_cstep(bottom);
    const char* src = (const char*)ncnn_mat_get_data(bottom);
    void* st = s->stream;
    int rows = 1, rc, q;
    ncnn_mat_t top;
    void *d_in, *d_out;
    const int8_t* d_xq;

    /* a 2-D blob whose rows are num_input long gives one output row per input row; anything else is one vector in channel
     * order (src/layer/innerproduct.cpp:100-166 / :168-273) */
    if (dims == 2 && w == num_input)
    {
        rows = h;
        top = ncnn_mat_create_2d_elem(s->num_output, rows, 4u, 1, NULL);
    }
    else
    {
        if (mat_count(bottom) != (size_t)num_input) return refuse(s, "the blob's value count is not the weights' num_input");
        top = ncnn_mat_create_1d_elem(s->num_output, 4u, 1, NULL);
    }
    if (!top || !ncnn_mat_get_data(top))
    {
        if (top) ncnn_mat_destroy(top);
        return -100;
    }
    *top_blob = top;

    d_in = scratch(s, SLOT_IN, (size_t)rows * num_input * elemsize);
    d_out = scratch(s, SLOT_OUT, (size_t)rows * s->num_output * 4);
    if (!d_in || !d_out) return fail(s, "device scratch");
    if (dims <= 2 || c == 1)
        rc = ncnnhip_memcpy_h2d(d_in, src, (size_t)rows * num_input * elemsize, st);
    else
    {
        /* planes are padded to 16 bytes in a 3-D Mat: flatten plane by plane */
        const size_t plane = (size_t)w * h * ncnn_mat_get_d(bottom) * elemsize;
        rc = 0;
        for (q = 0; q < c && rc == 0; q++) rc = ncnnhip_memcpy_h2d((char*)d_in + (size_t)q * plane, src + (size_t)q * cstep * elemsize, plane, st);
    }
    if (rc != 0) return fail(s, "upload bottom blob");

    d_xq = (const int8_t*)d_in;
    if (elemsize == 4u)
    {
        void* d_q = scratch(s, SLOT_QUANT, (size_t)rows * num_input);
        if (!d_q) return fail(s, "device scratch");
        rc = ncnnhip_quantize((const float*)d_in, (size_t)num_input, 0, (int8_t*)d_q, (size_t)num_input, 0, rows, num_input, 1,
                              (const float*)s->d_input_scales, 1, st);
        if (rc != 0) return fail(s, "ncnnhip_quantize");
        d_xq = (const int8_t*)d_q;
    }
    rc = ncnnhip_innerproduct_int8(d_xq, (size_t)num_input, rows, num_input, s->num_output, (const int8_t*)s->d_weight, (const float*)s->d_scale_in,
                                   (const float*)s->d_bias, make_activation(s), (float*)d_out, (size_t)s->num_output, 0, st);
    if (rc != 0) return fail(s, "ncnnhip_innerproduct_int8");
    rc = ncnnhip_memcpy_d2h(ncnn_mat_get_data(top), d_out, (size_t)rows * s->num_output * 4, st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return rc == 0 ? 0 : fail(s, "download top blob");
}

static int ip_forward_1(const ncnn_layer_t layer, const ncnn_mat_t bottom, ncnn_mat_t* top_blob, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    int ret;
    (void)opt;
    if (!s || !s->d_weight) return refuse(s, "forward before create_pipeline");
    if (ncnn_mat_get_elempack(bottom) != 1 || (ncnn_mat_get_elemsize(bottom) != 4u && ncnn_mat_get_elemsize(bottom) != 1u))
        return refuse(s, "needs a pack-1 fp32 or int8 blob");
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    pthread_mutex_lock(&s->lock);
    ret = ip_forward_locked(s, bottom, top_blob);
    pthread_mutex_unlock(&s->lock);
    return ret;
}

/* ------------------------------------------------------------------ Gemm */

/* quantize_term (src/layer/gemm.cpp:54-60): 1..3 dynamic int8; hundreds 4 / 6 / 8 = bits of block-quantised weights, tens 1 =
 * per-K input scales, units 0 / 1 / 2 = blocks of 32 / 64 / 128 */
static int term_is_block_quant(int term)
{
    const int bits = term / 100, tens = term % 100 / 10, code = term % 10;
    return (bits == 4 || bits == 6 || bits == 8) && tens <= 1 && code <= 2;
}
static int term_block(int term)
{
    const int code = term % 10;
    return code == 0 ? 32 : code == 1 ? 64 : 128;
}

static int gemm_load_param(ncnn_layer_t layer, const ncnn_paramdict_t pd)
{
    plugin_state* s = state_of(layer);
    if (!s) return -1;
    s->alpha = ncnn_paramdict_get_float(pd, 0, 1.f);
    s->beta = ncnn_paramdict_get_float(pd, 1, 1.f);
    s->transA = ncnn_paramdict_get_int(pd, 2, 0);
    s->transB = ncnn_paramdict_get_int(pd, 3, 0);
    s->constantA = ncnn_paramdict_get_int(pd, 4, 0);
    s->constantB = ncnn_paramdict_get_int(pd, 5, 0);
    s->constantC = ncnn_paramdict_get_int(pd, 6, 0);
    s->constantM = ncnn_paramdict_get_int(pd, 7, 0);
    s->constantN = ncnn_paramdict_get_int(pd, 8, 0);
    s->constantK = ncnn_paramdict_get_int(pd, 9, 0);
    s->constant_broadcast_type_C = ncnn_paramdict_get_int(pd, 10, 0);
    s->output_N1M = ncnn_paramdict_get_int(pd, 11, 0);
    s->output_elempack = ncnn_paramdict_get_int(pd, 12, 0);
    s->output_elemtype = ncnn_paramdict_get_int(pd, 13, 0);
    s->output_transpose = ncnn_paramdict_get_int(pd, 14, 0);
    s->quantize_term = ncnn_paramdict_get_int(pd, 18, 0);
    s->block_quant = term_is_block_quant(s->quantize_term);
    if (s->quantize_term == 0) return refuse(s, "no quantize_term; only the quantised paths run on this device");
    if (!s->block_quant && (s->quantize_term < 1 || s->quantize_term > 3)) return refuse(s, "unsupported quantize_term");
    if (s->block_quant
        && (s->constantA != 0 || s->constantB != 1 || s->transA != 0 || s->transB != 1 || s->output_N1M != 0 || s->output_elempack != 0
            || (s->output_elemtype != 0 && s->output_elemtype != 1) || s->output_transpose != 0))
        return refuse(s, "unsupported weight block quantize");
    if (s->constantA == 1 && (s->constantM == 0 || s->constantK == 0)) return refuse(s, "constantM and constantK must be non-zero when constantA enabled");
    if (s->constantB == 1 && (s->constantN == 0 || s->constantK == 0)) return refuse(s, "constantN and constantK must be non-zero when constantB enabled");
    if (s->constantC == 1 && (s->constant_broadcast_type_C < -1 || s->constant_broadcast_type_C > 4))
        return refuse(s, "constant_broadcast_type_C must be -1 or 0~4 when constantC enabled");
    /* one bottom blob is enough when two of the three operands are constants (src/layer/gemm.cpp:80-84) */
    ncnn_layer_set_one_blob_only(layer, s->constantA + s->constantB + s->constantC == 2);
    return 0;
}

static int gemm_load_model(ncnn_layer_t layer, const ncnn_modelbin_t mb)
{
    plugin_state* s = state_of(layer);
    if (!s) return -1;
    if (s->constantA == 1)
    {
        s->A_w = s->transA == 0 ? s->constantK : s->constantM;
        s->A_h = s->transA == 0 ? s->constantM : s->constantK;
        s->A_host = take_blob(mb->load_2d(mb, s->A_w, s->A_h, 0), &s->A_bytes, &s->A_elemsize);
        if (!s->A_host) return -100;
    }
    if (s->constantB == 1)
    {
        if (s->transB == 0)
        {
            s->B_w = s->constantN;
            s->B_h = s->constantK;
        }
        else if (s->block_quant)
        {
            s->B_w = (int)(((size_t)s->constantK * (size_t)(s->quantize_term / 100) + 7) / 8);
            s->B_h = s->constantN;
        }
        else
        {
            s->B_w = s->constantK;
            s->B_h = s->constantN;
        }
        s->B_host = take_blob(mb->load_2d(mb, s->B_w, s->B_h, 0), &s->B_bytes, &s->B_elemsize);
        if (!s->B_host) return -100;
    }
    if (s->constantC == 1 && s->constant_broadcast_type_C != -1)
    {
        ncnn_mat_t c = 0;
        size_t bytes = 0;
        int elemsize = 0;
        switch (s->constant_broadcast_type_C)
        {
        case 0: c = mb->load_1d(mb, 1, 0); break;
        case 1: c = mb->load_1d(mb, s->constantM, 0); break;
        case 2: c = mb->load_2d(mb, 1, s->constantM, 0); break;
        case 3: c = mb->load_2d(mb, s->constantN, s->constantM, 0); break;
        case 4: c = mb->load_2d(mb, s->constantN, 1, 0); break;
        }
        s->C_host = (float*)take_blob(c, &bytes, &elemsize);
        if (!s->C_host || elemsize != 4) return -100;
        s->C_count = bytes / 4;
    }
    if (s->block_quant)
    {
        const int block = term_block(s->quantize_term), nblocks = (s->constantK + block - 1) / block;
        size_t bytes = 0;
        int elemsize = 0;
        s->B_block_scales = (float*)take_blob(mb->load_2d(mb, nblocks, s->constantN, 1), &bytes, &elemsize);
        if (!s->B_block_scales || elemsize != 4) return -100;
        s->B_block_scales_count = bytes / 4;
        if (s->quantize_term % 100 / 10 == 1)
        {
            s->B_input_scales = take_floats(mb->load_1d(mb, s->constantK, 1), s->constantK);
            if (!s->B_input_scales) return -100;
        }
    }
    else
    {
        if (s->constantA == 1)
        {
            s->A_scales_host = take_floats(mb->load_1d(mb, s->constantM, 1), s->constantM);
            if (!s->A_scales_host) return -100;
        }
        if (s->constantB == 1)
        {
            float* b = take_floats(mb->load_1d(mb, 1, 1), 1);
            if (!b) return -100;
            s->B_scale = b[0];
            free(b);
        }
    }
    return 0;
}

static int gemm_destroy_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    if (!s) return -1;
    if (s->stream) ncnnhip_stream_synchronize(s->stream);
    free_device(&s->d_A);
    free_device(&s->d_B);
    free_device(&s->d_C);
    free_device(&s->d_A_scales);
    free_device(&s->d_B_scale);
    free_device(&s->d_B_block_scales);
    free_device(&s->d_B_input_scales);
    free_device(&s->d_B_packed);
    free_device(&s->d_B_packed_descales);
    s->b_ready_int8 = 0;
    return conv_destroy_pipeline(layer, opt); /* the scratch slots and the stream */
}

static int gemm_create_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    int rc = 0;
    if (!s) return -1;
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    if (ncnnhip_stream_create(&s->stream) != 0) return fail(s, "ncnnhip_stream_create");
    if (s->constantA == 1) rc = upload_constant(s->A_host, s->A_bytes, &s->d_A);
    if (rc == 0 && s->C_host) rc = upload_constant(s->C_host, s->C_count * 4, &s->d_C);
    if (rc == 0 && s->A_scales_host) rc = upload_constant(s->A_scales_host, (size_t)s->constantM * 4, &s->d_A_scales);
    if (rc == 0 && s->block_quant)
    {
        const int bits = s->quantize_term / 100, block = term_block(s->quantize_term);
        rc = upload_constant(s->B_host, (size_t)s->B_w * s->B_h, &s->d_B);
        if (rc == 0) rc = upload_constant(s->B_block_scales, s->B_block_scales_count * 4, &s->d_B_block_scales);
        if (rc == 0 && s->B_input_scales) rc = upload_constant(s->B_input_scales, (size_t)s->constantK * 4, &s->d_B_input_scales);
        if (rc == 0 && ncnnhip_gemm_blockquant_packed_supported(s->constantK))
        {
            /* second form of B for few activation rows (decoding): matrix-core tiles */
            size_t wb = 0, db = 0;
            uint8_t* pw = 0;
            float* pd = 0;
            rc = ncnnhip_blockquant_packed_size(s->constantN, s->constantK, bits, block, &wb, &db);
            if (rc == 0)
            {
                pw = (uint8_t*)malloc(wb ? wb : 1);
                pd = (float*)malloc(db ? db : 1);
                if (!pw || !pd) rc = -1;
            }
            if (rc == 0) rc = ncnnhip_blockquant_pack((const uint8_t*)s->B_host, s->B_block_scales, s->constantN, s->constantK, bits, block, pw, pd);
            if (rc == 0) rc = upload_constant(pw, wb, &s->d_B_packed);
            if (rc == 0) rc = upload_constant(pd, db, &s->d_B_packed_descales);
            free(pw);
            free(pd);
        }
    }
    else if (rc == 0 && s->constantB == 1)
    {
        rc = upload_constant(s->B_host, s->B_bytes, &s->d_B);
        if (rc == 0 && s->B_elemsize == 1)
        {
            rc = upload_constant(&s->B_scale, 4, &s->d_B_scale);
            if (rc == 0 && s->transB == 0)
            {
                /* stored [K][N]: brought to K-contiguous rows once */
                void* d_bt = 0;
                rc = ncnnhip_malloc(&d_bt, (size_t)s->constantN * s->constantK);
                if (rc == 0) rc = ncnnhip_transpose_s8((const int8_t*)s->d_B, (size_t)s->constantN, s->constantK, s->constantN, (int8_t*)d_bt, (size_t)s->constantK, 0);
                if (rc == 0) rc = ncnnhip_stream_synchronize(0);
                if (rc != 0)
                {
                    if (d_bt) ncnnhip_free(d_bt);
                }
                else
                {
                    ncnnhip_free(s->d_B);
                    s->d_B = d_bt;
                }
            }
            if (rc == 0) s->b_ready_int8 = 1;
        }
    }
    if (rc != 0)
    {
        fail(s, "create_pipeline");
        gemm_destroy_pipeline(layer, opt);
        return -1;
    }
    return 0;
}

/* a matrix held in a Mat: 2-D (h rows of w) or 3-D with h == 1 (c rows, cstep apart); a 1-D blob is one row */
static int mat_rows(const ncnn_mat_t m)
{
    return ncnn_mat_get_dims(m) == 3 ? ncnn_mat_get_c(m) : ncnn_mat_get_h(m);
}
static size_t mat_row_stride(const ncnn_mat_t m)
{
    return ncnn_mat_get_dims(m) == 3 ? ncnn_mat_get_cstep(m) : (size_t)ncnn_mat_get_w(m);
}

/* broadcast type of a C operand given as a blob (src/layer/gemm.cpp:887-943) */
static int classify_c(const ncnn_mat_t C, int M, int N)
{
    const int dims = ncnn_mat_get_dims(C), w = ncnn_mat_get_w(C), h = ncnn_mat_get_h(C);
    int bt = -2;
    if (dims == 1 && w == 1) bt = 0;
    if (dims == 1 && w == M) bt = 1;
    if (dims == 1 && w == N) bt = 4;
    if (dims == 2 && w == 1 && h == M) bt = 2;
    if (dims == 2 && w == N && h == M) bt = 3;
    if (dims == 2 && w == N && h == 1) bt = 4;
    return bt;
}

static ncnn_mat_t create_output(const plugin_state* s, int M, int N)
{
    const int ow = s->output_transpose ? M : N, oh = s->output_transpose ? N : M;
    return s->output_N1M ? ncnn_mat_create_3d_elem(ow, 1, oh, 4u, 1, NULL) : ncnn_mat_create_2d_elem(ow, oh, 4u, 1, NULL);
}

static int gemm_block_quant_locked(plugin_state* s, const ncnn_mat_t* bottoms, int n, ncnn_mat_t* tops)
{
    const ncnn_mat_t A = bottoms[0];
    const int K = ncnn_mat_get_w(A), M = mat_rows(A), N = s->constantN;
    const int bits = s->quantize_term / 100, block = term_block(s->quantize_term);
    void* st = s->stream;
    const float* d_c = 0;
    int bt = -1, rc;
    void *d_a, *d_out;
    ncnn_mat_t top;

    if (ncnn_mat_get_elemsize(A) != 4u || ncnn_mat_get_elempack(A) != 1) return refuse(s, "unsupported input");
    if (K != s->constantK) return refuse(s, "weight block quantize K mismatch");
    d_a = scratch(s, SLOT_IN, mat_bytes(A));
    d_out = scratch(s, SLOT_OUT, (size_t)M * N * 4);
    if (!d_a || !d_out) return fail(s, "device scratch");
    if (ncnnhip_memcpy_h2d(d_a, ncnn_mat_get_data(A), mat_bytes(A), st) != 0) return fail(s, "upload A");
    if (s->constantC)
    {
        bt = s->d_C ? s->constant_broadcast_type_C : -1;
        d_c = (const float*)s->d_C;
    }
    else if (n == 2 && ncnn_mat_get_data(bottoms[1]))
    {
        void* p;
        bt = classify_c(bottoms[1], M, N);
        if (bt < 0 || ncnn_mat_get_elemsize(bottoms[1]) != 4u || ncnn_mat_get_elempack(bottoms[1]) != 1) return refuse(s, "unsupported C");
        p = scratch(s, SLOT_C, mat_bytes(bottoms[1]));
        if (!p || ncnnhip_memcpy_h2d(p, ncnn_mat_get_data(bottoms[1]), mat_bytes(bottoms[1]), st) != 0) return fail(s, "upload C");
        d_c = (const float*)p;
    }
    top = ncnn_mat_create_2d_elem(N, M, 4u, 1, NULL);
    if (!top || !ncnn_mat_get_data(top))
    {
        if (top) ncnn_mat_destroy(top);
        return -100;
    }
    tops[0] = top;
    /* a few activation rows (decoding) read the matrix-core tiles; more rows the stored fields in one fp32 pass */
    if (M <= 4 && s->d_B_packed && mat_row_stride(A) % 4 == 0)
        rc = ncnnhip_gemm_blockquant_packed((const float*)d_a, mat_row_stride(A), M, N, K, (const uint8_t*)s->d_B_packed, (const float*)s->d_B_packed_descales,
                                            bits, block, (const float*)s->d_B_input_scales, d_c, d_c ? bt : -1, s->alpha, s->beta, (float*)d_out, (size_t)N, st);
    else
        rc = ncnnhip_gemm_blockquant((const float*)d_a, mat_row_stride(A), M, N, K, (const uint8_t*)s->d_B, bits, block, (const float*)s->d_B_block_scales,
                                     (const float*)s->d_B_input_scales, d_c, d_c ? bt : -1, s->alpha, s->beta, (float*)d_out, (size_t)N, st);
    if (rc != 0) return fail(s, "ncnnhip_gemm_blockquant");
    rc = ncnnhip_memcpy_d2h(ncnn_mat_get_data(top), d_out, (size_t)M * N * 4, st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return rc == 0 ? 0 : fail(s, "download top blob");
}

static int gemm_int8_locked(plugin_state* s, const ncnn_mat_t* bottoms, int n, ncnn_mat_t* tops)
{
    void* st = s->stream;
    int rc, M, K, N = 0, a_rows, a_cols, a_elemsize, bt = 0;
    size_t a_stride, aq_stride, bq_stride = 0, out_stride;
    const void* d_a0;
    const int8_t *d_aq, *d_bq = 0;
    const float *d_sa, *d_sb = (const float*)s->d_B_scale, *d_c = 0;
    ncnn_mat_t C = 0, top;
    void* d_out;

    if (n < 1 && !(s->constantA && s->constantB)) return -1;

    /* ---- A: [M][K] K-contiguous int8 + one scale per row */
    if (s->constantA)
    {
        a_rows = s->A_h;
        a_cols = s->A_w;
        a_elemsize = s->A_elemsize;
        a_stride = (size_t)s->A_w;
        d_a0 = s->d_A;
    }
    else
    {
        const ncnn_mat_t A0 = bottoms[0];
        void* p;
        if (ncnn_mat_get_elempack(A0) != 1 || (ncnn_mat_get_elemsize(A0) != 4u && ncnn_mat_get_elemsize(A0) != 1u)) return refuse(s, "A must be a pack-1 fp32 or int8 blob");
        a_rows = mat_rows(A0);
        a_cols = ncnn_mat_get_w(A0);
        a_elemsize = (int)ncnn_mat_get_elemsize(A0);
        a_stride = mat_row_stride(A0);
        p = scratch(s, SLOT_IN, mat_bytes(A0));
        if (!p || ncnnhip_memcpy_h2d(p, ncnn_mat_get_data(A0), mat_bytes(A0), st) != 0) return fail(s, "upload A");
        d_a0 = p;
    }
    M = s->transA ? a_cols : a_rows;
    K = s->transA ? a_rows : a_cols;
    if (s->transA)
    {
        void* p = scratch(s, SLOT_AT, (size_t)M * K * (size_t)a_elemsize);
        if (!p) return fail(s, "device scratch");
        rc = a_elemsize == 4 ? ncnnhip_transpose_f32((const float*)d_a0, a_stride, a_rows, a_cols, (float*)p, (size_t)K, st)
                             : ncnnhip_transpose_s8((const int8_t*)d_a0, a_stride, a_rows, a_cols, (int8_t*)p, (size_t)K, st);
        if (rc != 0) return fail(s, "transpose A");
        d_a0 = p;
        a_stride = (size_t)K;
    }
    d_aq = (const int8_t*)d_a0;
    d_sa = (const float*)s->d_A_scales;
    aq_stride = a_stride;
    if (a_elemsize == 4)
    {
        void *q, *sc;
        aq_stride = ((size_t)K + 15) / 16 * 16;
        q = scratch(s, SLOT_QUANT, (size_t)M * aq_stride);
        sc = scratch(s, SLOT_SCALES, (size_t)M * 4);
        if (!q || !sc) return fail(s, "device scratch");
        if (ncnnhip_gemm_quantize_rows((const float*)d_a0, a_stride, M, K, (int8_t*)q, aq_stride, (float*)sc, st) != 0) return fail(s, "ncnnhip_gemm_quantize_rows");
        d_aq = (const int8_t*)q;
        d_sa = (const float*)sc;
    }
    else if (!d_sa)
        return refuse(s, "int8 A without A_data_int8_scales");

    /* ---- B: [N][K] K-contiguous int8 + one scale */
    if (s->b_ready_int8)
    {
        N = s->constantN;
        if (s->constantK != K) return refuse(s, "K of A differs from constantK");
        d_bq = (const int8_t*)s->d_B;
        bq_stride = (size_t)K;
    }
    else
    {
        int b_rows, b_cols;
        size_t b_stride;
        const void* d_b0;
        void *q, *sc;
        if (s->constantB)
        {
            if (s->B_elemsize != 4) return refuse(s, "constant B is neither int8 nor fp32");
            b_rows = s->B_h;
            b_cols = s->B_w;
            b_stride = (size_t)s->B_w;
            d_b0 = s->d_B;
        }
        else
        {
            const ncnn_mat_t B0 = s->constantA ? (n > 0 ? bottoms[0] : 0) : (n > 1 ? bottoms[1] : 0);
            void* p;
            if (!B0 || !ncnn_mat_get_data(B0) || ncnn_mat_get_elempack(B0) != 1 || ncnn_mat_get_elemsize(B0) != 4u)
                return refuse(s, "B must be an fp32 blob or a constant int8 table");
            b_rows = mat_rows(B0);
            b_cols = ncnn_mat_get_w(B0);
            b_stride = mat_row_stride(B0);
            p = scratch(s, SLOT_B, mat_bytes(B0));
            if (!p || ncnnhip_memcpy_h2d(p, ncnn_mat_get_data(B0), mat_bytes(B0), st) != 0) return fail(s, "upload B");
            d_b0 = p;
        }
        N = s->transB ? b_rows : b_cols;
        if ((s->transB ? b_cols : b_rows) != K) return refuse(s, "A and B disagree on K");
        /* whole-tensor dynamic quantisation, then (if stored [K][N]) transposed to K-contiguous rows */
        q = scratch(s, SLOT_BQ, (size_t)b_rows * b_cols);
        sc = scratch(s, SLOT_BSCALE, 4);
        if (!q || !sc) return fail(s, "device scratch");
        if (ncnnhip_gemm_quantize_tensor((const float*)d_b0, b_stride, b_rows, b_cols, (int8_t*)q, (size_t)b_cols, (float*)sc, st) != 0)
            return fail(s, "ncnnhip_gemm_quantize_tensor");
        d_sb = (const float*)sc;
        if (s->transB)
        {
            d_bq = (const int8_t*)q;
            bq_stride = (size_t)b_cols;
        }
        else
        {
            void* t = scratch(s, SLOT_BT, (size_t)N * K);
            if (!t) return fail(s, "device scratch");
            if (ncnnhip_transpose_s8((const int8_t*)q, (size_t)b_cols, b_rows, b_cols, (int8_t*)t, (size_t)K, st) != 0) return fail(s, "transpose B");
            d_bq = (const int8_t*)t;
            bq_stride = (size_t)K;
        }
    }

    /* ---- C */
    if (s->constantC)
    {
        bt = s->constant_broadcast_type_C;
        d_c = bt >= 0 ? (const float*)s->d_C : 0;
    }
    else
    {
        if (s->constantA && s->constantB && n == 1)
            C = bottoms[0];
        else if ((s->constantA || s->constantB) && n == 2)
            C = bottoms[1];
        else if (n == 3)
            C = bottoms[2];
        if (C && ncnn_mat_get_data(C))
        {
            const int cls = classify_c(C, M, N);
            void* p = scratch(s, SLOT_C, mat_bytes(C));
            if (cls >= 0) bt = cls;
            if (!p || ncnnhip_memcpy_h2d(p, ncnn_mat_get_data(C), mat_bytes(C), st) != 0) return fail(s, "upload C");
            d_c = bt >= 0 ? (const float*)p : 0;
        }
    }

    /* ---- output */
    top = create_output(s, M, N);
    if (!top || !ncnn_mat_get_data(top))
    {
        if (top) ncnn_mat_destroy(top);
        return -100;
    }
    tops[0] = top;
    out_stride = mat_row_stride(top);
    d_out = scratch(s, SLOT_OUT, mat_bytes(top));
    if (!d_out) return fail(s, "device scratch");
    rc = ncnnhip_gemm_int8(d_aq, aq_stride, d_bq, bq_stride, M, N, K, d_sa, d_sb, 1, d_c, d_c ? bt : -1, s->alpha, s->beta, s->output_transpose,
                           (float*)d_out, out_stride, 0, st);
    if (rc != 0) return fail(s, "ncnnhip_gemm_int8");
    rc = ncnnhip_memcpy_d2h(ncnn_mat_get_data(top), d_out, mat_bytes(top), st);
    if (rc == 0) rc = ncnnhip_stream_synchronize(st);
    return rc == 0 ? 0 : fail(s, "download top blob");
}

static int gemm_forward_n(const ncnn_layer_t layer, const ncnn_mat_t* bottoms, int n, ncnn_mat_t* tops, int n2, const ncnn_option_t opt)
{
    plugin_state* s = state_of(layer);
    int ret;
    (void)opt;
    if (!s || !s->stream) return refuse(s, "forward before create_pipeline");
    if (n2 < 1) return -1;
    if (device_ready() != 0) return fail(s, "ncnnhip_init");
    pthread_mutex_lock(&s->lock);
    ret = s->block_quant ? (n >= 1 ? gemm_block_quant_locked(s, bottoms, n, tops) : -1) : gemm_int8_locked(s, bottoms, n, tops);
    pthread_mutex_unlock(&s->lock);
    return ret;
}

static int gemm_forward_1(const ncnn_layer_t layer, const ncnn_mat_t bottom, ncnn_mat_t* top_blob, const ncnn_option_t opt)
{
    ncnn_mat_t bottoms[1];
    bottoms[0] = bottom;
    return gemm_forward_n(layer, bottoms, 1, top_blob, 1, opt);
}

/* ------------------------------------------------------------------ factories and registration */

static ncnn_layer_t create_layer(int kind)
{
    ncnn_layer_t layer = ncnn_layer_create();
    plugin_state* s = (plugin_state*)calloc(1, sizeof(plugin_state));
    if (!layer || !s)
    {
        if (layer) ncnn_layer_destroy(layer);
        free(s);
        return 0;
    }
    s->layer = layer;
    s->kind = kind;
    pthread_mutex_init(&s->lock, 0);
    pthread_mutex_lock(&g_states_lock);
    s->next = g_states;
    g_states = s;
    pthread_mutex_unlock(&g_states_lock);

    ncnn_layer_set_support_inplace(layer, 0);
    if (kind == KIND_GEMM)
    {
        ncnn_layer_set_one_blob_only(layer, 0);
        layer->load_param = gemm_load_param;
        layer->load_model = gemm_load_model;
        layer->create_pipeline = gemm_create_pipeline;
        layer->destroy_pipeline = gemm_destroy_pipeline;
        layer->forward_1 = gemm_forward_1;
        layer->forward_n = gemm_forward_n;
    }
    else
    {
        ncnn_layer_set_one_blob_only(layer, 1);
        layer->load_param = kind == KIND_INNERPRODUCT ? ip_load_param : conv_load_param;
        layer->load_model = kind == KIND_INNERPRODUCT ? ip_load_model : conv_load_model;
        layer->create_pipeline = kind == KIND_INNERPRODUCT ? ip_create_pipeline : conv_create_pipeline;
        layer->destroy_pipeline = conv_destroy_pipeline;
        layer->forward_1 = kind == KIND_INNERPRODUCT ? ip_forward_1 : conv_forward_1;
    }
    return layer;
}

static ncnn_layer_t creator(void* userdata)
{
    return create_layer((int)(intptr_t)userdata);
}

static void destroyer(ncnn_layer_t layer, void* userdata)
{
    plugin_state *s = state_of(layer), **link;
    (void)userdata;
    if (s)
    {
        /* Net::clear calls destroy_pipeline before the destroyer (src/net.cpp:2419-2460); a layer dropped before that still
         * holds its device memory, so the call is repeated here (it is idempotent) */
        if (s->kind == KIND_GEMM)
            gemm_destroy_pipeline(layer, 0);
        else
            conv_destroy_pipeline(layer, 0);
        pthread_mutex_lock(&g_states_lock);
        for (link = &g_states; *link; link = &(*link)->next)
            if (*link == s)
            {
                *link = s->next;
                break;
            }
        pthread_mutex_unlock(&g_states_lock);
        free(s->weight_q);
        free(s->bias);
        free(s->weight_scales);
        free(s->bottom_scales);
        free(s->top_scales);
        free(s->A_host);
        free(s->B_host);
        free(s->C_host);
        free(s->A_scales_host);
        free(s->B_block_scales);
        free(s->B_input_scales);
        pthread_mutex_destroy(&s->lock);
        free(s);
    }
    ncnn_layer_destroy(layer);
}

#if defined(__GNUC__)
__attribute__((visibility("default")))
#endif
int ncnnhip_plugin_register(ncnn_net_t net)
{
    if (!net) return -1;
    ncnn_net_register_custom_layer_by_type(net, "Convolution", creator, destroyer, (void*)(intptr_t)KIND_CONVOLUTION);
    ncnn_net_register_custom_layer_by_type(net, "ConvolutionDepthWise", creator, destroyer, (void*)(intptr_t)KIND_DEPTHWISE);
    ncnn_net_register_custom_layer_by_type(net, "InnerProduct", creator, destroyer, (void*)(intptr_t)KIND_INNERPRODUCT);
    ncnn_net_register_custom_layer_by_type(net, "Gemm", creator, destroyer, (void*)(intptr_t)KIND_GEMM);
    return 0;
}
