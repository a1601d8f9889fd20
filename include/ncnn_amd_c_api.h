/*
 * C ABI of the host runtime (libncnn_amd.so): the subset of ncnn's own C API (src/c_api.h) that
 * drives the int8 path end to end -- load_param, load_model, create_extractor, input, extract --
 * plus the one call that installs the MI355X layers.  Names, argument meaning and return values
 * are those of src/c_api.h at the cited lines, so a program written against ncnn's C API links
 * against this library unchanged for these calls.
 */
#ifndef NCNN_AMD_C_API_H
#define NCNN_AMD_C_API_H

#include <stddef.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif

#pragma GCC visibility push(default)

/* src/c_api.h:18-19.  ncnn's version is 1.0.<date of the build>; this library gives the date its interface was taken from. */
const char* ncnn_version(void);
int ncnn_version_number(void);

/* allocator api, src/c_api.h:21-34: a host allocator as a table of function pointers (the C++ object calls through the table,
 * so an entry may be replaced); NULL wherever an allocator is asked for means the library's own */
typedef struct __ncnn_allocator_t* ncnn_allocator_t;
struct __ncnn_allocator_t
{
    void* pthis;
    void* (*fast_malloc)(ncnn_allocator_t allocator, size_t size);
    void (*fast_free)(ncnn_allocator_t allocator, void* ptr);
};
ncnn_allocator_t ncnn_allocator_create_pool_allocator(void);
ncnn_allocator_t ncnn_allocator_create_unlocked_pool_allocator(void);
void ncnn_allocator_destroy(ncnn_allocator_t allocator);
typedef struct __ncnn_option_t* ncnn_option_t;
typedef struct __ncnn_mat_t* ncnn_mat_t;
typedef struct __ncnn_net_t* ncnn_net_t;
typedef struct __ncnn_extractor_t* ncnn_extractor_t;

/* src/c_api.h:58-95 */
ncnn_option_t ncnn_option_create(void);
void ncnn_option_destroy(ncnn_option_t opt);
void ncnn_option_set_num_threads(ncnn_option_t opt, int num_threads);
void ncnn_option_set_blob_allocator(ncnn_option_t opt, ncnn_allocator_t allocator);      /* src/c_api.h:64 */
void ncnn_option_set_workspace_allocator(ncnn_option_t opt, ncnn_allocator_t allocator); /* src/c_api.h:65 */
void ncnn_option_set_lightmode(ncnn_option_t opt, int enable); /* Option::lightmode */
void ncnn_option_set_use_int8_inference(ncnn_option_t opt, int enable); /* Option::use_int8_inference */
int ncnn_option_get_use_int8_inference(const ncnn_option_t opt);
/* Option::use_hip_compute: layers with a device-resident overload keep their blobs in HBM between each other (the switch
 * ncnn_option_set_use_vulkan_compute, src/c_api.h:85, is for the reference's GPU path).  Set on the net's option before
 * ncnn_extractor_create. */
void ncnn_option_set_use_hip_compute(ncnn_option_t opt, int enable);
int ncnn_option_get_use_hip_compute(const ncnn_option_t opt);
/* the switches of src/c_api.h:61-99 that ncnn::Option has here; none of them changes what the int8 layers compute */
int ncnn_option_get_num_threads(const ncnn_option_t opt);
int ncnn_option_get_use_vulkan_compute(const ncnn_option_t opt);
int ncnn_option_get_use_local_pool_allocator(const ncnn_option_t opt);
int ncnn_option_get_use_winograd_convolution(const ncnn_option_t opt);
int ncnn_option_get_use_sgemm_convolution(const ncnn_option_t opt);
int ncnn_option_get_use_packing_layout(const ncnn_option_t opt);
int ncnn_option_get_use_fp16_packed(const ncnn_option_t opt);
int ncnn_option_get_use_fp16_storage(const ncnn_option_t opt);
int ncnn_option_get_use_fp16_arithmetic(const ncnn_option_t opt);
int ncnn_option_get_use_int8_packed(const ncnn_option_t opt);
int ncnn_option_get_use_int8_storage(const ncnn_option_t opt);
int ncnn_option_get_use_int8_arithmetic(const ncnn_option_t opt);
int ncnn_option_get_use_bf16_storage(const ncnn_option_t opt);
void ncnn_option_set_use_vulkan_compute(ncnn_option_t opt, int enable);
void ncnn_option_set_use_local_pool_allocator(ncnn_option_t opt, int enable);
void ncnn_option_set_use_winograd_convolution(ncnn_option_t opt, int enable);
void ncnn_option_set_use_sgemm_convolution(ncnn_option_t opt, int enable);
void ncnn_option_set_use_packing_layout(ncnn_option_t opt, int enable);
void ncnn_option_set_use_fp16_packed(ncnn_option_t opt, int enable);
void ncnn_option_set_use_fp16_storage(ncnn_option_t opt, int enable);
void ncnn_option_set_use_fp16_arithmetic(ncnn_option_t opt, int enable);
void ncnn_option_set_use_int8_packed(ncnn_option_t opt, int enable);
void ncnn_option_set_use_int8_storage(ncnn_option_t opt, int enable);
void ncnn_option_set_use_int8_arithmetic(ncnn_option_t opt, int enable);
void ncnn_option_set_use_bf16_storage(ncnn_option_t opt, int enable);

/* src/c_api.h:134-165; data is caller-owned memory laid out as ncnn::Mat lays it out */
ncnn_mat_t ncnn_mat_create_external_1d_elem(int w, void* data, size_t elemsize, int elempack, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_2d_elem(int w, int h, void* data, size_t elemsize, int elempack, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_3d_elem(int w, int h, int c, void* data, size_t elemsize, int elempack, ncnn_allocator_t allocator);
/* owning blobs of any element size (src/c_api.h:109,124-126): what a layer written in C creates its top blob with */
ncnn_mat_t ncnn_mat_create(void);
ncnn_mat_t ncnn_mat_create_1d_elem(int w, size_t elemsize, int elempack, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_2d_elem(int w, int h, size_t elemsize, int elempack, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_3d_elem(int w, int h, int c, size_t elemsize, int elempack, ncnn_allocator_t allocator);
/* owning, batched 3-D blobs (src/c_api.h:117,131: fp32, or any element size); fill them through ncnn_mat_get_batch_data */
ncnn_mat_t ncnn_mat_create_3d_batch(int w, int h, int c, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_3d_elem_batch(int w, int h, int c, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator);
/* the remaining constructors of src/c_api.h:110-137 (fp32 unless an element size is given; "external" wraps caller memory) */
ncnn_mat_t ncnn_mat_create_1d(int w, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_2d(int w, int h, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_3d(int w, int h, int c, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_4d(int w, int h, int d, int c, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_1d_batch(int w, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_2d_batch(int w, int h, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_4d_batch(int w, int h, int d, int c, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_1d(int w, void* data, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_2d(int w, int h, void* data, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_3d(int w, int h, int c, void* data, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_4d(int w, int h, int d, int c, void* data, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_4d_elem(int w, int h, int d, int c, size_t elemsize, int elempack, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_1d_elem_batch(int w, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_2d_elem_batch(int w, int h, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_4d_elem_batch(int w, int h, int d, int c, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_create_external_4d_elem(int w, int h, int d, int c, void* data, size_t elemsize, int elempack, ncnn_allocator_t allocator);
/* src/c_api.h:140-146,165: fill, deep copy (batch included), reshape (a new handle; shares the data where the layout allows) */
void ncnn_mat_fill_float(ncnn_mat_t mat, float v);
ncnn_mat_t ncnn_mat_clone(const ncnn_mat_t mat, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_reshape_1d(const ncnn_mat_t mat, int w, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_reshape_2d(const ncnn_mat_t mat, int w, int h, ncnn_allocator_t allocator);
ncnn_mat_t ncnn_mat_reshape_3d(const ncnn_mat_t mat, int w, int h, int c, ncnn_allocator_t allocator);
void* ncnn_mat_get_channel_data(const ncnn_mat_t mat, int c);
void ncnn_mat_destroy(ncnn_mat_t mat);
int ncnn_mat_get_dims(const ncnn_mat_t mat);
int ncnn_mat_get_w(const ncnn_mat_t mat);
int ncnn_mat_get_h(const ncnn_mat_t mat);
int ncnn_mat_get_d(const ncnn_mat_t mat);
int ncnn_mat_get_c(const ncnn_mat_t mat);
int ncnn_mat_get_n(const ncnn_mat_t mat);
size_t ncnn_mat_get_elemsize(const ncnn_mat_t mat);
int ncnn_mat_get_elempack(const ncnn_mat_t mat);
size_t ncnn_mat_get_cstep(const ncnn_mat_t mat);
size_t ncnn_mat_get_nstep(const ncnn_mat_t mat);
void* ncnn_mat_get_data(const ncnn_mat_t mat);
void* ncnn_mat_get_batch_data(const ncnn_mat_t mat, int b);

/* src/c_api.h:338-388 */
ncnn_net_t ncnn_net_create(void);
void ncnn_net_destroy(ncnn_net_t net);
ncnn_option_t ncnn_net_get_option(ncnn_net_t net); /* borrowed: the net's own Option */
void ncnn_net_set_option(ncnn_net_t net, ncnn_option_t opt);
int ncnn_net_load_param(ncnn_net_t net, const char* path);
int ncnn_net_load_model(ncnn_net_t net, const char* path);
int ncnn_net_load_param_memory(ncnn_net_t net, const char* mem);
/* src/c_api.h:357,373: the binary form of the .param text that tools/ncnn2mem.cpp writes (layers by the reference's type
 * numbers, blobs by number, no names: feed and extract with ncnn_extractor_input_index / _extract_index).  The memory form
 * returns the bytes consumed, 0 when the load failed. */
int ncnn_net_load_param_bin(ncnn_net_t net, const char* path);
size_t ncnn_net_load_param_bin_memory(ncnn_net_t net, const unsigned char* mem);
size_t ncnn_net_load_model_memory(ncnn_net_t net, const unsigned char* mem);
/* src/c_api.h:382,390-391 */
void ncnn_net_clear(ncnn_net_t net);
int ncnn_net_get_input_index(const ncnn_net_t net, int i);
int ncnn_net_get_output_index(const ncnn_net_t net, int i);
int ncnn_net_get_input_count(const ncnn_net_t net);
int ncnn_net_get_output_count(const ncnn_net_t net);
const char* ncnn_net_get_input_name(const ncnn_net_t net, int i);
const char* ncnn_net_get_output_name(const ncnn_net_t net, int i);

/* src/c_api.h:396-403 */
ncnn_extractor_t ncnn_extractor_create(ncnn_net_t net);
void ncnn_extractor_destroy(ncnn_extractor_t ex);
void ncnn_extractor_set_option(ncnn_extractor_t ex, const ncnn_option_t opt);
int ncnn_extractor_input(ncnn_extractor_t ex, const char* name, const ncnn_mat_t mat);
int ncnn_extractor_extract(ncnn_extractor_t ex, const char* name, ncnn_mat_t* mat);
/* by blob index (src/c_api.h:405-406); the indices of a net's inputs and outputs come from ncnn_net_get_input_index / _output_index */
int ncnn_extractor_input_index(ncnn_extractor_t ex, int index, const ncnn_mat_t mat);
int ncnn_extractor_extract_index(ncnn_extractor_t ex, int index, ncnn_mat_t* mat);

/* paramdict api, src/c_api.h:200-213: what a layer written in C reads its parameters from */
typedef struct __ncnn_paramdict_t* ncnn_paramdict_t;
ncnn_paramdict_t ncnn_paramdict_create(void);
void ncnn_paramdict_destroy(ncnn_paramdict_t pd);
int ncnn_paramdict_get_type(const ncnn_paramdict_t pd, int id);
int ncnn_paramdict_get_int(const ncnn_paramdict_t pd, int id, int def);
float ncnn_paramdict_get_float(const ncnn_paramdict_t pd, int id, float def);
ncnn_mat_t ncnn_paramdict_get_array(const ncnn_paramdict_t pd, int id, const ncnn_mat_t def); /* caller destroys the result */
void ncnn_paramdict_set_int(ncnn_paramdict_t pd, int id, int i);
void ncnn_paramdict_set_float(ncnn_paramdict_t pd, int id, float f);
void ncnn_paramdict_set_array(ncnn_paramdict_t pd, int id, const ncnn_mat_t v);

/* modelbin api, src/c_api.h:238-251: what a layer written in C reads its weights from (results are the caller's to destroy) */
typedef struct __ncnn_modelbin_t* ncnn_modelbin_t;
struct __ncnn_modelbin_t
{
    void* pthis;
    ncnn_mat_t (*load_1d)(const ncnn_modelbin_t mb, int w, int type);
    ncnn_mat_t (*load_2d)(const ncnn_modelbin_t mb, int w, int h, int type);
    ncnn_mat_t (*load_3d)(const ncnn_modelbin_t mb, int w, int h, int c, int type);
};
ncnn_modelbin_t ncnn_modelbin_create_from_mat_array(const ncnn_mat_t* weights, int n);
void ncnn_modelbin_destroy(ncnn_modelbin_t mb);

/* datareader api, src/c_api.h:218-235: where .param text and .bin bytes come from, as a table a C program may fill in with
 * functions of its own (pthis is then the program's to use).  ncnn_datareader_create gives a table that reads nothing. */
typedef struct __ncnn_datareader_t* ncnn_datareader_t;
struct __ncnn_datareader_t
{
    void* pthis;
    int (*scan)(ncnn_datareader_t dr, const char* format, void* p);
    size_t (*read)(ncnn_datareader_t dr, void* buf, size_t size);
};
ncnn_datareader_t ncnn_datareader_create(void);
ncnn_datareader_t ncnn_datareader_create_from_stdio(FILE* fp);
ncnn_datareader_t ncnn_datareader_create_from_memory(const unsigned char** mem); /* *mem is advanced as bytes are read */
void ncnn_datareader_destroy(ncnn_datareader_t dr);
/* src/c_api.h:248 */
ncnn_modelbin_t ncnn_modelbin_create_from_datareader(const ncnn_datareader_t dr);
/* src/c_api.h:377-380 */
int ncnn_net_load_param_datareader(ncnn_net_t net, const ncnn_datareader_t dr);
int ncnn_net_load_param_bin_datareader(ncnn_net_t net, const ncnn_datareader_t dr);
int ncnn_net_load_model_datareader(ncnn_net_t net, const ncnn_datareader_t dr);

/* layer api, src/c_api.h:254-320: a layer as a table of function pointers.  ncnn_layer_create gives a layer whose table
 * holds the base class's behaviour, for a C program to overwrite entry by entry; ncnn_layer_create_by_type / _by_typeindex
 * wrap one of the library's built-in layers (NULL for a type it has no host implementation of -- the four int8 types among
 * them); ncnnhip_layer_create_by_type (no counterpart in the reference) wraps the MI355X implementation of "Convolution",
 * "ConvolutionDepthWise", "InnerProduct", "Gemm" or "MultiHeadAttention", for registration through
 * ncnn_net_register_custom_layer_by_type below. */
typedef struct __ncnn_layer_t* ncnn_layer_t;
struct __ncnn_layer_t
{
    void* pthis;
    int (*load_param)(ncnn_layer_t layer, const ncnn_paramdict_t pd);
    int (*load_model)(ncnn_layer_t layer, const ncnn_modelbin_t mb);
    int (*create_pipeline)(ncnn_layer_t layer, const ncnn_option_t opt);
    int (*destroy_pipeline)(ncnn_layer_t layer, const ncnn_option_t opt);
    int (*forward_1)(const ncnn_layer_t layer, const ncnn_mat_t bottom_blob, ncnn_mat_t* top_blob, const ncnn_option_t opt);
    int (*forward_n)(const ncnn_layer_t layer, const ncnn_mat_t* bottom_blobs, int n, ncnn_mat_t* top_blobs, int n2, const ncnn_option_t opt);
    int (*forward_inplace_1)(const ncnn_layer_t layer, ncnn_mat_t bottom_top_blob, const ncnn_option_t opt);
    int (*forward_inplace_n)(const ncnn_layer_t layer, ncnn_mat_t* bottom_top_blobs, int n, const ncnn_option_t opt);
};
ncnn_layer_t ncnn_layer_create(void);
ncnn_layer_t ncnn_layer_create_by_typeindex(int typeindex);
ncnn_layer_t ncnn_layer_create_by_type(const char* type);
int ncnn_layer_type_to_index(const char* type);
ncnn_layer_t ncnnhip_layer_create_by_type(const char* type);
void ncnn_layer_destroy(ncnn_layer_t layer);
const char* ncnn_layer_get_name(const ncnn_layer_t layer);
int ncnn_layer_get_typeindex(const ncnn_layer_t layer);
const char* ncnn_layer_get_type(const ncnn_layer_t layer);
int ncnn_layer_get_one_blob_only(const ncnn_layer_t layer);
int ncnn_layer_get_support_inplace(const ncnn_layer_t layer);
int ncnn_layer_get_support_vulkan(const ncnn_layer_t layer);
int ncnn_layer_get_support_packing(const ncnn_layer_t layer);
int ncnn_layer_get_support_bf16_storage(const ncnn_layer_t layer);
int ncnn_layer_get_support_fp16_storage(const ncnn_layer_t layer);
int ncnn_layer_get_support_vulkan_packing(const ncnn_layer_t layer);
int ncnn_layer_get_support_any_packing(const ncnn_layer_t layer);
int ncnn_layer_get_support_vulkan_any_packing(const ncnn_layer_t layer);
void ncnn_layer_set_one_blob_only(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_inplace(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_vulkan(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_packing(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_bf16_storage(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_fp16_storage(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_vulkan_packing(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_any_packing(ncnn_layer_t layer, int enable);
void ncnn_layer_set_support_vulkan_any_packing(ncnn_layer_t layer, int enable);
int ncnn_layer_get_bottom_count(const ncnn_layer_t layer);
int ncnn_layer_get_bottom(const ncnn_layer_t layer, int i);
int ncnn_layer_get_top_count(const ncnn_layer_t layer);
int ncnn_layer_get_top(const ncnn_layer_t layer, int i);
void ncnn_blob_get_bottom_shape(const ncnn_layer_t layer, int i, int* dims, int* w, int* h, int* c);
void ncnn_blob_get_top_shape(const ncnn_layer_t layer, int i, int* dims, int* w, int* h, int* c);

/* layer factory functions and their registration on a net, src/c_api.h:322-352.  Registering under a built-in type name
 * replaces the built-in layer (src/net.cpp:1214-1237).  Call before ncnn_net_load_param; the factories live until
 * ncnn_net_destroy. */
typedef ncnn_layer_t (*ncnn_layer_creator_t)(void* userdata);
typedef void (*ncnn_layer_destroyer_t)(ncnn_layer_t layer, void* userdata);
void ncnn_net_register_custom_layer_by_type(ncnn_net_t net, const char* type, ncnn_layer_creator_t creator, ncnn_layer_destroyer_t destroyer, void* userdata);
void ncnn_net_register_custom_layer_by_typeindex(ncnn_net_t net, int typeindex, ncnn_layer_creator_t creator, ncnn_layer_destroyer_t destroyer, void* userdata);

/*
 * Installs the MI355X implementations of Convolution, ConvolutionDepthWise, InnerProduct and
 * Gemm on a net: four Net::register_custom_layer calls under the built-in type names
 * (src/net.cpp:1214-1237, the route tests/test_squeezenet.cpp:320-404 exercises).  Call it
 * before load_param.  Returns 0, or -1 if a registration was refused.
 */
int ncnnhip_register_int8_layers(ncnn_net_t net);
/* The same route for MultiHeadAttention with block-quantised weights (quantize_term 4xx / 6xx / 8xx,
 * src/layer/multiheadattention.cpp:561-912).  Registered separately: a net whose attention layers are not
 * block-quantised must keep the reference's own layer. */
int ncnnhip_register_attention_layer(ncnn_net_t net);

/* Device-resident ends of an inference (Option::use_hip_compute on): a blob uploaded once with ncnnhip_net_upload feeds any
 * number of extractors without another copy; ncnnhip_extractor_extract_hipmat enqueues the layers and returns the result
 * where it lies in HBM without waiting; ncnnhip_extractor_synchronize waits for what the extractor enqueued;
 * ncnnhip_hipmat_download waits and copies to a host Mat (caller destroys it).  The counterparts in the reference are the
 * VkMat overloads of Extractor::input / extract (src/net.h:226-239).  Destroy every hipmat before its net. */
typedef struct __ncnn_hipmat_t* ncnn_hipmat_t;
int ncnnhip_net_upload(ncnn_net_t net, const ncnn_mat_t mat, ncnn_hipmat_t* out);
void ncnnhip_hipmat_destroy(ncnn_hipmat_t m);
int ncnnhip_hipmat_download(const ncnn_hipmat_t m, ncnn_mat_t* out);
int ncnnhip_extractor_input_hipmat(ncnn_extractor_t ex, const char* name, const ncnn_hipmat_t m);
int ncnnhip_extractor_extract_hipmat(ncnn_extractor_t ex, const char* name, ncnn_hipmat_t* out);
int ncnnhip_extractor_synchronize(ncnn_extractor_t ex);
/* Per-layer timing, the run-time form of the reference's NCNN_BENCHMARK build switch (src/net.cpp:145-180, printed by
 * benchmark(), src/benchmark.cpp): while enabled, every layer the extractor runs is recorded (device layers between two
 * events on its stream, host layers by the wall clock).  ncnnhip_extractor_layer_timing waits for the stream and writes one
 * line per record, in execution order: "<layer index>\t<type>\t<name>\t<device|host>\t<milliseconds>\n"; `needed`
 * (may be NULL) receives the size of the whole text with its terminator, text (may be NULL) at most `capacity` bytes. */
void ncnnhip_extractor_set_layer_timing(ncnn_extractor_t ex, int enable);
int ncnnhip_extractor_layer_timing(ncnn_extractor_t ex, char* text, size_t capacity, size_t* needed);

/* A forward pass recorded once and replayed with one launch (the reference's GPU path records a VkCompute command buffer
 * and submits it, src/command.h:22-67).  record runs the pass from blob `input_name` (= input, resident) to `output_name`
 * once and then records it; update_input copies new values into that same input blob; launch enqueues one replay;
 * output hands out the result blob, which every launch rewrites (destroy the handle with ncnnhip_hipmat_destroy).
 * One launch at a time per graph; destroy the graph before the net. */
typedef struct __ncnn_hipgraph_t* ncnn_hipgraph_t;
int ncnnhip_graph_record(ncnn_net_t net, const char* input_name, const ncnn_hipmat_t input, const char* output_name, ncnn_hipgraph_t* out);
int ncnnhip_graph_update_input(ncnn_hipgraph_t g, const ncnn_mat_t mat);
int ncnnhip_graph_replay(ncnn_hipgraph_t g);
int ncnnhip_graph_synchronize(ncnn_hipgraph_t g);
int ncnnhip_graph_output(ncnn_hipgraph_t g, ncnn_hipmat_t* out);
void ncnnhip_graph_release(ncnn_hipgraph_t g);

/* Gives the extractor its own device stream and buffer pool (one hipStream per Extractor) by
 * installing a host blob allocator that carries them; the allocator lives until
 * ncnnhip_extractor_detach_stream or process end.  Optional: without it a per-thread stream is used. */
void* ncnnhip_extractor_attach_stream(ncnn_extractor_t ex);
void ncnnhip_extractor_detach_stream(void* handle);

/* Introspection used by the host-logic tests: fields a layer holds after load_param / load_model. */
int ncnn_net_get_layer_count(const ncnn_net_t net);
const char* ncnn_net_get_layer_type(const ncnn_net_t net, int i);
const char* ncnn_net_get_layer_name(const ncnn_net_t net, int i);
int ncnn_net_get_layer_flags(const ncnn_net_t net, int i); /* bit0 one_blob_only, bit1 support_inplace, bit2 support_int8_storage, bit3 support_batch, bit4 support_packing */
int ncnn_net_get_blob_count(const ncnn_net_t net);
const char* ncnn_net_get_blob_name(const ncnn_net_t net, int i);
int ncnn_net_get_blob_producer(const ncnn_net_t net, int i);
int ncnn_net_get_blob_consumer(const ncnn_net_t net, int i);

/* Parses one .param key=value tail ("0=64 1=3 10=0.0,6.0") and reports slot `id`: returns the slot
 * type (0 unset, 2 int, 3 float, 5 int array, 6 float array, 7 string, -1 parse error); the raw
 * 32-bit payload (or the array length) goes to *value_bits, array elements to array_bits[0..cap). */
int ncnn_paramdict_probe(const char* text, int id, unsigned int* value_bits, unsigned int* array_bits, int cap);
/* the same for the binary form (ParamDict::load_param_bin, src/paramdict.cpp:491-637); mem ends with the end mark -233 */
int ncnn_paramdict_probe_bin(const unsigned char* mem, int id, unsigned int* value_bits, unsigned int* array_bits, int cap);

/* Reads one blob of `w` elements of load-type `type` (0 tagged / 1 raw fp32) from a .bin image and
 * copies it as fp32 or int8 to out; returns the element size (4 or 1), 0 on failure. *consumed =
 * bytes of the image used. */
int ncnn_modelbin_probe(const unsigned char* mem, int w, int type, void* out, size_t* consumed);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif

#endif /* NCNN_AMD_C_API_H */
