#include "ncnn_amd_c_api.h"

#include <stdlib.h>
#include <string.h>

#include <string>
#include <string.h>

#include "layers/hip_layers.h"
#include "layers/hip_support.h"
#include "ncnn/datareader.h"
#include "ncnn/modelbin.h"
#include "ncnn/net.h"
#include "ncnn/paramdict.h"

using namespace ncnn;

namespace ncnn_amd {
void release_custom_layer_factories(const ncnn::Net* net); // c_api_layer.cpp
}

static Option* O(ncnn_option_t p)
{
    return (Option*)p;
}
static Mat* M(ncnn_mat_t p)
{
    return (Mat*)p;
}
static Net* N(ncnn_net_t p)
{
    return (Net*)p;
}
static Extractor* E(ncnn_extractor_t p)
{
    return (Extractor*)p;
}

// ---- allocators as tables of function pointers (src/c_api.cpp:55-150): the C++ object calls through the table, so a C
// program may replace an entry (that is how an out-of-memory test makes fastMalloc return NULL)
static Allocator* A(ncnn_allocator_t a)
{
    return a ? (Allocator*)a->pthis : 0;
}
class PoolAllocator_c_api : public PoolAllocator
{
public:
    explicit PoolAllocator_c_api(ncnn_allocator_t a) : allocator(a) {}
    virtual void* fastMalloc(size_t size)
    {
        return allocator->fast_malloc(allocator, size);
    }
    virtual void fastFree(void* ptr)
    {
        allocator->fast_free(allocator, ptr);
    }
    ncnn_allocator_t allocator;
};
class UnlockedPoolAllocator_c_api : public UnlockedPoolAllocator
{
public:
    explicit UnlockedPoolAllocator_c_api(ncnn_allocator_t a) : allocator(a) {}
    virtual void* fastMalloc(size_t size)
    {
        return allocator->fast_malloc(allocator, size);
    }
    virtual void fastFree(void* ptr)
    {
        allocator->fast_free(allocator, ptr);
    }
    ncnn_allocator_t allocator;
};
static void* pool_fast_malloc(ncnn_allocator_t a, size_t size)
{
    return ((PoolAllocator*)a->pthis)->PoolAllocator::fastMalloc(size);
}
static void pool_fast_free(ncnn_allocator_t a, void* ptr)
{
    ((PoolAllocator*)a->pthis)->PoolAllocator::fastFree(ptr);
}
static void* unlocked_pool_fast_malloc(ncnn_allocator_t a, size_t size)
{
    return ((UnlockedPoolAllocator*)a->pthis)->UnlockedPoolAllocator::fastMalloc(size);
}
static void unlocked_pool_fast_free(ncnn_allocator_t a, void* ptr)
{
    ((UnlockedPoolAllocator*)a->pthis)->UnlockedPoolAllocator::fastFree(ptr);
}

extern "C" {

ncnn_allocator_t ncnn_allocator_create_pool_allocator(void)
{
    ncnn_allocator_t a = (ncnn_allocator_t)malloc(sizeof(struct __ncnn_allocator_t));
    a->pthis = (void*)static_cast<Allocator*>(new PoolAllocator_c_api(a));
    a->fast_malloc = pool_fast_malloc;
    a->fast_free = pool_fast_free;
    return a;
}
ncnn_allocator_t ncnn_allocator_create_unlocked_pool_allocator(void)
{
    ncnn_allocator_t a = (ncnn_allocator_t)malloc(sizeof(struct __ncnn_allocator_t));
    a->pthis = (void*)static_cast<Allocator*>(new UnlockedPoolAllocator_c_api(a));
    a->fast_malloc = unlocked_pool_fast_malloc;
    a->fast_free = unlocked_pool_fast_free;
    return a;
}
void ncnn_allocator_destroy(ncnn_allocator_t allocator)
{
    if (!allocator) return;
    delete (Allocator*)allocator->pthis;
    free(allocator);
}
void ncnn_option_set_blob_allocator(ncnn_option_t opt, ncnn_allocator_t allocator)
{
    O(opt)->blob_allocator = A(allocator);
}
void ncnn_option_set_workspace_allocator(ncnn_option_t opt, ncnn_allocator_t allocator)
{
    O(opt)->workspace_allocator = A(allocator);
}

ncnn_option_t ncnn_option_create(void)
{
    return (ncnn_option_t) new Option;
}
void ncnn_option_destroy(ncnn_option_t opt)
{
    delete O(opt);
}
void ncnn_option_set_num_threads(ncnn_option_t opt, int num_threads)
{
    O(opt)->num_threads = num_threads;
}
void ncnn_option_set_lightmode(ncnn_option_t opt, int enable)
{
    O(opt)->lightmode = enable != 0;
}
void ncnn_option_set_use_int8_inference(ncnn_option_t opt, int enable)
{
    O(opt)->use_int8_inference = enable != 0;
}
int ncnn_option_get_use_int8_inference(const ncnn_option_t opt)
{
    return O(opt)->use_int8_inference;
}
void ncnn_option_set_use_hip_compute(ncnn_option_t opt, int enable)
{
    O(opt)->use_hip_compute = enable != 0;
}
int ncnn_option_get_use_hip_compute(const ncnn_option_t opt)
{
    return O(opt)->use_hip_compute;
}

ncnn_mat_t ncnn_mat_create_external_1d_elem(int w, void* data, size_t elemsize, int elempack, ncnn_allocator_t)
{
    Mat* m = new Mat(w, data, elemsize);
    m->elempack = elempack;
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_external_2d_elem(int w, int h, void* data, size_t elemsize, int elempack, ncnn_allocator_t)
{
    Mat* m = new Mat(w, h, data, elemsize);
    m->elempack = elempack;
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_external_3d_elem(int w, int h, int c, void* data, size_t elemsize, int elempack, ncnn_allocator_t)
{
    Mat* m = new Mat(w, h, c, data, elemsize);
    m->elempack = elempack;
    return (ncnn_mat_t)m;
}
static ncnn_mat_t made(int dims, int w, int h, int d, int c, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    if (dims == 1)
        m->create(w, elemsize, elempack, n, A(allocator));
    else if (dims == 2)
        m->create(w, h, elemsize, elempack, n, A(allocator));
    else if (dims == 3)
        m->create(w, h, c, elemsize, elempack, n, A(allocator));
    else
        m->create(w, h, d, c, elemsize, elempack, n, A(allocator));
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_1d(int w, ncnn_allocator_t allocator)
{
    return made(1, w, 1, 1, 1, 4u, 1, 1, allocator);
}
ncnn_mat_t ncnn_mat_create_2d(int w, int h, ncnn_allocator_t allocator)
{
    return made(2, w, h, 1, 1, 4u, 1, 1, allocator);
}
ncnn_mat_t ncnn_mat_create_3d(int w, int h, int c, ncnn_allocator_t allocator)
{
    return made(3, w, h, 1, c, 4u, 1, 1, allocator);
}
ncnn_mat_t ncnn_mat_create_4d(int w, int h, int d, int c, ncnn_allocator_t allocator)
{
    return made(4, w, h, d, c, 4u, 1, 1, allocator);
}
ncnn_mat_t ncnn_mat_create_1d_batch(int w, int n, ncnn_allocator_t allocator)
{
    return made(1, w, 1, 1, 1, 4u, 1, n, allocator);
}
ncnn_mat_t ncnn_mat_create_2d_batch(int w, int h, int n, ncnn_allocator_t allocator)
{
    return made(2, w, h, 1, 1, 4u, 1, n, allocator);
}
ncnn_mat_t ncnn_mat_create_4d_batch(int w, int h, int d, int c, int n, ncnn_allocator_t allocator)
{
    return made(4, w, h, d, c, 4u, 1, n, allocator);
}
ncnn_mat_t ncnn_mat_create_4d_elem(int w, int h, int d, int c, size_t elemsize, int elempack, ncnn_allocator_t allocator)
{
    return made(4, w, h, d, c, elemsize, elempack, 1, allocator);
}
ncnn_mat_t ncnn_mat_create_1d_elem_batch(int w, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator)
{
    return made(1, w, 1, 1, 1, elemsize, elempack, n, allocator);
}
ncnn_mat_t ncnn_mat_create_2d_elem_batch(int w, int h, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator)
{
    return made(2, w, h, 1, 1, elemsize, elempack, n, allocator);
}
ncnn_mat_t ncnn_mat_create_4d_elem_batch(int w, int h, int d, int c, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator)
{
    return made(4, w, h, d, c, elemsize, elempack, n, allocator);
}
ncnn_mat_t ncnn_mat_create_external_1d(int w, void* data, ncnn_allocator_t)
{
    return (ncnn_mat_t)(new Mat(w, data, (size_t)4u));
}
ncnn_mat_t ncnn_mat_create_external_2d(int w, int h, void* data, ncnn_allocator_t)
{
    return (ncnn_mat_t)(new Mat(w, h, data, (size_t)4u));
}
ncnn_mat_t ncnn_mat_create_external_3d(int w, int h, int c, void* data, ncnn_allocator_t)
{
    return (ncnn_mat_t)(new Mat(w, h, c, data, (size_t)4u));
}
ncnn_mat_t ncnn_mat_create_external_4d(int w, int h, int d, int c, void* data, ncnn_allocator_t)
{
    return (ncnn_mat_t)(new Mat(w, h, d, c, data, (size_t)4u));
}
ncnn_mat_t ncnn_mat_create_external_4d_elem(int w, int h, int d, int c, void* data, size_t elemsize, int elempack, ncnn_allocator_t)
{
    Mat* m = new Mat(w, h, d, c, data, elemsize);
    m->elempack = elempack;
    return (ncnn_mat_t)m;
}
void ncnn_mat_fill_float(ncnn_mat_t mat, float v)
{
    M(mat)->fill(v);
}
ncnn_mat_t ncnn_mat_clone(const ncnn_mat_t mat, ncnn_allocator_t allocator)
{
    return (ncnn_mat_t)(new Mat(M(mat)->clone(A(allocator))));
}
ncnn_mat_t ncnn_mat_reshape_1d(const ncnn_mat_t mat, int w, ncnn_allocator_t allocator)
{
    return (ncnn_mat_t)(new Mat(M(mat)->reshape(w, A(allocator))));
}
ncnn_mat_t ncnn_mat_reshape_2d(const ncnn_mat_t mat, int w, int h, ncnn_allocator_t allocator)
{
    return (ncnn_mat_t)(new Mat(M(mat)->reshape(w, h, A(allocator))));
}
ncnn_mat_t ncnn_mat_reshape_3d(const ncnn_mat_t mat, int w, int h, int c, ncnn_allocator_t allocator)
{
    return (ncnn_mat_t)(new Mat(M(mat)->reshape(w, h, c, A(allocator))));
}
void* ncnn_mat_get_channel_data(const ncnn_mat_t mat, int c)
{
    return M(mat)->channel(c).data;
}

#define OPTION_SWITCH(field)                                              \
    int ncnn_option_get_##field(const ncnn_option_t opt)                  \
    {                                                                     \
        return O(opt)->field;                                             \
    }                                                                     \
    void ncnn_option_set_##field(ncnn_option_t opt, int enable)           \
    {                                                                     \
        O(opt)->field = enable != 0;                                      \
    }
OPTION_SWITCH(use_vulkan_compute)
OPTION_SWITCH(use_local_pool_allocator)
OPTION_SWITCH(use_winograd_convolution)
OPTION_SWITCH(use_sgemm_convolution)
OPTION_SWITCH(use_packing_layout)
OPTION_SWITCH(use_fp16_packed)
OPTION_SWITCH(use_fp16_storage)
OPTION_SWITCH(use_fp16_arithmetic)
OPTION_SWITCH(use_int8_packed)
OPTION_SWITCH(use_int8_storage)
OPTION_SWITCH(use_int8_arithmetic)
OPTION_SWITCH(use_bf16_storage)
#undef OPTION_SWITCH
int ncnn_option_get_num_threads(const ncnn_option_t opt)
{
    return O(opt)->num_threads;
}

void ncnn_net_clear(ncnn_net_t net)
{
    N(net)->clear();
}
int ncnn_net_get_input_index(const ncnn_net_t net, int i)
{
    const std::vector<int>& v = N(net)->input_indexes();
    return (i >= 0 && (size_t)i < v.size()) ? v[(size_t)i] : -1;
}
int ncnn_net_get_output_index(const ncnn_net_t net, int i)
{
    const std::vector<int>& v = N(net)->output_indexes();
    return (i >= 0 && (size_t)i < v.size()) ? v[(size_t)i] : -1;
}
int ncnn_extractor_input_index(ncnn_extractor_t ex, int index, const ncnn_mat_t mat)
{
    return E(ex)->input(index, *M(mat));
}
int ncnn_extractor_extract_index(ncnn_extractor_t ex, int index, ncnn_mat_t* mat)
{
    Mat out;
    int ret = E(ex)->extract(index, out);
    *mat = (ncnn_mat_t) new Mat(out);
    return ret;
}

ncnn_mat_t ncnn_mat_create(void)
{
    return (ncnn_mat_t)(new Mat);
}
ncnn_mat_t ncnn_mat_create_1d_elem(int w, size_t elemsize, int elempack, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    m->create(w, elemsize, elempack, A(allocator));
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_2d_elem(int w, int h, size_t elemsize, int elempack, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    m->create(w, h, elemsize, elempack, A(allocator));
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_3d_elem(int w, int h, int c, size_t elemsize, int elempack, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    m->create(w, h, c, elemsize, elempack, A(allocator));
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_3d_batch(int w, int h, int c, int n, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    m->create(w, h, c, (size_t)4u, 1, n, A(allocator));
    return (ncnn_mat_t)m;
}
ncnn_mat_t ncnn_mat_create_3d_elem_batch(int w, int h, int c, size_t elemsize, int elempack, int n, ncnn_allocator_t allocator)
{
    Mat* m = new Mat;
    m->create(w, h, c, elemsize, elempack, n, A(allocator));
    return (ncnn_mat_t)m;
}
void ncnn_mat_destroy(ncnn_mat_t mat)
{
    delete M(mat);
}
int ncnn_mat_get_dims(const ncnn_mat_t mat)
{
    return M(mat)->dims;
}
int ncnn_mat_get_w(const ncnn_mat_t mat)
{
    return M(mat)->w;
}
int ncnn_mat_get_h(const ncnn_mat_t mat)
{
    return M(mat)->h;
}
int ncnn_mat_get_d(const ncnn_mat_t mat)
{
    return M(mat)->d;
}
int ncnn_mat_get_c(const ncnn_mat_t mat)
{
    return M(mat)->c;
}
int ncnn_mat_get_n(const ncnn_mat_t mat)
{
    return M(mat)->n;
}
size_t ncnn_mat_get_elemsize(const ncnn_mat_t mat)
{
    return M(mat)->elemsize;
}
int ncnn_mat_get_elempack(const ncnn_mat_t mat)
{
    return M(mat)->elempack;
}
size_t ncnn_mat_get_cstep(const ncnn_mat_t mat)
{
    return M(mat)->cstep;
}
size_t ncnn_mat_get_nstep(const ncnn_mat_t mat)
{
    return M(mat)->nstep;
}
void* ncnn_mat_get_data(const ncnn_mat_t mat)
{
    return M(mat)->data;
}
void* ncnn_mat_get_batch_data(const ncnn_mat_t mat, int b)
{
    return (unsigned char*)M(mat)->data + M(mat)->nstep * b * M(mat)->elemsize;
}

ncnn_net_t ncnn_net_create(void)
{
    return (ncnn_net_t) new Net;
}
void ncnn_net_destroy(ncnn_net_t net)
{
    delete N(net);
    ncnn_amd::release_custom_layer_factories(N(net)); // after the layers they made are gone
}
ncnn_option_t ncnn_net_get_option(ncnn_net_t net)
{
    return (ncnn_option_t)&N(net)->opt;
}
void ncnn_net_set_option(ncnn_net_t net, ncnn_option_t opt)
{
    N(net)->opt = *O(opt);
}
int ncnn_net_load_param(ncnn_net_t net, const char* path)
{
    return N(net)->load_param(path);
}
int ncnn_net_load_model(ncnn_net_t net, const char* path)
{
    return N(net)->load_model(path);
}
int ncnn_net_load_param_memory(ncnn_net_t net, const char* mem)
{
    return N(net)->load_param_mem(mem);
}
const char* ncnn_version(void)
{
    return "1.0.20251101";
}
int ncnn_version_number(void)
{
    return 20251101;
}
int ncnn_net_load_param_bin(ncnn_net_t net, const char* path)
{
    return N(net)->load_param_bin(path);
}
size_t ncnn_net_load_param_bin_memory(ncnn_net_t net, const unsigned char* mem)
{
    return N(net)->load_param_bin_mem(mem);
}
size_t ncnn_net_load_model_memory(ncnn_net_t net, const unsigned char* mem)
{
    return N(net)->load_model(mem);
}
int ncnn_net_get_input_count(const ncnn_net_t net)
{
    return (int)N(net)->input_names().size();
}
int ncnn_net_get_output_count(const ncnn_net_t net)
{
    return (int)N(net)->output_names().size();
}
const char* ncnn_net_get_input_name(const ncnn_net_t net, int i)
{
    return N(net)->input_names()[(size_t)i];
}
const char* ncnn_net_get_output_name(const ncnn_net_t net, int i)
{
    return N(net)->output_names()[(size_t)i];
}

ncnn_extractor_t ncnn_extractor_create(ncnn_net_t net)
{
    return (ncnn_extractor_t) new Extractor(N(net)->create_extractor());
}
void ncnn_extractor_destroy(ncnn_extractor_t ex)
{
    delete E(ex);
}
void ncnn_extractor_set_option(ncnn_extractor_t ex, const ncnn_option_t opt)
{
    E(ex)->set_light_mode(O(opt)->lightmode);
    E(ex)->set_num_threads(O(opt)->num_threads);
}
int ncnn_extractor_input(ncnn_extractor_t ex, const char* name, const ncnn_mat_t mat)
{
    return E(ex)->input(name, *M(mat));
}
int ncnn_extractor_extract(ncnn_extractor_t ex, const char* name, ncnn_mat_t* mat)
{
    Mat out;
    int ret = E(ex)->extract(name, out);
    *mat = (ncnn_mat_t) new Mat(out);
    return ret;
}

int ncnnhip_net_upload(ncnn_net_t net, const ncnn_mat_t mat, ncnn_hipmat_t* out)
{
    HipMat* m = new HipMat;
    int ret = N(net)->upload(*M(mat), *m);
    if (ret != 0)
    {
        delete m;
        m = 0;
    }
    *out = (ncnn_hipmat_t)m;
    return ret;
}
void ncnnhip_hipmat_destroy(ncnn_hipmat_t m)
{
    delete (HipMat*)m;
}
int ncnnhip_hipmat_download(const ncnn_hipmat_t m, ncnn_mat_t* out)
{
    const HipMat* hm = (const HipMat*)m;
    Mat host;
    // The command the blob came from may be gone (the blob keeps only its buffers alive), and whoever produced the values
    // may have enqueued them on any stream: wait for the device, then copy on this thread's own command.
    static thread_local HipCommand download_cmd;
    int ret = -1;
    if (hm && !hm->empty() && download_cmd.ensure_ready() == 0 && ncnnhip_device_synchronize() == 0) ret = download_cmd.download(*hm, host, 0);
    *out = (ncnn_mat_t) new Mat(host);
    return ret;
}
int ncnnhip_extractor_input_hipmat(ncnn_extractor_t ex, const char* name, const ncnn_hipmat_t m)
{
    return E(ex)->input(name, *(const HipMat*)m);
}
int ncnnhip_extractor_extract_hipmat(ncnn_extractor_t ex, const char* name, ncnn_hipmat_t* out)
{
    HipMat* m = new HipMat;
    int ret = E(ex)->extract(name, *m);
    *out = (ncnn_hipmat_t)m;
    return ret;
}
void ncnnhip_extractor_set_layer_timing(ncnn_extractor_t ex, int enable)
{
    E(ex)->set_layer_timing(enable != 0);
}
int ncnnhip_extractor_layer_timing(ncnn_extractor_t ex, char* text, size_t capacity, size_t* needed)
{
    std::vector<Extractor::LayerTime> t;
    int ret = E(ex)->layer_timing(t);
    if (ret != 0) return ret;
    std::string out;
    char line[512];
    for (size_t i = 0; i < t.size(); i++)
    {
        snprintf(line, sizeof(line), "%d\t%s\t%s\t%s\t%.6f\n", t[i].layer_index, t[i].type.c_str(), t[i].name.c_str(), t[i].on_device ? "device" : "host", t[i].ms);
        out += line;
    }
    if (needed) *needed = out.size() + 1;
    if (text && capacity)
    {
        const size_t n = out.size() < capacity - 1 ? out.size() : capacity - 1;
        memcpy(text, out.data(), n);
        text[n] = 0;
    }
    return 0;
}
int ncnnhip_extractor_synchronize(ncnn_extractor_t ex)
{
    return E(ex)->synchronize();
}

int ncnnhip_graph_record(ncnn_net_t net, const char* input_name, const ncnn_hipmat_t input, const char* output_name, ncnn_hipgraph_t* out)
{
    *out = 0;
    if (!input) return -1;
    HipGraph* g = new HipGraph;
    int ret = g->record(*N(net), input_name, *(const HipMat*)input, output_name);
    if (ret != 0)
    {
        delete g;
        return ret;
    }
    *out = (ncnn_hipgraph_t)g;
    return 0;
}
int ncnnhip_graph_update_input(ncnn_hipgraph_t g, const ncnn_mat_t mat)
{
    return ((HipGraph*)g)->update_input(*M(mat));
}
int ncnnhip_graph_replay(ncnn_hipgraph_t g)
{
    return ((HipGraph*)g)->launch();
}
int ncnnhip_graph_synchronize(ncnn_hipgraph_t g)
{
    return ((HipGraph*)g)->synchronize();
}
int ncnnhip_graph_output(ncnn_hipgraph_t g, ncnn_hipmat_t* out)
{
    *out = (ncnn_hipmat_t) new HipMat(((HipGraph*)g)->output());
    return 0;
}
void ncnnhip_graph_release(ncnn_hipgraph_t g)
{
    delete (HipGraph*)g;
}

int ncnnhip_register_int8_layers(ncnn_net_t net)
{
    using namespace ncnn_amd;
    int ret = 0;
    ret |= N(net)->register_custom_layer("Convolution", Convolution_hip_creator, hip_layer_destroyer, net);
    ret |= N(net)->register_custom_layer("ConvolutionDepthWise", ConvolutionDepthWise_hip_creator, hip_layer_destroyer, net);
    ret |= N(net)->register_custom_layer("InnerProduct", InnerProduct_hip_creator, hip_layer_destroyer, net);
    ret |= N(net)->register_custom_layer("Gemm", Gemm_hip_creator, hip_layer_destroyer, net);
    return ret ? -1 : 0;
}

int ncnnhip_register_attention_layer(ncnn_net_t net)
{
    return N(net)->register_custom_layer("MultiHeadAttention", ncnn_amd::MultiHeadAttention_hip_creator, ncnn_amd::hip_layer_destroyer, net) ? -1 : 0;
}

void* ncnnhip_extractor_attach_stream(ncnn_extractor_t ex)
{
    ncnn_amd::HipBlobAllocator* a = new ncnn_amd::HipBlobAllocator;
    E(ex)->set_blob_allocator(a);
    return a;
}
void ncnnhip_extractor_detach_stream(void* handle)
{
    delete (ncnn_amd::HipBlobAllocator*)handle;
}

int ncnn_net_get_layer_count(const ncnn_net_t net)
{
    return (int)N(net)->layers().size();
}
const char* ncnn_net_get_layer_type(const ncnn_net_t net, int i)
{
    return N(net)->layers()[(size_t)i]->type.c_str();
}
const char* ncnn_net_get_layer_name(const ncnn_net_t net, int i)
{
    return N(net)->layers()[(size_t)i]->name.c_str();
}
int ncnn_net_get_layer_flags(const ncnn_net_t net, int i)
{
    const Layer* l = N(net)->layers()[(size_t)i];
    return (l->one_blob_only ? 1 : 0) | (l->support_inplace ? 2 : 0) | (l->support_int8_storage ? 4 : 0) | (l->support_batch ? 8 : 0) | (l->support_packing ? 16 : 0);
}
int ncnn_net_get_blob_count(const ncnn_net_t net)
{
    return (int)N(net)->blobs().size();
}
const char* ncnn_net_get_blob_name(const ncnn_net_t net, int i)
{
    return N(net)->blobs()[(size_t)i].name.c_str();
}
int ncnn_net_get_blob_producer(const ncnn_net_t net, int i)
{
    return N(net)->blobs()[(size_t)i].producer;
}
int ncnn_net_get_blob_consumer(const ncnn_net_t net, int i)
{
    return N(net)->blobs()[(size_t)i].consumer;
}

static int paramdict_probe_slot(const ParamDict& pd, int id, unsigned int* value_bits, unsigned int* array_bits, int cap);

// the same for the binary form (ParamDict::load_param_bin): mem must hold the end mark -233
int ncnn_paramdict_probe_bin(const unsigned char* mem, int id, unsigned int* value_bits, unsigned int* array_bits, int cap)
{
    const unsigned char* cursor = mem;
    DataReaderFromMemory dr(cursor);
    ParamDict pd;
    if (pd.load_param_bin(dr) != 0) return -1;
    return paramdict_probe_slot(pd, id, value_bits, array_bits, cap);
}

int ncnn_paramdict_probe(const char* text, int id, unsigned int* value_bits, unsigned int* array_bits, int cap)
{
    const unsigned char* cursor = (const unsigned char*)text;
    DataReaderFromMemory dr(cursor);
    ParamDict pd;
    if (pd.load_param(dr) != 0) return -1;
    return paramdict_probe_slot(pd, id, value_bits, array_bits, cap);
}

static int paramdict_probe_slot(const ParamDict& pd, int id, unsigned int* value_bits, unsigned int* array_bits, int cap)
{
    const int t = pd.type(id);
    if (t == 1 || t == 2 || t == 3)
    {
        const int raw = pd.get(id, 0); // the slot's 32 bits, whichever way it was written
        memcpy(value_bits, &raw, 4);
    }
    else if (t == 4 || t == 5 || t == 6)
    {
        Mat v = pd.get(id, Mat());
        *value_bits = (unsigned)v.w;
        for (int i = 0; i < v.w && i < cap; i++) memcpy(array_bits + i, (const int*)v.data + i, 4);
    }
    else if (t == 7)
    {
        std::string s = pd.get(id, std::string());
        *value_bits = (unsigned)s.size();
        for (int i = 0; i < (int)s.size() && i < cap; i++) array_bits[i] = (unsigned char)s[(size_t)i];
    }
    return t;
}

int ncnn_modelbin_probe(const unsigned char* mem, int w, int type, void* out, size_t* consumed)
{
    const unsigned char* cursor = mem;
    DataReaderFromMemory dr(cursor);
    ModelBinFromDataReader mb(dr);
    Mat m = mb.load(w, type);
    if (consumed) *consumed = (size_t)(cursor - mem);
    if (m.empty()) return 0;
    memcpy(out, m.data, (size_t)w * m.elemsize);
    return (int)m.elemsize;
}

} // extern "C"
