// The layer half of ncnn's C API (src/c_api.h:196-352, src/c_api.cpp:800-1700): parameter dictionaries, model readers,
// layers as tables of function pointers, and custom-layer registration on a net through such tables.  With it the four
// MI355X layers can be plugged into a net from C (or any FFI) exactly the way a C program plugs its own layers into ncnn.
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <vector>

#include "layers/hip_layers.h"
#include "ncnn/layer.h"
#include "ncnn/datareader.h"
#include "ncnn/modelbin.h"
#include "ncnn/net.h"
#include "ncnn/paramdict.h"
#include "ncnn_amd_c_api.h"

using namespace ncnn;

static Layer* L(const ncnn_layer_t layer)
{
    return (Layer*)layer->pthis;
}

// ---- model reader handed to a C layer's load_model: the table points back into the C++ reader --------------------------
static ncnn_mat_t modelbin_load_1d(const ncnn_modelbin_t mb, int w, int type)
{
    return (ncnn_mat_t) new Mat(((const ModelBin*)mb->pthis)->load(w, type));
}
static ncnn_mat_t modelbin_load_2d(const ncnn_modelbin_t mb, int w, int h, int type)
{
    return (ncnn_mat_t) new Mat(((const ModelBin*)mb->pthis)->load(w, h, type));
}
static ncnn_mat_t modelbin_load_3d(const ncnn_modelbin_t mb, int w, int h, int c, int type)
{
    return (ncnn_mat_t) new Mat(((const ModelBin*)mb->pthis)->load(w, h, c, type));
}

// Weights handed over as an array of Mat handles, consumed in order (src/c_api.cpp:1115-1128); the handles are copied
// (refcounted views of the caller's data), so the array itself need not outlive the call.
class OwnedMatArrayModelBin : public ModelBin
{
public:
    OwnedMatArrayModelBin(const ncnn_mat_t* weights, int n) : keep(copy(weights, n)), reader(keep.empty() ? 0 : &keep[0]) {}
    virtual Mat load(int w, int type) const
    {
        return reader.load(w, type);
    }

private:
    static std::vector<Mat> copy(const ncnn_mat_t* weights, int n)
    {
        std::vector<Mat> v((size_t)(n > 0 ? n : 0));
        for (int i = 0; i < n; i++) v[(size_t)i] = *(const Mat*)weights[i];
        return v;
    }
    std::vector<Mat> keep;
    ModelBinFromMatArray reader;
};

// ---- a layer implemented by a table of function pointers (src/c_api.cpp:1152-1232) ------------------------------------
class Layer_c_api : public Layer
{
public:
    explicit Layer_c_api(ncnn_layer_t _layer) : Layer(), layer(_layer)
    {
        // the reference's executor hands a layer an int8 blob as it is (convert_layout, src/net.cpp:344-600, has no int8 cast):
        // a layer behind the table sees here what it would see there
        support_int8_storage = true;
    }

    virtual int load_param(const ParamDict& pd)
    {
        return layer->load_param(layer, (ncnn_paramdict_t)&pd);
    }
    virtual int load_model(const ModelBin& mb)
    {
        struct __ncnn_modelbin_t mb0;
        mb0.pthis = (void*)&mb;
        mb0.load_1d = modelbin_load_1d;
        mb0.load_2d = modelbin_load_2d;
        mb0.load_3d = modelbin_load_3d;
        return layer->load_model(layer, &mb0);
    }
    virtual int create_pipeline(const Option& opt)
    {
        return layer->create_pipeline(layer, (ncnn_option_t)&opt);
    }
    virtual int destroy_pipeline(const Option& opt)
    {
        return layer->destroy_pipeline(layer, (ncnn_option_t)&opt);
    }
    virtual int forward(const std::vector<Mat>& bottom_blobs, std::vector<Mat>& top_blobs, const Option& opt) const
    {
        const int n = (int)bottom_blobs.size(), n2 = (int)top_blobs.size();
        std::vector<ncnn_mat_t> bottoms0((size_t)n), tops0((size_t)n2, (ncnn_mat_t)0);
        for (int i = 0; i < n; i++) bottoms0[(size_t)i] = (ncnn_mat_t)&bottom_blobs[(size_t)i];
        int ret = layer->forward_n(layer, n ? &bottoms0[0] : 0, n, n2 ? &tops0[0] : 0, n2, (ncnn_option_t)&opt);
        for (int i = 0; i < n2; i++)
        {
            if (!tops0[(size_t)i]) continue; // (the reference dereferences a null handle here; a failed forward may leave one)
            top_blobs[(size_t)i] = *(Mat*)tops0[(size_t)i];
            ncnn_mat_destroy(tops0[(size_t)i]);
        }
        return ret;
    }
    virtual int forward(const Mat& bottom_blob, Mat& top_blob, const Option& opt) const
    {
        ncnn_mat_t top0 = 0;
        int ret = layer->forward_1(layer, (ncnn_mat_t)&bottom_blob, &top0, (ncnn_option_t)&opt);
        if (top0)
        {
            top_blob = *(Mat*)top0;
            ncnn_mat_destroy(top0);
        }
        return ret;
    }
    virtual int forward_inplace(std::vector<Mat>& bottom_top_blobs, const Option& opt) const
    {
        const int n = (int)bottom_top_blobs.size();
        std::vector<ncnn_mat_t> blobs0((size_t)n);
        for (int i = 0; i < n; i++) blobs0[(size_t)i] = (ncnn_mat_t)&bottom_top_blobs[(size_t)i];
        return layer->forward_inplace_n(layer, n ? &blobs0[0] : 0, n, (ncnn_option_t)&opt);
    }
    virtual int forward_inplace(Mat& bottom_top_blob, const Option& opt) const
    {
        return layer->forward_inplace_1(layer, (ncnn_mat_t)&bottom_top_blob, (ncnn_option_t)&opt);
    }

    ncnn_layer_t layer;
};

// table entries of ncnn_layer_create(): the base class's own behaviour (what a C layer gets for the calls it leaves alone)
static int base_load_param(ncnn_layer_t layer, const ncnn_paramdict_t pd)
{
    return L(layer)->Layer::load_param(*(const ParamDict*)pd);
}
static int base_load_model(ncnn_layer_t layer, const ncnn_modelbin_t mb)
{
    return L(layer)->Layer::load_model(*(const ModelBin*)mb->pthis);
}
static int base_create_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    return L(layer)->Layer::create_pipeline(*(const Option*)opt);
}
static int base_destroy_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    return L(layer)->Layer::destroy_pipeline(*(const Option*)opt);
}
static int base_forward_1(const ncnn_layer_t layer, const ncnn_mat_t bottom_blob, ncnn_mat_t* top_blob, const ncnn_option_t opt)
{
    Mat top;
    int ret = L(layer)->Layer::forward(*(const Mat*)bottom_blob, top, *(const Option*)opt);
    *top_blob = (ncnn_mat_t) new Mat(top);
    return ret;
}
static int base_forward_n(const ncnn_layer_t layer, const ncnn_mat_t* bottom_blobs, int n, ncnn_mat_t* top_blobs, int n2, const ncnn_option_t opt)
{
    std::vector<Mat> bottoms((size_t)n), tops((size_t)n2);
    for (int i = 0; i < n; i++) bottoms[(size_t)i] = *(const Mat*)bottom_blobs[i];
    int ret = L(layer)->Layer::forward(bottoms, tops, *(const Option*)opt);
    for (int i = 0; i < n2; i++) top_blobs[i] = (ncnn_mat_t) new Mat(tops[(size_t)i]);
    return ret;
}
static int base_forward_inplace_1(const ncnn_layer_t layer, ncnn_mat_t bottom_top_blob, const ncnn_option_t opt)
{
    return L(layer)->Layer::forward_inplace(*(Mat*)bottom_top_blob, *(const Option*)opt);
}
static int base_forward_inplace_n(const ncnn_layer_t layer, ncnn_mat_t* bottom_top_blobs, int n, const ncnn_option_t opt)
{
    std::vector<Mat> blobs((size_t)n);
    for (int i = 0; i < n; i++) blobs[(size_t)i] = *(Mat*)bottom_top_blobs[i];
    int ret = L(layer)->Layer::forward_inplace(blobs, *(const Option*)opt);
    for (int i = 0; i < n; i++) *(Mat*)bottom_top_blobs[i] = blobs[(size_t)i];
    return ret;
}

// table entries of a layer that exists in C++ (ncnn_layer_create_by_type, ncnnhip_layer_create_by_type): its virtuals
static int real_load_param(ncnn_layer_t layer, const ncnn_paramdict_t pd)
{
    return L(layer)->load_param(*(const ParamDict*)pd);
}
static int real_load_model(ncnn_layer_t layer, const ncnn_modelbin_t mb)
{
    return L(layer)->load_model(*(const ModelBin*)mb->pthis);
}
static int real_create_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    return L(layer)->create_pipeline(*(const Option*)opt);
}
static int real_destroy_pipeline(ncnn_layer_t layer, const ncnn_option_t opt)
{
    return L(layer)->destroy_pipeline(*(const Option*)opt);
}
static int real_forward_1(const ncnn_layer_t layer, const ncnn_mat_t bottom_blob, ncnn_mat_t* top_blob, const ncnn_option_t opt)
{
    Mat top;
    int ret = L(layer)->forward(*(const Mat*)bottom_blob, top, *(const Option*)opt);
    *top_blob = (ncnn_mat_t) new Mat(top);
    return ret;
}
static int real_forward_n(const ncnn_layer_t layer, const ncnn_mat_t* bottom_blobs, int n, ncnn_mat_t* top_blobs, int n2, const ncnn_option_t opt)
{
    std::vector<Mat> bottoms((size_t)n), tops((size_t)n2);
    for (int i = 0; i < n; i++) bottoms[(size_t)i] = *(const Mat*)bottom_blobs[i];
    int ret = L(layer)->forward(bottoms, tops, *(const Option*)opt);
    for (int i = 0; i < n2; i++) top_blobs[i] = (ncnn_mat_t) new Mat(tops[(size_t)i]);
    return ret;
}
static int real_forward_inplace_1(const ncnn_layer_t layer, ncnn_mat_t bottom_top_blob, const ncnn_option_t opt)
{
    return L(layer)->forward_inplace(*(Mat*)bottom_top_blob, *(const Option*)opt);
}
static int real_forward_inplace_n(const ncnn_layer_t layer, ncnn_mat_t* bottom_top_blobs, int n, const ncnn_option_t opt)
{
    std::vector<Mat> blobs((size_t)n);
    for (int i = 0; i < n; i++) blobs[(size_t)i] = *(Mat*)bottom_top_blobs[i];
    int ret = L(layer)->forward_inplace(blobs, *(const Option*)opt);
    for (int i = 0; i < n; i++) *(Mat*)bottom_top_blobs[i] = blobs[(size_t)i];
    return ret;
}

static ncnn_layer_t wrap_real_layer(Layer* layer)
{
    if (!layer) return 0;
    ncnn_layer_t h = (ncnn_layer_t)malloc(sizeof(struct __ncnn_layer_t));
    if (!h)
    {
        delete layer;
        return 0;
    }
    h->pthis = (void*)layer;
    h->load_param = real_load_param;
    h->load_model = real_load_model;
    h->create_pipeline = real_create_pipeline;
    h->destroy_pipeline = real_destroy_pipeline;
    h->forward_1 = real_forward_1;
    h->forward_n = real_forward_n;
    h->forward_inplace_1 = real_forward_inplace_1;
    h->forward_inplace_n = real_forward_inplace_n;
    return h;
}

// ---- custom-layer factories of a net: the handle is the Net itself here, so the list lives beside it -------------------
struct CustomLayerFactory
{
    ncnn_layer_creator_t creator;
    ncnn_layer_destroyer_t destroyer;
    void* userdata;
};
static std::mutex g_factory_lock;
static std::map<const Net*, std::vector<CustomLayerFactory*> > g_factories;

static Layer* c_api_layer_creator(void* userdata)
{
    CustomLayerFactory* ud = (CustomLayerFactory*)userdata;
    ncnn_layer_t layer0 = ud->creator(ud->userdata);
    if (!layer0) return 0;
    Layer* layer = (Layer*)layer0->pthis;
    layer->userdata = (void*)layer0;
    return layer; // (its flags are the object's own fields: nothing to copy, src/c_api.cpp:1648-1654 copies them onto itself)
}
static void c_api_layer_destroyer(Layer* layer, void* userdata)
{
    CustomLayerFactory* ud = (CustomLayerFactory*)userdata;
    ud->destroyer((ncnn_layer_t)layer->userdata, ud->userdata);
}

namespace ncnn_amd {
// called by ncnn_net_destroy once the net (and with it every layer the factories made) is gone
void release_custom_layer_factories(const ncnn::Net* net)
{
    std::lock_guard<std::mutex> g(g_factory_lock);
    std::map<const Net*, std::vector<CustomLayerFactory*> >::iterator it = g_factories.find(net);
    if (it == g_factories.end()) return;
    for (size_t i = 0; i < it->second.size(); i++) delete it->second[i];
    g_factories.erase(it);
}
} // namespace ncnn_amd

static CustomLayerFactory* new_factory(ncnn_net_t net, ncnn_layer_creator_t creator, ncnn_layer_destroyer_t destroyer, void* userdata)
{
    CustomLayerFactory* ud = new CustomLayerFactory;
    ud->creator = creator;
    ud->destroyer = destroyer;
    ud->userdata = userdata;
    std::lock_guard<std::mutex> g(g_factory_lock);
    g_factories[(const Net*)net].push_back(ud);
    return ud;
}

extern "C" {

/* paramdict api, src/c_api.cpp:800-843 */
ncnn_paramdict_t ncnn_paramdict_create(void)
{
    return (ncnn_paramdict_t) new ParamDict;
}
void ncnn_paramdict_destroy(ncnn_paramdict_t pd)
{
    delete (ParamDict*)pd;
}
int ncnn_paramdict_get_type(const ncnn_paramdict_t pd, int id)
{
    return ((const ParamDict*)pd)->type(id);
}
int ncnn_paramdict_get_int(const ncnn_paramdict_t pd, int id, int def)
{
    return ((const ParamDict*)pd)->get(id, def);
}
float ncnn_paramdict_get_float(const ncnn_paramdict_t pd, int id, float def)
{
    return ((const ParamDict*)pd)->get(id, def);
}
ncnn_mat_t ncnn_paramdict_get_array(const ncnn_paramdict_t pd, int id, const ncnn_mat_t def)
{
    return (ncnn_mat_t) new Mat(((const ParamDict*)pd)->get(id, def ? *(const Mat*)def : Mat()));
}
void ncnn_paramdict_set_int(ncnn_paramdict_t pd, int id, int i)
{
    ((ParamDict*)pd)->set(id, i);
}
void ncnn_paramdict_set_float(ncnn_paramdict_t pd, int id, float f)
{
    ((ParamDict*)pd)->set(id, f);
}
void ncnn_paramdict_set_array(ncnn_paramdict_t pd, int id, const ncnn_mat_t v)
{
    ((ParamDict*)pd)->set(id, *(const Mat*)v);
}

/* modelbin api, src/c_api.cpp:1115-1134 */
ncnn_modelbin_t ncnn_modelbin_create_from_mat_array(const ncnn_mat_t* weights, int n)
{
    ncnn_modelbin_t mb = (ncnn_modelbin_t)malloc(sizeof(struct __ncnn_modelbin_t));
    if (!mb) return 0;
    mb->pthis = (void*)static_cast<ModelBin*>(new OwnedMatArrayModelBin(weights, n));
    mb->load_1d = modelbin_load_1d;
    mb->load_2d = modelbin_load_2d;
    mb->load_3d = modelbin_load_3d;
    return mb;
}
void ncnn_modelbin_destroy(ncnn_modelbin_t mb)
{
    if (!mb) return;
    delete (ModelBin*)mb->pthis;
    free(mb);
}

/* datareader api, src/c_api.cpp:845-1000.  The table's entries forward to the reader that pthis holds; a C program may
 * replace them (a reader of its own over an asset, a decrypting one).  The loaders below read through the table, so the
 * replaced entries are the ones that run. */
namespace {
class TableDataReader : public DataReader
{
public:
    explicit TableDataReader(ncnn_datareader_t _table) : table(_table) {}
    virtual int scan(const char* format, void* p) const
    {
        return table && table->scan ? table->scan(table, format, p) : 0;
    }
    virtual size_t read(void* buf, size_t size) const
    {
        return table && table->read ? table->read(table, buf, size) : 0;
    }

private:
    ncnn_datareader_t table;
};

int held_reader_scan(ncnn_datareader_t dr, const char* format, void* p)
{
    return ((const DataReader*)dr->pthis)->scan(format, p);
}
size_t held_reader_read(ncnn_datareader_t dr, void* buf, size_t size)
{
    return ((const DataReader*)dr->pthis)->read(buf, size);
}
ncnn_datareader_t table_over(DataReader* held)
{
    ncnn_datareader_t dr = (ncnn_datareader_t)malloc(sizeof(struct __ncnn_datareader_t));
    if (!dr)
    {
        delete held;
        return 0;
    }
    dr->pthis = (void*)held;
    dr->scan = held_reader_scan;
    dr->read = held_reader_read;
    return dr;
}

// a ModelBin that reads through a table for as long as it lives
class TableModelBin : public ModelBin
{
public:
    explicit TableModelBin(ncnn_datareader_t table) : through(table), reader(through) {}
    virtual Mat load(int w, int type) const
    {
        return reader.load(w, type);
    }

private:
    TableDataReader through;
    ModelBinFromDataReader reader;
};
} // namespace

ncnn_datareader_t ncnn_datareader_create(void)
{
    return table_over(new DataReader()); // reads nothing until the caller fills the table in
}
ncnn_datareader_t ncnn_datareader_create_from_stdio(FILE* fp)
{
    return table_over(new DataReaderFromStdio(fp));
}
ncnn_datareader_t ncnn_datareader_create_from_memory(const unsigned char** mem)
{
    if (!mem) return 0;
    return table_over(new DataReaderFromMemory(*mem)); // *mem moves on as bytes are consumed
}
void ncnn_datareader_destroy(ncnn_datareader_t dr)
{
    if (!dr) return;
    delete (DataReader*)dr->pthis;
    free(dr);
}
ncnn_modelbin_t ncnn_modelbin_create_from_datareader(const ncnn_datareader_t dr)
{
    if (!dr) return 0;
    ncnn_modelbin_t mb = (ncnn_modelbin_t)malloc(sizeof(struct __ncnn_modelbin_t));
    if (!mb) return 0;
    mb->pthis = (void*)static_cast<ModelBin*>(new TableModelBin(dr));
    mb->load_1d = modelbin_load_1d;
    mb->load_2d = modelbin_load_2d;
    mb->load_3d = modelbin_load_3d;
    return mb;
}
int ncnn_net_load_param_datareader(ncnn_net_t net, const ncnn_datareader_t dr)
{
    if (!net || !dr) return -1;
    return ((Net*)net)->load_param(TableDataReader(dr));
}
int ncnn_net_load_param_bin_datareader(ncnn_net_t net, const ncnn_datareader_t dr)
{
    if (!net || !dr) return -1;
    return ((Net*)net)->load_param_bin(TableDataReader(dr));
}
int ncnn_net_load_model_datareader(ncnn_net_t net, const ncnn_datareader_t dr)
{
    if (!net || !dr) return -1;
    return ((Net*)net)->load_model(TableDataReader(dr));
}

/* layer api, src/c_api.cpp:1352-1600 */
ncnn_layer_t ncnn_layer_create(void)
{
    ncnn_layer_t layer = (ncnn_layer_t)malloc(sizeof(struct __ncnn_layer_t));
    if (!layer) return 0;
    layer->pthis = (void*)(new Layer_c_api(layer));
    layer->load_param = base_load_param;
    layer->load_model = base_load_model;
    layer->create_pipeline = base_create_pipeline;
    layer->destroy_pipeline = base_destroy_pipeline;
    layer->forward_1 = base_forward_1;
    layer->forward_n = base_forward_n;
    layer->forward_inplace_1 = base_forward_inplace_1;
    layer->forward_inplace_n = base_forward_inplace_n;
    return layer;
}
ncnn_layer_t ncnn_layer_create_by_typeindex(int typeindex)
{
    return wrap_real_layer(create_layer(typeindex));
}
ncnn_layer_t ncnn_layer_create_by_type(const char* type)
{
    return wrap_real_layer(create_layer(type));
}
int ncnn_layer_type_to_index(const char* type)
{
    return layer_to_index(type);
}
ncnn_layer_t ncnnhip_layer_create_by_type(const char* type)
{
    using namespace ncnn_amd;
    Layer* layer = 0;
    if (!type) return 0;
    if (strcmp(type, "Convolution") == 0) layer = Convolution_hip_creator(0);
    else if (strcmp(type, "ConvolutionDepthWise") == 0) layer = ConvolutionDepthWise_hip_creator(0);
    else if (strcmp(type, "InnerProduct") == 0) layer = InnerProduct_hip_creator(0);
    else if (strcmp(type, "Gemm") == 0) layer = Gemm_hip_creator(0);
    else if (strcmp(type, "MultiHeadAttention") == 0) layer = MultiHeadAttention_hip_creator(0);
    if (layer)
    {
        layer->type = type;
        layer->typeindex = layer_to_index(type);
    }
    return wrap_real_layer(layer);
}
void ncnn_layer_destroy(ncnn_layer_t layer)
{
    if (!layer) return;
    delete (Layer*)layer->pthis;
    free(layer);
}

const char* ncnn_layer_get_name(const ncnn_layer_t layer)
{
    return L(layer)->name.c_str();
}
int ncnn_layer_get_typeindex(const ncnn_layer_t layer)
{
    return L(layer)->typeindex;
}
const char* ncnn_layer_get_type(const ncnn_layer_t layer)
{
    return L(layer)->type.c_str();
}

#define NCNN_AMD_LAYER_FLAG(flag)                                     \
    int ncnn_layer_get_##flag(const ncnn_layer_t layer)               \
    {                                                                 \
        return L(layer)->flag;                                        \
    }                                                                 \
    void ncnn_layer_set_##flag(ncnn_layer_t layer, int enable)        \
    {                                                                 \
        L(layer)->flag = enable != 0;                                 \
    }
NCNN_AMD_LAYER_FLAG(one_blob_only)
NCNN_AMD_LAYER_FLAG(support_inplace)
NCNN_AMD_LAYER_FLAG(support_vulkan)
NCNN_AMD_LAYER_FLAG(support_packing)
NCNN_AMD_LAYER_FLAG(support_bf16_storage)
NCNN_AMD_LAYER_FLAG(support_fp16_storage)
NCNN_AMD_LAYER_FLAG(support_vulkan_packing)
NCNN_AMD_LAYER_FLAG(support_any_packing)
NCNN_AMD_LAYER_FLAG(support_vulkan_any_packing)
#undef NCNN_AMD_LAYER_FLAG

int ncnn_layer_get_bottom_count(const ncnn_layer_t layer)
{
    return (int)L(layer)->bottoms.size();
}
int ncnn_layer_get_bottom(const ncnn_layer_t layer, int i)
{
    return L(layer)->bottoms[(size_t)i];
}
int ncnn_layer_get_top_count(const ncnn_layer_t layer)
{
    return (int)L(layer)->tops.size();
}
int ncnn_layer_get_top(const ncnn_layer_t layer, int i)
{
    return L(layer)->tops[(size_t)i];
}
void ncnn_blob_get_bottom_shape(const ncnn_layer_t layer, int i, int* dims, int* w, int* h, int* c)
{
    const std::vector<Mat>& shapes = L(layer)->bottom_shapes;
    const Mat shape = (size_t)i < shapes.size() ? shapes[(size_t)i] : Mat();
    *dims = shape.dims, *w = shape.w, *h = shape.h, *c = shape.c;
}
void ncnn_blob_get_top_shape(const ncnn_layer_t layer, int i, int* dims, int* w, int* h, int* c)
{
    const std::vector<Mat>& shapes = L(layer)->top_shapes;
    const Mat shape = (size_t)i < shapes.size() ? shapes[(size_t)i] : Mat();
    *dims = shape.dims, *w = shape.w, *h = shape.h, *c = shape.c;
}

/* src/c_api.cpp:1665-1686; call before ncnn_net_load_param */
void ncnn_net_register_custom_layer_by_type(ncnn_net_t net, const char* type, ncnn_layer_creator_t creator, ncnn_layer_destroyer_t destroyer, void* userdata)
{
    ((Net*)net)->register_custom_layer(type, c_api_layer_creator, c_api_layer_destroyer, (void*)new_factory(net, creator, destroyer, userdata));
}
void ncnn_net_register_custom_layer_by_typeindex(ncnn_net_t net, int typeindex, ncnn_layer_creator_t creator, ncnn_layer_destroyer_t destroyer, void* userdata)
{
    ((Net*)net)->register_custom_layer(typeindex, c_api_layer_creator, c_api_layer_destroyer, (void*)new_factory(net, creator, destroyer, userdata));
}

} // extern "C"
