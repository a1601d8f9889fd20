#include "net.h"

#include <algorithm>

#include <stdint.h>
#include <string.h>

#include <map>
#include <chrono>
#include <memory>
#include <mutex>
#include <string>

#include "datareader.h"
#include "modelbin.h"
#include "ncnnhip.h"
#include "paramdict.h"

namespace ncnn {

struct CustomEntry
{
    std::string name; // empty for an overwritten built-in
    int typeindex;    // built-in index for an overwrite, -1 otherwise
    layer_creator_func creator;
    layer_destroyer_func destroyer;
    void* userdata;
};

static const int CUSTOM_BIT = 1 << 8; // type indexes of non-built-in custom layers carry this bit

// what one Extractor holds while it runs: every blob as a host Mat, a device HipMat, or both
// One entry per layer that ran, when the Extractor was asked to time its layers (the role of the reference's
// NCNN_BENCHMARK switch, src/net.cpp:145-180): a device layer is bracketed by two events on the command's stream, a host
// layer by the wall clock.
struct LayerTimingSlot
{
    int layer_index;
    void* start;    // events of a device layer (0 for a host layer)
    void* stop;
    double host_ms; // wall clock of a host layer
};

struct ExecState
{
    std::vector<Mat> host;
    std::vector<HipMat> dev;
    std::shared_ptr<HipCommand> cmd; // created on the first layer that runs device-resident
    int wanted;                      // the blob an extract call asked for (-1: none): it is produced as the model defines it
    bool time_layers;
    std::vector<LayerTimingSlot> timing;
    ExecState() : wanted(-1), time_layers(false) {}
    // a copy shares the blobs and the command but starts its own timing record (the events belong to one state)
    ExecState(const ExecState& r) : host(r.host), dev(r.dev), cmd(r.cmd), wanted(r.wanted), time_layers(r.time_layers) {}
    ExecState& operator=(const ExecState& r)
    {
        if (this != &r)
        {
            host = r.host;
            dev = r.dev;
            cmd = r.cmd;
            wanted = r.wanted;
            time_layers = r.time_layers;
            drop_timing();
        }
        return *this;
    }
    ~ExecState()
    {
        drop_timing();
    }
    void drop_timing()
    {
        for (size_t i = 0; i < timing.size(); i++)
        {
            if (timing[i].start) ncnnhip_event_destroy(timing[i].start);
            if (timing[i].stop) ncnnhip_event_destroy(timing[i].stop);
        }
        timing.clear();
    }

    bool has(int blob) const
    {
        return host[(size_t)blob].dims != 0 || !dev[(size_t)blob].empty();
    }
};

class NetPrivate
{
public:
    explicit NetPrivate(Option& _opt) : opt(_opt) {}

    Option& opt;
    std::vector<Blob> blobs;
    std::vector<Layer*> layers;
    std::vector<int> input_idx, output_idx;
    std::vector<const char*> input_nm, output_nm;
    std::vector<CustomEntry> custom;    // new type names
    std::vector<CustomEntry> overwrite; // replaced built-ins

    const CustomEntry* find_overwrite(int typeindex) const
    {
        for (size_t i = 0; i < overwrite.size(); i++)
            if (overwrite[i].typeindex == typeindex) return &overwrite[i];
        return 0;
    }

    Layer* make_layer(const char* type)
    {
        const int builtin = layer_to_index(type);
        Layer* layer = 0;
        if (builtin >= 0)
        {
            if (const CustomEntry* e = find_overwrite(builtin))
            {
                layer = e->creator(e->userdata);
                if (layer) layer->typeindex = builtin;
            }
            else
                layer = create_layer(builtin);
        }
        else
        {
            for (size_t i = 0; i < custom.size() && !layer; i++)
            {
                if (custom[i].name == type && custom[i].creator)
                {
                    layer = custom[i].creator(custom[i].userdata);
                    if (layer) layer->typeindex = CUSTOM_BIT | (int)i;
                }
            }
        }
        return layer;
    }

    // shape hints (id 30: [dims, w, h, c] per top blob), feature mask (id 31), then the layer's own load_param
    int configure_layer(Layer* layer, const ParamDict& pd)
    {
        const int nbottom = (int)layer->bottoms.size(), ntop = (int)layer->tops.size();
        const Mat hints = pd.get(30, Mat());
        if (!hints.empty())
        {
            const int* p = hints;
            int pos = 0;
            for (int j = 0; j < ntop && pos < hints.w; j++)
            {
                const int dims = p[pos];
                if (pos + 4 > hints.w) break;
                Blob& b = blobs[layer->tops[j]];
                Mat s;
                s.dims = dims;
                s.w = p[pos + 1];
                s.h = dims >= 2 ? p[pos + 2] : 1;
                s.c = dims >= 3 ? p[pos + 3] : 1;
                s.d = 1;
                b.shape = s;
                pos += 4;
            }
        }
        layer->bottom_shapes.resize((size_t)nbottom);
        for (int j = 0; j < nbottom; j++) layer->bottom_shapes[j] = blobs[layer->bottoms[j]].shape;
        layer->top_shapes.resize((size_t)ntop);
        for (int j = 0; j < ntop; j++) layer->top_shapes[j] = blobs[layer->tops[j]].shape;
        layer->featmask = pd.get(31, 0);
        return layer->load_param(pd);
    }

    // graph inputs are the tops of Input layers, outputs are blobs nobody consumes
    void index_inputs_and_outputs()
    {
        for (size_t li = 0; li < layers.size(); li++)
            if (layers[li]->type == "Input")
                for (size_t j = 0; j < layers[li]->tops.size(); j++) input_idx.push_back(layers[li]->tops[j]);
        for (size_t bi = 0; bi < blobs.size(); bi++)
            if (blobs[bi].producer >= 0 && blobs[bi].consumer < 0) output_idx.push_back((int)bi);
        for (size_t i = 0; i < input_idx.size(); i++) input_nm.push_back(blobs[input_idx[i]].name.c_str());
        for (size_t i = 0; i < output_idx.size(); i++) output_nm.push_back(blobs[output_idx[i]].name.c_str());
    }

    // a layer by the number a .param.bin file holds: a built-in type (possibly replaced) or a registered custom slot
    Layer* make_layer(int typeindex)
    {
        if (typeindex < 0) return 0;
        if (typeindex & CUSTOM_BIT)
        {
            const size_t i = (size_t)(typeindex & ~CUSTOM_BIT);
            if (i >= custom.size() || !custom[i].creator) return 0;
            Layer* layer = custom[i].creator(custom[i].userdata);
            if (layer)
            {
                layer->typeindex = typeindex;
                layer->type = custom[i].name;
            }
            return layer;
        }
        const char* type = layer_index_to_type(typeindex);
        if (!type) return 0;
        Layer* layer = make_layer(type);
        if (layer) layer->type = type;
        return layer;
    }

    void destroy_layer(Layer* layer)
    {
        const int ti = layer->typeindex;
        const CustomEntry* e = 0;
        if (ti >= 0 && (ti & CUSTOM_BIT))
        {
            const size_t i = (size_t)(ti & ~CUSTOM_BIT);
            if (i < custom.size()) e = &custom[i];
        }
        else if (ti >= 0)
            e = find_overwrite(ti);
        if (e && e->destroyer)
            e->destroyer(layer, e->userdata);
        else
            delete layer;
    }

    // Streams and buffer pools outlive the Extractors that use them: an Extractor takes an idle HipCommand (or a
    // new one) when its first device-resident layer runs and hands it back when it is cleared, so steady-state
    // inference allocates nothing.  Work left in flight by the previous user is ordered before the next user's
    // on the same stream.
    mutable std::mutex cmd_lock;
    mutable std::vector<std::shared_ptr<HipCommand> > idle_cmds;
    mutable std::shared_ptr<HipCommand> io_cmd; // carries blobs uploaded through Net::upload
    mutable std::mutex io_lock;                 // one upload at a time on it (a command's stream and scratch serve one caller)

    std::shared_ptr<HipCommand> acquire_command() const
    {
        std::lock_guard<std::mutex> g(cmd_lock);
        if (!idle_cmds.empty())
        {
            std::shared_ptr<HipCommand> c = idle_cmds.back();
            idle_cmds.pop_back();
            return c;
        }
        return std::shared_ptr<HipCommand>(new HipCommand);
    }
    void recycle_command(const std::shared_ptr<HipCommand>& c) const
    {
        std::lock_guard<std::mutex> g(cmd_lock);
        idle_cmds.push_back(c);
    }

    // ---- epilogue fusion of the device-resident path (built once the model is loaded) --------------------
    // tail_plan[L] for a layer L that is a plain ReLU or a plain two-input sum: the convolution whose epilogue can
    // produce L's output directly.  quantise_scale[b]: the one input scale with which every quantising consumer
    // of blob b (through Split layers) would quantise it, 0 if there is none or they differ.
    struct TailPlan
    {
        int conv;     // layer index, -1: none
        int eltwise;  // the sum layer
        int residual; // blob index of the sum's other input
        bool relu;
    };
    std::vector<TailPlan> tail_plan;
    // sibling_group[L]: the layers (L among them, in layer order) that read outputs of one Split, have equal sibling keys and
    // may therefore run as one launch; empty: none
    std::vector<std::vector<int> > sibling_group;
    int try_siblings(int layer_index, ExecState& st, const Option& opt, bool& done) const;
    std::vector<float> quantise_scale;
    // requant_scale[b] != 0: blob b is produced as int8, float2int8(value * scale), by its layer (a convolution
    // that agreed in hip_prepare_requantise): every consumer, through Split and windowed max pooling, quantises with
    // that one scale.  quantised_zone[b]: b holds such values when the plan is followed (b itself or downstream).
    std::vector<float> requant_scale;
    std::vector<char> quantised_zone;
    void build_fusion_plan();
    bool collect_quantise_scales(int blob, float& scale, bool& any) const;
    bool all_consumers_quantise(int blob, float& scale, bool& any, std::vector<int>& zone) const;
    bool follows_requant_plan(int blob, const ExecState& st, const Option& opt) const;
    int try_fused_tail(int layer_index, ExecState& st, const Option& opt, bool& done) const;

    int forward_layer(int layer_index, ExecState& st, const Option& opt) const;
    int run_layer(const Layer* layer, ExecState& st, const Option& opt) const;
    int run_layer_hip(const Layer* layer, ExecState& st, const Option& opt) const;
};

// int8 blob -> fp32 blob of the same shape (plain value conversion), batch aware
static int expand_int8(const Mat& src, Mat& dst, Allocator* allocator)
{
    if (src.dims == 1)
        dst.create(src.w, 4u, 1, src.n, allocator);
    else if (src.dims == 2)
        dst.create(src.w, src.h, 4u, 1, src.n, allocator);
    else if (src.dims == 3)
        dst.create(src.w, src.h, src.c, 4u, 1, src.n, allocator);
    else
        dst.create(src.w, src.h, src.d, src.c, 4u, 1, src.n, allocator);
    if (dst.empty()) return -100;
    const size_t plane = (size_t)src.w * src.h * src.d;
    for (int b = 0; b < src.n; b++)
        for (int q = 0; q < src.c; q++)
        {
            const signed char* p = (const signed char*)src.data + src.nstep * b + src.cstep * q;
            float* o = (float*)dst.data + dst.nstep * b + dst.cstep * q;
            for (size_t i = 0; i < plane; i++) o[i] = (float)p[i];
        }
    return 0;
}

// ---- fusion plan ----------------------------------------------------------------------------

// walks the consumers of a blob through Split layers; false when two quantising consumers disagree
bool NetPrivate::collect_quantise_scales(int blob, float& scale, bool& any) const
{
    const int ci = blobs[(size_t)blob].consumer;
    if (ci < 0) return true;
    const Layer* consumer = layers[(size_t)ci];
    if (consumer->type == "Split")
    {
        for (size_t i = 0; i < consumer->tops.size(); i++)
            if (!collect_quantise_scales(consumer->tops[i], scale, any)) return false;
        return true;
    }
    const float s = consumer->hip_input_quantise_scale();
    if (s == 0.f) return true; // reads the fp32 values
    if (any && s != scale) return false;
    scale = s;
    any = true;
    return true;
}

// true when every path from the blob ends, through Split and quantise-transparent layers, in a consumer that
// quantises with the same scale; zone collects the blobs on the way
bool NetPrivate::all_consumers_quantise(int blob, float& scale, bool& any, std::vector<int>& zone) const
{
    zone.push_back(blob);
    const int ci = blobs[(size_t)blob].consumer;
    if (ci < 0) return false; // a network output keeps the model's type
    const Layer* consumer = layers[(size_t)ci];
    if (consumer->type == "Split" || (consumer->support_hip && consumer->one_blob_only && consumer->hip_quantise_transparent()))
    {
        for (size_t i = 0; i < consumer->tops.size(); i++)
            if (!all_consumers_quantise(consumer->tops[i], scale, any, zone)) return false;
        return !consumer->tops.empty();
    }
    const float s = consumer->support_hip ? consumer->hip_input_quantise_scale() : 0.f;
    if (!(s > 0.f) || (any && s != scale)) return false;
    scale = s;
    any = true;
    return true;
}

bool NetPrivate::follows_requant_plan(int blob, const ExecState& st, const Option& opt) const
{
    if (!opt.use_hip_compute || !opt.lightmode || requant_scale.size() != blobs.size() || requant_scale[(size_t)blob] == 0.f) return false;
    // an extract call that asks for a blob of this zone gets the model's own fp32 values
    return st.wanted < 0 || !quantised_zone[(size_t)st.wanted];
}

void NetPrivate::build_fusion_plan()
{
    const TailPlan none = {-1, -1, -1, false};
    tail_plan.assign(layers.size(), none);
    quantise_scale.assign(blobs.size(), 0.f);
    requant_scale.assign(blobs.size(), 0.f);
    quantised_zone.assign(blobs.size(), 0);
    for (size_t b = 0; b < blobs.size(); b++)
    {
        const int p = blobs[b].producer;
        if (p < 0 || !layers[(size_t)p]->support_hip || !layers[(size_t)p]->one_blob_only || layers[(size_t)p]->tops.size() != 1) continue;
        float s = 0.f;
        bool any = false;
        std::vector<int> zone;
        if (!all_consumers_quantise((int)b, s, any, zone) || !any) continue;
        if (layers[(size_t)p]->hip_prepare_requantise(s) != 0) continue;
        requant_scale[b] = s;
        for (size_t i = 0; i < zone.size(); i++) quantised_zone[(size_t)zone[i]] = 1;
    }
    for (size_t b = 0; b < blobs.size(); b++)
    {
        float s = 0.f;
        bool any = false;
        if (collect_quantise_scales((int)b, s, any) && any) quantise_scale[b] = s;
    }
    // a sum whose (later) input is a convolution that can take the other input as a residual
    for (size_t li = 0; li < layers.size(); li++)
    {
        const Layer* e = layers[li];
        if (!e->support_hip || !e->hip_plain_sum() || e->bottoms.size() != 2 || e->tops.size() != 1) continue;
        int best = -1, best_slot = -1;
        for (int k = 0; k < 2; k++)
        {
            const int p = blobs[(size_t)e->bottoms[(size_t)k]].producer;
            if (p < 0) continue;
            const Layer* c = layers[(size_t)p];
            if (c->support_hip && c->one_blob_only && c->bottoms.size() == 1 && c->tops.size() == 1 && c->hip_can_fuse_tail() && p > best)
            {
                best = p;
                best_slot = k;
            }
        }
        if (best < 0) continue;
        TailPlan tp = {best, (int)li, e->bottoms[(size_t)(1 - best_slot)], false};
        tail_plan[li] = tp;
        // ... followed by a plain ReLU: that layer's output comes out of the same epilogue
        const int ri = blobs[(size_t)e->tops[0]].consumer;
        if (ri >= 0 && layers[(size_t)ri]->support_hip && layers[(size_t)ri]->hip_plain_relu() && layers[(size_t)ri]->bottoms.size() == 1)
        {
            tp.relu = true;
            tail_plan[(size_t)ri] = tp;
        }
    }
    // layers behind one Split that can share a launch (block-quantised Gemms on the same activation rows)
    sibling_group.assign(layers.size(), std::vector<int>());
    for (size_t li = 0; li < layers.size(); li++)
    {
        const Layer* sp = layers[li];
        if (sp->type != "Split" || sp->tops.size() < 2) continue;
        std::vector<int> members;
        unsigned long long key = 0;
        for (size_t t = 0; t < sp->tops.size(); t++)
        {
            const int ci = blobs[(size_t)sp->tops[t]].consumer;
            if (ci < 0) continue;
            const Layer* c = layers[(size_t)ci];
            if (!c->support_hip || c->featmask || c->bottoms.size() != 1 || c->tops.size() != 1) continue;
            const unsigned long long k = c->hip_sibling_key();
            if (!k) continue;
            if (members.empty()) key = k;
            if (k == key) members.push_back(ci);
        }
        if (members.size() < 2) continue;
        std::sort(members.begin(), members.end());
        for (size_t m = 0; m < members.size(); m++) sibling_group[(size_t)members[m]] = members;
    }
}

// Runs layer_index together with its siblings that have not run yet, as one launch, when their (shared) input is there.
// done = false: not applicable, the caller runs the layer on its own.
int NetPrivate::try_siblings(int layer_index, ExecState& st, const Option& opt, bool& done) const
{
    done = false;
    if (!opt.use_hip_compute || sibling_group.size() != layers.size()) return 0;
    const std::vector<int>& group = sibling_group[(size_t)layer_index];
    if (group.size() < 2) return 0;
    // the members whose output is still missing and whose input exists (all outputs of one Split: the same blob)
    std::vector<const Layer*> run;
    for (size_t m = 0; m < group.size(); m++)
    {
        const Layer* l = layers[(size_t)group[m]];
        if (!st.has(l->tops[0]) && st.has(l->bottoms[0])) run.push_back(l);
    }
    if (run.size() < 2) return 0;
    const Layer* self = layers[(size_t)layer_index];
    if (std::find(run.begin(), run.end(), self) == run.end()) return 0;
    if (!st.cmd) st.cmd = acquire_command();
    HipCommand& cmd = *st.cmd;
    int ret = cmd.ensure_ready();
    if (ret != 0) return ret;
    const size_t b0 = (size_t)run[0]->bottoms[0];
    if (st.dev[b0].empty())
    {
        ret = cmd.upload(st.host[b0], st.dev[b0]);
        if (ret != 0) return ret;
    }
    const HipMat bottom = st.dev[b0];
    // the members' inputs must be the very same device blob (a Split hands one blob to all its outputs)
    for (size_t m = 1; m < run.size(); m++)
    {
        const size_t bi = (size_t)run[m]->bottoms[0];
        if (st.dev[bi].empty() || st.dev[bi].data != bottom.data) return 0;
    }
    std::vector<HipMat> tops(run.size());
    ret = run[0]->forward_hip_siblings(run, bottom, tops, cmd, opt, done);
    if (ret != 0 || !done) return ret;
    for (size_t m = 0; m < run.size(); m++)
    {
        st.dev[(size_t)run[m]->tops[0]] = tops[m];
        st.host[(size_t)run[m]->tops[0]].release();
        if (opt.lightmode)
        {
            st.dev[(size_t)run[m]->bottoms[0]].release();
            st.host[(size_t)run[m]->bottoms[0]].release();
        }
    }
    return 0;
}

// Runs layer_index (a sum, or the ReLU after it) as the epilogue of the convolution in its plan, if nothing on the
// way has been computed yet and the intermediate blobs may be skipped (light mode).  done = false: not applicable,
// the caller runs the layers one by one.
// A layer's featmask (param id 31) switches features off for that layer alone, at create_pipeline and at forward time:
// NetPrivate::forward_layer with get_masked_option, src/net.cpp:100-121,163.  Bit 3 masks the int8 packing / storage /
// arithmetic switches (not use_int8_inference, which the reference never masks); bit 4 masks the GPU path, which here is
// use_hip_compute as well: such a layer sees host Mats.
static Option masked_option(const Option& opt, int featmask)
{
    Option o = opt;
    o.use_fp16_arithmetic = o.use_fp16_arithmetic && !(featmask & (1 << 0));
    o.use_fp16_packed = o.use_fp16_packed && !(featmask & (1 << 1));
    o.use_fp16_storage = o.use_fp16_storage && !(featmask & (1 << 1));
    o.use_bf16_storage = o.use_bf16_storage && !(featmask & (1 << 2));
    o.use_int8_packed = o.use_int8_packed && !(featmask & (1 << 3));
    o.use_int8_storage = o.use_int8_storage && !(featmask & (1 << 3));
    o.use_int8_arithmetic = o.use_int8_arithmetic && !(featmask & (1 << 3));
    o.use_vulkan_compute = o.use_vulkan_compute && !(featmask & (1 << 4));
    o.use_hip_compute = o.use_hip_compute && !(featmask & (1 << 4));
    o.use_sgemm_convolution = o.use_sgemm_convolution && !(featmask & (1 << 5));
    o.use_winograd_convolution = o.use_winograd_convolution && !(featmask & (1 << 6));
    if (featmask & (1 << 7)) o.num_threads = 1;
    return o;
}

int NetPrivate::try_fused_tail(int layer_index, ExecState& st, const Option& opt, bool& done) const
{
    done = false;
    if (!opt.use_hip_compute || !opt.lightmode || tail_plan.size() != layers.size()) return 0;
    const TailPlan& tp = tail_plan[(size_t)layer_index];
    if (tp.conv < 0) return 0;
    const Layer* conv = layers[(size_t)tp.conv];
    const Layer* sum = layers[(size_t)tp.eltwise];
    const Layer* last = layers[(size_t)layer_index];
    if (st.has(conv->tops[0]) || st.has(sum->tops[0])) return 0; // an intermediate exists already (fed or extracted)
    if (conv->featmask || sum->featmask || last->featmask) return 0; // a masked layer runs on its own, under its own options

    const int needed[2] = {conv->bottoms[0], tp.residual};
    for (int k = 0; k < 2; k++)
    {
        const int bi = needed[k];
        if (st.has(bi)) continue;
        const int producer = blobs[(size_t)bi].producer;
        if (producer < 0) return 0;
        int ret = forward_layer(producer, st, opt);
        if (ret != 0) return ret;
        if (!st.has(bi)) return 0;
    }
    if (!st.cmd) st.cmd = acquire_command();
    HipCommand& cmd = *st.cmd;
    int ret = cmd.ensure_ready();
    if (ret != 0) return ret;
    HipMat ins[2];
    for (int k = 0; k < 2; k++)
    {
        const size_t bi = (size_t)needed[k];
        if (st.dev[bi].empty())
        {
            ret = cmd.upload(st.host[bi], st.dev[bi]);
            if (ret != 0) return ret;
        }
        ins[k] = st.dev[bi];
    }
    if (ins[1].elemsize != 4u || ins[1].dims != 3 || ins[1].narrow()) return 0; // the residual must be an ordinary fp32 blob: take the plain route
    for (int k = 0; k < 2; k++)
    {
        st.dev[(size_t)needed[k]].release();
        st.host[(size_t)needed[k]].release();
    }
    HipMat top;
    ret = conv->forward_hip_fused(ins[0], &ins[1], tp.relu, quantise_scale[(size_t)last->tops[0]], top, cmd, opt);
    if (ret != 0) return ret;
    st.dev[(size_t)last->tops[0]] = top;
    st.host[(size_t)last->tops[0]].release();
    done = true;
    return 0;
}

// ---- executor -----------------------------------------------------------------------------

int NetPrivate::forward_layer(int layer_index, ExecState& st, const Option& opt) const
{
    const Layer* layer = layers[layer_index];
    if (layer->bottoms.empty() && layer->type == "Input") return 0; // inputs are fed, not computed

    {
        // (a tail folded into its producer's epilogue is timed as that one launch, under the layer that asked for it)
        LayerTimingSlot slot = {layer_index, 0, 0, 0.0};
        const bool timed = st.time_layers && st.cmd && ncnnhip_event_create(&slot.start) == 0 && ncnnhip_event_create(&slot.stop) == 0 &&
                           ncnnhip_event_record(slot.start, st.cmd->stream) == 0;
        bool done = false;
        int ret = try_fused_tail(layer_index, st, opt, done);
        if (timed && done && ret == 0 && ncnnhip_event_record(slot.stop, st.cmd->stream) == 0)
            st.timing.push_back(slot);
        else
        {
            if (slot.start) ncnnhip_event_destroy(slot.start);
            if (slot.stop) ncnnhip_event_destroy(slot.stop);
        }
        if (ret != 0 || done) return ret;
    }

    // make sure every input exists, computing producers depth-first
    for (size_t i = 0; i < layer->bottoms.size(); i++)
    {
        const int bi = layer->bottoms[i];
        if (!st.has(bi))
        {
            const int producer = blobs[bi].producer;
            if (producer < 0)
            {
                NCNN_LOGE("blob %s has no producer and was not fed", blobs[bi].name.c_str());
                return -1;
            }
            int ret = forward_layer(producer, st, opt);
            if (ret != 0) return ret;
            if (!st.has(bi))
            {
                NCNN_LOGE("blob %s was not produced (missing input?)", blobs[bi].name.c_str());
                return -1;
            }
        }
    }
    const Option lopt = layer->featmask ? masked_option(opt, layer->featmask) : opt;
    const bool on_device = lopt.use_hip_compute && layer->support_hip;
    if (on_device && !st.time_layers)
    {
        // siblings behind one Split that can share a launch (timed runs keep one record per layer and take the plain route)
        bool together = false;
        int ret = try_siblings(layer_index, st, lopt, together);
        if (ret != 0 || together) return ret;
    }
    if (!st.time_layers) return on_device ? run_layer_hip(layer, st, lopt) : run_layer(layer, st, lopt);

    LayerTimingSlot slot = {layer_index, 0, 0, 0.0};
    int ret;
    if (on_device)
    {
        if (!st.cmd) st.cmd = acquire_command();
        ret = st.cmd->ensure_ready();
        if (ret != 0) return ret;
        if (ncnnhip_event_create(&slot.start) != 0 || ncnnhip_event_create(&slot.stop) != 0 || ncnnhip_event_record(slot.start, st.cmd->stream) != 0)
        {
            if (slot.start) ncnnhip_event_destroy(slot.start);
            if (slot.stop) ncnnhip_event_destroy(slot.stop);
            return -1;
        }
        ret = run_layer_hip(layer, st, lopt);
        // a record is kept only when the layer ran and its stop event was recorded: a half-recorded pair could not be
        // read back and would cost the records around it
        if (ret != 0 || ncnnhip_event_record(slot.stop, st.cmd->stream) != 0)
        {
            ncnnhip_event_destroy(slot.start);
            ncnnhip_event_destroy(slot.stop);
            return ret != 0 ? ret : -1;
        }
    }
    else
    {
        const std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
        ret = run_layer(layer, st, lopt);
        slot.host_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        if (ret != 0) return ret;
    }
    st.timing.push_back(slot); // (copied as plain pointers: the state owns the events from here on)
    return ret;
}

// A layer with forward_hip: inputs are made device-resident (uploaded once if they only exist on the host), the
// outputs stay in HBM.  Nothing here waits for the GPU; only an upload out of pageable memory does.
int NetPrivate::run_layer_hip(const Layer* layer, ExecState& st, const Option& opt) const
{
    if (!st.cmd) st.cmd = acquire_command();
    HipCommand& cmd = *st.cmd;
    int ret = cmd.ensure_ready();
    if (ret != 0) return ret;

    std::vector<HipMat> ins(layer->bottoms.size());
    for (size_t i = 0; i < ins.size(); i++)
    {
        const size_t bi = (size_t)layer->bottoms[i];
        if (st.dev[bi].empty())
        {
            ret = cmd.upload(st.host[bi], st.dev[bi]);
            if (ret != 0) return ret;
        }
        ins[i] = st.dev[bi];
        if (opt.lightmode)
        {
            st.dev[bi].release();
            st.host[bi].release();
        }
        if (ins[i].narrow() && !layer->hip_accepts_narrow_input())
        {
            ret = cmd.widen(ins[i], ins[i]);
            if (ret != 0) return ret;
        }
        const bool passes_quantised = ins[i].elemsize == 1u && ins[i].q8_scale > 0.f && layer->one_blob_only && layer->hip_quantise_transparent();
        if (ins[i].elemsize == 1u && !layer->support_int8_storage && !passes_quantised)
        {
            HipMat wide;
            if (ins[i].dims == 3)
                wide.create(ins[i].w, ins[i].h, ins[i].c, 4u, ins[i].n, &cmd);
            else if (ins[i].dims == 2)
                wide.create(ins[i].w, ins[i].h, 4u, ins[i].n, &cmd);
            else
                wide.create(ins[i].w, 4u, ins[i].n, &cmd);
            if (wide.empty()) return -100;
            if (ncnnhip_int8_to_f32((const int8_t*)ins[i].data, (float*)wide.data, ins[i].count(), cmd.stream) != 0)
            {
                NCNN_LOGE("int8 -> fp32 cast failed: %s", ncnnhip_last_error());
                return -1;
            }
            ins[i] = wide;
        }
    }

    if (layer->one_blob_only)
    {
        HipMat top;
        if (layer->support_inplace)
        {
            top = ins[0];
            ins.clear();
            if (!top.exclusive())
            {
                // someone else still reads this blob (a Split sibling, or the table outside light mode)
                HipMat own;
                own.create_like(top, &cmd);
                if (own.empty()) return -100;
                if (ncnnhip_memcpy_d2d(own.data, top.data, top.bytes(), cmd.stream) != 0) return -1;
                top = own;
            }
            ret = layer->forward_inplace_hip(top, cmd, opt);
        }
        else
        {
            const float qs = quantise_scale.size() == blobs.size() ? quantise_scale[(size_t)layer->tops[0]] : 0.f;
            if (follows_requant_plan(layer->tops[0], st, opt))
                ret = layer->forward_hip_requantised(ins[0], requant_scale[(size_t)layer->tops[0]], top, cmd, opt); // only quantised values are wanted
            else if (qs != 0.f && layer->hip_can_fuse_tail())
                ret = layer->forward_hip_fused(ins[0], 0, false, qs, top, cmd, opt); // the consumers' Quantize rides along
            else
                ret = layer->forward_hip(ins[0], top, cmd, opt);
        }
        if (ret != 0) return ret;
        st.dev[(size_t)layer->tops[0]] = top;
        st.host[(size_t)layer->tops[0]].release();
        return 0;
    }

    std::vector<HipMat> outs(layer->tops.size());
    ret = layer->forward_hip(ins, outs, cmd, opt);
    if (ret != 0) return ret;
    for (size_t i = 0; i < outs.size(); i++)
    {
        st.dev[(size_t)layer->tops[i]] = outs[i];
        st.host[(size_t)layer->tops[i]].release();
    }
    return 0;
}

int NetPrivate::run_layer(const Layer* layer, ExecState& st, const Option& opt) const
{
    std::vector<Mat>& blob_mats = st.host;
    // a blob that only exists in HBM comes back to the host for a layer without a device overload
    for (size_t i = 0; i < layer->bottoms.size(); i++)
    {
        const size_t bi = (size_t)layer->bottoms[i];
        if (blob_mats[bi].dims == 0 && !st.dev[bi].empty())
        {
            // (a blob fed with Extractor::input(name, HipMat) may be the first thing this Extractor does on the device)
            if (!st.cmd) st.cmd = acquire_command();
            int ret = st.cmd->download(st.dev[bi], blob_mats[bi], opt.blob_allocator);
            if (ret != 0) return ret;
        }
        if (opt.lightmode) st.dev[bi].release();
    }
    // gather inputs; in light mode a blob is handed over (and dropped from the table) because
    // every blob has exactly one consumer
    std::vector<Mat> ins(layer->bottoms.size());
    for (size_t i = 0; i < ins.size(); i++)
    {
        Mat& slot = blob_mats[layer->bottoms[i]];
        ins[i] = slot;
        if (opt.lightmode) slot.release();
        if (ins[i].elemsize == 1u && !layer->support_int8_storage)
        {
            Mat wide;
            int ret = expand_int8(ins[i], wide, opt.blob_allocator);
            if (ret != 0) return ret;
            ins[i] = wide;
        }
    }

    if (layer->one_blob_only)
    {
        Mat bottom = ins[0];
        ins.clear();
        Mat top;
        const bool loop_samples = bottom.n > 1 && !layer->support_batch;
        if (layer->support_inplace)
        {
            // work on a private copy unless this is the only handle (light mode gave it to us)
            if (!(opt.lightmode && bottom.refcount && *bottom.refcount == 1))
            {
                Mat own = bottom.clone(opt.blob_allocator);
                if (own.empty()) return -100;
                bottom = own;
            }
            if (loop_samples)
            {
                for (int b = 0; b < bottom.n; b++)
                {
                    Mat one = bottom.batch(b);
                    int ret = layer->forward_inplace(one, opt);
                    if (ret != 0) return ret;
                }
            }
            else
            {
                int ret = layer->forward_inplace(bottom, opt);
                if (ret != 0) return ret;
            }
            top = bottom;
        }
        else if (loop_samples)
        {
            // a layer that does not understand batches sees one sample at a time
            for (int b = 0; b < bottom.n; b++)
            {
                Mat one_top;
                int ret = layer->forward(bottom.batch(b), one_top, opt);
                if (ret != 0) return ret;
                if (b == 0)
                {
                    top.create_like(one_top, bottom.n, opt.blob_allocator);
                    if (top.empty()) return -100;
                }
                memcpy((unsigned char*)top.data + top.nstep * b * top.elemsize, one_top.data, one_top.total() * one_top.elemsize);
            }
        }
        else
        {
            int ret = layer->forward(bottom, top, opt);
            if (ret != 0) return ret;
        }
        blob_mats[layer->tops[0]] = top;
        st.dev[(size_t)layer->tops[0]].release();
        return 0;
    }

    std::vector<Mat> outs(layer->tops.size());
    bool any_batch = false;
    for (size_t i = 0; i < ins.size(); i++) any_batch = any_batch || ins[i].n > 1;
    if (any_batch && !layer->support_batch)
    {
        const int B = ins[0].n;
        for (int b = 0; b < B; b++)
        {
            std::vector<Mat> one_in(ins.size()), one_out(outs.size());
            for (size_t i = 0; i < ins.size(); i++) one_in[i] = ins[i].n > 1 ? ins[i].batch(b) : ins[i];
            int ret = layer->forward(one_in, one_out, opt);
            if (ret != 0) return ret;
            for (size_t i = 0; i < outs.size(); i++)
            {
                if (b == 0)
                {
                    outs[i].create_like(one_out[i], B, opt.blob_allocator);
                    if (outs[i].empty()) return -100;
                }
                memcpy((unsigned char*)outs[i].data + outs[i].nstep * b * outs[i].elemsize, one_out[i].data, one_out[i].total() * one_out[i].elemsize);
            }
        }
    }
    else
    {
        int ret = layer->forward(ins, outs, opt);
        if (ret != 0) return ret;
    }
    for (size_t i = 0; i < outs.size(); i++)
    {
        blob_mats[layer->tops[i]] = outs[i];
        st.dev[(size_t)layer->tops[i]].release();
    }
    return 0;
}

// ---- Net ----------------------------------------------------------------------------------

Net::Net() : d(new NetPrivate(opt)) {}

Net::~Net()
{
    clear();
    delete d;
}

int Net::register_custom_layer(const char* type, layer_creator_func creator, layer_destroyer_func destroyer, void* userdata)
{
    const int builtin = layer_to_index(type);
    if (builtin >= 0)
    {
        for (size_t i = 0; i < d->overwrite.size(); i++)
        {
            if (d->overwrite[i].typeindex == builtin)
            {
                NCNN_LOGE("overwrite existing overwritten built-in layer type %s", type);
                d->overwrite[i].creator = creator;
                d->overwrite[i].destroyer = destroyer;
                d->overwrite[i].userdata = userdata;
                return 0;
            }
        }
        CustomEntry e = {std::string(), builtin, creator, destroyer, userdata};
        d->overwrite.push_back(e);
        return 0;
    }
    for (size_t i = 0; i < d->custom.size(); i++)
    {
        if (d->custom[i].name == type)
        {
            NCNN_LOGE("overwrite existing custom layer type %s", type);
            d->custom[i].creator = creator;
            d->custom[i].destroyer = destroyer;
            d->custom[i].userdata = userdata;
            return 0;
        }
    }
    CustomEntry e = {std::string(type), -1, creator, destroyer, userdata};
    d->custom.push_back(e);
    return 0;
}

int Net::register_custom_layer(int index, layer_creator_func creator, layer_destroyer_func destroyer, void* userdata)
{
    if (index < 0) return -1;
    if (!(index & CUSTOM_BIT))
    {
        for (size_t i = 0; i < d->overwrite.size(); i++)
        {
            if (d->overwrite[i].typeindex == index)
            {
                d->overwrite[i].creator = creator;
                d->overwrite[i].destroyer = destroyer;
                d->overwrite[i].userdata = userdata;
                return 0;
            }
        }
        CustomEntry e = {std::string(), index, creator, destroyer, userdata};
        d->overwrite.push_back(e);
        return 0;
    }
    const size_t slot = (size_t)(index & ~CUSTOM_BIT);
    if (d->custom.size() <= slot)
    {
        CustomEntry empty = {std::string(), -1, 0, 0, 0};
        d->custom.resize(slot + 1, empty);
    }
    d->custom[slot].creator = creator;
    d->custom[slot].destroyer = destroyer;
    d->custom[slot].userdata = userdata;
    return 0;
}

int Net::custom_layer_to_index(const char* type)
{
    for (size_t i = 0; i < d->custom.size(); i++)
        if (d->custom[i].name == type) return (int)i;
    return -1;
}

int Net::load_param(const DataReader& dr)
{
    int magic = 0;
    if (dr.scan("%d", &magic) != 1)
    {
        NCNN_LOGE("parse magic failed");
        return -1;
    }
    if (magic != 7767517)
    {
        NCNN_LOGE("param is too old, please regenerate");
        return -1;
    }
    int layer_count = 0, blob_count = 0;
    // (counts are bounded so that a damaged file gives an error instead of an allocation of gigabytes)
    if (dr.scan("%d", &layer_count) != 1 || dr.scan("%d", &blob_count) != 1 || layer_count <= 0 || blob_count <= 0 || layer_count > (1 << 24) ||
        blob_count > (1 << 24))
    {
        NCNN_LOGE("invalid layer_count or blob_count");
        return -1;
    }

    d->layers.assign((size_t)layer_count, (Layer*)0);
    d->blobs.assign((size_t)blob_count, Blob());
    std::map<std::string, int> blob_of;
    ParamDict pd;

    for (int li = 0; li < layer_count; li++)
    {
        char type[256], name[256];
        int nbottom = 0, ntop = 0;
        if (dr.scan("%255s", type) != 1 || dr.scan("%255s", name) != 1 || dr.scan("%d", &nbottom) != 1 || dr.scan("%d", &ntop) != 1)
        {
            NCNN_LOGE("parse layer header failed at layer %d", li);
            clear();
            return -1;
        }
        if (nbottom < 0 || ntop < 0 || nbottom > blob_count || ntop > blob_count)
        {
            NCNN_LOGE("layer %d %s: %d bottom and %d top blobs in a net of %d blobs", li, name, nbottom, ntop, blob_count);
            clear();
            return -1;
        }
        Layer* layer = d->make_layer(type);
        if (!layer)
        {
            NCNN_LOGE("layer %s not exists or registered", type);
            clear();
            return -1;
        }
        layer->type = type;
        layer->name = name;
        d->layers[li] = layer;

        layer->bottoms.resize((size_t)nbottom);
        for (int j = 0; j < nbottom; j++)
        {
            char bname[256];
            if (dr.scan("%255s", bname) != 1)
            {
                NCNN_LOGE("parse bottom_name failed");
                clear();
                return -1;
            }
            std::map<std::string, int>::iterator it = blob_of.find(bname);
            int bi;
            if (it == blob_of.end())
            {
                bi = (int)blob_of.size();
                if (bi >= blob_count)
                {
                    NCNN_LOGE("more blobs than declared (%d)", blob_count);
                    clear();
                    return -1;
                }
                blob_of[bname] = bi;
                d->blobs[bi].name = bname;
            }
            else
                bi = it->second;
            d->blobs[bi].consumer = li;
            layer->bottoms[j] = bi;
        }
        layer->tops.resize((size_t)ntop);
        for (int j = 0; j < ntop; j++)
        {
            char bname[256];
            if (dr.scan("%255s", bname) != 1)
            {
                NCNN_LOGE("parse blob_name failed");
                clear();
                return -1;
            }
            int bi;
            std::map<std::string, int>::iterator it = blob_of.find(bname);
            if (it == blob_of.end())
            {
                bi = (int)blob_of.size();
                if (bi >= blob_count)
                {
                    NCNN_LOGE("more blobs than declared (%d)", blob_count);
                    clear();
                    return -1;
                }
                blob_of[bname] = bi;
                d->blobs[bi].name = bname;
            }
            else
                bi = it->second;
            d->blobs[bi].producer = li;
            layer->tops[j] = bi;
        }

        if (pd.load_param(dr) != 0)
        {
            // a parameter line that cannot be read ends the load, as in the reference (src/net.cpp:1477-1484): going on would leave
            // a layer whose load_param never ran
            NCNN_LOGE("ParamDict load_param %d %s failed", li, name);
            clear();
            return -1;
        }

        if (d->configure_layer(layer, pd) != 0)
        {
            NCNN_LOGE("layer load_param %d %s failed", li, name);
            clear();
            return -1;
        }
    }
    d->index_inputs_and_outputs();
    return 0;
}

// The binary form of the .param text (src/net.cpp:1667-2018; tools/ncnn2mem.cpp writes it): 32-bit little-endian words, no
// names.  magic, layer count, blob count; per layer its type number, bottom count, top count, the blob numbers, and the
// parameters as ParamDict::load_param_bin reads them.  Layers and blobs are then known by number (the .id.h file that
// ncnn2mem writes beside it holds the numbers); a layer also gets the name of its type, which the executor reads.
int Net::load_param_bin(const DataReader& dr)
{
    int head[3] = {0, 0, 0};
    if (dr.read(head, sizeof(head)) != sizeof(head))
    {
        NCNN_LOGE("read magic and counts failed");
        return -1;
    }
    if (head[0] != 7767517)
    {
        NCNN_LOGE("param is too old, please regenerate");
        return -1;
    }
    const int layer_count = head[1], blob_count = head[2];
    if (layer_count <= 0 || blob_count <= 0 || layer_count > (1 << 24) || blob_count > (1 << 24))
    {
        NCNN_LOGE("invalid layer_count or blob_count");
        return -1;
    }
    d->layers.assign((size_t)layer_count, (Layer*)0);
    d->blobs.assign((size_t)blob_count, Blob());
    ParamDict pd;
    for (int li = 0; li < layer_count; li++)
    {
        int lh[3] = {0, 0, 0}; // type number, bottom count, top count
        if (dr.read(lh, sizeof(lh)) != sizeof(lh) || lh[1] < 0 || lh[2] < 0 || lh[1] > blob_count || lh[2] > blob_count)
        {
            NCNN_LOGE("read layer header failed at layer %d", li);
            clear();
            return -1;
        }
        Layer* layer = d->make_layer(lh[0]);
        if (!layer)
        {
            NCNN_LOGE("layer %d not exists or registered", lh[0]);
            clear();
            return -1;
        }
        d->layers[li] = layer;
        layer->bottoms.resize((size_t)lh[1]);
        layer->tops.resize((size_t)lh[2]);
        for (int j = 0; j < lh[1] + lh[2]; j++)
        {
            int bi = -1;
            if (dr.read(&bi, 4) != 4 || bi < 0 || bi >= blob_count)
            {
                NCNN_LOGE("layer %d: blob number %d in a net of %d blobs", li, bi, blob_count);
                clear();
                return -1;
            }
            if (j < lh[1])
            {
                d->blobs[bi].consumer = li;
                layer->bottoms[j] = bi;
            }
            else
            {
                d->blobs[bi].producer = li;
                layer->tops[j - lh[1]] = bi;
            }
        }
        if (pd.load_param_bin(dr) != 0)
        {
            NCNN_LOGE("ParamDict load_param_bin %d failed", li);
            clear();
            return -1;
        }
        if (d->configure_layer(layer, pd) != 0)
        {
            NCNN_LOGE("layer load_param %d failed", li);
            clear();
            return -1;
        }
    }
    // the reference leaves layers and blobs of such a net without names; here each is named by its number in decimal, so that
    // the entry points that take a name (the device-resident ones among them) reach it too
    for (int li = 0; li < layer_count; li++) d->layers[li]->name = std::to_string(li);
    for (int bi = 0; bi < blob_count; bi++) d->blobs[bi].name = std::to_string(bi);
    d->index_inputs_and_outputs();
    return 0;
}

int Net::load_param_bin(FILE* fp)
{
    DataReaderFromStdio dr(fp);
    return load_param_bin(dr);
}

int Net::load_param_bin(const char* protopath)
{
    FILE* fp = fopen(protopath, "rb");
    if (!fp)
    {
        NCNN_LOGE("fopen %s failed", protopath);
        return -1;
    }
    int ret = load_param_bin(fp);
    fclose(fp);
    return ret;
}

size_t Net::load_param_bin_mem(const unsigned char* mem)
{
    const unsigned char* cursor = mem;
    DataReaderFromMemory dr(cursor);
    if (load_param_bin(dr) != 0) return 0;
    return (size_t)(cursor - mem);
}

int Net::load_param(FILE* fp)
{
    DataReaderFromStdio dr(fp);
    return load_param(dr);
}

int Net::load_param(const char* protopath)
{
    FILE* fp = fopen(protopath, "rb");
    if (!fp)
    {
        NCNN_LOGE("fopen %s failed", protopath);
        return -1;
    }
    int ret = load_param(fp);
    fclose(fp);
    return ret;
}

int Net::load_param_mem(const char* mem)
{
    const unsigned char* cursor = (const unsigned char*)mem;
    DataReaderFromMemory dr(cursor);
    return load_param(dr);
}

int Net::load_model(const DataReader& dr)
{
    if (d->layers.empty())
    {
        NCNN_LOGE("network graph not ready");
        return -1;
    }
    ModelBinFromDataReader mb(dr);
    int status = 0;
    for (size_t i = 0; i < d->layers.size(); i++)
    {
        Layer* layer = d->layers[i];
        if (!layer)
        {
            NCNN_LOGE("load_model error at layer %d, parameter file has inconsistent content.", (int)i);
            status = -1;
            break;
        }
        int ret = layer->load_model(mb);
        if (ret != 0)
        {
            NCNN_LOGE("layer load_model %d %s failed", (int)i, layer->name.c_str());
            status = -1;
            break;
        }
        ret = layer->create_pipeline(layer->featmask ? masked_option(opt, layer->featmask) : opt);
        if (ret != 0)
        {
            NCNN_LOGE("layer create_pipeline %d %s failed", (int)i, layer->name.c_str());
            status = -1;
            break;
        }
    }
    if (status == 0) d->build_fusion_plan();
    return status;
}

int Net::load_model(FILE* fp)
{
    DataReaderFromStdio dr(fp);
    return load_model(dr);
}

int Net::load_model(const char* modelpath)
{
    FILE* fp = fopen(modelpath, "rb");
    if (!fp)
    {
        NCNN_LOGE("fopen %s failed", modelpath);
        return -1;
    }
    int ret = load_model(fp);
    fclose(fp);
    return ret;
}

size_t Net::load_model(const unsigned char* mem)
{
    const unsigned char* cursor = mem;
    DataReaderFromMemory dr(cursor);
    load_model(dr);
    return (size_t)(cursor - mem);
}

void Net::clear()
{
    for (size_t i = 0; i < d->layers.size(); i++)
    {
        Layer* layer = d->layers[i];
        if (!layer) continue;
        if (layer->destroy_pipeline(opt) != 0) NCNN_LOGE("layer destroy_pipeline failed");
        d->destroy_layer(layer);
    }
    d->layers.clear();
    d->blobs.clear();
    d->input_idx.clear();
    d->output_idx.clear();
    d->input_nm.clear();
    d->output_nm.clear();
    d->tail_plan.clear();
    d->sibling_group.clear();
    d->quantise_scale.clear();
    d->requant_scale.clear();
    d->quantised_zone.clear();
    std::lock_guard<std::mutex> g(d->cmd_lock);
    d->idle_cmds.clear();
    d->io_cmd.reset();
}

Extractor Net::create_extractor() const
{
    return Extractor(this, d->blobs.size());
}

int Net::upload(const Mat& src, HipMat& dst) const
{
    {
        std::lock_guard<std::mutex> g(d->cmd_lock);
        if (!d->io_cmd) d->io_cmd.reset(new HipCommand(true)); // its blobs are read on the Extractors' streams
    }
    std::lock_guard<std::mutex> g(d->io_lock);
    return d->io_cmd->upload(src, dst);
}

const std::vector<int>& Net::input_indexes() const
{
    return d->input_idx;
}
const std::vector<int>& Net::output_indexes() const
{
    return d->output_idx;
}
const std::vector<const char*>& Net::input_names() const
{
    return d->input_nm;
}
const std::vector<const char*>& Net::output_names() const
{
    return d->output_nm;
}
const std::vector<Blob>& Net::blobs() const
{
    return d->blobs;
}
const std::vector<Layer*>& Net::layers() const
{
    return d->layers;
}

int Net::find_blob_index_by_name(const char* name) const
{
    for (size_t i = 0; i < d->blobs.size(); i++)
        if (d->blobs[i].name == name) return (int)i;
    NCNN_LOGE("find_blob_index_by_name %s failed", name);
    return -1;
}

int Net::find_layer_index_by_name(const char* name) const
{
    for (size_t i = 0; i < d->layers.size(); i++)
        if (d->layers[i]->name == name) return (int)i;
    NCNN_LOGE("find_layer_index_by_name %s failed", name);
    return -1;
}

// ---- Extractor ----------------------------------------------------------------------------

class ExtractorPrivate
{
public:
    const Net* net;
    ExecState st;
    Option opt;
};

Extractor::Extractor(const Net* net, size_t blob_count) : d(new ExtractorPrivate)
{
    d->net = net;
    d->st.host.resize(blob_count);
    d->st.dev.resize(blob_count);
    d->opt = net->opt;
}

Extractor::~Extractor()
{
    clear();
    delete d;
}

Extractor::Extractor(const Extractor& rhs) : d(new ExtractorPrivate)
{
    *d = *rhs.d;
}

Extractor& Extractor::operator=(const Extractor& rhs)
{
    if (this != &rhs) *d = *rhs.d;
    return *this;
}

void Extractor::clear()
{
    d->st.host.clear();
    d->st.dev.clear(); // device blobs return to the command's pool before the command itself moves on
    if (d->st.cmd && d->st.cmd.use_count() == 1) d->net->d->recycle_command(d->st.cmd);
    d->st.cmd.reset();
}
void Extractor::set_light_mode(bool enable)
{
    d->opt.lightmode = enable;
}
void Extractor::set_num_threads(int num_threads)
{
    d->opt.num_threads = num_threads;
}
void Extractor::set_blob_allocator(Allocator* allocator)
{
    d->opt.blob_allocator = allocator;
}
void Extractor::set_workspace_allocator(Allocator* allocator)
{
    d->opt.workspace_allocator = allocator;
}

int Extractor::input(const char* blob_name, const Mat& in)
{
    const int bi = d->net->find_blob_index_by_name(blob_name);
    if (bi < 0) return -1;
    return input(bi, in);
}

int Extractor::input(int blob_index, const Mat& in)
{
    if (blob_index < 0 || blob_index >= (int)d->st.host.size()) return -1;
    d->st.host[(size_t)blob_index] = in;
    d->st.dev[(size_t)blob_index].release();
    return 0;
}

int Extractor::input(const char* blob_name, const HipMat& in)
{
    const int bi = d->net->find_blob_index_by_name(blob_name);
    if (bi < 0) return -1;
    return input(bi, in);
}

int Extractor::input(int blob_index, const HipMat& in)
{
    if (blob_index < 0 || blob_index >= (int)d->st.dev.size()) return -1;
    d->st.dev[(size_t)blob_index] = in;
    d->st.host[(size_t)blob_index].release();
    return 0;
}

int Extractor::extract(const char* blob_name, HipMat& feat)
{
    const int bi = d->net->find_blob_index_by_name(blob_name);
    if (bi < 0) return -1;
    return extract(bi, feat);
}

int Extractor::extract(int blob_index, HipMat& feat)
{
    if (blob_index < 0 || blob_index >= (int)d->st.dev.size()) return -1;
    const size_t bi = (size_t)blob_index;
    int ret = 0;
    // quantised stand-in values (see requant_scale) are not what the model defines for this blob: compute it again
    if (!d->st.dev[bi].empty() && d->st.dev[bi].elemsize == 1u && d->st.dev[bi].q8_scale != 0.f)
    {
        d->st.dev[bi].release();
        d->st.host[bi].release();
    }
    if (!d->st.has(blob_index))
    {
        const int producer = d->net->d->blobs[bi].producer;
        if (producer < 0) return -1;
        d->st.wanted = blob_index;
        ret = d->net->d->forward_layer(producer, d->st, d->opt);
        d->st.wanted = -1;
    }
    if (ret == 0 && d->st.dev[bi].empty())
    {
        // produced by a layer without a device overload
        if (!d->st.cmd) d->st.cmd = d->net->d->acquire_command();
        ret = d->st.cmd->upload(d->st.host[bi], d->st.dev[bi]);
    }
    feat = d->st.dev[bi];
    return ret;
}

int Extractor::synchronize()
{
    return d->st.cmd ? d->st.cmd->synchronize() : 0;
}

void Extractor::set_layer_timing(bool enable)
{
    d->st.time_layers = enable;
    if (!enable) d->st.drop_timing();
}

int Extractor::layer_timing(std::vector<LayerTime>& out)
{
    out.clear();
    if (d->st.cmd)
    {
        int ret = d->st.cmd->synchronize();
        if (ret != 0) return ret;
    }
    const std::vector<Layer*>& layers = d->net->d->layers;
    for (size_t i = 0; i < d->st.timing.size(); i++)
    {
        const LayerTimingSlot& s = d->st.timing[i];
        LayerTime t;
        t.layer_index = s.layer_index;
        t.name = layers[(size_t)s.layer_index]->name;
        t.type = layers[(size_t)s.layer_index]->type;
        t.on_device = s.start != 0;
        t.ms = s.host_ms;
        if (s.start)
        {
            // a pair that cannot be read (recorded while the stream was being captured into a graph) is reported as
            // -1 ms; the other records stay valid
            float ms = 0.f;
            t.ms = ncnnhip_event_elapsed_ms(s.start, s.stop, &ms) == 0 ? ms : -1.0;
        }
        out.push_back(t);
    }
    return 0;
}

int Extractor::extract(const char* blob_name, Mat& feat, int type)
{
    const int bi = d->net->find_blob_index_by_name(blob_name);
    if (bi < 0) return -1;
    return extract(bi, feat, type);
}

int Extractor::extract(int blob_index, Mat& feat, int type)
{
    if (blob_index < 0 || blob_index >= (int)d->st.host.size()) return -1;
    const size_t bi = (size_t)blob_index;
    int ret = 0;
    // quantised stand-in values (see requant_scale) are not what the model defines for this blob: compute it again
    if (!d->st.dev[bi].empty() && d->st.dev[bi].elemsize == 1u && d->st.dev[bi].q8_scale != 0.f)
    {
        d->st.dev[bi].release();
        d->st.host[bi].release();
    }
    if (!d->st.has(blob_index))
    {
        const int producer = d->net->d->blobs[bi].producer;
        if (producer < 0) return -1;
        d->st.wanted = blob_index;
        ret = d->net->d->forward_layer(producer, d->st, d->opt);
        d->st.wanted = -1;
    }
    if (ret == 0 && d->st.host[bi].dims == 0 && !d->st.dev[bi].empty())
    {
        if (!d->st.cmd) d->st.cmd = d->net->d->acquire_command(); // the blob was fed as a HipMat and nothing ran yet
        ret = d->st.cmd->download(d->st.dev[bi], d->st.host[bi], d->opt.blob_allocator); // waits for the stream
    }
    feat = d->st.host[bi];
    if (ret == 0 && type == 0 && feat.elemsize == 1u && !feat.empty())
    {
        Mat wide;
        ret = expand_int8(feat, wide, d->opt.blob_allocator);
        if (ret == 0) feat = wide;
    }
    return ret;
}

// ---- HipGraph --------------------------------------------------------------------------------

class HipGraphPrivate
{
public:
    HipGraphPrivate() : exec(0) {}
    std::shared_ptr<HipCommand> cmd; // this graph's alone while it lives: its pool holds the recorded buffers
    void* exec;
    HipMat input, output;
};

HipGraph::HipGraph() : d(new HipGraphPrivate) {}

HipGraph::~HipGraph()
{
    clear();
    delete d;
}

void HipGraph::clear()
{
    if (d->cmd) d->cmd->synchronize();
    if (d->exec) ncnnhip_graph_destroy(d->exec);
    d->exec = 0;
    d->output.release();
    d->input.release();
    d->cmd.reset(); // not handed back to the net: the net may be gone
}

int HipGraph::record(const Net& net, const char* input_name, const HipMat& input, const char* output_name)
{
    clear();
    if (!net.opt.use_hip_compute || !net.opt.lightmode)
    {
        NCNN_LOGE("HipGraph::record: needs a net with use_hip_compute and lightmode");
        return -1;
    }
    if (input.empty() || net.find_blob_index_by_name(input_name) < 0 || net.find_blob_index_by_name(output_name) < 0) return -1;
    std::shared_ptr<HipCommand> cmd = net.d->acquire_command();
    int ret = cmd->ensure_ready();
    if (ret != 0) return ret;
    // Plain passes first: every pool buffer, workspace and lazily created table exists afterwards, so the recorded pass
    // allocates nothing.  One pass is not enough: it starts on an empty pool and gives every request a buffer of its own
    // size, while the recorded pass starts with all of those idle and may hand an early request a buffer that a later,
    // smaller one had made -- whose own request then finds only buffers the pool holds too wasteful for it and would
    // allocate, which a stream under capture cannot.  So passes are repeated until one adds nothing to the pool; the
    // recorded pass starts from the same state as that one (everything idle) and takes the same buffers.
    size_t pooled = 0;
    for (int pass = 0; pass < 8 && ret == 0; pass++)
    {
        {
            Extractor ex = net.create_extractor();
            ex.d->st.cmd = cmd;
            HipMat warm;
            ret = ex.input(input_name, input);
            if (ret == 0) ret = ex.extract(output_name, warm);
            if (ret == 0) ret = cmd->synchronize();
        }
        const size_t now = cmd->pooled_bytes();
        if (pass > 0 && now == pooled) break;
        pooled = now;
    }
    if (ret != 0) return ret;
    if (ncnnhip_stream_begin_capture(cmd->stream) != 0)
    {
        NCNN_LOGE("HipGraph::record: %s", ncnnhip_last_error());
        return -1;
    }
    HipMat out;
    {
        Extractor ex = net.create_extractor();
        ex.d->st.cmd = cmd;
        ret = ex.input(input_name, input);
        if (ret == 0) ret = ex.extract(output_name, out);
    }
    void* exec = 0;
    const int rc = ncnnhip_stream_end_capture(cmd->stream, &exec); // also when the pass failed: the stream must leave capture mode
    if (ret == 0 && rc != 0)
    {
        NCNN_LOGE("HipGraph::record: %s (a layer without a device overload on the way?)", ncnnhip_last_error());
        ret = -1;
    }
    if (ret != 0)
    {
        if (exec) ncnnhip_graph_destroy(exec);
        return ret;
    }
    d->cmd = cmd;
    d->exec = exec;
    d->input = input;
    d->output = out;
    return 0;
}

int HipGraph::update_input(const Mat& src)
{
    if (!d->exec) return -1;
    return d->cmd->upload_into(src, d->input);
}

int HipGraph::launch()
{
    if (!d->exec) return -1;
    if (ncnnhip_graph_launch(d->exec, d->cmd->stream) != 0)
    {
        NCNN_LOGE("HipGraph::launch: %s", ncnnhip_last_error());
        return -1;
    }
    return 0;
}

int HipGraph::synchronize()
{
    return d->cmd ? d->cmd->synchronize() : 0;
}

const HipMat& HipGraph::output() const
{
    return d->output;
}

} // namespace ncnn
