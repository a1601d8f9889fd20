// Net and Extractor: the caller-facing API that stays unchanged around the int8 layers
// (public surface of src/net.h that the path uses; Vulkan and platform loaders left out).
#ifndef NCNN_NET_H
#define NCNN_NET_H

#include <stdio.h>

#include <string>
#include <vector>

#include "blob.h"
#include "layer.h"
#include "mat.h"
#include "option.h"
#include "platform.h"

namespace ncnn {

class DataReader;
class Extractor;
class NetPrivate;
class NCNN_EXPORT Net
{
public:
    Net();
    virtual ~Net();

    Option opt;

    // A built-in type name replaces that built-in (the route the HIP layers take); any other name
    // adds a new type.  Must be called before load_param.
    int register_custom_layer(const char* type, layer_creator_func creator, layer_destroyer_func destroyer = 0, void* userdata = 0);
    int register_custom_layer(int index, layer_creator_func creator, layer_destroyer_func destroyer = 0, void* userdata = 0);
    virtual int custom_layer_to_index(const char* type);

    int load_param(const DataReader& dr);
    int load_param(FILE* fp);
    int load_param(const char* protopath);
    int load_param_mem(const char* mem);
    // the binary form (32-bit words, layers and blobs by number)
    int load_param_bin(const DataReader& dr);
    int load_param_bin(FILE* fp);
    int load_param_bin(const char* protopath);
    size_t load_param_bin_mem(const unsigned char* mem); // bytes consumed, 0 on failure

    int load_model(const DataReader& dr);
    int load_model(FILE* fp);
    int load_model(const char* modelpath);
    size_t load_model(const unsigned char* mem); // bytes consumed

    void clear();

    Extractor create_extractor() const;

    // host Mat -> device-resident blob that any Extractor of this net accepts as an input (the copy has completed
    // on return).  The blob's memory belongs to the net: release it before the net is cleared or destroyed.
    int upload(const Mat& src, HipMat& dst) const;

    const std::vector<int>& input_indexes() const;
    const std::vector<int>& output_indexes() const;
    const std::vector<const char*>& input_names() const;
    const std::vector<const char*>& output_names() const;
    const std::vector<Blob>& blobs() const;
    const std::vector<Layer*>& layers() const;

protected:
    friend class Extractor;
    friend class HipGraph;
    int find_blob_index_by_name(const char* name) const;
    int find_layer_index_by_name(const char* name) const;

private:
    Net(const Net&);
    Net& operator=(const Net&);
    NetPrivate* const d;
};

class ExtractorPrivate;
class NCNN_EXPORT Extractor
{
public:
    virtual ~Extractor();
    Extractor(const Extractor&);
    Extractor& operator=(const Extractor&);

    void clear();
    void set_light_mode(bool enable);
    void set_num_threads(int num_threads);
    void set_blob_allocator(Allocator* allocator);
    void set_workspace_allocator(Allocator* allocator);

    int input(const char* blob_name, const Mat& in);
    int input(int blob_index, const Mat& in);
    // type 0: int8 results are expanded to fp32; type 1: returned as stored
    int extract(const char* blob_name, Mat& feat, int type = 0);
    int extract(int blob_index, Mat& feat, int type = 0);

    // device-resident ends of the pipeline (the VkMat overloads of src/net.h:226-239): a blob that is already in
    // HBM goes in without a copy; extract enqueues the work and hands back the blob where it lies, without waiting.
    // synchronize() waits for everything this Extractor has enqueued.
    int input(const char* blob_name, const HipMat& in);
    int input(int blob_index, const HipMat& in);
    int extract(const char* blob_name, HipMat& feat);
    int extract(int blob_index, HipMat& feat);
    int synchronize();

    // Per-layer timing (what the reference prints under its NCNN_BENCHMARK build switch, src/net.cpp:145-180, a run-time
    // switch here): while enabled every layer this Extractor runs is recorded, device layers between two events on the
    // Extractor's stream, host layers by the wall clock.  layer_timing() waits for the stream and returns the records in
    // execution order; a layer folded into its producer's epilogue appears as that one launch.
    struct LayerTime
    {
        int layer_index;
        std::string name, type;
        bool on_device;
        double ms;
    };
    void set_layer_timing(bool enable);
    int layer_timing(std::vector<LayerTime>& out);

protected:
    friend Extractor Net::create_extractor() const;
    friend class HipGraph;
    Extractor(const Net* net, size_t blob_count);

private:
    ExtractorPrivate* const d;
};

// One forward pass of a device-resident net, recorded once and replayed with a single launch: at batch 1 a pass is
// dozens of kernels of a few microseconds each and the host cannot describe them as fast as the GPU runs them.  The
// reference's GPU path has the same split between recording and submitting (VkCompute, src/command.h:22-67).
//   HipGraph g;  g.record(net, "data", in_dev, "prob");        // runs the pass once, then records it
//   g.update_input(host_mat);  g.launch();  g.synchronize();   // any number of times
//   g.output()                                                  // the result blob, rewritten by every launch
// The recording reads the input blob's buffer and owns every buffer in between, so: one launch at a time per graph,
// take what you need from output() before the next launch, and keep the net loaded while the graph lives.  Needs
// use_hip_compute and light mode, and a path from input to output on which every layer has a device overload.
class HipGraphPrivate;
class NCNN_EXPORT HipGraph
{
public:
    HipGraph();
    ~HipGraph();
    int record(const Net& net, const char* input_name, const HipMat& input, const char* output_name);
    int update_input(const Mat& src); // same shape as the recorded input; the copy has completed on return
    int launch();
    int synchronize();
    const HipMat& output() const;
    void clear();

private:
    HipGraph(const HipGraph&);
    HipGraph& operator=(const HipGraph&);
    HipGraphPrivate* const d;
};

} // namespace ncnn

#endif // NCNN_NET_H
