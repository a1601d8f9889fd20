// Device-side counterparts of Mat and of the per-inference command object: the roles VkMat (src/mat.h:383-560)
// and VkCompute (src/command.h:20-120) play for the reference's GPU path, shaped for one HIP stream.
//
// HipMat is a refcounted handle to a blob in HBM:
//   dims 3: channels-last [n][h*w][cp], cp = 16*ceil(c/16), pad channels zero  (fp32 or int8)
//   dims 1: dense [n][w]            dims 2: dense [n][h][w]
// HipCommand owns the stream every kernel of one Extractor runs on and shares a pool of device buffers (HipPool) with the
// blobs cut from it: the pool lives until the command AND every such blob are gone, so a blob may outlive its command, its
// Extractor and its Net.  All work of an Extractor is stream-ordered, so a buffer that goes back to the pool can be handed
// out again at once: whatever still reads it was enqueued earlier on the same stream.  A pool whose blobs are read on
// OTHER streams (the net's upload command) defers reuse instead: a returned buffer is handed out again only after a
// device-wide synchronisation.
#ifndef NCNN_HIPMAT_H
#define NCNN_HIPMAT_H

#include <stddef.h>

#include <memory>
#include <mutex>
#include <vector>

#include "mat.h"
#include "platform.h"

namespace ncnn {

class HipCommand;

// Device buffers of one command, shared (std::shared_ptr) with every blob allocated from it; the last owner frees them.
// Safe to use from several threads.
class NCNN_EXPORT HipPool
{
public:
    explicit HipPool(bool defer_reuse);
    ~HipPool();
    void* take(size_t bytes, int state); // state 1 blob, 2 borrowed scratch; 0 when the device cannot serve the request
    void give_back(void* ptr);
    void give_back_all_borrowed();
    size_t pooled_bytes() const;

private:
    HipPool(const HipPool&);
    HipPool& operator=(const HipPool&);
    struct Slot
    {
        void* ptr;
        size_t bytes;
        int state; // 0 idle, 1 blob, 2 borrowed scratch, 3 returned but possibly still read on another stream
        unsigned long long retired; // state 3: the pool's return count when the buffer came back
    };
    unsigned long long returns; // buffers given back so far (orders the state-3 slots against a device-wide wait)
    mutable std::mutex lock;
    std::vector<Slot> slots;
    bool defer_reuse;
};

class NCNN_EXPORT HipMat
{
public:
    HipMat();
    HipMat(const HipMat& m);
    ~HipMat();
    HipMat& operator=(const HipMat& m);

    // all return with empty() true when the pool cannot serve the request
    void create(int w, size_t elemsize, int n, HipCommand* cmd);
    void create(int w, int h, size_t elemsize, int n, HipCommand* cmd);
    void create(int w, int h, int c, size_t elemsize, int n, HipCommand* cmd);
    void create_like(const HipMat& m, HipCommand* cmd);
    // fp32 image of at most 4 channels at 4 floats per pixel (cp = 4): how such an input arrives from the host.  Only
    // layers that say so (Layer::hip_accepts_narrow_input) see it; the executor widens it for everyone else.
    void create_narrow(int w, int h, int c, int n, HipCommand* cmd);
    bool narrow() const
    {
        return dims == 3 && cp < 16;
    }
    void release();

    bool empty() const
    {
        return data == 0;
    }
    // elements as they lie in memory, padding included
    size_t count() const
    {
        return dims == 3 ? (size_t)n * h * w * cp : (size_t)n * h * w;
    }
    size_t bytes() const
    {
        return count() * elemsize;
    }
    // true when this handle is the only one (an in-place kernel may overwrite the blob)
    bool exclusive() const
    {
        return refcount && *refcount == 1;
    }

    void* data;
    int* refcount; // host side
    std::shared_ptr<HipPool> pool; // where data goes back to; keeps the buffers alive after the command is gone
    int dims, w, h, c, n;
    int cp; // channels as padded in memory (dims 3), else 0.  16*ceil(c/16), or 4 for a narrow fp32 image (create_narrow)
    size_t elemsize;
    // An fp32 blob may travel with an int8 copy of itself, float2int8(value * q8_scale), written by the kernel
    // that produced it: the convolution that consumes the blob with that input scale then skips its Quantize pass.
    // An int8 blob (elemsize 1, no twin) with q8_scale != 0 stands in for an fp32 blob of the model: the executor
    // had its producer emit float2int8(value * q8_scale) directly because every consumer would quantise it so.
    std::shared_ptr<HipMat> q8;
    float q8_scale;

private:
    void allocate(HipCommand* cmd);
};

class NCNN_EXPORT HipCommand
{
public:
    // blobs_cross_streams: blobs of this command are consumed on other commands' streams (see HipPool)
    explicit HipCommand(bool blobs_cross_streams = false);
    ~HipCommand();
    int ensure_ready(); // selects the device and creates the stream on first use
    void* stream;

    // blob memory (returned when the last HipMat handle goes)
    void* alloc(size_t bytes);
    void free(void* ptr);
    // scratch for one forward call: everything borrowed goes back with give_back_all()
    void* borrow(size_t bytes);
    void give_back_all();
    // one persistent buffer, zero-filled when it is (re)allocated, for kernels that keep their scratch "zero at rest"
    // (the arrival counters of the K-split convolution); used by one kernel at a time, like everything on this stream
    void* zeroed_workspace(size_t bytes);

    // host Mat (planar, any batch) -> device blob and back; download synchronises the stream
    int upload(const Mat& src, HipMat& dst);
    int upload_into(const Mat& src, HipMat& dst); // dst exists and has src's shape: new values for the same buffer
    int widen(const HipMat& src, HipMat& dst);    // narrow blob -> ordinary 16-channel-padded blob (enqueued, not waited for)
    int download(const HipMat& src, Mat& dst, Allocator* allocator);
    int synchronize();

    size_t pooled_bytes() const;

private:
    HipCommand(const HipCommand&);
    HipCommand& operator=(const HipCommand&);
    friend class HipMat;
    bool ready;
    std::shared_ptr<HipPool> pool;
    void* zero_ws;
    size_t zero_ws_bytes;
};

// scratch borrowed during one forward() returns to the pool when this goes out of scope
class ScopedScratch
{
public:
    explicit ScopedScratch(HipCommand* c) : cmd(c) {}
    ~ScopedScratch()
    {
        cmd->give_back_all();
    }
    void* get(size_t bytes)
    {
        return cmd->borrow(bytes);
    }

private:
    HipCommand* cmd;
};

} // namespace ncnn

#endif // NCNN_HIPMAT_H
