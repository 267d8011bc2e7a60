// Layer graph over device-resident Blobs: the shape of feather::Layer in the
// reference's layer.h:29-84 (bottom/top blobs by name, GenerateTopBlobs / Init /
// Forward, a CommonMemPool shared by all layers plus a PrivateMemPool per
// layer), reduced to what a convolution trunk needs.  The reference declares
// this interface but never compiles it (layer.h includes a missing rt_param.h);
// here it runs: ConvolutionLayer picks Winograd or implicit GEMM per layer,
// fuses bias + ReLU into the kernel epilogue, and draws its V / M / split
// workspace from the shared pool, so a whole stack runs back to back on the
// device with no host round trip.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "fastconv_hip.h"
#include "utility/blob.h"
#include "utility/mempool.h"

namespace feather {

class Layer {
   public:
    Layer(const std::string &name, const std::string &type) : _name(name), _type(type), common_mempool(NULL), private_mempool(NULL) {}
    virtual ~Layer() {
        for (size_t i = 0; i < _top_blobs_owned.size(); i++) delete _top_blobs_owned[i];
        delete private_mempool;
    }
    int SetupBottomBlob(const Blob<float> *p_blob, std::string name) {
        _bottom_blobs[name] = p_blob;
        _bottom.push_back(name);
        return 0;
    }
    void SetPools(CommonMemPool<float> *common, fastconv::RangeAllocator *alloc) {
        common_mempool = common;
        _alloc = alloc;
        private_mempool = new PrivateMemPool<float>(alloc);
    }
    // Shapes (and allocates) the output blobs from the bottom blobs.
    virtual int GenerateTopBlobs() = 0;
    // Other initialisation: plans, filter transforms, scratch requests to the common pool.
    virtual int Init() { return 0; }
    virtual int Forward() = 0;

    std::string name() { return _name; }
    std::string type() { return _type; }
    size_t top_size() { return _top.size(); }
    const Blob<float> *top_blob(size_t idx) { return _top_blobs[_top[idx]]; }
    const Blob<float> *top_blob(std::string name) { return _top_blobs.count(name) ? _top_blobs[name] : NULL; }

   protected:
    Blob<float> *NewTop(const std::string &name, size_t n, size_t c, size_t h, size_t w) {
        Blob<float> *b = new Blob<float>(NULL, n, c, h, w, name);
        b->SetAllocator(_alloc);
        b->Alloc();
        _top_blobs_owned.push_back(b);
        _top_blobs[name] = b;
        _top.push_back(name);
        return b;
    }
    std::string _name, _type;
    std::vector<std::string> _bottom, _top;
    std::map<std::string, const Blob<float> *> _bottom_blobs;
    std::map<std::string, Blob<float> *> _top_blobs;
    std::vector<Blob<float> *> _top_blobs_owned;
    CommonMemPool<float> *common_mempool;
    PrivateMemPool<float> *private_mempool;
    fastconv::RangeAllocator *_alloc = NULL;
};

// kernel x kernel convolution, optional per-channel bias and ReLU fused into the epilogue.
class ConvolutionLayer : public Layer {
   public:
    ConvolutionLayer(const std::string &name, size_t oc, size_t kernel, size_t stride, size_t pad, const float *weights,
                     const float *bias, bool relu)
        : Layer(name, "Convolution"), oc_(oc), k_(kernel), s_(stride), p_(pad), w_host_(weights), b_host_(bias),
          relu_(relu), winograd_(false), fused_(false), onepass_(false), w_dev_(NULL), b_dev_(NULL), U_(NULL), Wp_(NULL), table_(NULL),
          shape_(), wplan_(), iplan_(), v_off_(0), m_off_(0) {}

    int GenerateTopBlobs();
    int Init();
    int Forward();
    bool uses_winograd() const { return winograd_; }

   private:
    size_t oc_, k_, s_, p_;
    const float *w_host_, *b_host_;
    bool relu_, winograd_, fused_, onepass_;
    float *w_dev_, *b_dev_, *U_, *Wp_;
    int32_t *table_;
    fc_conv_shape shape_;
    fc_wino_plan wplan_;
    fc_igemm_plan iplan_;
    size_t v_off_, m_off_;      // offsets of V and M (or the split workspace) inside the common pool
};

class MaxPool2x2Layer : public Layer {
   public:
    explicit MaxPool2x2Layer(const std::string &name) : Layer(name, "Pooling") {}
    int GenerateTopBlobs();
    int Forward();
};

// A chain of layers: layer i reads the top blob of layer i-1.
class Net {
   public:
    explicit Net(size_t arena_bytes);
    ~Net();
    void SetInput(size_t n, size_t c, size_t h, size_t w);
    void Add(Layer *layer);                 // takes ownership
    int Init();                             // GenerateTopBlobs + Init of every layer, then one common-pool Alloc
    int Forward(const float *input_host);   // upload, run all layers, no download
    // Runs the layers once, then records them into a graph: every later Forward() replays the
    // recording with one launch call (worth it when the kernels are short, e.g. batch 1).
    int RecordGraph();
    const Blob<float> *output() const;
    const Blob<float> *blob_of(size_t layer) const { return layers_[layer]->top_blob((size_t)0); }
    size_t num_layers() const { return layers_.size(); }
    Layer *layer(size_t i) { return layers_[i]; }
    size_t common_bytes() const { return common_->common_bytes(); }

   private:
    fastconv::RangeAllocator *alloc_;
    CommonMemPool<float> *common_;
    Blob<float> *input_;
    std::vector<Layer *> layers_;
    void *arena_block_;
    size_t arena_mark_;     // pool usage before the arena block was taken
    size_t arena_top_;      // and right after: the block is the top of the stack while usage equals this
    fc_graph *graph_;
};

}  // namespace feather
