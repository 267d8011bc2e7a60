#include "layer.h"

#include <stdio.h>
#include <stdlib.h>

#include "select_algorithm.h"

using fastconv::Device;

namespace feather {

static size_t round256(size_t v) { return (v + 255) / 256 * 256; }

// Init() and Forward() return int with 0 = success (the pools report failure as `false`).
#define POOL_OK_OR_FAIL(call)                                                \
    do {                                                                     \
        if (!(call)) {                                                       \
            fprintf(stderr, "Err in file %s line %d\n", __FILE__, __LINE__); \
            return -1;                                                       \
        }                                                                    \
    } while (0)

int ConvolutionLayer::GenerateTopBlobs() {
    const Blob<float> *in = _bottom_blobs[_bottom[0]];
    shape_.N = (int)in->num(); shape_.C = (int)in->channels(); shape_.H = (int)in->height(); shape_.W = (int)in->width();
    shape_.K = (int)oc_; shape_.kh = shape_.kw = (int)k_; shape_.sh = shape_.sw = (int)s_;
    shape_.pt = shape_.pb = shape_.pl = shape_.pr = (int)p_;
    const size_t oh = (in->height() + 2 * p_ - k_) / s_ + 1, ow = (in->width() + 2 * p_ - k_) / s_ + 1;
    NewTop(_name, in->num(), oc_, oh, ow);
    return 0;
}

int ConvolutionLayer::Init() {
    Device &d = Device::Get();
    const size_t w_elems = oc_ * shape_.C * k_ * k_;
    POOL_OK_OR_FAIL(private_mempool->Alloc(&w_dev_, w_elems * sizeof(float)));
    d.Check(fc_upload(d.ctx(), w_dev_, w_host_, w_elems * sizeof(float)), "upload weights");
    if (b_host_) {
        POOL_OK_OR_FAIL(private_mempool->Alloc(&b_dev_, oc_ * sizeof(float)));
        d.Check(fc_upload(d.ctx(), b_dev_, b_host_, oc_ * sizeof(float)), "upload bias");
    }
    nnp_size ks = {k_, k_}, st = {s_, s_}, os = {_top_blobs[_name]->width(), _top_blobs[_name]->height()};
    const nnp_convolution_algorithm algo = select_algorithm(ks, st, os, shape_.C, oc_, shape_.N);
    winograd_ = algo == nnp_convolution_algorithm_winograd;
    onepass_ = winograd_ && fc_wino_prefer_onepass(&shape_) != 0;
    if (onepass_) {
        // the whole layer in one kernel: no shared scratch at all
        d.Check(fc_wino_make_onepass_plan(&shape_, &wplan_), "fc_wino_make_onepass_plan");
        POOL_OK_OR_FAIL(private_mempool->Alloc(&U_, wplan_.U_bytes));
        d.Check(fc_wino_onepass_filter_transform(d.ctx(), &wplan_, w_dev_, U_), "fc_wino_onepass_filter_transform");
    } else if (winograd_) {
        d.Check(fc_wino_make_plan(&shape_, fc_wino_gemm_default_config(&shape_), &wplan_), "fc_wino_make_plan");
        fused_ = fc_wino_prefer_fused(&shape_) != 0;
        POOL_OK_OR_FAIL(private_mempool->Alloc(&U_, wplan_.U_bytes));
        // weights are constant: the filter transform is done once, here
        d.Check(fc_wino_filter_transform(d.ctx(), &wplan_, w_dev_, U_), "fc_wino_filter_transform");
        v_off_ = 0;
        m_off_ = round256(wplan_.V_bytes);
        common_mempool->Request(m_off_ + (fused_ ? 0 : wplan_.M_bytes));
    } else {
        d.Check(fc_igemm_make_plan(&shape_, fc_igemm_default_config(&shape_), &iplan_), "fc_igemm_make_plan");
        POOL_OK_OR_FAIL(private_mempool->Alloc(&Wp_, iplan_.Wp_bytes));
        float *tab = NULL;
        POOL_OK_OR_FAIL(private_mempool->Alloc(&tab, iplan_.table_bytes));
        table_ = (int32_t *)tab;
        d.Check(fc_igemm_pack_filter(d.ctx(), &iplan_, w_dev_, Wp_, table_), "fc_igemm_pack_filter");
        if (iplan_.ws_bytes) common_mempool->Request(iplan_.ws_bytes);
    }
    return 0;
}

int ConvolutionLayer::Forward() {
    Device &d = Device::Get();
    const float *x = _bottom_blobs[_bottom[0]]->data();
    float *y = _top_blobs[_name]->data();
    float *scratch = NULL;
    if (onepass_) {
        d.Check(fc_wino_conv_onepass(d.ctx(), &wplan_, x, U_, b_dev_, relu_, y), "fc_wino_conv_onepass");
        return 0;
    }
    if (winograd_ || iplan_.ws_bytes) POOL_OK_OR_FAIL(common_mempool->GetPtr(&scratch));
    if (winograd_) {
        float *V = scratch, *M = (float *)((char *)scratch + m_off_);
        if (fused_)
            d.Check(fc_wino_forward_fused(d.ctx(), &wplan_, x, w_dev_, b_dev_, relu_, 1, U_, V, y), "fc_wino_forward_fused");
        else
            d.Check(fc_wino_forward(d.ctx(), &wplan_, x, w_dev_, b_dev_, relu_, 1, U_, V, M, y), "fc_wino_forward");
    } else {
        d.Check(fc_conv_implicit_gemm(d.ctx(), &iplan_, x, Wp_, table_, b_dev_, relu_, scratch, y), "fc_conv_implicit_gemm");
    }
    return 0;
}

int MaxPool2x2Layer::GenerateTopBlobs() {
    const Blob<float> *in = _bottom_blobs[_bottom[0]];
    NewTop(_name, in->num(), in->channels(), in->height() / 2, in->width() / 2);
    return 0;
}

int MaxPool2x2Layer::Forward() {
    Device &d = Device::Get();
    const Blob<float> *in = _bottom_blobs[_bottom[0]];
    d.Check(fc_maxpool2x2(d.ctx(), in->data(), _top_blobs[_name]->data(), (int)in->num(), (int)in->channels(),
                          (int)in->height(), (int)in->width()),
            "fc_maxpool2x2");
    return 0;
}

Net::Net(size_t arena_bytes) : input_(NULL), graph_(NULL) {
    Device &d = Device::Get();
    arena_mark_ = d.Mark();
    arena_block_ = d.Alloc(arena_bytes, "layer graph arena");
    arena_top_ = d.Mark();
    alloc_ = new fastconv::RangeAllocator(arena_block_, arena_bytes, 256);
    common_ = new CommonMemPool<float>(alloc_);
}

Net::~Net() {
    if (graph_) fc_graph_destroy(graph_);
    for (size_t i = 0; i < layers_.size(); i++) delete layers_[i];
    delete input_;
    delete common_;
    delete alloc_;
    // The device arena is a stack: the block goes back only while it is still the top of it.  When
    // something was allocated after it (and is still alive) the block stays until that owner releases.
    Device &d = Device::Get();
    if (d.Mark() == arena_top_) d.Release(arena_mark_);
    else fprintf(stderr, "Net: device buffers were allocated after the layer graph arena; its block stays in the pool\n");
}

void Net::SetInput(size_t n, size_t c, size_t h, size_t w) {
    input_ = new Blob<float>(NULL, n, c, h, w, "data");
    input_->SetAllocator(alloc_);
    input_->Alloc();
}

void Net::Add(Layer *layer) {
    const Blob<float> *bottom = layers_.empty() ? input_ : layers_.back()->top_blob((size_t)0);
    layer->SetPools(common_, alloc_);
    layer->SetupBottomBlob(bottom, layers_.empty() ? "data" : layers_.back()->name());
    layer->GenerateTopBlobs();
    layers_.push_back(layer);
}

int Net::Init() {
    for (size_t i = 0; i < layers_.size(); i++)
        if (layers_[i]->Init() != 0) return -1;
    if (common_->common_bytes() > 0 && !common_->Alloc()) {
        fprintf(stderr, "Error: the arena is too small for the shared scratch (%zu bytes)\n", common_->common_bytes());
        return -1;
    }
    return 0;
}

int Net::Forward(const float *input_host) {
    if (input_host) input_->CopyData(input_host);
    if (graph_) {
        Device &d = Device::Get();
        d.Check(fc_graph_launch(d.ctx(), graph_), "fc_graph_launch");
        return 0;
    }
    for (size_t i = 0; i < layers_.size(); i++)
        if (layers_[i]->Forward() != 0) return -1;
    return 0;
}

int Net::RecordGraph() {
    Device &d = Device::Get();
    if (graph_) return 0;
    if (Forward(NULL) != 0) return -1;      // every kernel has run once: LDS grants are in place
    d.Check(fc_sync(d.ctx()), "fc_sync");
    d.Check(fc_graph_begin(d.ctx()), "fc_graph_begin");
    int failed = 0;
    for (size_t i = 0; i < layers_.size() && !failed; i++) failed = layers_[i]->Forward() != 0;
    // the recording is always closed, also when a layer refused: the stream must not stay in capture mode
    fc_graph *g = NULL;
    const int rc = fc_graph_end(d.ctx(), &g);
    if (failed || rc != FC_OK) {
        if (g) fc_graph_destroy(g);
        fprintf(stderr, "Error: recording the layer graph failed%s%s\n", rc != FC_OK ? ": " : "",
                rc != FC_OK ? fc_last_error(d.ctx()) : "");
        return -1;
    }
    graph_ = g;
    return 0;
}

const Blob<float> *Net::output() const { return layers_.back()->top_blob((size_t)0); }

}  // namespace feather
