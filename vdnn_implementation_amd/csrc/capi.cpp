// C ABI over Network (include/vdnn_capi.h).
#include "vdnn_capi.h"

#include <cstring>

#include "network.h"
#include "seeded_init.h"

struct vdnn_network { Network* net; };

static NetworkOptions to_options(const vdnn_network_options* o) {
    NetworkOptions n;
    if (!o) return n;
    n.seed = o->seed; n.poolBytes = o->pool_bytes; n.capBytes = o->cap_bytes;
    n.planOnly = o->plan_only != 0; n.hostSync = o->host_sync != 0; n.capture = o->capture != 0;
    n.verbose = o->verbose != 0; n.device = o->device;
    n.refinedLifetimes = o->refined_lifetimes != 0;
    n.dataType = o->data_type;
    n.offloadLag = o->offload_lag;
    n.prefetchDepth = o->prefetch_depth < 1 ? 1 : o->prefetch_depth;
    n.unfusedOptimizer = o->unfused_optimizer != 0;
    n.deferOptimizer = o->defer_optimizer != 0;
    n.fuseActivations = o->fuse_activations != 0;
    n.compressOffload = o->compress_offload != 0;
    n.keepTailBytes = o->keep_tail_bytes;
    n.keepPackedOnDevice = o->keep_packed_on_device != 0;
    n.planPackedFraction = o->plan_packed_fraction;
    n.prefetchWithinPeak = o->prefetch_within_peak != 0;
    n.hbmBudgetBytes = o->hbm_budget_bytes;
    n.inPlaceBackward = o->in_place_backward != 0;
    n.recomputeFirstLayer = o->recompute_first_layer != 0;
    n.planLinkBytes = o->plan_link_bytes;
    return n;
}

extern "C" {

void vdnn_network_default_options(vdnn_network_options* o) {
    if (!o) return;
    memset(o, 0, sizeof *o); /* padding and every field a later version adds start at zero */
    const NetworkOptions d;
    o->seed = d.seed; o->pool_bytes = d.poolBytes; o->cap_bytes = d.capBytes;
    o->plan_only = d.planOnly; o->host_sync = d.hostSync; o->capture = d.capture; o->verbose = d.verbose;
    o->device = d.device;
    o->refined_lifetimes = d.refinedLifetimes;
    o->unfused_optimizer = d.unfusedOptimizer; o->defer_optimizer = d.deferOptimizer;
    o->offload_lag = d.offloadLag; o->prefetch_depth = d.prefetchDepth;
    o->data_type = d.dataType;
    o->fuse_activations = d.fuseActivations;
    o->keep_tail_bytes = d.keepTailBytes;
    o->prefetch_within_peak = d.prefetchWithinPeak;
    o->keep_packed_on_device = d.keepPackedOnDevice;
    o->plan_packed_fraction = d.planPackedFraction;
    o->compress_offload = d.compressOffload;
    o->hbm_budget_bytes = d.hbmBudgetBytes;
    o->in_place_backward = d.inPlaceBackward;
    o->recompute_first_layer = d.recomputeFirstLayer;
    o->plan_link_bytes = d.planLinkBytes;
}

vdnn_network* vdnn_network_create(int cnn, int policy, int algo, int batch, const vdnn_network_options* o) {
    if (Network::tableFor((CNN_t)cnn, 1).empty()) return nullptr;
    vdnn_network* h = new vdnn_network;
    h->net = new Network((CNN_t)cnn, (vdnn_t)policy, (vdnnAlgoMode_t)algo, batch > 0 ? batch : DEFAULT_BATCH_SIZE, to_options(o));
    return h;
}

vdnn_network* vdnn_network_create_custom(const vdnn_layer_spec* layers, int num_layers, int policy, int algo,
                                         const vdnn_network_options* o) {
    if (!layers || num_layers <= 0 || num_layers > DEFAULT_NUM_LAYER) return nullptr;
    std::vector<LayerSpec> t;
    for (int i = 0; i < num_layers; i++) {
        const vdnn_layer_spec& s = layers[i];
        t.push_back(LayerSpec{(Layer_t)s.type, s.n, s.c, s.h, s.w, s.pad_h, s.pad_w, s.stride_h, s.stride_w, s.k, s.r, s.s, false});
    }
    vdnn_network* h = new vdnn_network;
    h->net = new Network(t, (vdnn_t)policy, (vdnnAlgoMode_t)algo, to_options(o));
    return h;
}

void vdnn_network_destroy(vdnn_network* h) {
    if (!h) return;
    delete h->net;
    delete h;
}

int vdnn_network_forward(vdnn_network* h, int is_dynamic) { return h->net->forwardPropagation(is_dynamic != 0); }
int vdnn_network_backward(vdnn_network* h, int is_dynamic) { return h->net->backwardPropagation(is_dynamic != 0); }
void vdnn_network_synchronize(vdnn_network* h) { h->net->synchronize(); }
float vdnn_network_loss(vdnn_network* h) { return h->net->loss(); }
int vdnn_network_num_layers(vdnn_network* h) { return h->net->numLayersCount(); }
int vdnn_network_batch(vdnn_network* h) { return h->net->batch(); }
int vdnn_network_policy(vdnn_network* h) { return (int)h->net->policy(); }
int vdnn_network_algo(vdnn_network* h) { return (int)h->net->algo(); }

int vdnn_network_layer_spec(vdnn_network* h, int l, vdnn_layer_spec* out) {
    if (!out || l < 0 || l >= h->net->numLayersCount()) return -1;
    const LayerSpec& s = h->net->table()[l];
    Layer* L = h->net->layerArray()[l];
    *out = vdnn_layer_spec{(int)s.type, s.n, s.c, s.h, s.w, s.pad_h, s.pad_w, s.stride_h, s.stride_w, s.k, s.r, s.s,
                           L->OutputN(), L->OutputC(), L->OutputH(), L->OutputW()};
    return 0;
}

size_t vdnn_network_input_size(vdnn_network* h) { return h->net->getInputSize(); }
size_t vdnn_network_output_size(vdnn_network* h) { return h->net->getOutputSize(); }
void vdnn_network_set_input(vdnn_network* h, const float* host) { h->net->setInput(host); }
void vdnn_network_get_input(vdnn_network* h, float* host) { h->net->getInput(host); }
void vdnn_network_set_labels(vdnn_network* h, const int32_t* labels) { h->net->setLabels(labels); }
void vdnn_network_set_label_tensor(vdnn_network* h, const float* host) { h->net->setLabelTensor(host); }
int vdnn_network_set_layer_params(vdnn_network* h, int l, const float* f, const float* b) { return h->net->setLayerParams(l, f, b); }
int vdnn_network_get_layer_params(vdnn_network* h, int l, float* f, float* b) { return h->net->getLayerParams(l, f, b); }
int vdnn_network_get_layer_gradients(vdnn_network* h, int l, float* f, float* b) { return h->net->getLayerGradients(l, f, b); }
int vdnn_network_apply_gradients(vdnn_network* h) { return h->net->applyGradients(); }
int vdnn_network_train(vdnn_network* h, int steps, int is_dynamic, float* losses) {
    const std::vector<float> v = h->net->train(steps, is_dynamic != 0);
    if (losses) for (size_t i = 0; i < v.size(); i++) losses[i] = v[i];
    return (int)v.size();
}

size_t vdnn_network_filter_count(vdnn_network* h, int l) {
    return (l < 0 || l >= h->net->numLayersCount()) ? 0 : h->net->layerArray()[l]->FilterDataSize();
}
size_t vdnn_network_bias_count(vdnn_network* h, int l) {
    return (l < 0 || l >= h->net->numLayersCount()) ? 0 : h->net->layerArray()[l]->BiasDataSize();
}

static size_t copy_out(const std::vector<float>& v, float* host, size_t capacity) {
    if (host && capacity >= v.size() && !v.empty()) memcpy(host, v.data(), v.size() * sizeof(float));
    return v.size();
}
size_t vdnn_network_captured_dst(vdnn_network* h, int l, float* host, size_t capacity) {
    if (l < 0 || l >= h->net->numLayersCount()) return 0;
    return copy_out(h->net->capturedDst(l), host, capacity);
}
size_t vdnn_network_captured_grad(vdnn_network* h, int l, float* host, size_t capacity) {
    if (l < 0 || l >= h->net->numLayersCount()) return 0;
    return copy_out(h->net->capturedGrad(l), host, capacity);
}

void vdnn_network_stats_get(vdnn_network* h, vdnn_network_stats* out) {
    if (!out) return;
    const NetworkStats s = h->net->stats();
    *out = vdnn_network_stats{s.peakBytesInUse, s.peakExtent, s.offloadBytes, s.prefetchBytes, s.pinnedBytes, s.poolBytes, s.weightBytes};
}
void vdnn_network_reset_peak(vdnn_network* h) { h->net->resetPeak(); }
int vdnn_network_is_offloaded(vdnn_network* h, int l) {
    return (l >= 0 && l < h->net->numLayersCount() && h->net->isOffloaded(l)) ? 1 : 0;
}

int vdnn_network_grad_over_src(vdnn_network* h, int l) { return h->net->gradOverSrc(l) ? 1 : 0; }
int vdnn_network_offload_lag(vdnn_network* h) { return h->net->offloadLagInUse(); }
int vdnn_network_recomputed_layer(vdnn_network* h) { return h->net->recomputedSrcLayer(); }

int vdnn_network_placement(vdnn_network* h, int l) { return (int)h->net->placementOf(l); }
int vdnn_network_plan_feasible(vdnn_network* h) { return h->net->planFeasible() ? 1 : 0; }
size_t vdnn_network_plan_peak_bytes(vdnn_network* h) { return h->net->planPeakBytes(); }

int vdnn_network_prefetch_trace(vdnn_network* h, int* bwd_layer, int* prefetched_layer, int capacity) {
    const auto& t = h->net->prefetchTrace();
    for (int i = 0; i < (int)t.size() && i < capacity; i++) {
        if (bwd_layer) bwd_layer[i] = t[i].first;
        if (prefetched_layer) prefetched_layer[i] = t[i].second;
    }
    return (int)t.size();
}

size_t vdnn_network_max_dxdy_bytes(vdnn_network* h) { return h->net->findMaxDxDySize(); }
size_t vdnn_network_max_workspace_bytes(vdnn_network* h) { return h->net->findMaxWorkSpaceSize(); }
struct vdnn_ctx* vdnn_network_context(vdnn_network* h) { return h->net->context(); }

/* vdnn.cu:12-27 */
int vdnn_parse_cnn(const char* w, int* cnn) {
    static const struct { const char* name; int v; } tab[] = {
        {"ALEXNET", ALEXNET}, {"OVERFEAT", OVERFEAT}, {"GOOGLENET", GOOGLENET}, {"VGG16_64", VGG16_64}, {"VGG16_128", VGG16_128},
        {"VGG16_256", VGG16_256}, {"CUSTOM_CNN", CUSTOM_CNN}, {"ALEXNET_LRN", ALEXNET_LRN}, {"VGG16_512", VGG16_512}};
    for (const auto& e : tab) if (w && strcmp(w, e.name) == 0) { *cnn = e.v; return 0; }
    return -1;
}
/* vdnn.cu:29-38 */
int vdnn_parse_policy(const char* w, int* policy) {
    static const struct { const char* name; int v; } tab[] = {{"BASELINE", BASELINE}, {"VDNN_NONE", VDNN_NONE}, {"VDNN_ALL", VDNN_ALL}, {"VDNN_CONV", VDNN_CONV}};
    for (const auto& e : tab) if (w && strcmp(w, e.name) == 0) { *policy = e.v; return 0; }
    return -1;
}
/* vdnn.cu:40-47 */
int vdnn_parse_algo(const char* w, int* algo) {
    static const struct { const char* name; int v; } tab[] = {
        {"VDNN_MEMORY_OPT_ALGO", VDNN_MEMORY_OPT_ALGO}, {"VDNN_PERF_OPT_ALGO", VDNN_PERF_OPT_ALGO}, {"VDNN_DYNAMIC_ALGO", VDNN_DYNAMIC_ALGO}};
    for (const auto& e : tab) if (w && strcmp(w, e.name) == 0) { *algo = e.v; return 0; }
    return -1;
}

void vdnn_seeded_fill_normal(float* p, size_t count, uint64_t seed, uint64_t stream, float mean, float stddev) {
    vdnn::seeded_fill_normal(p, count, seed, stream, mean, stddev);
}
void vdnn_seeded_fill_labels(int32_t* p, size_t count, uint64_t seed, uint64_t stream, int classes) {
    vdnn::seeded_fill_labels(p, count, seed, stream, classes);
}

} // extern "C"
