/* C ABI over the C++ host classes (Network, Layer): what a foreign-function binding of the
 * reference's upper boundary needs. The reference exposes C++ classes only (network.h:15-95,
 * layer.h:130-255, constructed by main at vdnn.cu:69); each entry point names the member it wraps.
 * Status: 0 ok, -1 out of memory (dynamic mode), other failures abort like the reference's macros.
 */
#ifndef VDNN_AMD_CAPI_H_
#define VDNN_AMD_CAPI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct vdnn_network vdnn_network;

typedef struct {
    uint64_t seed;
    size_t   pool_bytes;   /* 0: sized from the layer table */
    size_t   cap_bytes;    /* 0: no artificial limit */
    int      plan_only;    /* replay the allocation schedule without a device */
    int      host_sync;    /* synchronise both streams after every layer (network.cu:1090-1091) */
    int      capture;      /* keep host copies of every layer's dstData / gradData */
    int      verbose;
    int      device;
    int      refined_lifetimes; /* value-preserving lifetime refinements of the vDNN policies (0 = literal schedule) */
    int      unfused_optimizer; /* keep dW / db per layer and step after backward instead of inside it (same bits) */
    int      defer_optimizer;   /* with unfused_optimizer: backward leaves the step to vdnn_network_apply_gradients */
    int      offload_lag;       /* layers enqueued before an offloaded block is recycled (0 = the reference's schedule) */
    int      prefetch_depth;    /* offloaded tensors fetched ahead of their backward (1 = the reference's schedule) */
    int      data_type;         /* element type of activation tensors: VDNN_DTYPE_F32 (the reference, vdnn.h:11-12) or VDNN_DTYPE_BF16 */
    int      fuse_activations;  /* a ReLU after a CONV / FC layer runs inside the neighbouring layers' kernels (same bits, layer.cu:766-814) */
    size_t   keep_tail_bytes;   /* the deepest tensors of the policy's offload set stay on the device, up to this many bytes (0 = the reference's policies, network.cu:898-921) */
    int      prefetch_within_peak; /* backward fetches tensors ahead of the reference's schedule (network.cu:1198-1208) wherever a replay of the schedule shows that the peak cannot rise */
    int      keep_packed_on_device; /* with compress_offload: the packed tensors stay in device memory (about 0.6 of their size) instead of crossing the link */
    double   plan_packed_fraction;  /* what a plan-only network assumes a packed stream to be of its tensor (0 = the longest possible, 1.03) */
    int      compress_offload;  /* offloaded rectified tensors cross the link without their zero elements (lossless; layer.cu:969-987 copies them whole) */
    size_t   hbm_budget_bytes;  /* a limit on pool bytes in use that the policy meets by choosing, per member of its offload set (network.cu:898-936), between the device, a packed stream on the device and host memory (0 = the policy's own set) */
    int      in_place_backward; /* a layer's input gradient is written over its input where nothing reads that again (layer.cu:599 allocates it beside x and dy); needs refined_lifetimes */
    int      recompute_first_layer; /* the output of a first convolution over at most four channels is computed again before its consumer's backward instead of kept or offloaded (network.cu:916-936 keeps or moves it); needs refined_lifetimes */
    size_t   plan_link_bytes;   /* with hbm_budget_bytes: bytes per step and direction that the plan sends over the link before it packs anything on the device (0 = pack first) */
} vdnn_network_options;

typedef struct {
    int type;              /* Layer_t */
    int n, c, h, w;
    int pad_h, pad_w, stride_h, stride_w;
    int k, r, s;
    int n_out, c_out, h_out, w_out; /* filled in by vdnn_network_layer_spec; ignored on input */
} vdnn_layer_spec;

typedef struct {
    size_t peak_bytes_in_use, peak_extent, offload_bytes, prefetch_bytes, pinned_bytes, pool_bytes, weight_bytes;
} vdnn_network_stats;

void vdnn_network_default_options(vdnn_network_options* o);
/* Network::Network (network.cu:10-92); cnn is a CNN_t, policy a vdnn_t, algo a vdnnAlgoMode_t */
vdnn_network* vdnn_network_create(int cnn, int policy, int algo, int batch, const vdnn_network_options* o);
/* a network from an explicit table (Network::setLayersCustomCNN is an empty stub, network.cu:815-817) */
vdnn_network* vdnn_network_create_custom(const vdnn_layer_spec* layers, int num_layers, int policy, int algo,
                                         const vdnn_network_options* o);
void vdnn_network_destroy(vdnn_network* net);
/* Network::forwardPropagation / backwardPropagation (network.cu:1056-1191) */
int  vdnn_network_forward(vdnn_network* net, int is_dynamic);
int  vdnn_network_backward(vdnn_network* net, int is_dynamic);
void vdnn_network_synchronize(vdnn_network* net);
float vdnn_network_loss(vdnn_network* net);
int  vdnn_network_num_layers(vdnn_network* net);
int  vdnn_network_batch(vdnn_network* net);
int  vdnn_network_policy(vdnn_network* net);
int  vdnn_network_algo(vdnn_network* net);
int  vdnn_network_layer_spec(vdnn_network* net, int l, vdnn_layer_spec* out);
/* Network::getInputSize / getOutputSize (network.h:56-57) */
size_t vdnn_network_input_size(vdnn_network* net);
size_t vdnn_network_output_size(vdnn_network* net);
void vdnn_network_set_input(vdnn_network* net, const float* host);
void vdnn_network_get_input(vdnn_network* net, float* host);
void vdnn_network_set_labels(vdnn_network* net, const int32_t* labels);
void vdnn_network_set_label_tensor(vdnn_network* net, const float* host);
int  vdnn_network_set_layer_params(vdnn_network* net, int l, const float* filter, const float* bias);
int  vdnn_network_get_layer_params(vdnn_network* net, int l, float* filter, float* bias);
/* unfused optimizer (no counterpart in the reference, which fuses SGD into backward: layer.cu:651-660, 736-761) */
int  vdnn_network_get_layer_gradients(vdnn_network* net, int l, float* filter, float* bias);
int  vdnn_network_apply_gradients(vdnn_network* net);
/* `steps` training steps; writes the loss seen by each step's forward into losses[0..return) */
int  vdnn_network_train(vdnn_network* net, int steps, int is_dynamic, float* losses);
size_t vdnn_network_filter_count(vdnn_network* net, int l);
size_t vdnn_network_bias_count(vdnn_network* net, int l);
/* host copies taken during the last step when options.capture is set; returns the element count */
size_t vdnn_network_captured_dst(vdnn_network* net, int l, float* host, size_t capacity);
size_t vdnn_network_captured_grad(vdnn_network* net, int l, float* host, size_t capacity);
void vdnn_network_stats_get(vdnn_network* net, vdnn_network_stats* out);
void vdnn_network_reset_peak(vdnn_network* net);
/* Network::isOffload[] after setVdnnType (network.cu:875-940) */
int  vdnn_network_is_offloaded(vdnn_network* net, int l);
/* in_place_backward: 1 where layer l's backward writes its input gradient over its input */
int  vdnn_network_grad_over_src(vdnn_network* net, int l);
/* recompute_first_layer: the layer whose input layer 0 computes again before that layer's backward, or -1 */
int  vdnn_network_recomputed_layer(vdnn_network* net);
/* hbm_budget_bytes: the place of layer l's input (0 no plan / not a member of the offload set, 1 on the device, 2 packed on
 * the device, 3 host memory), whether the plan's replay met the budget, and what it peaked at */
int  vdnn_network_placement(vdnn_network* net, int l);
int  vdnn_network_plan_feasible(vdnn_network* net);
/* the offload lag in use: offload_lag, or the one the placement plan chose where that is negative */
int  vdnn_network_offload_lag(vdnn_network* net);
size_t vdnn_network_plan_peak_bytes(vdnn_network* net);
/* (backward layer, prefetched layer) pairs of the last backward, Network::findPrefetchLayer
 * (network.cu:1198-1208); returns the number of pairs */
int  vdnn_network_prefetch_trace(vdnn_network* net, int* bwd_layer, int* prefetched_layer, int capacity);
/* Network::findMaxDxDySize / findMaxWorkSpaceSize (network.cu:1010-1040), bytes */
size_t vdnn_network_max_dxdy_bytes(vdnn_network* net);
size_t vdnn_network_max_workspace_bytes(vdnn_network* net);
/* the context of the network, for calling include/vdnn_backend.h directly (timing events) */
struct vdnn_ctx* vdnn_network_context(vdnn_network* net);
/* parseVdnnInputs (vdnn.cu:8-54): 0 on success, -1 for an unknown word */
int vdnn_parse_cnn(const char* word, int* cnn);
int vdnn_parse_policy(const char* word, int* policy);
int vdnn_parse_algo(const char* word, int* algo);
/* host-side seeded generator, so a binding can reproduce the synthetic tensors */
void vdnn_seeded_fill_normal(float* p, size_t count, uint64_t seed, uint64_t stream, float mean, float stddev);
void vdnn_seeded_fill_labels(int32_t* p, size_t count, uint64_t seed, uint64_t stream, int classes);

#ifdef __cplusplus
}
#endif
#endif
