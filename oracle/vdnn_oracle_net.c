/* TEST INFRASTRUCTURE — CPU restatement of the reference's network tables and of one training step
 * (see vdnn_oracle.h). Memory policies do not change the arithmetic, so a single schedule (every
 * tensor resident) stands for all four. */
#include "vdnn_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

enum { T_FC_GEMM = 0, T_CONV = 1, T_FC_CONV = 2, T_RELU = 3, T_TANH = 4, T_SIGMOID = 5, T_SOFTMAX = 6, T_POOL = 7, T_LRN = 10 };
#define ORC_MAX_LAYERS 64
#define ORC_LR 1e-5 /* vdnn.h:8 */

struct orc_net {
    int num_layers;
    orc_layer_desc L[ORC_MAX_LAYERS];
    float* filter[ORC_MAX_LAYERS];
    float* bias[ORC_MAX_LAYERS];
    float* dst[ORC_MAX_LAYERS];
    float* grad[ORC_MAX_LAYERS];
    float* input;
    float* label;
    float* diff_last;
    int bf16; /* activations are stored as bfloat16: every layer output and gradient is rounded once, and the
                 products of forward and backward data take the filter rounded to bfloat16 (the update acts
                 on the float master copy) */
};

static size_t src_count(const orc_layer_desc* d) { return (size_t)d->g.n * d->g.c * d->g.h * d->g.w; }
static size_t dst_count(const orc_layer_desc* d) { return (size_t)d->n_out * d->c_out * d->h_out * d->w_out; }

static void add_layer(orc_net* net, int type, int n, int c, int h, int w,
                      int pad_h, int pad_w, int stride_h, int stride_w, int k, int r, int s) {
    orc_layer_desc* d = &net->L[net->num_layers++];
    memset(d, 0, sizeof(*d));
    d->type = type;
    d->g.n = n; d->g.c = c; d->g.h = h; d->g.w = w;
    d->g.k = k; d->g.r = r; d->g.s = s;
    d->g.pad_h = pad_h; d->g.pad_w = pad_w; d->g.stride_h = stride_h; d->g.stride_w = stride_w;
    switch (type) {
    case T_FC_GEMM: /* layer.cu:84-91 */
        d->n_out = n; d->c_out = k; d->h_out = 1; d->w_out = 1; break;
    case T_CONV: case T_FC_CONV: /* layer.cu:208-216 */
        d->n_out = n; d->c_out = k;
        d->h_out = orc_out_dim(h, pad_h, r, stride_h); d->w_out = orc_out_dim(w, pad_w, s, stride_w); break;
    case T_POOL: /* layer.cu:432-439 */
        d->n_out = n; d->c_out = c;
        d->h_out = orc_out_dim(h, pad_h, r, stride_h); d->w_out = orc_out_dim(w, pad_w, s, stride_w); break;
    default: /* layer.cu:301-304 */
        d->n_out = n; d->c_out = c; d->h_out = h; d->w_out = w; break;
    }
}

static void conv(orc_net* t, int n, int c, int hw, int pad, int stride, int k, int r) {
    add_layer(t, T_FC_CONV, n, c, hw, hw, pad, pad, stride, stride, k, r, r);
}
static void relu(orc_net* t, int n, int c, int hw) { add_layer(t, T_RELU, n, c, hw, hw, 0, 0, 0, 0, 0, 0, 0); }
static void lrn(orc_net* t, int n, int c, int hw) { add_layer(t, T_LRN, n, c, hw, hw, 0, 0, 0, 0, 0, 0, 0); }
static void pool(orc_net* t, int n, int c, int hw, int win) { add_layer(t, T_POOL, n, c, hw, hw, 0, 0, 2, 2, 0, win, win); }
static void fc(orc_net* t, int n, int cin, int cout) { add_layer(t, T_FC_GEMM, n, cin, 1, 1, 0, 0, 0, 0, cout, 1, 1); }
static void softmax(orc_net* t, int n, int c) { add_layer(t, T_SOFTMAX, n, c, 1, 1, 0, 0, 0, 0, 0, 0, 0); }

/* network.cu:156-323; with_lrn inserts the two normalisation layers after ReLU 1 and ReLU 2 */
static void table_alexnet(orc_net* t, int n, int with_lrn) {
    conv(t, n, 3, 227, 0, 4, 96, 11);  relu(t, n, 96, 55);  if (with_lrn) lrn(t, n, 96, 55);  pool(t, n, 96, 55, 3);
    conv(t, n, 96, 27, 2, 1, 256, 5);  relu(t, n, 256, 27); if (with_lrn) lrn(t, n, 256, 27); pool(t, n, 256, 27, 3);
    conv(t, n, 256, 13, 1, 1, 384, 3); relu(t, n, 384, 13);
    conv(t, n, 384, 13, 1, 1, 384, 3); relu(t, n, 384, 13);
    conv(t, n, 384, 13, 1, 1, 256, 3); relu(t, n, 256, 13); pool(t, n, 256, 13, 3);
    fc(t, n, 9216, 4096); relu(t, n, 4096, 1);
    fc(t, n, 4096, 4096); relu(t, n, 4096, 1);
    fc(t, n, 4096, 1000); softmax(t, n, 1000);
}

/* network.cu:325-495 */
static void table_overfeat(orc_net* t, int n) {
    conv(t, n, 3, 231, 0, 4, 96, 11);    relu(t, n, 96, 56);   pool(t, n, 96, 56, 2);
    conv(t, n, 96, 28, 0, 1, 256, 5);    relu(t, n, 256, 24);  pool(t, n, 256, 24, 2);
    conv(t, n, 256, 12, 1, 1, 512, 3);   relu(t, n, 512, 12);
    conv(t, n, 512, 12, 1, 1, 1024, 3);  relu(t, n, 1024, 12);
    conv(t, n, 1024, 12, 1, 1, 1024, 3); relu(t, n, 1024, 12); pool(t, n, 1024, 12, 2);
    conv(t, n, 1024, 6, 0, 1, 3072, 6);  relu(t, n, 3072, 1);
    conv(t, n, 3072, 1, 0, 1, 4096, 1);  relu(t, n, 4096, 1);
    conv(t, n, 4096, 1, 0, 1, 1000, 1);  softmax(t, n, 1000);
}

/* network.cu:501-813 */
static void table_vgg16(orc_net* t, int n) {
    static const int cfg[13][3] = { /* c_in, c_out, hw */
        {3, 64, 224}, {64, 64, 224}, {64, 128, 112}, {128, 128, 112}, {128, 256, 56}, {256, 256, 56}, {256, 256, 56},
        {256, 512, 28}, {512, 512, 28}, {512, 512, 28}, {512, 512, 14}, {512, 512, 14}, {512, 512, 14}};
    static const int pool_after[13] = {0, 1, 0, 1, 0, 0, 1, 0, 0, 1, 0, 0, 1};
    for (int i = 0; i < 13; i++) {
        conv(t, n, cfg[i][0], cfg[i][2], 1, 1, cfg[i][1], 3);
        relu(t, n, cfg[i][1], cfg[i][2]);
        if (pool_after[i]) pool(t, n, cfg[i][1], cfg[i][2], 2);
    }
    fc(t, n, 512 * 7 * 7, 4096); relu(t, n, 4096, 1);
    fc(t, n, 4096, 4096);        relu(t, n, 4096, 1);
    fc(t, n, 4096, 1000);        softmax(t, n, 1000);
}

static int has_params(int type) { return type == T_FC_GEMM || type == T_CONV || type == T_FC_CONV; }

size_t orc_net_filter_count(const orc_net* net, int l) {
    const orc_layer_desc* d = &net->L[l];
    if (!has_params(d->type)) return 0;
    return (size_t)d->g.k * d->g.c * d->g.r * d->g.s; /* layer.h:243 */
}
size_t orc_net_bias_count(const orc_net* net, int l) {
    const orc_layer_desc* d = &net->L[l];
    return has_params(d->type) ? (size_t)d->c_out : 0;
}

static void alloc_tensors(orc_net* net) {
    for (int l = 0; l < net->num_layers; l++) {
        const orc_layer_desc* d = &net->L[l];
        net->dst[l] = (float*)calloc(dst_count(d), sizeof(float));
        net->grad[l] = (float*)calloc(src_count(d), sizeof(float));
        const size_t fcnt = orc_net_filter_count(net, l), bcnt = orc_net_bias_count(net, l);
        net->filter[l] = fcnt ? (float*)calloc(fcnt, sizeof(float)) : NULL;
        net->bias[l] = bcnt ? (float*)calloc(bcnt, sizeof(float)) : NULL;
    }
    net->input = (float*)calloc(src_count(&net->L[0]), sizeof(float));
    const size_t out = dst_count(&net->L[net->num_layers - 1]);
    net->label = (float*)calloc(out, sizeof(float));
    net->diff_last = (float*)calloc(out, sizeof(float));
}

orc_net* orc_net_create(int cnn, int batch) {
    orc_net* net = (orc_net*)calloc(1, sizeof(orc_net));
    switch (cnn) {
    case 0: table_alexnet(net, batch > 0 ? batch : 128, 0); break;
    case 7: table_alexnet(net, batch > 0 ? batch : 128, 1); break;
    case 1: table_overfeat(net, batch > 0 ? batch : 128); break;
    case 3: table_vgg16(net, batch > 0 ? batch : 64); break;   /* network.cu:142-143 */
    case 4: table_vgg16(net, batch > 0 ? batch : 128); break;  /* network.cu:144-145 */
    case 5: table_vgg16(net, batch > 0 ? batch : 256); break;  /* network.cu:146-147 */
    case 8: table_vgg16(net, batch > 0 ? batch : 512); break;
    default: free(net); return NULL;
    }
    alloc_tensors(net);
    return net;
}

orc_net* orc_net_create_custom(const orc_layer_desc* layers, int num_layers) {
    if (num_layers <= 0 || num_layers > ORC_MAX_LAYERS) return NULL;
    orc_net* net = (orc_net*)calloc(1, sizeof(orc_net));
    for (int l = 0; l < num_layers; l++) {
        const orc_shape* g = &layers[l].g;
        add_layer(net, layers[l].type, g->n, g->c, g->h, g->w, g->pad_h, g->pad_w, g->stride_h, g->stride_w, g->k, g->r, g->s);
    }
    alloc_tensors(net);
    return net;
}

void orc_net_destroy(orc_net* net) {
    if (!net) return;
    for (int l = 0; l < net->num_layers; l++) {
        free(net->dst[l]); free(net->grad[l]); free(net->filter[l]); free(net->bias[l]);
    }
    free(net->input); free(net->label); free(net->diff_last);
    free(net);
}

int orc_net_num_layers(const orc_net* net) { return net->num_layers; }
void orc_net_layer_desc(const orc_net* net, int l, orc_layer_desc* out) { *out = net->L[l]; }
float* orc_net_filter(orc_net* net, int l) { return net->filter[l]; }
float* orc_net_bias(orc_net* net, int l) { return net->bias[l]; }
float* orc_net_input(orc_net* net) { return net->input; }
float* orc_net_label(orc_net* net) { return net->label; }
float* orc_net_dst(orc_net* net, int l) { return net->dst[l]; }
float* orc_net_grad(orc_net* net, int l) { return net->grad[l]; }

void orc_net_set_labels(orc_net* net, const int32_t* labels) {
    const orc_layer_desc* last = &net->L[net->num_layers - 1];
    const int n = last->n_out, classes = last->c_out * last->h_out * last->w_out;
    memset(net->label, 0, sizeof(float) * (size_t)n * classes);
    for (int i = 0; i < n; i++) net->label[(size_t)i * classes + labels[i]] = 1.0f;
}

/* Streams of the seeded generator: 1 input, 2 labels, 100+2l filter of layer l, 101+2l its bias. */
void orc_net_init_seeded(orc_net* net, uint64_t seed) {
    orc_fill_normal(net->input, src_count(&net->L[0]), seed, 1, 0.0f, 1.0f);
    const orc_layer_desc* last = &net->L[net->num_layers - 1];
    const int n = last->n_out, classes = last->c_out * last->h_out * last->w_out;
    int32_t* lab = (int32_t*)malloc(sizeof(int32_t) * (size_t)n);
    orc_fill_labels(lab, (size_t)n, seed, 2, classes);
    orc_net_set_labels(net, lab);
    free(lab);
    for (int l = 0; l < net->num_layers; l++) {
        const size_t fcnt = orc_net_filter_count(net, l);
        if (!fcnt) continue;
        const orc_layer_desc* d = &net->L[l];
        const double fan_in = (double)d->g.c * d->g.r * d->g.s;
        orc_fill_normal(net->filter[l], fcnt, seed, 100 + 2 * (uint64_t)l, 0.0f, (float)sqrt(2.0 / fan_in));
        memset(net->bias[l], 0, sizeof(float) * orc_net_bias_count(net, l));
    }
}

/* forwardPropagation (network.cu:1056-1110): src[l] = dst[l-1] (:1080-1083), Layer::forward
 * dispatch (layer.cu:489-512) */
void orc_net_set_bf16(orc_net* net, int on) { net->bf16 = on != 0; }

/* the filter as forward / backward data multiply it: the master copy, or its bfloat16 rounding in a scratch copy */
static const float* product_filter(const orc_net* net, int l, float** scratch) {
    *scratch = NULL;
    if (!net->bf16) return net->filter[l];
    const size_t count = orc_net_filter_count(net, l);
    *scratch = (float*)malloc(sizeof(float) * count);
    orc_round_bf16(count, net->filter[l], *scratch);
    return *scratch;
}

float orc_net_forward(orc_net* net) {
    if (net->bf16) orc_round_bf16(src_count(&net->L[0]), net->input, net->input);
    for (int l = 0; l < net->num_layers; l++) {
        const orc_layer_desc* d = &net->L[l];
        const float* src = l == 0 ? net->input : net->dst[l - 1];
        float* dst = net->dst[l];
        switch (d->type) {
        case T_FC_GEMM: { float* tmp; const float* w = product_filter(net, l, &tmp); orc_fc_fwd(d->g.n, d->g.c, d->g.k, src, w, net->bias[l], dst); free(tmp); } break;
        case T_CONV: case T_FC_CONV: { float* tmp; const float* w = product_filter(net, l, &tmp); orc_conv_fwd(&d->g, src, w, net->bias[l], dst); free(tmp); } break;
        case T_RELU: orc_relu_fwd(src_count(d), src, dst); break;
        case T_TANH: orc_tanh_fwd(src_count(d), src, dst); break;
        case T_SIGMOID: orc_sigmoid_fwd(src_count(d), src, dst); break;
        case T_LRN: orc_lrn_fwd(d->g.n, d->g.c, d->g.h * d->g.w, src, dst); break;
        case T_POOL: orc_maxpool_fwd(&d->g, src, dst); break;
        case T_SOFTMAX: orc_softmax_fwd(d->g.n, d->g.c * d->g.h * d->g.w, src, dst); break;
        default: break;
        }
        if (net->bf16) orc_round_bf16(dst_count(d), dst, dst);
    }
    const orc_layer_desc* last = &net->L[net->num_layers - 1];
    (void)last;
    return orc_cross_entropy_dense(last->n_out, last->c_out * last->h_out * last->w_out,
                                   net->dst[net->num_layers - 1], net->label);
}

/* backwardPropagation (network.cu:1112-1191): first diff = y - label (:1042-1054), then
 * Layer::backward from the last layer down (layer.cu:514-537); diff[l] = grad[l+1] (:1144-1147).
 * Inside a conv layer: bwd-data with the old filter, then bias, then filter (layer.cu:616-660);
 * inside an FC layer: dX, then W, then bias (layer.cu:725-761). lr = (float)(1e-5 * -1). */
void orc_net_backward(orc_net* net) {
    const float alpha = (float)(ORC_LR * -1.0f);
    const int L = net->num_layers;
    const orc_layer_desc* last = &net->L[L - 1];
    orc_sub(dst_count(last), net->dst[L - 1], net->label, net->diff_last);
    if (net->bf16) orc_round_bf16(dst_count(last), net->diff_last, net->diff_last);
    for (int l = L - 1; l >= 0; l--) {
        const orc_layer_desc* d = &net->L[l];
        const float* src = l == 0 ? net->input : net->dst[l - 1];
        const float* dst = net->dst[l];
        const float* diff = l == L - 1 ? net->diff_last : net->grad[l + 1];
        float* grad = net->grad[l];
        switch (d->type) {
        case T_FC_GEMM:
            { float* tmp; const float* w = product_filter(net, l, &tmp); orc_fc_bwd_data(d->g.n, d->g.c, d->g.k, diff, w, grad); free(tmp); }
            orc_fc_bwd_weight_sgd(d->g.n, d->g.c, d->g.k, src, diff, net->filter[l], alpha);
            orc_fc_bwd_bias_sgd(d->g.n, d->g.k, diff, net->bias[l], alpha);
            break;
        case T_CONV: case T_FC_CONV:
            { float* tmp; const float* w = product_filter(net, l, &tmp); orc_conv_bwd_data(&d->g, diff, w, grad); free(tmp); }
            orc_conv_bwd_bias_sgd(&d->g, diff, net->bias[l], alpha);
            orc_conv_bwd_filter_sgd(&d->g, src, diff, net->filter[l], alpha);
            break;
        case T_RELU: orc_relu_bwd(src_count(d), src, dst, diff, grad); break;
        case T_TANH: orc_tanh_bwd(src_count(d), dst, diff, grad); break;
        case T_SIGMOID: orc_sigmoid_bwd(src_count(d), dst, diff, grad); break;
        case T_LRN: orc_lrn_bwd(d->g.n, d->g.c, d->g.h * d->g.w, src, dst, diff, grad); break;
        case T_POOL: orc_maxpool_bwd(&d->g, src, dst, diff, grad); break;
        case T_SOFTMAX: orc_softmax_bwd(d->g.n, d->g.c * d->g.h * d->g.w, dst, diff, grad); break;
        default: break;
        }
        if (net->bf16) orc_round_bf16(src_count(d), grad, grad);
    }
}
