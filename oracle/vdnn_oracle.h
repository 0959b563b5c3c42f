/* TEST INFRASTRUCTURE — CPU restatement of the reference's layer math and training step.
 *
 * This is the checker that the HIP path is compared against, and the timed CPU baseline. It is not
 * part of the product: nothing under the package may include, link or call it.
 *
 * Where the arithmetic comes from: the reference delegates every layer to cuDNN 7.6.5 / cuBLAS 10.2
 * (closed source, absent from the reference tree; build.sh:2), so each function restates the
 * published definition of the library call at the cited call site, with the scalars (alpha, beta)
 * the reference passes. The reference has no tests, golden vectors or fixtures.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   conv fwd / bwd-data / bwd-filter : torch-CPU conv2d + autograd fixtures (tests/golden), adjoint
 *                                      identities in fp64, brute-force 7-deep loops; torch's float64
 *                                      conv2d + autograd at test time on geometries drawn from a seeded
 *                                      generator (asymmetric windows, strides to 3, paddings to window - 1)
 *   bias add / bias grad / sub / fill: closed form
 *   fc fwd / bwd-data / bwd-weight   : numpy matmul
 *   relu                             : closed form incl. -0, NaN, inf
 *   bfloat16 rounding                : torch's float32 -> bfloat16 conversion on random values, exact ties,
 *                                      subnormals, infinities and NaN
 *   tanh / sigmoid fwd / bwd         : torch.tanh / torch.sigmoid + autograd in float64, special values,
 *                                      the identities tanh(-x) = -tanh(x), sigmoid(x) + sigmoid(-x) = 1
 *   maxpool fwd / bwd                : torch max_pool2d + autograd fixtures on tie-free data
 *                                      (3x3 s2 overlapping and 2x2 s2), and at test time on five more
 *                                      window / stride / plane shapes; brute force.
 *                                      TIE RULE OF maxpool bwd: PARITY UNPINNED (cuDNN closed, no
 *                                      test in the reference). First maximum in row-major window
 *                                      order is chosen here.
 *   lrn fwd / bwd                    : torch local_response_norm fixtures, finite differences
 *   softmax fwd / bwd, softmax-CE    : torch fixtures; rows sum to 1; sum dx = 0; shift invariance
 *   network step                     : torch-CPU autograd fixture of a small net built from the same
 *                                      layer kinds; finite differences of the loss; torch's float64
 *                                      autograd at test time on ten layer tables drawn from a seeded generator
 *   seeded generator                 : fixture of first values + moments
 */
#ifndef VDNN_ORACLE_H_
#define VDNN_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int n, c, h, w;
    int k, r, s;
    int pad_h, pad_w, stride_h, stride_w;
} orc_shape;

/* accumulate convolution / GEMM sums in double (1) or float (0, default) */
void orc_set_accumulate_double(int on);
int  orc_get_accumulate_double(void);
/* Route stride-1 convolutions (forward, backward data, backward filter) through im2col + cache-blocked SGEMM
 * (vdnn_oracle_gemm.c) instead of the direct loops: the same sums in another order, several times faster. For the
 * timed CPU baseline; off by default, ignored while sums are accumulated in double. Pinned by comparison with the
 * direct loops on every convolution geometry of the fixtures (tests/test_oracle_layers.py). */
void orc_set_blocked_gemm(int on);
int  orc_get_blocked_gemm(void);
int  orc_blocked_conv_ok(const orc_shape* g);
void orc_blocked_conv_fwd(const orc_shape* g, const float* x, const float* w, const float* bias, float* y);
void orc_blocked_conv_bwd_data(const orc_shape* g, const float* dy, const float* w, float* dx);
void orc_blocked_conv_bwd_filter_sgd(const orc_shape* g, const float* x, const float* dy, float* w, float alpha);
void orc_set_threads(int n);
int  orc_get_threads(void);

int orc_out_dim(int in, int pad, int window, int stride);

/* layer.cu:560-582 */
void orc_conv_fwd(const orc_shape* g, const float* x, const float* w, const float* bias, float* y);
/* layer.cu:616-625 */
void orc_conv_bwd_data(const orc_shape* g, const float* dy, const float* w, float* dx);
/* layer.cu:631-637 */
void orc_conv_bwd_bias_sgd(const orc_shape* g, const float* dy, float* bias, float alpha);
/* layer.cu:651-660 */
void orc_conv_bwd_filter_sgd(const orc_shape* g, const float* x, const float* dy, float* w, float alpha);
/* brute-force forms (double accumulation, one loop per index), used to pin the fast ones */
void orc_conv_fwd_brute(const orc_shape* g, const float* x, const float* w, const float* bias, float* y);
void orc_conv_bwd_data_brute(const orc_shape* g, const float* dy, const float* w, float* dx);
void orc_conv_bwd_filter_brute(const orc_shape* g, const float* x, const float* dy, float* dw);

/* layer.cu:677-706 */
void orc_fc_fwd(int n, int c_in, int c_out, const float* x, const float* w, const float* bias, float* y);
/* layer.cu:725-733 */
void orc_fc_bwd_data(int n, int c_in, int c_out, const float* dy, const float* w, float* dx);
/* layer.cu:736-744 */
void orc_fc_bwd_weight_sgd(int n, int c_in, int c_out, const float* x, const float* dy, float* w, float alpha);
/* layer.cu:747-761 */
void orc_fc_bwd_bias_sgd(int n, int c_out, const float* dy, float* bias, float alpha);

/* layer.cu:774-781, 802-811 */
void orc_relu_fwd(size_t count, const float* x, float* y);
void orc_relu_bwd(size_t count, const float* x, const float* y, const float* dy, float* dx);
void orc_round_bf16(size_t count, const float* x, float* y);
void orc_tanh_fwd(size_t count, const float* x, float* y);
void orc_tanh_bwd(size_t count, const float* y, const float* dy, float* dx);
void orc_sigmoid_fwd(size_t count, const float* x, float* y);
void orc_sigmoid_bwd(size_t count, const float* y, const float* dy, float* dx);
/* layer.cu:875-882, 903-912 */
void orc_maxpool_fwd(const orc_shape* g, const float* x, float* y);
void orc_maxpool_bwd(const orc_shape* g, const float* x, const float* y, const float* dy, float* dx);
/* no counterpart in the reference (window 5, alpha 1e-4, beta 0.75, k 2, alpha divided by window) */
void orc_lrn_fwd(int n, int c, int hw, const float* x, float* y);
void orc_lrn_bwd(int n, int c, int hw, const float* x, const float* y, const float* dy, float* dx);
/* layer.cu:824-832, 853-862 */
void orc_softmax_fwd(int n, int classes, const float* x, float* y);
void orc_softmax_bwd(int n, int classes, const float* y, const float* dy, float* dx);
/* network.cu:3-8 */
void orc_sub(size_t count, const float* a, const float* b, float* r);
/* fused softmax-CE on integer labels; returns the mean loss */
float orc_softmax_ce_fwd(int n, int classes, const float* logits, const int32_t* labels, float* prob);
void  orc_softmax_ce_bwd(int n, int classes, const float* prob, const int32_t* labels, float* dlogits);
float orc_cross_entropy_dense(int n, int classes, const float* prob, const float* target);

/* ---- seeded synthetic data ---------------------------------------------------------------- */
/* counter-based generator: element i of stream `stream` under `seed` */
uint64_t orc_rng_u64(uint64_t seed, uint64_t stream, uint64_t i);
void orc_fill_normal(float* p, size_t count, uint64_t seed, uint64_t stream, float mean, float std);
void orc_fill_uniform(float* p, size_t count, uint64_t seed, uint64_t stream, float lo, float hi);
void orc_fill_labels(int32_t* p, size_t count, uint64_t seed, uint64_t stream, int classes);

/* ---- whole networks (network.cu:156-813 tables, 1056-1191 drivers) --------------------------- */
typedef struct orc_net orc_net;
/* layer kinds use the reference's Layer_t numbering (vdnn.h:38-50) plus 10 for LRN */
typedef struct {
    int type;
    orc_shape g;          /* input n,c,h,w and k,r,s,pad,stride */
    int n_out, c_out, h_out, w_out;
} orc_layer_desc;

/* cnn: 0 AlexNet (19 layers), 1 OverFeat, 3/4/5 VGG16, 7 AlexNet+LRN; batch overrides the table's
 * batch when > 0 */
orc_net* orc_net_create(int cnn, int batch);
/* a net from an explicit table (used by the small-net fixture) */
orc_net* orc_net_create_custom(const orc_layer_desc* layers, int num_layers);
void orc_net_destroy(orc_net* net);
int  orc_net_num_layers(const orc_net* net);
void orc_net_layer_desc(const orc_net* net, int l, orc_layer_desc* out);
/* He-normal filters (std sqrt(2/fan_in)), zero biases, N(0,1) input, integer labels */
void orc_net_init_seeded(orc_net* net, uint64_t seed);
/* bfloat16 activation storage: the input, every layer's output, the first difference and every
 * layer's input gradient are rounded to bfloat16 once; parameters and their updates stay float */
void orc_net_set_bf16(orc_net* net, int on);
size_t orc_net_filter_count(const orc_net* net, int l);
size_t orc_net_bias_count(const orc_net* net, int l);
float* orc_net_filter(orc_net* net, int l);
float* orc_net_bias(orc_net* net, int l);
float* orc_net_input(orc_net* net);
float* orc_net_label(orc_net* net);              /* dense n x classes target */
void   orc_net_set_labels(orc_net* net, const int32_t* labels); /* one-hot into the dense target */
/* forwardPropagation (network.cu:1056-1110): returns the mean cross-entropy against the target */
float orc_net_forward(orc_net* net);
/* backwardPropagation (network.cu:1112-1191): dy_last = y - label, then every layer's backward with
 * the fused SGD updates, lr = 1e-5 */
void  orc_net_backward(orc_net* net);
float* orc_net_dst(orc_net* net, int l);   /* y of layer l after forward */
float* orc_net_grad(orc_net* net, int l);  /* dx of layer l after backward */

#ifdef __cplusplus
}
#endif
#endif
