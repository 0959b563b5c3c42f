// Layer: per-layer forward/backward, offload/prefetch copies and pool requests.
// Follows the control flow of the reference's layer.cu (cited per function); the cuDNN/cuBLAS calls
// become calls into the device back end's C ABI.
#include "layer.h"

#include <cmath>
#include <cstring>
#include <iostream>

#include "seeded_init.h"

static const char* type_name(Layer_t t) {
    switch (t) {
    case FC_GEMM: return "FC_GEMM";
    case CONV: case FC_CONV: return "FC_CONV"; // the reference prints FC_CONV for both (layer.cu:154)
    case RELU: return "RELU";
    case TANH: return "TANH";
    case SIGMOID: return "SIGMOID";
    case SOFTMAX: return "SOFTMAX";
    case POOL: return "POOL";
    case LRN: return "LRN";
    default: return "";
    }
}

/* FC_GEMM constructor (layer.cu:40-102) */
Layer::Layer(vdnn_t _vdnnMode, vdnnAlgoMode_t _vdnnAlgoMode, Layer_t _layerType, vdnnGemmHandle_t* _gemmHandle,
             vdnn_stream_t* _stream_compute, vdnn_stream_t* _stream_memory, int _id,
             int _n, int _c, int _h, int _w, int _pad_h, int _pad_w, int _stride_h, int _stride_w, int _k, int _r, int _s)
    : vdnnMode(_vdnnMode), vdnnAlgoMode(_vdnnAlgoMode), layerType(_layerType), layerId(_id), ctx(nullptr),
      n_in(_n), c_in(_c), h_in(_h), w_in(_w), pad_h(_pad_h), pad_w(_pad_w), stride_h(_stride_h), stride_w(_stride_w),
      k(_k), r(_r), s(_s), stream_compute(_stream_compute), stream_memory(_stream_memory),
      convHandle(nullptr), gemmHandle(_gemmHandle) {
    /* Make sure only FC layer is initialized with the GEMM handle (layer.cu:79-81) */
    M_ASSERT(_layerType == FC_GEMM, "Layer type is not FC_GEMM!");
    M_ASSERT(h_in == 1 && w_in == 1 && r == 1 && s == 1, "Invalid dimensions!");
    M_ASSERT(_gemmHandle && _gemmHandle->ctx, "null GEMM handle");
    construct(_gemmHandle->ctx, _gemmHandle->settings);
}

/* Constructor of every other layer kind (layer.cu:104-485) */
Layer::Layer(vdnn_t _vdnnMode, vdnnAlgoMode_t _vdnnAlgoMode, Layer_t _layerType, vdnnConvHandle_t* _convHandle,
             vdnn_stream_t* _stream_compute, vdnn_stream_t* _stream_memory, int _id,
             int _n, int _c, int _h, int _w, int _pad_h, int _pad_w, int _stride_h, int _stride_w, int _k, int _r, int _s)
    : vdnnMode(_vdnnMode), vdnnAlgoMode(_vdnnAlgoMode), layerType(_layerType), layerId(_id), ctx(nullptr),
      n_in(_n), c_in(_c), h_in(_h), w_in(_w), pad_h(_pad_h), pad_w(_pad_w), stride_h(_stride_h), stride_w(_stride_w),
      k(_k), r(_r), s(_s), stream_compute(_stream_compute), stream_memory(_stream_memory),
      convHandle(_convHandle), gemmHandle(nullptr) {
    M_ASSERT(_layerType != FC_GEMM, "FC_GEMM type layer cannot be initialized with the convolution handle!");
    M_ASSERT(_convHandle && _convHandle->ctx, "null convolution handle");
    construct(_convHandle->ctx, _convHandle->settings);
}

void Layer::construct(vdnn_ctx* _ctx, const vdnnLayerSettings& _settings) {
    ctx = _ctx;
    settings = _settings;
    /* Basic settings (layer.cu:58-77, 122-142) */
    insideInceptionModule = headOfFork = tailOfFork = inPlaceOp = false;
    fuseRelu = elided = elidedBackward = gateGrad = false;
    forkId = -1;
    concatenateChannelOffset = 0;
    refCntFwd = refCntBwd = 0;
    srcData = filterData = biasData = dstData = diffData = gradData = nullptr;
    filterGrad = biasGrad = nullptr;
    actBytes = vdnn_ctx_activation_dtype(ctx) == VDNN_DTYPE_BF16 ? 2 : 4;
    fwdWorkSpaceSize = bwdDataWorkSpaceSize = bwdFilterWorkSpaceSize = 0;
    srcReadyEvent = offloadDoneEvent = nullptr;
    prefetchBlockFreeEvent = prefetchHostReadyEvent = prefetchDoneEvent = nullptr;
    shape = vdnn_shape_t{n_in, c_in, h_in, w_in, k, r, s, pad_h, pad_w, stride_h, stride_w};

    switch (layerType) {
    case FC_GEMM: /* layer.cu:83-91 */
        n_out = n_in; c_out = k; h_out = 1; w_out = 1;
        initializeFullyConnectedFilterAndBias();
        break;
    case CONV:
    case FC_CONV: /* output extent: layer.cu:208-216 */
        n_out = n_in; c_out = k;
        h_out = vdnn_out_dim(h_in, pad_h, r, stride_h);
        w_out = vdnn_out_dim(w_in, pad_w, s, stride_w);
        M_ASSERT(h_out > 0 && w_out > 0, "Convolution output is empty!");
        initializeConvolutionFilterAndBias();
        setAlgoMode(vdnnAlgoMode); /* layer.cu:255-294 */
        break;
    case RELU:
    case TANH:
    case SIGMOID: /* layer.cu:298-304: the three activation modes share one layer kind */
    case SOFTMAX:
    case LRN:
        n_out = n_in; c_out = c_in; h_out = h_in; w_out = w_in;
        break;
    case POOL: /* layer.cu:432-439 */
        n_out = n_in; c_out = c_in;
        h_out = vdnn_out_dim(h_in, pad_h, r, stride_h);
        w_out = vdnn_out_dim(w_in, pad_w, s, stride_w);
        M_ASSERT(h_out > 0 && w_out > 0, "Pooling output is empty!");
        break;
    case CONCATENATE: /* empty in the reference (layer.cu:464-468) */
    default:
        M_ASSERT(false, "Layer type not supported");
    }

    /* Allocate GPU memory for dstData (layer.cu:94, 472) */
    if (vdnnMode == BASELINE) cnmemMallocDstData(false);

    if (settings.verbose) {
        printf("----------------------- Layer %d -----------------------\n", layerId);
        printf("Layer Type: %s\n", type_name(layerType));
        printf("Input (n, c, h, w): (%d, %d, %d, %d)\n", n_in, c_in, h_in, w_in);
        printf("Output (n, c, h, w): (%d, %d, %d, %d)\n", n_out, c_out, h_out, w_out);
        printf("Filter (k, c, r, s): (%d, %d, %d, %d)\n", k, c_in, r, s);
        printf("Stride: (%d, %d), Padding: (%d, %d)\n", stride_h, stride_w, pad_h, pad_w);
        if (layerType == FC_CONV || layerType == CONV) {
            printf("CONV Layer %d fwdWorkSpaceSize: %lu\n", layerId, (unsigned long)fwdWorkSpaceSize);
            printf("CONV Layer %d bwdDataWorkSpaceSize: %lu\n", layerId, (unsigned long)bwdDataWorkSpaceSize);
            printf("CONV Layer %d bwdFilterWorkSpaceSize: %lu\n", layerId, (unsigned long)bwdFilterWorkSpaceSize);
        }
    }
}

/* The reference never releases a layer (layer.cu:487); here the parameters and a BASELINE dstData
 * go back to the pool. Activations of the other policies belong to the Network's schedule. */
Layer::~Layer() {
    if (filterData) vdnn_pool_free(ctx, filterData);
    if (biasData) vdnn_pool_free(ctx, biasData);
    if (filterGrad) vdnn_pool_free(ctx, filterGrad);
    if (biasGrad) vdnn_pool_free(ctx, biasGrad);
    if (vdnnMode == BASELINE && dstData && !elided) vdnn_pool_free(ctx, dstData);
    if (evBiasFork) vdnn_event_destroy(ctx, evBiasFork);
    if (evBiasJoin) vdnn_event_destroy(ctx, evBiasJoin);
}

/* an elided ReLU has no output block of its own: under BASELINE the one taken at construction goes back */
void Layer::setElided(bool v) {
    if (v == elided) return;
    if (v && vdnnMode == BASELINE && dstData) { vdnn_pool_free(ctx, dstData); dstData = nullptr; }
    if (!v && vdnnMode == BASELINE) { dstData = nullptr; cnmemMallocDstData(false); }
    elided = v;
    if (!v) elidedBackward = false;
}

void Layer::setAlgoMode(vdnnAlgoMode_t m) {
    vdnnAlgoMode = m;
    if (layerType != CONV && layerType != FC_CONV) return;
    if (m == VDNN_PERF_OPT_ALGO) {
        findPerfOptFwdAlgo(); findPerfOptBwdFilterAlgo(); findPerfOptBwdDataAlgo();
    } else {
        findMemOptFwdAlgo(); findMemOptBwdFilterAlgo(); findMemOptBwdDataAlgo();
    }
}

/* layer.cu:1013-1089: the two-way switch between workspace-free and workspace-using kernels; the
 * workspace sizes come from the back end (cudnnGet*WorkspaceSize, layer.cu:268-294) */
void Layer::findMemOptFwdAlgo()       { fwdWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_MEMORY_OPT_ALGO, VDNN_PASS_FWD, vdnn_ctx_activation_dtype(ctx)); }
void Layer::findMemOptBwdFilterAlgo() { bwdFilterWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_MEMORY_OPT_ALGO, VDNN_PASS_BWD_FILTER, vdnn_ctx_activation_dtype(ctx)); }
void Layer::findMemOptBwdDataAlgo()   { bwdDataWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_MEMORY_OPT_ALGO, VDNN_PASS_BWD_DATA, vdnn_ctx_activation_dtype(ctx)); }
void Layer::findPerfOptFwdAlgo()      { fwdWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_FWD, vdnn_ctx_activation_dtype(ctx)); }
void Layer::findPerfOptBwdFilterAlgo(){ bwdFilterWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_BWD_FILTER, vdnn_ctx_activation_dtype(ctx)); }
void Layer::findPerfOptBwdDataAlgo()  { bwdDataWorkSpaceSize = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_BWD_DATA, vdnn_ctx_activation_dtype(ctx)); }

/* layer.cu:1091-1147: per-layer greedy choice by trial allocation. With two variants per pass this
 * reduces to: use the workspace variant when its workspace can be allocated right now. */
void Layer::findDynamicAlgo() {
    if (layerType != CONV && layerType != FC_CONV) return;
    size_t need = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_FWD, vdnn_ctx_activation_dtype(ctx));
    size_t t = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_BWD_DATA, vdnn_ctx_activation_dtype(ctx));
    if (t > need) need = t;
    t = vdnn_conv_workspace_bytes_dtype(&shape, VDNN_PERF_OPT_ALGO, VDNN_PASS_BWD_FILTER, vdnn_ctx_activation_dtype(ctx));
    if (t > need) need = t;
    void* probe = nullptr;
    if (need == 0 || vdnn_pool_malloc(ctx, &probe, need) == VDNN_OK) {
        if (probe) vdnn_pool_free(ctx, probe);
        setAlgoMode(VDNN_PERF_OPT_ALGO);
    } else {
        setAlgoMode(VDNN_MEMORY_OPT_ALGO);
    }
}

/* layer.cu:489-512 */
int Layer::forward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic) {
    switch (layerType) {
    case FC_GEMM: return fullyConnectedForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    case CONV:
    case FC_CONV: return convolutionForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    case RELU:
    case TANH:
    case SIGMOID: return activationForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    case SOFTMAX: return softmaxForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    case POOL: return poolingForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    case LRN: return lrnForward(_offloaded, _offloadedSrcData_h, workSpace, isDynamic);
    default: return 0;
    }
}

/* layer.cu:514-537 */
void Layer::waitSrcFetched() {
    if (!srcFetchedEvent) return;
    checkVDNN(vdnn_stream_wait_event(ctx, *stream_compute, srcFetchedEvent));
    srcFetchedEvent = nullptr;
}

int Layer::backward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                    unsigned long _prefetch_bytes, void* workSpace, bool isDynamic) {
    /* CONV / FC layers wait in front of their first reader of srcData, everything else here */
    if (layerType != CONV && layerType != FC_CONV && layerType != FC_GEMM) waitSrcFetched();
    switch (layerType) {
    case FC_GEMM: return fullyConnectedBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    case CONV:
    case FC_CONV: return convolutionBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    case RELU:
    case TANH:
    case SIGMOID: return activationBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    case SOFTMAX: return softmaxBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    case POOL: return poolingBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    case LRN: return lrnBackward(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    default: return 0;
    }
}

/* Workspace protocol of layer.cu:544-551 / 606-613 / 640-647: BASELINE hands in the shared buffer,
 * the other policies take the pass's workspace from the pool for the duration of the call. */
int Layer::mallocWorkSpace(void* shared, size_t bytes, void** cur, bool isDynamic) {
    *cur = nullptr;
    if (shared != nullptr) {
        M_ASSERT(vdnnMode == BASELINE, "vdnn mode should be BASELINE");
        *cur = shared;
    } else if (bytes > 0) {
        if (ASSERT_EQ(vdnn_pool_malloc(ctx, cur, bytes), isDynamic) < 0) return -1;
    }
    return 0;
}

void Layer::freeWorkSpace(void* shared, size_t bytes, void* cur, bool isDynamic) {
    if (shared == nullptr && bytes > 0 && cur) ASSERT_EQ(vdnn_pool_free(ctx, cur), isDynamic);
}

/* layer.cu:539-589. The bias is added in the convolution kernel's epilogue: one fp32 add after the
 * complete reduction, the same value cudnnAddTensor (layer.cu:576-582) produces in a second pass. */
int Layer::convolutionForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic) {
    void* curWorkSpace = nullptr;
    if (mallocWorkSpace(workSpace, fwdWorkSpaceSize, &curWorkSpace, isDynamic) < 0) return -1;

    /* Allocate GPU memory for dstData */
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) {
            freeWorkSpace(workSpace, fwdWorkSpaceSize, curWorkSpace, isDynamic);
            return -1;
        }
    }

    if (fuseRelu)
        checkVDNN(vdnn_conv_fwd_relu(ctx, *stream_compute, &shape, vdnnAlgoMode, srcData, (const float*)filterData,
                                     (const float*)biasData, dstData, curWorkSpace, fwdWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_fwd(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)filterData,
                                (const float*)biasData, (float*)dstData, curWorkSpace, fwdWorkSpaceSize));

    /* Offload srcData to host */
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);

    freeWorkSpace(workSpace, fwdWorkSpaceSize, curWorkSpace, isDynamic);
    return 0;
}

/* The bias gradient (layer.cu:631-637) reads the output gradient once at memory speed and shares nothing with the two
 * matrix-core kernels of the layer's backward but that input: it is enqueued on the context's fourth stream, behind
 * whatever produced the output gradient, and runs beside them (its partial sums have a part of the staging area to
 * themselves). joinBiasGradient makes the compute stream wait for it before the layer's backward returns: the caller
 * may recycle the output gradient's block after that, and the next forward reads the bias. Same kernels, same bits. */
void Layer::biasGradientBeside(DATATYPE lr) {
    if (!evBiasFork) {
        checkVDNN(vdnn_event_create(ctx, &evBiasFork, 0));
        checkVDNN(vdnn_event_create(ctx, &evBiasJoin, 0));
    }
    vdnn_stream_t beside = vdnn_ctx_stream_pack(ctx);
    checkVDNN(vdnn_event_record(ctx, evBiasFork, *stream_compute));
    checkVDNN(vdnn_stream_wait_event(ctx, beside, evBiasFork));
    if (filterGrad) checkVDNN(vdnn_conv_bwd_bias(ctx, beside, &shape, (const float*)diffData, (float*)biasGrad));
    else checkVDNN(vdnn_conv_bwd_bias_sgd(ctx, beside, &shape, (const float*)diffData, (float*)biasData, lr));
    checkVDNN(vdnn_event_record(ctx, evBiasJoin, beside));
}

/* Whether this layer's backward filter adds up the bias gradient itself (a property of the shape, the algorithm mode and
 * the element type: the same answer under every policy, so the same sums). */
bool Layer::biasGradientInFilterKernel() const {
    return biasData != nullptr && vdnn_conv_bwd_filter_sums_bias(&shape, vdnnAlgoMode, vdnn_ctx_activation_dtype(ctx)) != 0;
}

void Layer::joinBiasGradient() {
    checkVDNN(vdnn_stream_wait_event(ctx, *stream_compute, evBiasJoin));
}

/* Addition (recomputeFirstLayer): what convolutionForward computed, again, from the same input and filter into `into`
 * (the workspace of the pass comes from the pool as in the forward of the offloading policies). */
int Layer::forwardAgainInto(void* into, bool isDynamic) {
    M_ASSERT((layerType == CONV || layerType == FC_CONV) && srcData && into, "only a convolution with its input on the device computes its output again");
    void* curWorkSpace = nullptr;
    if (mallocWorkSpace(nullptr, fwdWorkSpaceSize, &curWorkSpace, isDynamic) < 0) return -1;
    if (fuseRelu)
        checkVDNN(vdnn_conv_fwd_relu(ctx, *stream_compute, &shape, vdnnAlgoMode, srcData, (const float*)filterData,
                                     (const float*)biasData, into, curWorkSpace, fwdWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_fwd(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)filterData,
                                (const float*)biasData, (float*)into, curWorkSpace, fwdWorkSpaceSize));
    freeWorkSpace(nullptr, fwdWorkSpaceSize, curWorkSpace, isDynamic);
    return 0;
}

/* The kernels that may write a layer's input gradient over its input: every lane reads what it overwrites before it
 * does, and nothing else reads the input (vdnn_conv_bwd_data_in_place_ok / vdnn_maxpool_bwd_in_place_ok). */
bool Layer::canGradOverSrc() const {
    if (layerType == CONV || layerType == FC_CONV) return vdnn_conv_bwd_data_in_place_ok(&shape) != 0;
    if (layerType == POOL) return vdnn_maxpool_bwd_in_place_ok(&shape) != 0;
    return false;
}

/* Addition (gradOverSrc): the filter gradient first, into a block of its own, because it is the last reader of the
 * input; then the data gradient over the input - with the filter as it was, the order of layer.cu:616-660 - and only
 * then the update, param += alpha * grad with the fused call's arithmetic. */
int Layer::convolutionBackwardOverSrc(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                                      unsigned long _prefetch_bytes, void* workSpace, bool isDynamic) {
    void* curWorkSpace = nullptr;
    const DATATYPE lr = LEARNING_RATE * -1.0f;
    gradData = srcData;
    if (_layer_id_to_prefetch >= 0) prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);

    /* the bias gradient: inside the filter-gradient kernel where that kernel sums the dy it streams, else beside it */
    const bool biasInFilter = biasGradientInFilterKernel();
    auto joinBias = [&]() { if (!biasInFilter) joinBiasGradient(); };
    if (!biasInFilter) biasGradientBeside(lr);

    void* dw = filterGrad;
    if (!dw && ASSERT_EQ(vdnn_pool_malloc(ctx, &dw, sizeof(DATATYPE) * (size_t)k * c_in * r * s), isDynamic) < 0) { joinBias(); return -1; }
    /* a trial of the dynamic mode that runs out of memory gives up here: the caller recycles the output gradient's
     * block next, so the bias gradient's stream is joined on these paths too */
    auto releaseDw = [&]() { if (!filterGrad) ASSERT_EQ(vdnn_pool_free(ctx, dw), isDynamic); };
    if (mallocWorkSpace(workSpace, bwdFilterWorkSpaceSize, &curWorkSpace, isDynamic) < 0) { releaseDw(); joinBias(); return -1; }
    waitSrcFetched();
    if (biasInFilter && filterGrad)
        checkVDNN(vdnn_conv_bwd_filter_bias(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                            (float*)dw, (float*)biasGrad, curWorkSpace, bwdFilterWorkSpaceSize));
    else if (biasInFilter)
        checkVDNN(vdnn_conv_bwd_filter_then_bias_sgd(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                                     (float*)dw, (float*)biasData, lr, curWorkSpace, bwdFilterWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_bwd_filter(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                       (float*)dw, curWorkSpace, bwdFilterWorkSpaceSize));
    freeWorkSpace(workSpace, bwdFilterWorkSpaceSize, curWorkSpace, isDynamic);

    if (mallocWorkSpace(workSpace, bwdDataWorkSpaceSize, &curWorkSpace, isDynamic) < 0) { releaseDw(); joinBias(); return -1; }
    if (gateGrad)
        checkVDNN(vdnn_conv_bwd_data_relu(ctx, *stream_compute, &shape, vdnnAlgoMode, diffData, (const float*)filterData,
                                          srcData, gradData, curWorkSpace, bwdDataWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_bwd_data(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)diffData, (const float*)filterData,
                                     (float*)gradData, curWorkSpace, bwdDataWorkSpaceSize));
    freeWorkSpace(workSpace, bwdDataWorkSpaceSize, curWorkSpace, isDynamic);

    if (!filterGrad) {
        checkVDNN(vdnn_sgd_apply(ctx, *stream_compute, (size_t)k * c_in * r * s, lr, (const float*)dw, (float*)filterData));
        releaseDw();
    }
    joinBias();
    return 0;
}

/* layer.cu:591-665: gradData, prefetch, backward data (old filter), bias update, filter update */
int Layer::convolutionBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                               unsigned long _prefetch_bytes, void* workSpace, bool isDynamic) {
    if (gradOverSrc && vdnnMode != BASELINE)
        return convolutionBackwardOverSrc(_layer_id_to_prefetch, _prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes, workSpace, isDynamic);
    void* curWorkSpace = nullptr;
    const DATATYPE lr = LEARNING_RATE * -1.0f;

    if (vdnnMode != BASELINE) {
        if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }

    /* Prefetch srcData of previous layer */
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);

    if (mallocWorkSpace(workSpace, bwdDataWorkSpaceSize, &curWorkSpace, isDynamic) < 0) return -1;
    if (gateGrad) waitSrcFetched(); /* the masked data gradient reads this layer's input */
    if (gateGrad)
        checkVDNN(vdnn_conv_bwd_data_relu(ctx, *stream_compute, &shape, vdnnAlgoMode, diffData, (const float*)filterData,
                                          srcData, gradData, curWorkSpace, bwdDataWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_bwd_data(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)diffData, (const float*)filterData,
                                     (float*)gradData, curWorkSpace, bwdDataWorkSpaceSize));
    freeWorkSpace(workSpace, bwdDataWorkSpaceSize, curWorkSpace, isDynamic);

    /* Backward Bias Propagation (layer.cu:631-637), the learning rate folded into the update: summed inside the
     * filter-gradient kernel below where that kernel can (it streams the same dy), else by a kernel of its own beside it */
    const bool biasInFilter = biasGradientInFilterKernel();
    if (!biasInFilter) biasGradientBeside(lr);

    /* a trial of the dynamic mode that runs out of memory gives up here: the caller recycles the output gradient's
     * block next, so the bias gradient's stream is joined first */
    if (mallocWorkSpace(workSpace, bwdFilterWorkSpaceSize, &curWorkSpace, isDynamic) < 0) { if (!biasInFilter) joinBiasGradient(); return -1; }
    waitSrcFetched();
    if (filterGrad && biasInFilter)
        checkVDNN(vdnn_conv_bwd_filter_bias(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                            (float*)filterGrad, (float*)biasGrad, curWorkSpace, bwdFilterWorkSpaceSize));
    else if (filterGrad)
        checkVDNN(vdnn_conv_bwd_filter(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                       (float*)filterGrad, curWorkSpace, bwdFilterWorkSpaceSize));
    else if (biasInFilter)
        checkVDNN(vdnn_conv_bwd_filter_bias_sgd(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                                (float*)filterData, (float*)biasData, lr, curWorkSpace, bwdFilterWorkSpaceSize));
    else
        checkVDNN(vdnn_conv_bwd_filter_sgd(ctx, *stream_compute, &shape, vdnnAlgoMode, (const float*)srcData, (const float*)diffData,
                                           (float*)filterData, lr, curWorkSpace, bwdFilterWorkSpaceSize));
    freeWorkSpace(workSpace, bwdFilterWorkSpaceSize, curWorkSpace, isDynamic);
    if (!biasInFilter) joinBiasGradient();
    return 0;
}

/* layer.cu:667-709: the rank-1 bias GEMM with its temporary ones vector (:692-706) is fused into
 * the GEMM epilogue / split reduction */
int Layer::fullyConnectedForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) return -1;
    }
    if (fuseRelu)
        checkVDNN(vdnn_fc_fwd_relu(ctx, *stream_compute, n_out, c_in, c_out, srcData, (const float*)filterData,
                                   (const float*)biasData, dstData));
    else
        checkVDNN(vdnn_fc_fwd(ctx, *stream_compute, n_out, c_in, c_out, (const float*)srcData, (const float*)filterData,
                              (const float*)biasData, (float*)dstData));
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);
    return 0;
}

/* layer.cu:711-764: dX with the old filter, then the filter update, then the bias update */
int Layer::fullyConnectedBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                                  unsigned long _prefetch_bytes, void*, bool isDynamic) {
    const DATATYPE lr = LEARNING_RATE * -1.0f;
    if (vdnnMode != BASELINE) {
        if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);
    if (gateGrad) waitSrcFetched();
    if (gateGrad)
        checkVDNN(vdnn_fc_bwd_data_relu(ctx, *stream_compute, n_out, c_in, c_out, diffData, (const float*)filterData, srcData, gradData));
    else
        checkVDNN(vdnn_fc_bwd_data(ctx, *stream_compute, n_out, c_in, c_out, (const float*)diffData, (const float*)filterData, (float*)gradData));
    waitSrcFetched();
    if (filterGrad) {
        checkVDNN(vdnn_fc_bwd_weight(ctx, *stream_compute, n_out, c_in, c_out, (const float*)srcData, (const float*)diffData, (float*)filterGrad));
        checkVDNN(vdnn_fc_bwd_bias(ctx, *stream_compute, n_out, c_out, (const float*)diffData, (float*)biasGrad));
    } else {
        checkVDNN(vdnn_fc_bwd_weight_sgd(ctx, *stream_compute, n_out, c_in, c_out, (const float*)srcData, (const float*)diffData, (float*)filterData, lr));
        checkVDNN(vdnn_fc_bwd_bias_sgd(ctx, *stream_compute, n_out, c_out, (const float*)diffData, (float*)biasData, lr));
    }
    return 0;
}

/* layer.cu:766-788 */
int Layer::activationForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void*, bool isDynamic) {
    if (elided) { /* the producer has rectified already: the output is the input block */
        dstData = srcData;
        return 0;
    }
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) return -1;
    }
    /* the activation mode follows the layer type (layer.cu:357-372) */
    if (layerType == TANH) checkVDNN(vdnn_tanh_fwd(ctx, *stream_compute, SrcDataSize(), (const float*)srcData, (float*)dstData));
    else if (layerType == SIGMOID) checkVDNN(vdnn_sigmoid_fwd(ctx, *stream_compute, SrcDataSize(), (const float*)srcData, (float*)dstData));
    else checkVDNN(vdnn_relu_fwd(ctx, *stream_compute, SrcDataSize(), (const float*)srcData, (float*)dstData));
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);
    return 0;
}

/* layer.cu:790-814: cuDNN is handed x, y and dy */
int Layer::activationBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                              unsigned long _prefetch_bytes, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (inPlaceOp || elidedBackward) gradData = diffData; /* elementwise: dx may overwrite dy */
        else if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);
    if (elidedBackward) return 0; /* the consumer's backward has applied the mask */
    if (layerType == TANH)
        checkVDNN(vdnn_tanh_bwd(ctx, *stream_compute, SrcDataSize(), (const float*)dstData, (const float*)diffData, (float*)gradData));
    else if (layerType == SIGMOID)
        checkVDNN(vdnn_sigmoid_bwd(ctx, *stream_compute, SrcDataSize(), (const float*)dstData, (const float*)diffData, (float*)gradData));
    else
        checkVDNN(vdnn_relu_bwd(ctx, *stream_compute, SrcDataSize(), (const float*)srcData, (const float*)dstData,
                                (const float*)diffData, (float*)gradData));
    return 0;
}

/* layer.cu:816-839 */
int Layer::softmaxForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) return -1;
    }
    checkVDNN(vdnn_softmax_fwd(ctx, *stream_compute, n_in, c_in * h_in * w_in, (const float*)srcData, (float*)dstData));
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);
    return 0;
}

/* layer.cu:841-865 */
int Layer::softmaxBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                           unsigned long _prefetch_bytes, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);
    checkVDNN(vdnn_softmax_bwd(ctx, *stream_compute, n_in, c_in * h_in * w_in, (const float*)dstData, (const float*)diffData, (float*)gradData));
    return 0;
}

/* layer.cu:867-889 */
int Layer::poolingForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) return -1;
    }
    checkVDNN(vdnn_maxpool_fwd(ctx, *stream_compute, &shape, (const float*)srcData, (float*)dstData));
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);
    return 0;
}

/* layer.cu:891-915 */
int Layer::poolingBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                           unsigned long _prefetch_bytes, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (gradOverSrc) gradData = srcData; /* every thread reads its windows whole before it writes them back */
        else if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);
    if (gateGrad)
        checkVDNN(vdnn_maxpool_bwd_relu(ctx, *stream_compute, &shape, srcData, dstData, diffData, gradData));
    else
        checkVDNN(vdnn_maxpool_bwd(ctx, *stream_compute, &shape, (const float*)srcData, (const float*)dstData,
                                   (const float*)diffData, (float*)gradData));
    return 0;
}

int Layer::lrnForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocDstData(isDynamic) < 0) return -1;
    }
    checkVDNN(vdnn_lrn_fwd(ctx, *stream_compute, n_in, c_in, h_in * w_in, (const float*)srcData, (float*)dstData));
    if (_offloaded[layerId]) offloadSrcData(_offloaded, _offloadedSrcData_h);
    return 0;
}

int Layer::lrnBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch,
                       unsigned long _prefetch_bytes, void*, bool isDynamic) {
    if (vdnnMode != BASELINE) {
        if (cnmemMallocGradData(isDynamic) < 0) return -1;
    }
    if (vdnnMode != BASELINE && _layer_id_to_prefetch >= 0)
        prefetchPreviousSrcData(_prefetchedSrcData_h, _srcDataToPrefetch, _prefetch_bytes);
    checkVDNN(vdnn_lrn_bwd(ctx, *stream_compute, n_in, c_in, h_in * w_in, (const float*)srcData, (const float*)dstData,
                           (const float*)diffData, (float*)gradData));
    return 0;
}

int Layer::concatenateForward() { return 0; }
int Layer::concatenateBackward() { return 0; }

/* layer.cu:925-945. He-normal filter (std sqrt(2 / (c*r*s))), zero bias, from the seeded generator:
 * stream 100 + 2*layerId for the filter. */
void Layer::initializeConvolutionFilterAndBias() {
    const size_t filterDataSize = (size_t)k * c_in * r * s;
    const size_t biasDataSize = (size_t)k;
    ASSERT_EQ(vdnn_pool_malloc(ctx, &filterData, sizeof(DATATYPE) * filterDataSize));
    ASSERT_EQ(vdnn_pool_malloc(ctx, &biasData, sizeof(DATATYPE) * biasDataSize));
    if (settings.skipParameterValues) return;
    std::vector<DATATYPE> filterData_h(filterDataSize), biasData_h(biasDataSize, 0.0f);
    const double fan_in = (double)c_in * r * s;
    vdnn::seeded_fill_normal(filterData_h.data(), filterDataSize, settings.initSeed, 100 + 2 * (uint64_t)layerId, 0.0f, (float)std::sqrt(2.0 / fan_in));
    checkVDNN(vdnn_memcpy_h2d(ctx, filterData, filterData_h.data(), sizeof(DATATYPE) * filterDataSize));
    checkVDNN(vdnn_memcpy_h2d(ctx, biasData, biasData_h.data(), sizeof(DATATYPE) * biasDataSize));
}

/* addition: gradient buffers of a layer with parameters, for an optimizer step outside backward */
void Layer::keepGradients() {
    if (!filterData || filterGrad) return;
    ASSERT_EQ(vdnn_pool_malloc(ctx, &filterGrad, sizeof(DATATYPE) * (size_t)k * c_in * r * s));
    ASSERT_EQ(vdnn_pool_malloc(ctx, &biasGrad, sizeof(DATATYPE) * (size_t)k));
}

int Layer::applyGradients(DATATYPE alpha) {
    if (!filterGrad) return 0;
    checkVDNN(vdnn_sgd_apply(ctx, *stream_compute, (size_t)k * c_in * r * s, alpha, (const float*)filterGrad, (float*)filterData));
    checkVDNN(vdnn_sgd_apply(ctx, *stream_compute, (size_t)k, alpha, (const float*)biasGrad, (float*)biasData));
    return 0;
}

/* layer.cu:947-967 */
void Layer::initializeFullyConnectedFilterAndBias() {
    initializeConvolutionFilterAndBias(); // r = s = 1: the same element counts and fan-in
}

/* layer.cu:969-977: asynchronous D2H of the whole srcData into this layer's pinned buffer. The copy
 * stream first waits for the event that marks srcData as completely written, and signals an event
 * the driver waits on before the block is recycled. */
void Layer::offloadSrcData(bool*, DATATYPE** _offloadedSrcData_h) {
    if (srcPacked) {
        /* the packing kernel runs on a stream of its own, so that it overlaps the copy of the tensor before */
        vdnn_stream_t pack = srcPackedEvent ? vdnn_ctx_stream_pack(ctx) : *stream_memory;
        if (srcReadyEvent) checkVDNN(vdnn_stream_wait_event(ctx, pack, srcReadyEvent));
        checkVDNN(vdnn_zvc_offload_staged_async(ctx, _offloadedSrcData_h[layerId], offloadStaging, offloadStagingBytes, srcData, SrcDataSize(),
                                                actBytes, offloadLengthWord, pack, *stream_memory, srcPackedEvent, offloadKeep ? 1 : 0));
    } else {
        if (srcReadyEvent) checkVDNN(vdnn_stream_wait_event(ctx, *stream_memory, srcReadyEvent));
        checkVDNN(vdnn_memcpy_d2h_async(ctx, _offloadedSrcData_h[layerId], srcData, SrcDataSize() * actBytes, *stream_memory));
    }
    if (offloadDoneEvent) checkVDNN(vdnn_event_record(ctx, offloadDoneEvent, *stream_memory));
}

/* layer.cu:979-987: asynchronous H2D into the freshly allocated srcData of an earlier layer, on the
 * host-to-device stream. It waits until (a) kernels that last used the recycled block have been
 * enqueued before it on the compute stream and finished, (b) the pinned buffer has been filled. */
void Layer::prefetchPreviousSrcData(DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch, unsigned long _prefetch_bytes) {
    vdnn_stream_t h2d = vdnn_ctx_stream_h2d(ctx);
    if (prefetchBlockFreeEvent) {
        checkVDNN(vdnn_event_record(ctx, prefetchBlockFreeEvent, *stream_compute));
        checkVDNN(vdnn_stream_wait_event(ctx, h2d, prefetchBlockFreeEvent));
    }
    if (prefetchHostReadyEvent) checkVDNN(vdnn_stream_wait_event(ctx, h2d, prefetchHostReadyEvent));
    if (prefetchPacked)
        checkVDNN(vdnn_zvc_prefetch_staged_async(ctx, _srcDataToPrefetch, prefetchStaging, prefetchStagingBytes, _prefetchedSrcData_h,
                                                 _prefetch_bytes / actBytes, actBytes, h2d));
    else
        checkVDNN(vdnn_memcpy_h2d_async(ctx, _srcDataToPrefetch, _prefetchedSrcData_h, _prefetch_bytes, h2d));
    if (prefetchDoneEvent) checkVDNN(vdnn_event_record(ctx, prefetchDoneEvent, h2d));
}

void Layer::fetchPackedSrcData(DATATYPE* _packed_h, void* _staging, size_t _bytes) {
    vdnn_stream_t h2d = vdnn_ctx_stream_h2d(ctx);
    if (prefetchBlockFreeEvent) {
        checkVDNN(vdnn_event_record(ctx, prefetchBlockFreeEvent, *stream_compute));
        checkVDNN(vdnn_stream_wait_event(ctx, h2d, prefetchBlockFreeEvent));
    }
    if (prefetchHostReadyEvent) checkVDNN(vdnn_stream_wait_event(ctx, h2d, prefetchHostReadyEvent));
    checkVDNN(vdnn_memcpy_h2d_async(ctx, _staging, _packed_h, _bytes, h2d));
    if (prefetchDoneEvent) checkVDNN(vdnn_event_record(ctx, prefetchDoneEvent, h2d));
}

void Layer::expandPackedSrcData(DATATYPE* _packed_h, const void* _staging, size_t _stagingBytes, vdnn_event_t _blockFilled, vdnn_event_t _hostFilled) {
    if (_blockFilled) checkVDNN(vdnn_stream_wait_event(ctx, *stream_compute, _blockFilled));
    if (_hostFilled) checkVDNN(vdnn_stream_wait_event(ctx, *stream_compute, _hostFilled));
    checkVDNN(vdnn_zvc_prefetch_staged_async(ctx, srcData, _staging, _stagingBytes, _packed_h, SrcDataSize(), actBytes, *stream_compute));
}

/* layer.cu:989-1011 */
int Layer::cnmemMallocSrcData(bool isDynamic) {
    if (ASSERT_EQ(vdnn_pool_malloc(ctx, &srcData, actBytes * SrcDataSize()), isDynamic) < 0) return -1;
    return 0;
}
int Layer::cnmemMallocDstData(bool isDynamic) {
    if (ASSERT_EQ(vdnn_pool_malloc(ctx, &dstData, actBytes * DstDataSize()), isDynamic) < 0) return -1;
    return 0;
}
/* the reference sizes diffData by SrcDataSize (layer.cu:1001-1005); it is only called for the last
 * layer, a softmax, where input and output extents agree */
int Layer::cnmemMallocDiffData(bool isDynamic) {
    if (ASSERT_EQ(vdnn_pool_malloc(ctx, &diffData, actBytes * (SrcDataSize() > DstDataSize() ? SrcDataSize() : DstDataSize())), isDynamic) < 0) return -1;
    return 0;
}
int Layer::cnmemMallocGradData(bool isDynamic) {
    if (ASSERT_EQ(vdnn_pool_malloc(ctx, &gradData, actBytes * SrcDataSize()), isDynamic) < 0) return -1;
    return 0;
}

/* layer.cu:1149-1185 (debug dumps; the reference indexes rows with h*h_out+w, here h*w_out+w) */
void Layer::printDstData() {
    std::vector<DATATYPE> h(DstDataSize());
    if (actBytes == 2) {
        std::vector<uint16_t> raw(h.size());
        checkVDNN(vdnn_memcpy_d2h(ctx, raw.data(), dstData, raw.size() * sizeof(uint16_t)));
        for (size_t i = 0; i < h.size(); i++) h[i] = vdnn::bf16_to_float_host(raw[i]);
    } else {
        checkVDNN(vdnn_memcpy_d2h(ctx, h.data(), dstData, h.size() * sizeof(DATATYPE)));
    }
    printf("Layer %d dstData:\n", layerId);
    for (int n = 0; n < n_out; n++) for (int c = 0; c < c_out; c++) {
        for (int y = 0; y < h_out; y++) {
            for (int x = 0; x < w_out; x++) printf("%g ", h[(((size_t)n * c_out + c) * h_out + y) * w_out + x]);
            printf("\n");
        }
        printf("\n");
    }
}

void Layer::printFilterData() {
    if (!hasParams()) return;
    std::vector<DATATYPE> h(FilterDataSize());
    checkVDNN(vdnn_memcpy_d2h(ctx, h.data(), filterData, h.size() * sizeof(DATATYPE)));
    printf("Layer %d filterData:\n", layerId);
    for (size_t i = 0; i < h.size(); i++) printf("%g%c", h[i], (i + 1) % (size_t)(r * s) == 0 ? '\n' : ' ');
}
