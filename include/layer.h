// One layer of a network: geometry, parameter and activation pointers, forward/backward, the
// offload/prefetch copies. Mirrors the reference's class Layer (layer.h:130-342): same public
// method names, argument order and return convention (0 ok, -1 out of memory when isDynamic).
// Everything device-side is reached through the C ABI of include/vdnn_backend.h; the cuDNN/cuBLAS
// descriptors of the reference have no counterpart (geometry is a plain vdnn_shape_t).
#pragma once
#include <cassert>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "vdnn.h"
#include "vdnn_backend.h"

/* Macro related to kernel execution (layer.h:32) */
#define CEIL(a, b) (((a) + (b) - 1) / (b))

/* Error conventions of layer.h:60-128: assertion-style aborts outside dynamic mode */
#define M_ASSERT(EXPR, MESSAGE)                                                        \
    do {                                                                               \
        if (!(EXPR)) {                                                                 \
            fprintf(stderr, "Assertion failed: %s (%s:%d)\n", MESSAGE, __FILE__, __LINE__); \
            abort();                                                                   \
        }                                                                              \
    } while (0)

#define FatalError(s)                                                                  \
    do {                                                                               \
        fprintf(stderr, "%s\n%s:%d\nAborting...\n", std::string(s).c_str(), __FILE__, __LINE__); \
        exit(EXIT_FAILURE);                                                            \
    } while (0)

/* checkCUDNN / checkCUBLAS / checkCudaErrors / checkCuda collapse into one check of the back end's
 * status (layer.h:72-107) */
#define checkVDNN(status)                                                              \
    do {                                                                               \
        int s_ = (status);                                                             \
        if (s_ != VDNN_OK) {                                                           \
            fprintf(stderr, "vDNN back end failure %d: %s\n", s_, vdnn_last_error());  \
            FatalError("back end failure");                                            \
        }                                                                              \
    } while (0)

/* layer.h:109-128: pool status -> 0 / -1 (out of memory) / -2; aborts outside dynamic mode */
inline int ASSERT_EQ(int result, bool isDynamicMode = false) {
    if (!isDynamicMode) {
        if (result != VDNN_OK) {
            fprintf(stderr, "\n[POOL FAILED with error %d: %s]\n", result, vdnn_last_error());
            abort();
        }
        return 0;
    }
    if (result == VDNN_OOM) return -1;
    if (result == VDNN_OK) return 0;
    return -2;
}

/* The two handle types of the reference's constructors (cudnnHandle_t*, cublasHandle_t*) survive as
 * two distinct thin types over the same back-end context. */
/* Settings every layer made through a handle takes over at construction (addition): the seed of the synthetic
 * initialisation (the reference draws from std::random_device), the per-layer shape dump on stdout of the
 * reference's constructors (layer.cu:96-101, 474-484), and whether parameter values are drawn and uploaded at
 * all (a plan-only network allocates the blocks and leaves them as they are). They travel with the handle, so
 * two networks in one process never see each other's. */
struct vdnnLayerSettings {
    uint64_t initSeed = 0;
    bool     verbose = false;
    bool     skipParameterValues = false;
};
struct vdnnConvHandle_t { vdnn_ctx* ctx; vdnnLayerSettings settings; };
struct vdnnGemmHandle_t { vdnn_ctx* ctx; vdnnLayerSettings settings; };

class Layer {
public:
    Layer(
        vdnn_t            _vdnnMode,
        vdnnAlgoMode_t    _vdnnAlgoMode,
        Layer_t           _layerType,
        vdnnConvHandle_t* _convHandle,
        vdnn_stream_t*    _stream_compute,
        vdnn_stream_t*    _stream_memory,
        int _id,
        int _n, int _c, int _h, int _w,
        int _pad_h, int _pad_w, int _stride_h, int _stride_w,
        int _k, int _r, int _s);
    Layer(
        vdnn_t            _vdnnMode,
        vdnnAlgoMode_t    _vdnnAlgoMode,
        Layer_t           _layerType,
        vdnnGemmHandle_t* _gemmHandle,
        vdnn_stream_t*    _stream_compute,
        vdnn_stream_t*    _stream_memory,
        int _id,
        int _n, int _c, int _h, int _w,
        int _pad_h, int _pad_w, int _stride_h, int _stride_w,
        int _k, int _r, int _s);
    ~Layer();
    Layer(const Layer&) = delete;
    Layer& operator=(const Layer&) = delete;

    uint64_t        InitSeed() const { return settings.initSeed; }
    /* addition: keep dW / db in buffers of their own instead of fusing the SGD step into backward
     * (layer.cu:651-660, 736-761 fuse it); applyGradients then performs the step */
    void            keepGradients();
    int             applyGradients(DATATYPE alpha);
    void*           FilterGrad()             { return filterGrad; }
    void*           BiasGrad()               { return biasGrad; }

    // Seeded initialisation of filter/bias: He-normal filters, zero biases
    void    initializeConvolutionFilterAndBias();
    void    initializeFullyConnectedFilterAndBias();

    // Algorithm selection: memory-optimal (no workspace) or perf-optimal (workspace) kernel variants
    void    findMemOptFwdAlgo();
    void    findMemOptBwdFilterAlgo();
    void    findMemOptBwdDataAlgo();
    void    findPerfOptFwdAlgo();
    void    findPerfOptBwdFilterAlgo();
    void    findPerfOptBwdDataAlgo();
    void    findDynamicAlgo();

    // General fwd/bwd function
    int     forward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     backward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                     void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);

    // CONV layer
    int     convolutionForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     convolutionBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                                void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    /* Addition (recomputeFirstLayer): the forward kernel once more, from this layer's srcData into the given block */
    int     forwardAgainInto(void* into, bool isDynamic);
    void    biasGradientBeside(DATATYPE lr);
    bool    biasGradientInFilterKernel() const;
    void    joinBiasGradient();
    int     convolutionBackwardOverSrc(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                                       void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // FC_GEMM layer
    int     fullyConnectedForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     fullyConnectedBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                                   void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // Activation (RELU) layer
    int     activationForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     activationBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                               void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // SOFTMAX layer
    int     softmaxForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     softmaxBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                            void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // POOL layer
    int     poolingForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     poolingBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                            void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // LRN layer (addition)
    int     lrnForward(bool* _offloaded, DATATYPE** _offloadedSrcData_h, void* workSpace, bool isDynamic);
    int     lrnBackward(int _layer_id_to_prefetch, DATATYPE* _prefetchedSrcData_h,
                        void* _srcDataToPrefetch, unsigned long _prefetch_bytes, void* workSpace, bool isDynamic);
    // CONCATENATE layer (empty in the reference, layer.cu:917-923)
    int     concatenateForward();
    int     concatenateBackward();

    // Offloading and prefetching functions
    void    offloadSrcData(bool* _offloaded, DATATYPE** _offloadedSrcData_h);
    void    prefetchPreviousSrcData(DATATYPE* _prefetchedSrcData_h, void* _srcDataToPrefetch, unsigned long _prefetch_bytes);
    /* additions (compressed offload). fetchPackedSrcData: the copy engine brings the first `bytes` of a packed stream
       from pinned host memory into a block on the device, on the host-to-device stream, ordered like
       prefetchPreviousSrcData. expandPackedSrcData: this layer's srcData is written from its packed stream - the first
       stagingBytes of it in a block on the device, the rest (if any) in pinned host memory - by a kernel on the compute
       stream, behind the events given (the copy that filled the block, the offload that filled the host buffer). */
    void    fetchPackedSrcData(DATATYPE* _packed_h, void* _staging, size_t _bytes);
    void    expandPackedSrcData(DATATYPE* _packed_h, const void* _staging, size_t _stagingBytes, vdnn_event_t _blockFilled, vdnn_event_t _hostFilled);

    // Allocate device memory from the pool (the reference's names, layer.cu:989-1011)
    int     cnmemMallocSrcData(bool isDynamic);
    int     cnmemMallocDstData(bool isDynamic);
    int     cnmemMallocDiffData(bool isDynamic);
    int     cnmemMallocGradData(bool isDynamic);

    // Copy pointers
    void    copySrcData(void* _srcData)   { srcData = _srcData;   }
    void    copyDstData(void* _dstData)   { dstData = _dstData;   }
    void    copyDiffData(void* _diffData) { diffData = _diffData; }
    void    copyGradData(void* _gradData) { gradData = _gradData; }

    /* Set functions */
    void    setVdnnMode(vdnn_t _vdnnMode) { vdnnMode = _vdnnMode; }
    // ReLU only: backward writes dx over dy instead of into a freshly allocated gradData
    void    setInPlaceOp(bool v) { inPlaceOp = v; }
    /* Addition: a ReLU fused into its neighbours. The producing CONV / FC layer rectifies in its own
       kernel (setFuseRelu); the RELU layer then launches nothing in forward and its dstData is its
       srcData (setElided). Where the consumer's backward zeroes its gradData at non-positive inputs
       (setGateGrad), the RELU layer launches nothing in backward either (setElidedBackward). */
    void    setFuseRelu(bool v) { fuseRelu = v; }
    bool    FuseRelu() const { return fuseRelu; }
    void    setElided(bool v);
    bool    Elided() const { return elided; }
    void    setElidedBackward(bool v) { elidedBackward = v; }
    bool    ElidedBackward() const { return elidedBackward; }
    void    setGateGrad(bool v) { gateGrad = v; }
    bool    GateGrad() const { return gateGrad; }
    bool    InPlaceOp() const { return inPlaceOp; }
    /* Addition: backward writes gradData over srcData (CONV with stride 1 and more than four input channels, 2x2 /
       stride 2 POOL): gradData then *is* srcData and no block is taken for it. The Network sets it where the layer
       below does not read that tensor in its own backward. */
    void    setGradOverSrc(bool v) { gradOverSrc = v; }
    bool    GradOverSrc() const { return gradOverSrc; }
    bool    canGradOverSrc() const;
    void    setAlgoMode(vdnnAlgoMode_t m);
    // Event the offload copy waits for (srcData fully written) and the events this layer's copies
    // signal; owned by the Network. Null events mean "no ordering needed" (plan-only contexts).
    void    setSrcReadyEvent(vdnn_event_t e)     { srcReadyEvent = e; }
    void    setOffloadDoneEvent(vdnn_event_t e)  { offloadDoneEvent = e; }
    void    setPrefetchEvents(vdnn_event_t blockFree, vdnn_event_t hostReady, vdnn_event_t done) {
        prefetchBlockFreeEvent = blockFree; prefetchHostReadyEvent = hostReady; prefetchDoneEvent = done;
    }
    // This layer's offloaded input / the tensor this layer fetches next crosses the link without its zeros.
    // The event behind which this layer's prefetched srcData is complete (null: it never left). Backward waits
    // for it in front of the first kernel that reads srcData: for a CONV / FC layer that is the filter gradient
    // (or backward data, if that masks by the input), so the data gradient runs while the copy still lands.
    void    setSrcFetchedEvent(vdnn_event_t e)   { srcFetchedEvent = e; }
    void    setSrcPacked(bool on)                { srcPacked = on; }
    bool    SrcPacked() const                    { return srcPacked; }
    void    setPrefetchPacked(bool on)           { prefetchPacked = on; }
    // Where the packed stream of this layer's input is staged on its way out (bytes may be 0: the kernel stores
    // all of it into host memory itself), the pinned word that receives its length, and the event recorded when
    // the packing kernel has read srcData.
    // With `keep` the staging block is where the stream stays (no copy to the host but of what did not fit).
    void    setOffloadStaging(void* staging, size_t bytes, unsigned long long* lengthWord, vdnn_event_t packed, bool keep) {
        offloadStaging = staging; offloadStagingBytes = bytes; offloadLengthWord = lengthWord; srcPackedEvent = packed;
        offloadKeep = keep;
    }
    // The block that holds the first bytes of the packed stream this layer fetches next (null: all of it is on the host).
    void    setPrefetchStaging(void* staging, size_t bytes) { prefetchStaging = staging; prefetchStagingBytes = bytes; }

    /* Get functions */
    Layer_t LayerType()              { return layerType; }
    int     LayerId()                { return layerId; }
    void*   SrcData()                { return srcData;  }
    void*   DstData()                { return dstData;  }
    void*   DiffData()               { return diffData; }
    void*   GradData()               { return gradData; }
    void*   FilterData()             { return filterData; }
    void*   BiasData()               { return biasData; }
    int     InputN()                 { return n_in;  }
    int     InputC()                 { return c_in;  }
    int     InputH()                 { return h_in;  }
    int     InputW()                 { return w_in;  }
    int     OutputN()                { return n_out; }
    int     OutputC()                { return c_out; }
    int     OutputH()                { return h_out; }
    int     OutputW()                { return w_out; }
    // element counts are size_t: the reference's int overflows from VGG16 batch 256 on (layer.h:240)
    size_t  SrcDataSize()            { return (size_t)n_in * c_in * h_in * w_in;      }
    size_t  DstDataSize()            { return (size_t)n_out * c_out * h_out * w_out;  }
    size_t  FwdWorkSpaceSize()       { return fwdWorkSpaceSize;       }
    size_t  BwdDataWorkSpaceSize()   { return bwdDataWorkSpaceSize;   }
    size_t  BwdFilterWorkSpaceSize() { return bwdFilterWorkSpaceSize; }
    size_t  FilterDataSize()         { return hasParams() ? (size_t)k * c_in * r * s : 0; }
    size_t  BiasDataSize()           { return hasParams() ? (size_t)c_out : 0; }
    bool    hasParams() const        { return layerType == FC_GEMM || layerType == CONV || layerType == FC_CONV; }
    const vdnn_shape_t& Shape() const { return shape; }
    vdnnAlgoMode_t AlgoMode() const  { return vdnnAlgoMode; }
    vdnnConvHandle_t* ConvHandle()   { return convHandle; }
    vdnnGemmHandle_t* GemmHandle()   { return gemmHandle; }
    int     RefCntFwd()              { return refCntFwd; }
    int     RefCntBwd()              { return refCntBwd; }

    /* Reference Count Management (unused by the three networks, kept for interface parity) */
    void    decrementRefCntFwd()  { assert(refCntFwd > 0);  refCntFwd--; }
    void    decrementRefCntBwd()  { assert(refCntBwd > 0);  refCntBwd--; }

    /* For debugging */
    void    printDstData();
    void    printFilterData();

private:
    void    construct(vdnn_ctx* _ctx, const vdnnLayerSettings& _settings);
    int     mallocWorkSpace(void* shared, size_t bytes, void** cur, bool isDynamic);
    void    freeWorkSpace(void* shared, size_t bytes, void* cur, bool isDynamic);

    vdnnLayerSettings settings; // copied from the handle the layer was made through

    /* General layer info */
    vdnn_t         vdnnMode;
    vdnnAlgoMode_t vdnnAlgoMode;
    Layer_t        layerType;
    int            layerId;
    vdnn_ctx*      ctx;

    /* Input NCHW, filter, output NCHW */
    int n_in, c_in, h_in, w_in;
    int pad_h, pad_w, stride_h, stride_w, k, r, s;
    int n_out, c_out, h_out, w_out;
    vdnn_shape_t shape;

    /* Workspace size */
    size_t fwdWorkSpaceSize, bwdDataWorkSpaceSize, bwdFilterWorkSpaceSize;

    /* Streams */
    vdnn_stream_t* stream_compute;
    vdnn_stream_t* stream_memory;

    /* Pointers to memory (data) */
    void* srcData;    // x
    void* filterData; // w
    void* biasData;   // bias
    size_t actBytes;  // bytes per activation element (the context's activation dtype)
    void* filterGrad; // dW (only with keepGradients)
    void* biasGrad;   // db
    void* dstData;    // y
    void* diffData;   // dy
    void* gradData;   // dx

    /* Ordering of the copies */
    vdnn_event_t srcReadyEvent, offloadDoneEvent;
    vdnn_event_t prefetchBlockFreeEvent, prefetchHostReadyEvent, prefetchDoneEvent;
    vdnn_event_t srcFetchedEvent = nullptr;
    void    waitSrcFetched();
    bool    srcPacked = false, prefetchPacked = false;
    void*   offloadStaging = nullptr;
    size_t  offloadStagingBytes = 0;
    unsigned long long* offloadLengthWord = nullptr;
    bool    offloadKeep = false;
    void*   prefetchStaging = nullptr;
    size_t  prefetchStagingBytes = 0;
    vdnn_event_t srcPackedEvent = nullptr;

    /* Connection to other layers (GoogLeNet plumbing of the reference, unused) */
    std::vector<int> producerLayerId, consumerLayerId;
    int  refCntFwd, refCntBwd;
    bool inPlaceOp, insideInceptionModule, headOfFork, tailOfFork;
    bool fuseRelu, elided, elidedBackward, gateGrad;
    bool gradOverSrc = false;
    vdnn_event_t evBiasFork = nullptr, evBiasJoin = nullptr; // order the bias gradient's stream against the compute stream
    int  forkId, concatenateChannelOffset;

    vdnnConvHandle_t* convHandle;
    vdnnGemmHandle_t* gemmHandle;
};
