// Network: layer tables, memory-policy setup, forward/backward drivers and the prefetch scheduler.
// Mirrors the reference's class Network (network.h:15-95): same public method names and return
// convention. Additions (marked) cover what the reference cannot do: seeded data, a loss value,
// tensor capture for parity checks, usage statistics, real teardown.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "layer.h"

/* Optional settings of a Network (addition). The reference's constructor takes none of these. */
struct NetworkOptions {
    uint64_t seed = 1;           // seed of inputs, labels and filters
    size_t   poolBytes = 0;      // size of the device pool; 0 = sized from the layer table
    size_t   capBytes = 0;       // artificial limit on pool bytes in use; 0 = none
    bool     planOnly = false;   // replay the allocation schedule without a device
    bool     hostSync = false;   // synchronise both streams after every layer like the reference
                                 // (network.cu:1090-1091, 1168-1169) instead of ordering by events
    bool     capture = false;    // keep host copies of every layer's dstData and gradData
    bool     verbose = false;    // the reference's per-layer printouts
    // Value-preserving lifetime refinements of the vDNN policies (off = the reference's literal
    // schedule): (1) a tensor no backward kernel reads is released instead of kept or offloaded:
    // the input of a ReLU layer, whose backward needs only its output (y > 0 selects the same
    // elements as x > 0); (2) the output of a convolution, FC or pooling layer is released before
    // that layer's backward instead of after it (those backward kernels never read y);
    // (3) a ReLU layer writes dx over dy instead of into a new block.
    bool     refinedLifetimes = false;
    // Keep every layer's dW / db in buffers of their own and perform the SGD step after the last
    // backward layer (applyGradients) instead of inside the backward kernels as the reference does
    // (layer.cu:651-660, 736-761). Same bits as the fused step; what a data-parallel exchange or
    // another optimizer needs. deferOptimizer leaves the step to the caller.
    // Element type of activation tensors (layer inputs, outputs, their gradients, the network input and
    // target): VDNN_DTYPE_F32 as in the reference (vdnn.h:11-12) or VDNN_DTYPE_BF16, which halves device
    // memory and offload traffic. Parameters and their gradients stay float (the master copy is what the
    // kernels read), arithmetic and accumulation are float, results are rounded once when stored.
    int      dataType = VDNN_DTYPE_F32;
    // Scheduling slack of the offloading policies (0 / 1 = the reference's schedule; values unchanged, only
    // lifetimes). offloadLag: the block of an offloaded srcData is recycled - and the compute stream made to
    // wait for its device-to-host copy - only after `offloadLag` further layers have been enqueued, so a
    // copy that is longer than its own layer's kernels overlaps the following layers instead of stalling
    // them. prefetchDepth: up to that many offloaded tensors below the current layer are in flight or
    // resident ahead of their backward (the reference fetches one, network.cu:1193-1208).
    int      offloadLag = 0;        // negative with hbmBudgetBytes: the placement plan chooses the lag as well (0 otherwise)
    int      prefetchDepth = 1;
    bool     unfusedOptimizer = false;
    bool     deferOptimizer = false;
    // A ReLU layer that follows a CONV / FC layer is applied by that layer's own kernel, and its backward
    // by the backward of the CONV / FC / POOL layer that consumes it (where one does); the ReLU layer then
    // launches nothing and owns no tensor: its dstData is its srcData and its gradData its diffData. Same
    // bits as the separate layers of the reference (layer.cu:766-814); two passes over the tensor fewer.
    // Such a ReLU layer is never offloaded (its input is not a tensor of its own any more).
    bool     fuseActivations = false;
    // Offloaded tensors that hold rectified values (the output of a ReLU, also behind max-pool and LRN
    // layers, which keep zeros zero) cross the link to host memory without their zero elements: a kernel on
    // the copy stream compacts the tensor into the pinned buffer and another expands it on the way back.
    // Lossless; the reference copies every tensor whole (layer.cu:969-987). Other tensors are copied as before.
    bool     compressOffload = false;
    // The deepest tensors that the policy would offload stay on the device instead, as many as fit in this
    // many bytes counted from the last layer down. They are the last into the copy queue and the first that
    // backward asks for, so offloading them makes backward wait for the queue to drain, and they are small and
    // gone before the large tensors of the shallow layers come back: the peak is elsewhere. 0: the reference's
    // policies (network.cu:898-921).
    size_t   keepTailBytes = 0;
    // With compressOffload: the packed stream of a tensor stays in its staging block on the device instead of
    // going to the host, and backward expands it from there; the link carries only what a block sized from the
    // step before could not hold. Trades the link for HBM: a rectified tensor then occupies about 0.6 of its size
    // between its forward and its backward, at the price of reading and writing it once more each way.
    bool     keepPackedOnDevice = false;
    // What a plan-only context assumes a packed stream to be of its tensor (it has no data): 0 = the longest
    // possible stream, 1.03 of the tensor.
    double   planPackedFraction = 0.0;
    // Backward fetches further tensors ahead whenever that cannot raise the step's peak: the network replays
    // its own schedule on a context without a device, notes the bytes in use during every layer's backward,
    // and fetches a tensor early only if, at every layer between here and the layer that would have fetched
    // it, those bytes plus everything fetched early stay at or below the replay's highest value (or below what
    // the pool has already held, this step's forward for one, if that is more). The large
    // tensors of the shallow layers then start their way back while the small deep layers run, whose working
    // set is far below the peak. Same values, same peak, fewer waits for the link.
    bool     prefetchWithinPeak = false;
    // A limit on pool bytes in use that the policy has to meet, instead of an offload set fixed by the policy's name
    // (network.cu:898-936 offloads every member whatever the device could hold). With a budget, every member of the
    // policy's offload set gets the cheapest of three places that keeps a replay of the schedule within the budget:
    // it stays on the device as it is, it stays on the device as a packed stream (needs compressOffload and a
    // rectified tensor), or it crosses the link (packed where it can be). Tensors are moved one place down, the
    // largest one that is stored at the moment of the replay's peak first, until the replay fits; if it never does,
    // the last plan stands and Network::planFeasible() says so. The replay has no data: planPackedFraction is what it
    // takes a packed stream to be of its tensor. 0: no budget, the policy's own offload set.
    size_t   hbmBudgetBytes = 0;
    // With hbmBudgetBytes: how many bytes per step and direction the plan may send over the host link BEFORE it packs
    // anything on the device. The planner's own order is the other way round (a stream on the device costs two passes
    // at HBM speed, the link a hundred times that), which leaves the link idle until the budget forces a tensor out. A
    // step whose kernels take T seconds can hide about T x 56 GB/s each way if the copies are spread well: with this
    // many bytes allowed, the members that must leave the device go over the link first (the largest gain first, a
    // rectified tensor as its packed stream, counted at planPackedFraction of its size), and are packed on the device
    // only once the allowance is used up. 0: pack first (the planner's own order).
    size_t   planLinkBytes = 0;
    // Backward writes a layer's input gradient over the layer's own input where nothing reads that input again: a
    // convolution (stride 1, more than four input channels) computes its filter gradient first, into a block of the
    // filter's size, then the data gradient - still with the old filter, as layer.cu:616-660 has it - over its
    // srcData, then applies the update (param += alpha * grad, the fused call's arithmetic: same bits); a 2x2 / stride 2
    // max-pool reads its two windows and writes them back. The layer below must be one whose backward does not read
    // its own output (with refinedLifetimes: convolution, FC, pooling, or a ReLU that is fused away), and the filter
    // must be smaller than the input (or the block for its gradient would outweigh the one saved). The reference
    // holds x, dy and dx of a layer together (layer.cu:599, 999-1011); here the largest layer holds two of them.
    // Needs refinedLifetimes; not BASELINE (whose dx/dy pair is shared by all layers).
    bool     inPlaceBackward = false;
    // The output of a first layer that is a convolution over at most four input channels (half a millisecond for
    // VGG16's, against 16 ms on the link or 1.6 GB of device memory for the tensor) is released once its consumer's
    // forward has read it and computed again, by the same kernel from the same filter (layer 0's update comes last), into
    // a fresh block just before the consumer's backward: the same bits. The network input then stays on the device
    // whatever the policy says. Applies where the consumer is layer 1, or layer 2 behind a ReLU that layer 0 applies
    // itself (fuseActivations); needs refinedLifetimes; not BASELINE. The reference keeps or offloads every such
    // tensor (network.cu:916-936).
    bool     recomputeFirstLayer = false;
    std::vector<unsigned char> forcedPlacement; // (internal: the replay's placement per layer, see Placement)
    bool     tracePeaks = false;          // (internal: the replay records bytes in use per forward and backward layer)
    int      device = DEFAULT_DEVICE;
};

/* One row of a layer table (the argument list of the reference's Layer constructor). */
struct LayerSpec {
    Layer_t type;
    int n, c, h, w;
    int pad_h, pad_w, stride_h, stride_w;
    int k, r, s;
    bool forceMemOpt; // OverFeat's FC-as-conv layers ignore the algorithm mode (network.cu:449, 465, 481)
};

/* Per-step statistics (addition). */
struct NetworkStats {
    size_t peakBytesInUse = 0;     // pool high-water mark (bytes in use)
    size_t peakExtent = 0;         // highest pool offset handed out
    size_t offloadBytes = 0;       // bytes copied device-to-host by the last forward
    size_t prefetchBytes = 0;      // bytes copied host-to-device by the last backward
    size_t pinnedBytes = 0;        // pinned host memory held for offloaded tensors
    size_t poolBytes = 0;
    size_t weightBytes = 0;
};

/* Where a member of the policy's offload set waits between its forward and its backward (addition, see
 * NetworkOptions::hbmBudgetBytes). */
enum Placement : unsigned char {
    PLACE_POLICY   = 0, // no plan: what the policy and the other options say
    PLACE_RESIDENT = 1, // on the device, as it is
    PLACE_PACKED   = 2, // on the device, as a packed stream
    PLACE_LINK     = 3, // in pinned host memory
};

class Network {
public:
    Network(
        CNN_t          _cnnType,
        vdnn_t         _vdnnType,
        vdnnAlgoMode_t _algoMode,
        int            _batchSize = DEFAULT_BATCH_SIZE);
    /* addition: explicit options */
    Network(CNN_t _cnnType, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode, int _batchSize, const NetworkOptions& _options);
    /* addition: a network from an explicit layer table (the reference's CUSTOM_CNN is an empty stub) */
    Network(const std::vector<LayerSpec>& table, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode, const NetworkOptions& _options);
    ~Network();
    Network(const Network&) = delete;
    Network& operator=(const Network&) = delete;

    /* Reset network */
    void            reset(CNN_t _cnnType, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode);

    /* Setup */
    void            setLayers(CNN_t _cnnType);
    void            setLayersAlexnet();
    void            setLayersOverfeat();
    void            setLayersGooglenet();
    bool            fusesRelu(int l) const;
    bool            srcIsRectified(int l) const;
    void            setLayersVgg16(int givenBatch);
    void            setLayersCustomCNN();
    void            randomInitializeData(void* data, size_t size);
    void            sanityCheck();
    void            setVdnnType(vdnn_t newVdnnType);
    void            setAlgoType(vdnnAlgoMode_t newAlgoMode);
    void            vdnnDynamicAlgo();

    /* Find max dx, dy, workspace size (bytes) */
    size_t          findMaxDxDySize();
    size_t          findMaxWorkSpaceSize();

    /* Computation for training network */
    void            calculateFirstDiffData(void* result, void* first, void* second);
    int             forwardPropagation(bool isDynamic = false);
    int             backwardPropagation(bool isDynamic = false);

    /* Find prefetch layer */
    void            resetIsPrefetchedArray();
    int             findPrefetchLayer(int currLayerId);
    int             findPrefetchLayerDeep(int currLayerId); /* addition: see NetworkOptions::prefetchDepth */

    /* Get functions */
    Layer**         layerArray()            { return layer;              }
    DATATYPE**      offloadedSrcDataArray() { return offloadedSrcData_h; }
    size_t          getInputSize()          { return (size_t)n_in * c_in * h_in * w_in;     }
    size_t          getOutputSize()         { return (size_t)n_out * c_out * h_out * w_out; }

    /* ---- additions ---- */
    int             numLayersCount() const  { return numLayers; }
    int             batch() const           { return batchSize; }
    vdnn_t          policy() const          { return vdnnType; }
    vdnnAlgoMode_t  algo() const            { return algoMode; }
    vdnn_ctx*       context()               { return ctx; }
    bool            isOffloaded(int l) const { return isOffload[l]; }
    // recomputeFirstLayer: the layer whose input is computed again before its backward (-1: none)
    int             recomputedSrcLayer() const { return recomputedLayer; }
    // inPlaceBackward: layer l's backward writes its input gradient over its input
    bool            gradOverSrc(int l) const { return l >= 0 && l < numLayers && layer[l] && layer[l]->GradOverSrc(); }
    // synthetic data: N(0,1) input, integer labels in [0, classes) as a one-hot target, seeded filters
    void            setInput(const float* host);
    void            setLabels(const int32_t* labels);
    void            setLabelTensor(const float* host);
    void            getInput(float* host);
    int             setLayerParams(int l, const float* filter, const float* bias);
    int             getLayerParams(int l, float* filter, float* bias);
    // mean cross-entropy of the last forward's output against the target (waits for the device)
    float           loss();
    // the optimizer step of unfusedOptimizer: w += (-lr) * dW, b += (-lr) * db for every layer
    int             applyGradients();
    int             getLayerGradients(int l, float* filter, float* bias);
    // `steps` training steps (forward, backward, optimizer); returns the loss before each step's update
    std::vector<float> train(int steps, bool isDynamic = false);
    void            synchronize();
    NetworkStats    stats();
    void            resetPeak();
    // host copies of dstData / gradData of layer l taken during the last step (options.capture)
    const std::vector<float>& capturedDst(int l) const { return capDst[l]; }
    const std::vector<float>& capturedGrad(int l) const { return capGrad[l]; }
    // the sequence (backward layer, prefetched layer) of the last backward
    const std::vector<std::pair<int, int>>& prefetchTrace() const { return prefetchLog; }
    const std::vector<size_t>& backwardPeakTrace() const { return bwdPeakTrace; }
    const std::vector<size_t>& forwardPeakTrace() const { return fwdPeakTrace; }
    // hbmBudgetBytes: the place each layer's input got (PLACE_POLICY for layers outside the offload set), whether the
    // replay met the budget, what it peaked at, and the bytes the plan sends over the link each way per step
    Placement       placementOf(int l) const { return l >= 0 && l < (int)placement.size() ? (Placement)placement[l] : PLACE_POLICY; }
    bool            planFeasible() const { return planFeasibleFlag; }
    size_t          planPeakBytes() const { return planBudgetPeak; }
    // the offload lag the step runs with: offloadLag, or - where that is negative - the one the placement plan chose
    int             offloadLagInUse() const { return options.offloadLag >= 0 ? options.offloadLag : plannedLag; }
    const std::vector<LayerSpec>& table() const { return specs; }
    static std::vector<LayerSpec> tableFor(CNN_t cnn, int batch);

private:
    void            construct(vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode);
    void            initPool();
    void            buildLayers();
    void            releaseLayers();
    void            releasePolicyBuffers();
    void            allocIoBuffers();
    void            captureLayer(int l, bool grad);
    size_t          actBytes() const { return options.dataType == VDNN_DTYPE_BF16 ? 2 : 4; }
    void            uploadActivations(void* dev, const float* host, size_t count);
    void            downloadActivations(float* host, const void* dev, size_t count);
    void            afterLayerSync();
    void            printUsage(const char* tag, int l, size_t workspace);

    CNN_t               cnnType;
    vdnn_t              vdnnType;
    vdnnAlgoMode_t      algoMode;
    NetworkOptions      options;
    vdnn_ctx*           ctx;
    vdnnConvHandle_t    convHandle;   // in place of cudnnHandle
    vdnnGemmHandle_t    gemmHandle;   // in place of cublasHandle
    vdnn_stream_t       stream_compute;
    vdnn_stream_t       stream_memory; // device-to-host copies; host-to-device copies use the context's third stream
    int                 batchSize;
    int                 numLayers;
    bool                customTable;

    /* Input / Output */
    int n_in, c_in, h_in, w_in;
    int n_out, c_out, h_out, w_out;

    /* Data */
    void*               inputData;
    void*               labelData;
    void*               networkDiffData;
    void*               networkGradData;
    void*               workSpace;
    float*              lossData;          // one float on the device (addition)
    std::vector<float>  inputHost;         // the seeded input, kept for re-upload (addition)

    /* Layers */
    std::vector<LayerSpec> specs;
    Layer*              layer[DEFAULT_NUM_LAYER];
    bool                isOffload[DEFAULT_NUM_LAYER];
    bool                isPrefetched[DEFAULT_NUM_LAYER];
    bool                dropSrcAfterFwd[DEFAULT_NUM_LAYER]; // refined lifetimes: srcData is dead after forward
    int                 recomputedLayer = -1;               // recomputeFirstLayer: the layer whose srcData layer 0 computes again in backward
    DATATYPE*           offloadedSrcData_h[DEFAULT_NUM_LAYER];

    /* Events that order the copy streams against the compute stream (addition) */
    vdnn_event_t        evFwdDone[DEFAULT_NUM_LAYER];     // compute: layer l's forward kernels enqueued
    vdnn_event_t        evOffloadDone[DEFAULT_NUM_LAYER]; // d2h: srcData of layer l is in pinned memory
    vdnn_event_t        evBlockFree[DEFAULT_NUM_LAYER];   // compute: everything enqueued before the prefetch of l
    vdnn_event_t        evPrefetchDone[DEFAULT_NUM_LAYER];// h2d: srcData of layer l is back on the device
    /* compressOffload: the packed stream of an offloaded input waits in device memory for the copy engine */
    vdnn_event_t        evPacked[DEFAULT_NUM_LAYER];      // d2h: the packing kernel has read srcData of layer l
    void*               zvcStaging[DEFAULT_NUM_LAYER];    // staging block of layer l's stream (null: none this step)
    size_t              zvcStagingBytes[DEFAULT_NUM_LAYER];
    size_t              zvcLengthSeen[DEFAULT_NUM_LAYER] = {};   // the stream length a step's forward sized its block from (0: none known)
    bool                zvcKept[DEFAULT_NUM_LAYER];       // the block holds the stream until layer l's backward has expanded it
    bool                zvcFetched[DEFAULT_NUM_LAYER];    // ... and was filled by a copy from host memory during this backward
    bool                srcReleasedEarly[DEFAULT_NUM_LAYER]; // srcData of layer l went back to the pool behind its forward
    unsigned long long* zvcLength_h;                       // pinned: length of each layer's stream, reported by the packing kernel
    std::vector<int>    pendingOffload;                    // offloaded layers whose block is not yet recycled (offloadLag)
    bool                inputResident;                     // inputData currently holds the input (addition)

    NetworkStats        lastStats;
    std::vector<std::vector<float>> capDst, capGrad;
    std::vector<std::pair<int, int>> prefetchLog;
    /* prefetchWithinPeak: from the replay - bytes in use during backward of each layer, their highest value, the
       layer whose backward fetches each offloaded tensor; and what this backward has fetched ahead of that */
    std::vector<size_t> bwdPeakTrace, fwdPeakTrace, planBwdPeak, fetchedAhead;
    /* hbmBudgetBytes */
    std::vector<unsigned char> placement;
    bool                keepPackedLayer[DEFAULT_NUM_LAYER]; // the packed stream of layer l's input stays on the device
    bool                planFeasibleFlag = true;
    size_t              planBudgetPeak = 0;
    int                 plannedLag = 0;
    std::vector<unsigned char> planPlacement(vdnn_t policy, const std::vector<bool>& member);
    std::vector<int>    planIssueLayer;
    size_t              planPeak = 0, peakBudget = 0;
    void                buildPeakPlan(vdnn_t policy);
    int                 findPrefetchWithinPeak(int currLayerId);
    size_t              stagedFetchBytes(int id) const;
    int                 fetchPackedToStaging(int issuingLayer, int id, bool isDynamic);
};
