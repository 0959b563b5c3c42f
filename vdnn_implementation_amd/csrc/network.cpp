// Network: tables, policy setup, forward/backward drivers, prefetch scheduler.
// Control flow follows the reference's network.cu (cited per function). Differences that change no
// value: copies are ordered against compute with events instead of two host-side stream syncs per
// layer (options.hostSync restores those), byte counts are size_t, the input block is released after
// its offload like every other offloaded tensor (the reference leaks one input-sized block per
// step, network.cu:1156/1185), and everything is torn down in the destructor.
#include "network.h"

#include <algorithm>
#include <cmath>
#include <cstring>

#include "seeded_init.h"

namespace {

bool is_conv(Layer_t t) { return t == FC_CONV || t == CONV; }

struct TableBuilder {
    std::vector<LayerSpec>& t;
    int n;
    void conv(int c, int hw, int pad, int stride, int k, int r, bool forceMemOpt = false) {
        t.push_back(LayerSpec{FC_CONV, n, c, hw, hw, pad, pad, stride, stride, k, r, r, forceMemOpt});
    }
    void relu(int c, int hw) { t.push_back(LayerSpec{RELU, n, c, hw, hw, 0, 0, 0, 0, 0, 0, 0, false}); }
    void lrn(int c, int hw) { t.push_back(LayerSpec{LRN, n, c, hw, hw, 0, 0, 0, 0, 0, 0, 0, false}); }
    void pool(int c, int hw, int win) { t.push_back(LayerSpec{POOL, n, c, hw, hw, 0, 0, 2, 2, 0, win, win, false}); }
    void fc(int cin, int cout) { t.push_back(LayerSpec{FC_GEMM, n, cin, 1, 1, 0, 0, 0, 0, cout, 1, 1, false}); }
    void softmax(int c) { t.push_back(LayerSpec{SOFTMAX, n, c, 1, 1, 0, 0, 0, 0, 0, 0, 0, false}); }
};

/* network.cu:156-323 (19 layers); withLrn adds conv-ReLU-LRN-pool normalisation after the first two
 * convolutions (21 layers) */
void table_alexnet(std::vector<LayerSpec>& t, int n, bool withLrn) {
    TableBuilder b{t, n};
    b.conv(3, 227, 0, 4, 96, 11);  b.relu(96, 55);  if (withLrn) b.lrn(96, 55);  b.pool(96, 55, 3);
    b.conv(96, 27, 2, 1, 256, 5);  b.relu(256, 27); if (withLrn) b.lrn(256, 27); b.pool(256, 27, 3);
    b.conv(256, 13, 1, 1, 384, 3); b.relu(384, 13);
    b.conv(384, 13, 1, 1, 384, 3); b.relu(384, 13);
    b.conv(384, 13, 1, 1, 256, 3); b.relu(256, 13); b.pool(256, 13, 3);
    b.fc(9216, 4096); b.relu(4096, 1);
    b.fc(4096, 4096); b.relu(4096, 1);
    b.fc(4096, 1000); b.softmax(1000);
}

/* network.cu:325-495: the three classifier layers are convolutions pinned to the memory-optimal mode */
void table_overfeat(std::vector<LayerSpec>& t, int n) {
    TableBuilder b{t, n};
    b.conv(3, 231, 0, 4, 96, 11);    b.relu(96, 56);   b.pool(96, 56, 2);
    b.conv(96, 28, 0, 1, 256, 5);    b.relu(256, 24);  b.pool(256, 24, 2);
    b.conv(256, 12, 1, 1, 512, 3);   b.relu(512, 12);
    b.conv(512, 12, 1, 1, 1024, 3);  b.relu(1024, 12);
    b.conv(1024, 12, 1, 1, 1024, 3); b.relu(1024, 12); b.pool(1024, 12, 2);
    b.conv(1024, 6, 0, 1, 3072, 6, true); b.relu(3072, 1);
    b.conv(3072, 1, 0, 1, 4096, 1, true); b.relu(4096, 1);
    b.conv(4096, 1, 0, 1, 1000, 1, true); b.softmax(1000);
}

/* network.cu:501-813 */
void table_vgg16(std::vector<LayerSpec>& t, int n) {
    TableBuilder b{t, n};
    const int stages[5][3] = {{64, 2, 224}, {128, 2, 112}, {256, 3, 56}, {512, 3, 28}, {512, 3, 14}}; // channels, convs, extent
    int c = 3;
    for (const auto& st : stages) {
        for (int i = 0; i < st[1]; i++) { b.conv(c, st[2], 1, 1, st[0], 3); b.relu(st[0], st[2]); c = st[0]; }
        b.pool(st[0], st[2], 2);
    }
    b.fc(512 * 7 * 7, 4096); b.relu(4096, 1);
    b.fc(4096, 4096);        b.relu(4096, 1);
    b.fc(4096, 1000);        b.softmax(1000);
}

size_t spec_src_count(const LayerSpec& s) { return (size_t)s.n * s.c * s.h * s.w; }

void spec_out(const LayerSpec& s, int& n, int& c, int& h, int& w) {
    n = s.n;
    switch (s.type) {
    case FC_GEMM: c = s.k; h = 1; w = 1; break;
    case CONV: case FC_CONV: c = s.k; h = vdnn_out_dim(s.h, s.pad_h, s.r, s.stride_h); w = vdnn_out_dim(s.w, s.pad_w, s.s, s.stride_w); break;
    case POOL: c = s.c; h = vdnn_out_dim(s.h, s.pad_h, s.r, s.stride_h); w = vdnn_out_dim(s.w, s.pad_w, s.s, s.stride_w); break;
    default: c = s.c; h = s.h; w = s.w; break;
    }
}

size_t spec_dst_count(const LayerSpec& s) {
    int n, c, h, w;
    spec_out(s, n, c, h, w);
    return (size_t)n * c * h * w;
}

} // namespace

std::vector<LayerSpec> Network::tableFor(CNN_t cnn, int batch) {
    std::vector<LayerSpec> t;
    switch (cnn) {
    case ALEXNET: table_alexnet(t, batch, false); break;
    case ALEXNET_LRN: table_alexnet(t, batch, true); break;
    case OVERFEAT: table_overfeat(t, batch); break;
    case VGG16_64: case VGG16_128: case VGG16_256: case VGG16_512: table_vgg16(t, batch); break;
    default: break; // GOOGLENET and CUSTOM_CNN are empty stubs in the reference (network.cu:497-499, 815-817)
    }
    return t;
}

Network::Network(CNN_t _cnnType, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode, int _batchSize)
    : cnnType(_cnnType), options(), batchSize(_batchSize), customTable(false) {
    construct(_vdnnType, _algoMode);
}

Network::Network(CNN_t _cnnType, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode, int _batchSize, const NetworkOptions& _options)
    : cnnType(_cnnType), options(_options), batchSize(_batchSize), customTable(false) {
    construct(_vdnnType, _algoMode);
}

Network::Network(const std::vector<LayerSpec>& table, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode, const NetworkOptions& _options)
    : cnnType(CUSTOM_CNN), options(_options), batchSize(table.empty() ? 0 : table[0].n), customTable(true), specs(table) {
    construct(_vdnnType, _algoMode);
}

/* network.cu:10-92 */
void Network::construct(vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode) {
    vdnnType = _vdnnType;
    algoMode = _algoMode;
    numLayers = 0;
    inputData = labelData = networkDiffData = networkGradData = workSpace = nullptr;
    lossData = nullptr;
    inputResident = false;
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        layer[i] = nullptr;
        isOffload[i] = isPrefetched[i] = false;
        dropSrcAfterFwd[i] = false;
        offloadedSrcData_h[i] = nullptr;
        evFwdDone[i] = evOffloadDone[i] = evBlockFree[i] = evPrefetchDone[i] = evPacked[i] = nullptr;
        zvcStaging[i] = nullptr;
        zvcStagingBytes[i] = 0; zvcLengthSeen[i] = 0;
        zvcKept[i] = zvcFetched[i] = false;
        srcReleasedEarly[i] = false;
        keepPackedLayer[i] = false;
    }
    zvcLength_h = nullptr;

    /* context = handles + streams (network.cu:39-42) */
    ctx = nullptr;
    checkVDNN(vdnn_ctx_create(&ctx, options.device, options.planOnly ? VDNN_CTX_PLAN_ONLY : 0));
    checkVDNN(vdnn_ctx_set_activation_dtype(ctx, options.dataType));
    convHandle.ctx = ctx;
    gemmHandle.ctx = ctx;
    /* every layer of this network, also those rebuilt by reset(), takes these from its handle */
    convHandle.settings = gemmHandle.settings = vdnnLayerSettings{options.seed, options.verbose, options.planOnly};
    stream_compute = vdnn_ctx_stream_compute(ctx);
    stream_memory = vdnn_ctx_stream_d2h(ctx);

    if (_algoMode == VDNN_DYNAMIC_ALGO) {
        /* network.cu:59-78: start from (VDNN_ALL, memory-optimal), then walk the ladder */
        algoMode = VDNN_MEMORY_OPT_ALGO;
        vdnnType = VDNN_ALL;
        setLayers(cnnType);
        setVdnnType(VDNN_ALL);
        allocIoBuffers();
        vdnnDynamicAlgo();
    } else {
        setLayers(cnnType);
        setVdnnType(vdnnType);
        allocIoBuffers();
    }
}

Network::~Network() {
    if (ctx) vdnn_device_synchronize(ctx);
    releasePolicyBuffers();
    releaseLayers();
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        for (vdnn_event_t* e : {&evFwdDone[i], &evOffloadDone[i], &evBlockFree[i], &evPrefetchDone[i], &evPacked[i]}) {
            if (*e) vdnn_event_destroy(ctx, *e);
            *e = nullptr;
        }
    }
    if (ctx) {
        vdnn_pool_finalize(ctx);
        vdnn_ctx_destroy(ctx);
    }
}

void Network::releaseLayers() {
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        delete layer[i];
        layer[i] = nullptr;
    }
    numLayers = 0;
}

void Network::releasePolicyBuffers() {
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        if (offloadedSrcData_h[i]) vdnn_host_free_pinned(ctx, offloadedSrcData_h[i]);
        offloadedSrcData_h[i] = nullptr;
        isOffload[i] = isPrefetched[i] = false;
    }
    if (zvcLength_h) vdnn_host_free_pinned(ctx, zvcLength_h);
    zvcLength_h = nullptr;
}

/* network.cu:101-132: drop every allocation, rebuild layers and buffers for a new configuration */
void Network::reset(CNN_t _cnnType, vdnn_t _vdnnType, vdnnAlgoMode_t _algoMode) {
    vdnn_device_synchronize(ctx);
    releasePolicyBuffers();
    releaseLayers();
    vdnn_pool_finalize(ctx); /* cnmemFinalize: everything carved from the pool is gone */
    inputData = labelData = networkDiffData = networkGradData = workSpace = nullptr;
    lossData = nullptr;
    inputResident = false;
    /* so is every block the last step still held: a trial step of the dynamic ladder may have stopped half-way */
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        zvcStaging[i] = nullptr;
        zvcStagingBytes[i] = 0; zvcLengthSeen[i] = 0;
        zvcKept[i] = zvcFetched[i] = false;
        srcReleasedEarly[i] = false;
    }
    pendingOffload.clear();
    cnnType = _cnnType;
    algoMode = _algoMode;
    vdnnType = _vdnnType;
    setLayers(_cnnType);
    setVdnnType(_vdnnType);
    allocIoBuffers();
}

/* network.cu:47-53 reserves floor(totalGlobalMem / 1e9) GB. On a 288 GB device that would take the
 * whole card for a network that needs a fraction of it, so the reservation is sized from the layer
 * table instead: everything BASELINE keeps resident plus slack; options.poolBytes overrides. */
void Network::initPool() {
    size_t bytes = options.poolBytes;
    if (bytes == 0) {
        size_t sum = 0, maxAct = 0, params = 0;
        for (const LayerSpec& s : specs) {
            const size_t src = spec_src_count(s), dst = spec_dst_count(s);
            sum += dst;
            maxAct = std::max(maxAct, std::max(src, dst));
            if (s.type == FC_GEMM || is_conv(s.type)) params += ((size_t)s.k * s.c * s.r * s.s + s.k) * (options.unfusedOptimizer ? 2 : 1);
        }
        sum += spec_src_count(specs[0]) * 2 + spec_dst_count(specs.back()) * 2 + 3 * maxAct;
        bytes = sum * actBytes() + params * sizeof(float);
        bytes += bytes / 8 + (size_t(384) << 20); // rounding of ~100 blocks, staging area, headroom
        size_t freeB = 0, totalB = 0;
        checkVDNN(vdnn_device_mem_info(ctx, &freeB, &totalB));
        const size_t limit = freeB - freeB / 16;
        if (bytes > limit) bytes = limit;
    }
    ASSERT_EQ(vdnn_pool_init(ctx, bytes));
    if (options.capBytes) checkVDNN(vdnn_pool_set_cap(ctx, options.capBytes));
}

/* network.cu:134-154 */
void Network::setLayers(CNN_t _cnnType) {
    cnnType = _cnnType;
    if (_cnnType == ALEXNET || _cnnType == ALEXNET_LRN) setLayersAlexnet();
    else if (_cnnType == OVERFEAT) setLayersOverfeat();
    else if (_cnnType == GOOGLENET) setLayersGooglenet();
    else if (_cnnType == VGG16_64) setLayersVgg16(64);
    else if (_cnnType == VGG16_128) setLayersVgg16(128);
    else if (_cnnType == VGG16_256) setLayersVgg16(256);
    else if (_cnnType == VGG16_512) setLayersVgg16(512);
    else if (_cnnType == CUSTOM_CNN) setLayersCustomCNN();
    else M_ASSERT(false, "Invalid CNN Type!");
    if (options.verbose) printf("-------------------------------------------------------\n\n");
    sanityCheck();
}

void Network::setLayersAlexnet() {
    specs = tableFor(cnnType, batchSize);
    buildLayers();
}

void Network::setLayersOverfeat() {
    specs = tableFor(OVERFEAT, batchSize);
    buildLayers();
}

void Network::setLayersGooglenet() {
    M_ASSERT(false, "GOOGLENET is an empty stub in the reference (network.cu:497-499); not available");
}

/* network.cu:501-503: the VGG16 variants carry their batch in the enum; a batch given to the
 * constructor that differs from the default overrides it (addition, used for small test batches) */
void Network::setLayersVgg16(int givenBatch) {
    if (batchSize == DEFAULT_BATCH_SIZE || batchSize <= 0) batchSize = givenBatch;
    specs = tableFor(VGG16_128, batchSize);
    buildLayers();
}

void Network::setLayersCustomCNN() {
    M_ASSERT(customTable && !specs.empty(), "CUSTOM_CNN needs an explicit layer table");
    buildLayers();
}

/* Creates the Layer objects of `specs` (the bodies of the reference's setLayers* functions). */
void Network::buildLayers() {
    M_ASSERT(!specs.empty() && (int)specs.size() <= DEFAULT_NUM_LAYER, "layer table empty or too long");
    numLayers = (int)specs.size();
    batchSize = specs[0].n;
    n_in = specs[0].n; c_in = specs[0].c; h_in = specs[0].h; w_in = specs[0].w;
    spec_out(specs.back(), n_out, c_out, h_out, w_out);
    initPool();
    for (int l = 0; l < numLayers; l++) {
        const LayerSpec& s = specs[l];
        const vdnnAlgoMode_t mode = s.forceMemOpt ? VDNN_MEMORY_OPT_ALGO : algoMode;
        if (s.type == FC_GEMM)
            layer[l] = new Layer(vdnnType, mode, s.type, &gemmHandle, &stream_compute, &stream_memory, l,
                                 s.n, s.c, s.h, s.w, s.pad_h, s.pad_w, s.stride_h, s.stride_w, s.k, s.r, s.s);
        else
            layer[l] = new Layer(vdnnType, mode, s.type, &convHandle, &stream_compute, &stream_memory, l,
                                 s.n, s.c, s.h, s.w, s.pad_h, s.pad_w, s.stride_h, s.stride_w, s.k, s.r, s.s);
        if (options.unfusedOptimizer) layer[l]->keepGradients();
        /* before the next layer takes its blocks: an elided ReLU hands its BASELINE output block back */
        if (fusesRelu(l)) layer[l]->setElided(true);
    }
    capDst.assign(numLayers, {});
    capGrad.assign(numLayers, {});
}

/* addition (fuseActivations): layer l is a ReLU that the CONV / FC layer before it applies */
bool Network::fusesRelu(int l) const {
    if (!options.fuseActivations || l <= 0 || l >= (int)specs.size() || specs[l].type != RELU) return false;
    return is_conv(specs[l - 1].type) || specs[l - 1].type == FC_GEMM;
}

/* addition (compressOffload): the input of layer l holds rectified values - it is the output of a ReLU,
 * directly or behind max-pool / LRN layers, which map zero to zero and keep a tensor of many zeros one */
bool Network::srcIsRectified(int l) const {
    int p = l - 1;
    while (p >= 0 && (specs[p].type == POOL || specs[p].type == LRN)) p--;
    return p >= 0 && specs[p].type == RELU;
}

/* network.cu:819-829: the reference draws U(-0.01, 0.01) from an unseeded generator on every call;
 * here the draw is seeded (stream 1) and N(0,1) */
void Network::randomInitializeData(void* data, size_t size) {
    std::vector<DATATYPE> data_h(size);
    vdnn::seeded_fill_normal(data_h.data(), size, options.seed, 1, 0.0f, 1.0f);
    uploadActivations(data, data_h.data(), size);
}

/* network.cu:831-873 */
void Network::sanityCheck() {
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        if (i < numLayers) { M_ASSERT(layer[i] != NULL, "Not enough layers!"); }
        else { M_ASSERT(layer[i] == NULL, "Too many layers!"); }
    }
    M_ASSERT((layer[0]->InputN() == n_in && layer[0]->InputC() == c_in && layer[0]->InputH() == h_in && layer[0]->InputW() == w_in),
             "Layer 0 input and network input have different dimensions");
    M_ASSERT((layer[numLayers - 1]->OutputN() == n_out && layer[numLayers - 1]->OutputC() == c_out &&
              layer[numLayers - 1]->OutputH() == h_out && layer[numLayers - 1]->OutputW() == w_out),
             "Layer L output and network output have different dimensions");
    for (int i = 0; i < numLayers - 1; i++) {
        bool check;
        if (layer[i + 1]->LayerType() == FC_GEMM) {
            check = layer[i]->DstDataSize() == layer[i + 1]->SrcDataSize();
        } else {
            check = layer[i]->OutputN() == layer[i + 1]->InputN() && layer[i]->OutputC() == layer[i + 1]->InputC() &&
                    layer[i]->OutputH() == layer[i + 1]->InputH() && layer[i]->OutputW() == layer[i + 1]->InputW();
        }
        if (!check) {
            printf("Sanity check error at layer %d and %d!\n", i, i + 1);
            M_ASSERT(0, "Sanity check error!");
        }
    }
}

/* network.cu:875-940 */
void Network::setVdnnType(vdnn_t newVdnnType) {
    vdnnType = newVdnnType;
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) {
        isOffload[i] = false;
        isPrefetched[i] = false;
        dropSrcAfterFwd[i] = false;
        if (offloadedSrcData_h[i] != NULL) vdnn_host_free_pinned(ctx, offloadedSrcData_h[i]);
        offloadedSrcData_h[i] = NULL;
        if (layer[i] != NULL) {
            layer[i]->setVdnnMode(newVdnnType);
            layer[i]->setInPlaceOp(false);
            layer[i]->setSrcPacked(false);
            layer[i]->setFuseRelu(false);
            layer[i]->setElidedBackward(false);
            layer[i]->setGateGrad(false);
        }
    }
    /* fused rectifiers: producer l-1 rectifies, consumer l+1 masks its gradient */
    if (options.fuseActivations) {
        for (int l = 1; l < numLayers; l++) {
            if (!fusesRelu(l)) continue;
            layer[l - 1]->setFuseRelu(true);
            layer[l]->setElided(true);
            layer[l]->setInPlaceOp(true);
            if (l + 1 < numLayers) {
                const Layer_t next = layer[l + 1]->LayerType();
                /* a convolution over at most four channels computes its input gradient with a kernel of
                   its own that has no masked store: the ReLU's backward stays a launch there */
                const bool few_channels = is_conv(next) && layer[l + 1]->InputC() <= 4;
                if ((is_conv(next) || next == FC_GEMM || next == POOL) && !few_channels) {
                    layer[l + 1]->setGateGrad(true);
                    layer[l]->setElidedBackward(true);
                }
            }
        }
    }
    lastStats.pinnedBytes = 0;
    /* refined lifetimes: an activation layer's input is dead once its forward has run (never layer 0: the
       network input outlives the step) and its backward runs in place */
    const bool refined = options.refinedLifetimes && newVdnnType != BASELINE;
    if (refined) {
        for (int l = 0; l < numLayers; l++) {
            const Layer_t kind = layer[l]->LayerType(); /* all three activations differentiate from y alone */
            if (kind != RELU && kind != TANH && kind != SIGMOID) continue;
            layer[l]->setInPlaceOp(true);
            if (l > 0 && !layer[l]->Elided()) dropSrcAfterFwd[l] = true;
        }
    }

    /* recomputeFirstLayer: the first layer's output is dead after its consumer's forward and comes back by running layer 0
       again; the network input stays on the device for that */
    recomputedLayer = -1;
    if (options.recomputeFirstLayer && refined && numLayers > 2 && is_conv(layer[0]->LayerType()) && layer[0]->InputC() <= 4) {
        const int consumer = layer[1]->Elided() ? 2 : (specs[1].type == RELU || specs[1].type == TANH || specs[1].type == SIGMOID ? -1 : 1);
        if (consumer > 0 && consumer < numLayers - 1) {
            recomputedLayer = consumer;
            dropSrcAfterFwd[consumer] = true;
        }
    }

    /* keepTailBytes: the deepest members of the offload set stay on the device */
    int tailStart = numLayers;
    {
        size_t tail = 0;
        for (int l = numLayers - 2; l >= 0 && options.keepTailBytes > 0; l--) {
            const bool member = (newVdnnType == VDNN_ALL || (newVdnnType == VDNN_CONV && is_conv(layer[l]->LayerType()))) &&
                                !dropSrcAfterFwd[l] && !layer[l]->Elided();
            if (!member) continue;
            const size_t bytes = layer[l]->SrcDataSize() * actBytes();
            if (tail + bytes > options.keepTailBytes) break;
            tail += bytes;
            tailStart = l;
        }
    }

    /* the policy's offload set (network.cu:916-922, 928-936), less what the refinements above take out of it */
    std::vector<bool> member(numLayers, false);
    for (int l = 0; l < numLayers - 1; l++) {
        const bool named = newVdnnType == VDNN_ALL || (newVdnnType == VDNN_CONV && is_conv(layer[l]->LayerType()));
        member[l] = named && !dropSrcAfterFwd[l]     /* released, not moved: nothing reads it again (or layer 0 computes it again) */
                    && !(l == 0 && recomputedLayer > 0)  /* the input that layer 0 will read again */
                    && !layer[l]->Elided()           /* its input is the next layer's srcData, which has its own turn */
                    && l < tailStart;
    }
    /* hbmBudgetBytes: each member's place comes from a plan (the replay is handed one, the network itself makes one) */
    placement.assign(numLayers, PLACE_POLICY);
    planFeasibleFlag = true;
    plannedLag = 0;
    if (newVdnnType == VDNN_ALL || newVdnnType == VDNN_CONV) {
        if ((int)options.forcedPlacement.size() == numLayers) placement = options.forcedPlacement;
        else if (options.hbmBudgetBytes > 0 && !options.tracePeaks) placement = planPlacement(newVdnnType, member);
    }

    auto offload = [&](int l) {
        keepPackedLayer[l] = false;
        if (!member[l]) return;
        if (placement[l] == PLACE_RESIDENT) return;
        isOffload[l] = true;
        const bool packed = options.compressOffload && srcIsRectified(l);
        M_ASSERT(placement[l] != PLACE_PACKED || packed, "only a rectified tensor with compressOffload can wait as a packed stream");
        keepPackedLayer[l] = packed && (placement[l] == PLACE_PACKED || (placement[l] == PLACE_POLICY && options.keepPackedOnDevice));
        layer[l]->setSrcPacked(packed);
        const size_t bytes = packed ? vdnn_zvc_buffer_bytes(layer[l]->SrcDataSize(), (int)actBytes())
                                    : layer[l]->SrcDataSize() * actBytes();
        checkVDNN(vdnn_host_alloc_pinned(ctx, (void**)&offloadedSrcData_h[l], bytes));
        lastStats.pinnedBytes += bytes;
    };

    switch (newVdnnType) {
    case BASELINE: {
        /* one dx/dy ping-pong pair and one workspace, each sized for the largest user */
        const size_t dxdySize = findMaxDxDySize();
        ASSERT_EQ(vdnn_pool_malloc(ctx, &networkDiffData, dxdySize));
        ASSERT_EQ(vdnn_pool_malloc(ctx, &networkGradData, dxdySize));
        const size_t workSpaceSize = findMaxWorkSpaceSize();
        if (workSpaceSize > 0) ASSERT_EQ(vdnn_pool_malloc(ctx, &workSpace, workSpaceSize));
    } break;
    case VDNN_NONE:
        break;
    case VDNN_ALL:
    case VDNN_CONV:
        for (int l = 0; l < numLayers - 1; l++) offload(l);
        break;
    }

    /* fused rectifiers: a layer whose input comes back by prefetch does not mask its data gradient by that input -
       the data gradient then needs dy and W only and runs while the copy still lands (Layer::waitSrcFetched); the
       ReLU below it does its own backward, as below a consumer that cannot mask */
    for (int l = 1; l < numLayers; l++) {
        if (!layer[l]->GateGrad() || !isOffload[l]) continue;
        const Layer_t t = layer[l]->LayerType();
        if (!is_conv(t) && t != FC_GEMM) continue; /* a pooling layer reads its input anyway */
        /* a packed input that stays on the device is expanded by the layer itself before its first kernel */
        if (layer[l]->SrcPacked()) continue; /* (also one that crosses the link: it comes back into a staging block) */
        layer[l]->setGateGrad(false);
        layer[l - 1]->setElidedBackward(false);
    }

    /* inPlaceBackward: the input gradient of a convolution or a 2x2 pooling layer goes over the layer's input where the
       layer below does not read that tensor - its own output - in its backward: convolution, FC and pooling layers
       (refined lifetimes release it before their backward as it is), and a ReLU whose backward is fused away. Never
       layer 0: the network input outlives the step. */
    for (int l = 0; l < numLayers; l++) layer[l]->setGradOverSrc(false);
    if (options.inPlaceBackward && refined) {
        for (int l = 1; l < numLayers; l++) {
            if (!layer[l]->canGradOverSrc()) continue;
            /* a convolution then takes a block of its filter's size for the filter gradient: no gain where that is the larger one */
            if (layer[l]->FilterDataSize() * sizeof(DATATYPE) >= layer[l]->SrcDataSize() * actBytes()) continue;
            const Layer_t below = layer[l - 1]->LayerType();
            const bool belowLeavesIt = is_conv(below) || below == FC_GEMM || below == POOL ||
                                       (layer[l - 1]->Elided() && layer[l - 1]->ElidedBackward());
            if (belowLeavesIt) layer[l]->setGradOverSrc(true);
        }
    }

    if (newVdnnType != BASELINE) {
        for (int l = 0; l < numLayers; l++)
            for (vdnn_event_t* e : {&evFwdDone[l], &evOffloadDone[l], &evBlockFree[l], &evPrefetchDone[l], &evPacked[l]})
                if (!*e) checkVDNN(vdnn_event_create(ctx, e, 0));
        if (options.prefetchWithinPeak && !options.tracePeaks) buildPeakPlan(newVdnnType);
        if (options.compressOffload && !options.planOnly && !zvcLength_h) {
            checkVDNN(vdnn_host_alloc_pinned(ctx, (void**)&zvcLength_h, sizeof(unsigned long long) * DEFAULT_NUM_LAYER));
            for (int l = 0; l < DEFAULT_NUM_LAYER; l++) zvcLength_h[l] = 0; /* 0: not known yet */
        }
    }
}

/* network.cu:942-944 is empty in the reference; here it switches every convolution's variant */
void Network::setAlgoType(vdnnAlgoMode_t newAlgoMode) {
    algoMode = newAlgoMode;
    for (int l = 0; l < numLayers; l++)
        if (!specs[l].forceMemOpt) layer[l]->setAlgoMode(newAlgoMode);
}

/* network.cu:87-90: input and label tensors; plus the loss scalar and the seeded contents */
void Network::allocIoBuffers() {
    ASSERT_EQ(vdnn_pool_malloc(ctx, &inputData, actBytes() * getInputSize()));
    ASSERT_EQ(vdnn_pool_malloc(ctx, &labelData, actBytes() * getOutputSize()));
    ASSERT_EQ(vdnn_pool_malloc(ctx, (void**)&lossData, sizeof(DATATYPE)));
    if (!options.planOnly) {
        inputHost.resize(getInputSize());
        vdnn::seeded_fill_normal(inputHost.data(), inputHost.size(), options.seed, 1, 0.0f, 1.0f);
        uploadActivations(inputData, inputHost.data(), inputHost.size());
        const int classes = c_out * h_out * w_out;
        std::vector<int32_t> lab((size_t)n_out);
        vdnn::seeded_fill_labels(lab.data(), lab.size(), options.seed, 2, classes);
        setLabels(lab.data());
    }
    inputResident = true;
}

/* network.cu:946-1008 */
void Network::vdnnDynamicAlgo() {
    int ret = 0;
    if (options.verbose) printf("\n1. Test VDNN_ALL and VDNN_MEMORY_OPT_ALGO\n");
    if (forwardPropagation(true) < 0 || backwardPropagation(true) < 0) {
        printf("This CNN model cannot be trained\n");
        M_ASSERT(0, "This CNN model cannot be trained");
    }
    const vdnn_t ladder[3] = {VDNN_NONE, VDNN_CONV, VDNN_ALL};
    const char* names[3] = {"VDNN_NONE", "VDNN_CONV", "VDNN_ALL"};
    for (int i = 0; i < 3; i++) {
        if (options.verbose) printf("\n%d. Test %s and VDNN_PERF_OPT_ALGO\n", i + 2, names[i]);
        reset(cnnType, ladder[i], VDNN_PERF_OPT_ALGO);
        ret = forwardPropagation(true);
        if (ret >= 0) ret = backwardPropagation(true);
        if (ret >= 0) {
            reset(cnnType, ladder[i], VDNN_PERF_OPT_ALGO);
            if (options.verbose) printf("%s and VDNN_PERF_OPT_ALGO Passed!\n", names[i]);
            return;
        }
    }
    if (options.verbose) printf("\n5. Dynamic Algorithm with VDNN_ALL\n");
    /* network.cu:89-98 stops at the per-layer choice, which tries every workspace against an empty pool: a workspace of
     * hundreds of megabytes chosen that way need not fit once the activations are there, and the first training step
     * would return -1. Here the choice is tried like the rungs above; while the trial step fails, the layer with the
     * largest workspace still in use goes back to the memory-optimal kernels (with all of them there it is rung 1,
     * which passed). */
    std::vector<bool> demoted(DEFAULT_NUM_LAYER, false);
    bool verified = false;
    for (;;) {
        reset(cnnType, VDNN_ALL, VDNN_PERF_OPT_ALGO);
        for (int id = 0; id < DEFAULT_NUM_LAYER; id++) {
            if (layer[id] == NULL || !is_conv(layer[id]->LayerType())) continue;
            if (demoted[id]) layer[id]->setAlgoMode(VDNN_MEMORY_OPT_ALGO);
            else layer[id]->findDynamicAlgo();
        }
        int largest = -1;
        size_t most = 0;
        for (int id = 0; id < DEFAULT_NUM_LAYER; id++) {
            if (layer[id] == NULL || !is_conv(layer[id]->LayerType()) || layer[id]->AlgoMode() != VDNN_PERF_OPT_ALGO) continue;
            const size_t w = std::max(layer[id]->FwdWorkSpaceSize(), std::max(layer[id]->BwdDataWorkSpaceSize(), layer[id]->BwdFilterWorkSpaceSize()));
            if (w > most) { most = w; largest = id; }
        }
        if (verified || largest < 0) return; /* the tried choice, rebuilt; or nothing left to give up */
        ret = forwardPropagation(true);
        if (ret >= 0) ret = backwardPropagation(true);
        if (ret >= 0) { verified = true; continue; } /* rebuild once more: the trial step changed the parameters */
        if (options.verbose) printf("layer %d goes back to the memory-optimal kernels\n", largest);
        demoted[largest] = true;
    }
}

/* network.cu:1010-1023 */
size_t Network::findMaxDxDySize() {
    size_t ret = 0;
    for (int i = 0; i < numLayers; i++) ret = std::max(ret, layer[i]->SrcDataSize());
    ret = std::max(ret, layer[numLayers - 1]->DstDataSize());
    return ret * actBytes();
}

/* network.cu:1025-1040 */
size_t Network::findMaxWorkSpaceSize() {
    size_t ret = 0;
    for (int i = 0; i < numLayers; i++) {
        if (!is_conv(layer[i]->LayerType())) continue;
        ret = std::max(ret, layer[i]->FwdWorkSpaceSize());
        ret = std::max(ret, layer[i]->BwdDataWorkSpaceSize());
        ret = std::max(ret, layer[i]->BwdFilterWorkSpaceSize());
    }
    return ret;
}

/* network.cu:1042-1054: result = first - second on the compute stream (the reference launches it on
 * the default stream and redraws the label here; the label is fixed at construction instead) */
void Network::calculateFirstDiffData(void* result, void* first, void* second) {
    checkVDNN(vdnn_sub(ctx, stream_compute, getOutputSize(), (const float*)first, (const float*)second, (float*)result));
}

void Network::printUsage(const char* tag, int l, size_t workspace) {
    if (!options.verbose) return;
    size_t freeB = 0, totalB = 0;
    vdnn_pool_info(ctx, &freeB, &totalB);
    printf("[%s] Layer %d, Free Memory: %lu, Total Memory: %lu, Memory Usage: %lu\n", tag, l,
           (unsigned long)freeB, (unsigned long)totalB, (unsigned long)(totalB - freeB + workspace));
}

void Network::captureLayer(int l, bool grad) {
    if (!options.capture || options.planOnly) return;
    std::vector<float>& dstv = grad ? capGrad[l] : capDst[l];
    const size_t count = grad ? layer[l]->SrcDataSize() : layer[l]->DstDataSize();
    dstv.resize(count);
    downloadActivations(dstv.data(), grad ? layer[l]->GradData() : layer[l]->DstData(), count);
}

/* network.cu:1090-1091, 1168-1169 */
void Network::afterLayerSync() {
    checkVDNN(vdnn_stream_synchronize(ctx, stream_compute));
    checkVDNN(vdnn_stream_synchronize(ctx, stream_memory));
    checkVDNN(vdnn_stream_synchronize(ctx, vdnn_ctx_stream_h2d(ctx)));
}

/* network.cu:1056-1110 */
int Network::forwardPropagation(bool isDynamic) {
    M_ASSERT(inputResident && inputData, "forwardPropagation needs the input on the device (run backwardPropagation after a forward)");
    lastStats.offloadBytes = 0;
    pendingOffload.clear();
    if (vdnnType == BASELINE) {
        for (int l = 0; l < numLayers; l++) {
            layer[l]->copySrcData(l == 0 ? inputData : layer[l - 1]->DstData());
            if (layer[l]->forward(isOffload, offloadedSrcData_h, workSpace, isDynamic) < 0) return -1;
            captureLayer(l, false);
            printUsage("Fwd", l, layer[l]->FwdWorkSpaceSize());
        }
    } else {
        /* everything enqueued so far (the previous step's last prefetch included) precedes this event */
        checkVDNN(vdnn_event_record(ctx, evBlockFree[0], stream_compute));
        /* packed streams that a forward without a backward left on the device */
        for (int l = 0; l < numLayers; l++) {
            if (zvcKept[l] && zvcStaging[l]) ASSERT_EQ(vdnn_pool_free(ctx, zvcStaging[l]), isDynamic);
            zvcKept[l] = zvcFetched[l] = false;
            zvcStaging[l] = nullptr;
        }
        if (options.tracePeaks) fwdPeakTrace.assign(numLayers, 0);
        for (int l = 0; l < numLayers; l++) {
            if (options.tracePeaks) vdnn_pool_reset_peak(ctx);
            layer[l]->copySrcData(l == 0 ? inputData : layer[l - 1]->DstData());
            if (isOffload[l]) {
                layer[l]->setSrcReadyEvent(l == 0 ? evBlockFree[0] : evFwdDone[l - 1]);
                layer[l]->setOffloadDoneEvent(evOffloadDone[l]);
            }
            /* compressOffload: the stream is packed into a staging block sized from its length one step ago (plus
               a margin; what does not fit the kernel stores into host memory itself) and the copy engine moves
               the block. The first step has no length to go by and stores everything from the kernel; planning
               without a device assumes the longest stream. */
            zvcStaging[l] = nullptr;
            srcReleasedEarly[l] = false;
            if (isOffload[l] && layer[l]->SrcPacked()) {
                const size_t longest = vdnn_zvc_buffer_bytes(layer[l]->SrcDataSize(), (int)actBytes());
                const size_t assumed = options.planPackedFraction > 0.0
                                           ? (size_t)(options.planPackedFraction * (double)(layer[l]->SrcDataSize() * actBytes())) : longest;
                const size_t known = options.planOnly ? assumed : (size_t)zvcLength_h[l];
                zvcLengthSeen[l] = known; /* backward sizes the way back from the same figure, whatever the word holds by then */
                size_t want = known ? known + known / 32 + 65536 : 0;
                want = std::min(longest, (want + 15) / 16 * 16);
                if (want && ASSERT_EQ(vdnn_pool_malloc(ctx, &zvcStaging[l], want), isDynamic) < 0) return -1;
                if (want) {
                    /* the packing stream writes a recycled block: whatever the compute stream was told to wait
                       for before the block went back to the pool (a copy out of it, say) comes first */
                    checkVDNN(vdnn_event_record(ctx, evBlockFree[l], stream_compute));
                    layer[l]->setSrcReadyEvent(evBlockFree[l]);
                }
                zvcStagingBytes[l] = want;
                zvcKept[l] = keepPackedLayer[l] && want > 0;
                layer[l]->setOffloadStaging(zvcStaging[l], want, options.planOnly ? nullptr : &zvcLength_h[l], evPacked[l], zvcKept[l]);
            }

            /* Forward propagation */
            if (layer[l]->forward(isOffload, offloadedSrcData_h, workSpace, isDynamic) < 0) return -1;
            checkVDNN(vdnn_event_record(ctx, evFwdDone[l], stream_compute));
            captureLayer(l, false);

            /* The reference synchronises both streams on the host here. Ordering is what matters:
               the block may be recycled once this layer's kernels (stream order) and its offload
               copy (event) are done with it. */
            if (options.hostSync) afterLayerSync();

            /* Release srcData of this layer. The reference keeps layer 0's block and later allocates
               a second one for its prefetch; releasing it here avoids that leak. With offloadLag the
               wait for the copy and the release move behind the next `offloadLag` layers. */
            if (isOffload[l]) {
                if (!zvcKept[l]) lastStats.offloadBytes += layer[l]->SrcDataSize() * actBytes();
                pendingOffload.push_back(l);
                if (zvcStaging[l]) {
                    /* the staging block has the tensor: srcData goes back behind this layer's kernels and the
                       packing kernel, which works at HBM speed and started when this layer did */
                    if (!options.hostSync) checkVDNN(vdnn_stream_wait_event(ctx, stream_compute, evPacked[l]));
                    ASSERT_EQ(vdnn_pool_free(ctx, layer[l]->SrcData()), isDynamic);
                    srcReleasedEarly[l] = true;
                }
            } else if (dropSrcAfterFwd[l]) {
                /* refined lifetimes: every reader (this layer's forward) is already enqueued */
                ASSERT_EQ(vdnn_pool_free(ctx, layer[l]->SrcData()), isDynamic);
                layer[l]->copySrcData(nullptr);
            }
            const int lag = options.hostSync ? 0 : offloadLagInUse();
            while (!pendingOffload.empty() && (pendingOffload.front() + lag <= l || l == numLayers - 1)) {
                const int j = pendingOffload.front();
                pendingOffload.erase(pendingOffload.begin());
                if (!options.hostSync) checkVDNN(vdnn_stream_wait_event(ctx, stream_compute, evOffloadDone[j]));
                if (zvcStaging[j] && !zvcKept[j]) {
                    ASSERT_EQ(vdnn_pool_free(ctx, zvcStaging[j]), isDynamic);
                    zvcStaging[j] = nullptr;
                }
                if (!srcReleasedEarly[j]) ASSERT_EQ(vdnn_pool_free(ctx, layer[j]->SrcData()), isDynamic);
                if (j == 0) { inputData = nullptr; inputResident = false; }
            }
            printUsage("Fwd", l, layer[l]->FwdWorkSpaceSize());
            if (options.tracePeaks) {
                size_t inUse = 0, extent = 0;
                vdnn_pool_peak(ctx, &inUse, &extent);
                fwdPeakTrace[l] = inUse;
            }
        }
    }
    /* addition: mean cross-entropy of the output against the target, for monitoring */
    checkVDNN(vdnn_cross_entropy_dense(ctx, stream_compute, n_out, c_out * h_out * w_out,
                                       (const float*)layer[numLayers - 1]->DstData(), (const float*)labelData, lossData));
    return 0;
}

/* network.cu:1112-1191 */
int Network::backwardPropagation(bool isDynamic) {
    lastStats.prefetchBytes = 0;
    prefetchLog.clear();
    if (vdnnType == BASELINE) {
        calculateFirstDiffData(networkDiffData, layer[numLayers - 1]->DstData(), labelData);
        for (int l = numLayers - 1; l >= 0; l--) {
            if (l == numLayers - 1) {
                layer[l]->copyDiffData(networkDiffData);
                layer[l]->copyGradData(networkGradData);
            } else {
                layer[l]->copyDiffData(layer[l + 1]->GradData());
                layer[l]->copyGradData(layer[l + 1]->DiffData());
            }
            if (layer[l]->ElidedBackward()) {
                /* the masked gradient is already in place: it is this layer's gradData, and the other
                   buffer of the pair stays free for the layer below */
                void* masked = layer[l]->DiffData();
                layer[l]->copyDiffData(layer[l]->GradData());
                layer[l]->copyGradData(masked);
                captureLayer(l, true);
                continue;
            }
            if (layer[l]->backward(-1, NULL, NULL, 0, workSpace, isDynamic) < 0) return -1;
            captureLayer(l, true);
            printUsage("Bwd", l, layer[l]->BwdDataWorkSpaceSize() + layer[l]->BwdFilterWorkSpaceSize());
        }
    } else {
        resetIsPrefetchedArray();
        if (layer[numLayers - 1]->cnmemMallocDiffData(isDynamic) < 0) return -1;
        calculateFirstDiffData(layer[numLayers - 1]->DiffData(), layer[numLayers - 1]->DstData(), labelData);

        if (options.tracePeaks) bwdPeakTrace.assign(numLayers, 0);
        fetchedAhead.assign(numLayers, 0);
        {
            /* what backward may hold: the highest value of the replay's backward, or what the pool has already
               held (this step's forward, say) if that is more - either way the peak does not move */
            size_t held = 0, extent = 0;
            vdnn_pool_peak(ctx, &held, &extent);
            peakBudget = std::max(planPeak, held);
        }
        for (int l = numLayers - 1; l >= 0; l--) {
            if (options.tracePeaks) vdnn_pool_reset_peak(ctx);
            if (l != numLayers - 1) {
                layer[l]->copyDiffData(layer[l + 1]->GradData());
                layer[l]->copyDstData(layer[l + 1]->SrcData());
                /* an elided ReLU's input and output are one block: the next layer's srcData, by now
                   possibly a prefetched copy at another address */
                if (layer[l]->Elided()) layer[l]->copySrcData(layer[l]->DstData());
            }
            /* refined lifetimes: convolution, FC and pooling backward never read their output, so
               its block (the next layer's srcData) goes back to the pool before anything is
               allocated for this layer */
            /* the layer above wrote its input gradient over its input: this layer's output and the gradient that
               arrives for it are one block, released once, as the gradient */
            const bool dstIsDiff = l != numLayers - 1 && layer[l]->DstData() == layer[l]->DiffData();
            bool dstReleased = false;
            if (options.refinedLifetimes && l != numLayers - 1 && !dstIsDiff) {
                const Layer_t t = layer[l]->LayerType();
                if (is_conv(t) || t == FC_GEMM || t == POOL) {
                    ASSERT_EQ(vdnn_pool_free(ctx, layer[l]->DstData()), isDynamic);
                    layer[l]->copyDstData(nullptr);
                    dstReleased = true;
                }
            }
            /* recomputeFirstLayer: this layer's input was released behind its forward; layer 0 computes it again */
            if (l == recomputedLayer) {
                M_ASSERT(inputResident && layer[0]->SrcData() != nullptr, "the first layer's input has to be on the device to compute its output again");
                if (layer[l]->cnmemMallocSrcData(isDynamic) < 0) return -1;
                if (layer[0]->forwardAgainInto(layer[l]->SrcData(), isDynamic) < 0) return -1;
            }
            /* a packed input that stayed on the device is expanded now, not a layer ahead: that takes HBM time only
               (a millisecond for the largest), and so the tensor, its packed block and the working set of the
               layer above are never held together; the block goes back before this layer allocates anything */
            if (isOffload[l] && zvcKept[l] && !isPrefetched[l]) {
                isPrefetched[l] = true;
                if (layer[l]->cnmemMallocSrcData(isDynamic) < 0) return -1;
                /* on the compute stream: behind everything that used the recycled block, behind the copy that filled
                   the staging block (if the stream came back over the link) and behind the offload that wrote what
                   the block is too short for into host memory */
                layer[l]->expandPackedSrcData(offloadedSrcData_h[l], zvcStaging[l], zvcStagingBytes[l],
                                              zvcFetched[l] && !options.hostSync ? evPrefetchDone[l] : nullptr,
                                              options.hostSync ? nullptr : evOffloadDone[l]);
                if (!zvcFetched[l]) prefetchLog.emplace_back(l, l);
                if (l == 0) { inputData = layer[0]->SrcData(); inputResident = true; }
                if (options.hostSync) afterLayerSync();
                ASSERT_EQ(vdnn_pool_free(ctx, zvcStaging[l]), isDynamic);
                zvcStaging[l] = nullptr;
                zvcKept[l] = zvcFetched[l] = false;
                layer[l]->setSrcFetchedEvent(nullptr);
            } else {
                /* this layer reads its own srcData: if that was prefetched, the copy must have landed */
                layer[l]->setSrcFetchedEvent(!options.hostSync && isPrefetched[l] ? evPrefetchDone[l] : nullptr);
            }

            int prefId = l == 0 ? -1 : (options.prefetchDepth > 1 ? findPrefetchLayerDeep(l) : findPrefetchLayer(l));
            /* a packed stream comes back through the copy engine into a block of its own length; its layer expands it */
            if (prefId >= 0 && stagedFetchBytes(prefId) > 0) {
                if (fetchPackedToStaging(l, prefId, isDynamic) < 0) return -1;
                prefId = -1;
            }
            if (prefId >= 0) {
                if (layer[prefId]->cnmemMallocSrcData(isDynamic) < 0) return -1;
                layer[l]->setPrefetchEvents(evBlockFree[prefId], evOffloadDone[prefId], evPrefetchDone[prefId]);
                layer[l]->setPrefetchPacked(layer[prefId]->SrcPacked());
                layer[l]->setPrefetchStaging(nullptr, 0);
                const size_t bytes = actBytes() * layer[prefId]->SrcDataSize();
                if (layer[l]->backward(prefId, offloadedSrcData_h[prefId], layer[prefId]->SrcData(), bytes, workSpace, isDynamic) < 0) return -1;
                lastStats.prefetchBytes += bytes;
                prefetchLog.emplace_back(l, prefId);
                if (prefId == 0) { inputData = layer[0]->SrcData(); inputResident = true; }
            } else {
                if (layer[l]->backward(-1, NULL, NULL, 0, workSpace, isDynamic) < 0) return -1;
            }
            /* deeper prefetch: further tensors below, enqueued behind this layer's kernels */
            while ((options.prefetchDepth > 1 || options.prefetchWithinPeak) && l > 0) {
                int extra = options.prefetchDepth > 1 ? findPrefetchLayerDeep(l) : -1;
                if (extra < 0 && options.prefetchWithinPeak) extra = findPrefetchWithinPeak(l);
                if (extra < 0) break;
                if (stagedFetchBytes(extra) > 0) {
                    if (fetchPackedToStaging(l, extra, isDynamic) < 0) return -1;
                    continue;
                }
                if (layer[extra]->cnmemMallocSrcData(isDynamic) < 0) return -1;
                layer[l]->setPrefetchEvents(evBlockFree[extra], evOffloadDone[extra], evPrefetchDone[extra]);
                layer[l]->setPrefetchPacked(layer[extra]->SrcPacked());
                layer[l]->setPrefetchStaging(nullptr, 0);
                const size_t bytes = actBytes() * layer[extra]->SrcDataSize();
                layer[l]->prefetchPreviousSrcData(offloadedSrcData_h[extra], layer[extra]->SrcData(), bytes);
                lastStats.prefetchBytes += bytes;
                prefetchLog.emplace_back(l, extra);
                if (extra == 0) { inputData = layer[0]->SrcData(); inputResident = true; }
            }
            captureLayer(l, true);

            if (options.hostSync) afterLayerSync();

            /* Release dstData and diffData: every reader is already enqueued on the compute stream.
               An in-place ReLU's diffData is its gradData and lives on as the next layer's diffData. */
            /* an elided ReLU's block is released by the layer below, as its dstData */
            if (!dstReleased && !dstIsDiff && !layer[l]->Elided()) ASSERT_EQ(vdnn_pool_free(ctx, layer[l]->DstData()), isDynamic);
            if (!(layer[l]->InPlaceOp() && layer[l]->GradData() == layer[l]->DiffData()))
                ASSERT_EQ(vdnn_pool_free(ctx, layer[l]->DiffData()), isDynamic);
            /* this layer's packed input has been expanded (its backward waited for that): the block goes back */
            if (zvcKept[l] && zvcStaging[l]) {
                ASSERT_EQ(vdnn_pool_free(ctx, zvcStaging[l]), isDynamic);
                zvcStaging[l] = nullptr;
                zvcKept[l] = false;
            }
            printUsage("Bwd", l, layer[l]->BwdDataWorkSpaceSize() + layer[l]->BwdFilterWorkSpaceSize());
            if (options.tracePeaks) {
                size_t inUse = 0, extent = 0;
                vdnn_pool_peak(ctx, &inUse, &extent);
                bwdPeakTrace[l] = inUse;
            }
        }
        ASSERT_EQ(vdnn_pool_free(ctx, layer[0]->GradData()), isDynamic);
        inputData = layer[0]->SrcData(); /* network.cu:1185 */
        inputResident = true;
    }
    if (options.unfusedOptimizer && !options.deferOptimizer) return applyGradients();
    return 0;
}

/* addition: the optimizer step of unfusedOptimizer, with the reference's scalar (alpha = -lr, layer.cu:593) */
int Network::applyGradients() {
    const DATATYPE lr = LEARNING_RATE * -1.0f;
    for (int l = 0; l < numLayers; l++)
        if (layer[l]->applyGradients(lr) < 0) return -1;
    return 0;
}

int Network::getLayerGradients(int l, float* filter, float* bias) {
    if (l < 0 || l >= numLayers || !layer[l]->hasParams() || !layer[l]->FilterGrad()) return -1;
    if (filter) checkVDNN(vdnn_memcpy_d2h(ctx, filter, layer[l]->FilterGrad(), layer[l]->FilterDataSize() * sizeof(float)));
    if (bias) checkVDNN(vdnn_memcpy_d2h(ctx, bias, layer[l]->BiasGrad(), layer[l]->BiasDataSize() * sizeof(float)));
    return 0;
}

/* addition: the reference's main runs one step (vdnn.cu:71-75); this is the loop around it */
std::vector<float> Network::train(int steps, bool isDynamic) {
    std::vector<float> losses;
    for (int i = 0; i < steps; i++) {
        if (forwardPropagation(isDynamic) < 0) break;
        losses.push_back(loss());
        if (backwardPropagation(isDynamic) < 0) break;
        if (options.unfusedOptimizer && options.deferOptimizer && applyGradients() < 0) break;
    }
    return losses;
}

/* addition (compressOffload): the bytes of the device block that a packed stream on its way back is copied into - the
 * stream's length one step ago plus a margin, as on the way out - or 0 if the tensor comes back the plain way: it is
 * not packed, or its length is not known yet (first step; the expanding kernel then reads pinned memory itself). */
size_t Network::stagedFetchBytes(int id) const {
    if (!isOffload[id] || !layer[id]->SrcPacked() || zvcKept[id]) return 0;
    const size_t longest = vdnn_zvc_buffer_bytes(layer[id]->SrcDataSize(), (int)actBytes());
    const size_t assumed = options.planPackedFraction > 0.0
                               ? (size_t)(options.planPackedFraction * (double)(layer[id]->SrcDataSize() * actBytes())) : longest;
    /* the length this step's forward went by (the step before's; none in a first step, whose streams then come back
       through the expanding kernel): the pinned word itself changes while the step runs */
    const size_t known = options.planOnly ? assumed : zvcLengthSeen[id];
    if (!known) return 0;
    return std::min(longest, (known + known / 32 + 65536 + 15) / 16 * 16);
}

/* addition (compressOffload): during layer `issuingLayer`'s backward the copy engine starts to bring the packed stream
 * of layer id's input back into a block of the pool; from here on the tensor counts as kept on the device, and its own
 * layer expands it at the start of its backward (behind evPrefetchDone[id]). Only the stream's length is held a layer
 * ahead, not the tensor, and the link runs at the copy engine's rate whatever the kernels beside it do. */
int Network::fetchPackedToStaging(int issuingLayer, int id, bool isDynamic) {
    const size_t want = stagedFetchBytes(id);
    if (ASSERT_EQ(vdnn_pool_malloc(ctx, &zvcStaging[id], want), isDynamic) < 0) return -1;
    zvcStagingBytes[id] = want;
    layer[issuingLayer]->setPrefetchEvents(evBlockFree[id], evOffloadDone[id], evPrefetchDone[id]);
    layer[issuingLayer]->fetchPackedSrcData(offloadedSrcData_h[id], zvcStaging[id], want);
    zvcKept[id] = zvcFetched[id] = true;
    isPrefetched[id] = false; /* its own layer's turn comes at the start of its backward */
    lastStats.prefetchBytes += actBytes() * layer[id]->SrcDataSize();
    prefetchLog.emplace_back(issuingLayer, id);
    return 0;
}

/* network.cu:1193-1196 */
void Network::resetIsPrefetchedArray() {
    for (int i = 0; i < DEFAULT_NUM_LAYER; i++) isPrefetched[i] = false;
}

/* addition (prefetchDepth > 1): the nearest offloaded, not yet fetched layer below currLayerId, as long
 * as fewer than prefetchDepth fetched tensors below currLayerId are still waiting for their backward. A packed
 * stream that the copy engine has brought back into a staging block (fetchPackedToStaging: zvcFetched) waits for
 * its backward like a tensor fetched whole, and counts. */
int Network::findPrefetchLayerDeep(int currLayerId) {
    int outstanding = 0;
    for (int id = currLayerId - 1; id >= 0; id--)
        if (isOffload[id] && (isPrefetched[id] || zvcFetched[id])) outstanding++;
    if (outstanding >= options.prefetchDepth) return -1;
    for (int id = currLayerId - 1; id >= 0; id--) {
        if (isOffload[id] && !isPrefetched[id] && !zvcKept[id]) {
            isPrefetched[id] = true;
            return id;
        }
    }
    return -1;
}

/* addition (prefetchWithinPeak): one step of this network's schedule on a context without a device, with the
 * bytes in use noted per backward layer */
void Network::buildPeakPlan(vdnn_t policy) {
    planBwdPeak.clear();
    planIssueLayer.assign(numLayers, -1);
    planPeak = 0;
    if (policy == BASELINE) return;
    NetworkOptions o = options;
    o.planOnly = true; o.tracePeaks = true; o.prefetchWithinPeak = false;
    o.capture = false; o.verbose = false; o.capBytes = 0;
    o.hbmBudgetBytes = 0; o.forcedPlacement = placement; /* the replay takes this network's plan, it makes none */
    o.offloadLag = offloadLagInUse();
    Network replay(specs, policy, algoMode == VDNN_DYNAMIC_ALGO ? VDNN_MEMORY_OPT_ALGO : algoMode, o);
    if (replay.forwardPropagation(false) < 0 || replay.backwardPropagation(false) < 0) return;
    planBwdPeak = replay.backwardPeakTrace();
    for (const auto& p : replay.prefetchTrace()) planIssueLayer[p.second] = p.first;
    for (size_t b : planBwdPeak) planPeak = std::max(planPeak, b);
}

/* addition (hbmBudgetBytes): a place for every member of the offload set such that a replay of one step stays
 * within the budget. Everything starts on the device as it is; while the replay peaks above the budget, the largest
 * member that is stored at the moment of the peak (its forward is over, its backward has not begun) moves one place
 * down: to a packed stream on the device if it is rectified and streams are packed at all, else - or from there - to
 * host memory. Ends when the replay fits or nothing that is stored at the peak can move any further: then the peak is
 * the working set of the layer itself, which no placement changes. */
std::vector<unsigned char> Network::planPlacement(vdnn_t policy, const std::vector<bool>& member) {
    NetworkOptions o = options;
    o.planOnly = true; o.tracePeaks = true; o.prefetchWithinPeak = false; o.hbmBudgetBytes = 0;
    o.capture = false; o.verbose = false; o.capBytes = 0; o.keepPackedOnDevice = false; o.keepTailBytes = 0;
    const vdnnAlgoMode_t mode = algoMode == VDNN_DYNAMIC_ALGO ? VDNN_MEMORY_OPT_ALGO : algoMode;
    struct Plan { std::vector<unsigned char> place; bool feasible = false; size_t peak = 0; double link = 0.0; int lag = 0; };
    auto plan_with = [&](int lag) {
        Plan p;
        p.lag = lag;
        p.place.assign(numLayers, PLACE_POLICY);
        std::vector<unsigned char>& place = p.place;
        for (int l = 0; l < numLayers; l++) if (member[l]) place[l] = PLACE_RESIDENT;
        o.offloadLag = lag;
        for (int round = 0; round <= 2 * numLayers; round++) {
            o.forcedPlacement = place;
            size_t peak = 0; int at = 0;
            {
                Network replay(specs, policy, mode, o);
                /* two steps: the first forward of a packed stream has no length to size its block by */
                for (int step = 0; step < 2; step++)
                    if (replay.forwardPropagation(true) < 0 || replay.backwardPropagation(true) < 0) return p;
                for (int l = 0; l < numLayers; l++) {
                    if (replay.forwardPeakTrace()[l] > peak) { peak = replay.forwardPeakTrace()[l]; at = l; }
                    if (replay.backwardPeakTrace()[l] > peak) { peak = replay.backwardPeakTrace()[l]; at = l; }
                }
            }
            p.peak = peak;
            if (peak <= options.hbmBudgetBytes) { p.feasible = true; break; }
            /* stored at the peak: every member below the layer at work (in forward it has been written and left behind,
               in backward it still waits for its turn) */
            const double f = options.planPackedFraction > 0.0 ? options.planPackedFraction : 1.04;
            /* a stream on the device costs two passes at HBM speed, the link a hundred times that: everything stored at
               the peak that can be packed is packed before anything crosses the link; within a kind, the largest gain first */
            int pick = -1; double best = 0.0; unsigned char to = PLACE_LINK;
            /* planLinkBytes: an allowance of bytes on the link that is spent first - whatever is stored at the peak and
               whose bytes on the link (its packed stream where it can be packed) still fit goes there, the largest gain
               first; packing on the device begins when nothing fits the rest of the allowance */
            if (options.planLinkBytes > 0) {
                double on_link = 0.0;
                auto link_bytes = [&](int l) {
                    const double size = (double)(layer[l]->SrcDataSize() * actBytes());
                    return (options.compressOffload && srcIsRectified(l) && f < 1.0) ? f * size : size;
                };
                for (int l = 0; l < numLayers; l++) if (member[l] && place[l] == PLACE_LINK) on_link += link_bytes(l);
                for (int l = 0; l < at; l++) {
                    if (!member[l] || place[l] == PLACE_LINK || on_link + link_bytes(l) > (double)options.planLinkBytes) continue;
                    const double size = (double)(layer[l]->SrcDataSize() * actBytes());
                    const double gain = place[l] == PLACE_PACKED ? f * size : size;
                    if (gain > best) { best = gain; pick = l; to = PLACE_LINK; }
                }
            }
            for (int pass = 0; pass < 2 && pick < 0; pass++) {
                for (int l = 0; l < at; l++) {
                    if (!member[l] || place[l] == PLACE_LINK) continue;
                    const double size = (double)(layer[l]->SrcDataSize() * actBytes());
                    const bool canPack = options.compressOffload && srcIsRectified(l) && f < 1.0;
                    const bool pack = place[l] == PLACE_RESIDENT && canPack;
                    if (pack != (pass == 0)) continue;
                    /* what the step down gives back: packing leaves f of the tensor, the link takes what is there */
                    const double gain = pack ? (1.0 - f) * size : (place[l] == PLACE_PACKED ? f * size : size);
                    if (gain > best) { best = gain; pick = l; to = pack ? PLACE_PACKED : PLACE_LINK; }
                }
            }
            if (pick < 0) break;
            place[pick] = to;
        }
        for (int l = 0; l < numLayers; l++)
            if (place[l] == PLACE_LINK) p.link += (double)(layer[l]->SrcDataSize() * actBytes());
        return p;
    };
    /* offloadLag < 0: the lag is part of the plan. What waits for its copy counts against the budget for as many layers
       as the lag is long, so a long lag may force more tensors out than a short one; what crosses the link costs time
       whatever the lag, a short lag only makes the compute stream wait for it sooner. So: of the lags tried, the one
       whose plan fits with the fewest bytes on the link, the longest of those; if none fits, the lowest peak. */
    Plan chosen;
    if (options.offloadLag >= 0) {
        chosen = plan_with(options.offloadLag);
    } else {
        bool have = false;
        for (int lag : {14, 10, 8, 6, 4, 2, 0}) {
            Plan p = plan_with(lag);
            const bool better = !have || (p.feasible != chosen.feasible ? p.feasible
                                          : p.feasible ? p.link < chosen.link : p.peak < chosen.peak);
            if (better) { chosen = p; have = true; }
        }
    }
    plannedLag = chosen.lag;
    planFeasibleFlag = chosen.feasible;
    planBudgetPeak = chosen.peak;
    return chosen.place;
}

/* addition (prefetchWithinPeak): the nearest offloaded tensor below currLayerId that is still on the host, if
 * holding it from now on keeps every layer down to the one that would have fetched it at or below the
 * replay's peak */
int Network::findPrefetchWithinPeak(int currLayerId) {
    if (planBwdPeak.size() != (size_t)numLayers) return -1;
    for (int id = currLayerId - 1; id >= 0; id--) {
        if (!isOffload[id] || isPrefetched[id] || zvcKept[id]) continue;
        const int issue = planIssueLayer[id];
        if (issue < 0 || issue >= currLayerId) return -1;
        const size_t staged = stagedFetchBytes(id); /* a packed stream is held ahead as its own length, not the tensor's */
        const size_t bytes = staged ? staged : actBytes() * layer[id]->SrcDataSize();
        for (int k = issue; k <= currLayerId; k++)
            if (planBwdPeak[k] + fetchedAhead[k] + bytes > peakBudget) return -1;
        for (int k = issue; k <= currLayerId; k++) fetchedAhead[k] += bytes;
        isPrefetched[id] = true;
        return id;
    }
    return -1;
}

/* network.cu:1198-1208: scan downward from currLayerId-1; the first layer that is offloaded and not
 * yet prefetched is the one to fetch; stop at the first convolution that is not eligible */
int Network::findPrefetchLayer(int currLayerId) {
    for (int id = currLayerId - 1; id >= 0; id--) {
        if (isOffload[id] == true && isPrefetched[id] == false && !zvcKept[id]) { /* (a kept packed input is expanded by its own layer) */
            isPrefetched[id] = true;
            return id;
        } else if (is_conv(layer[id]->LayerType())) {
            return -1;
        }
    }
    return -1;
}

/* ---- additions ------------------------------------------------------------------------------ */
/* Host tensors are float; a bfloat16 network converts at the boundary (round to nearest even). */
void Network::uploadActivations(void* dev, const float* host, size_t count) {
    if (options.dataType == VDNN_DTYPE_BF16) {
        std::vector<uint16_t> h(count);
        for (size_t i = 0; i < count; i++) h[i] = vdnn::float_to_bf16_host(host[i]);
        checkVDNN(vdnn_memcpy_h2d(ctx, dev, h.data(), count * sizeof(uint16_t)));
    } else {
        checkVDNN(vdnn_memcpy_h2d(ctx, dev, host, count * sizeof(float)));
    }
}

void Network::downloadActivations(float* host, const void* dev, size_t count) {
    if (options.dataType == VDNN_DTYPE_BF16) {
        std::vector<uint16_t> h(count);
        checkVDNN(vdnn_memcpy_d2h(ctx, h.data(), dev, count * sizeof(uint16_t)));
        for (size_t i = 0; i < count; i++) host[i] = vdnn::bf16_to_float_host(h[i]);
    } else {
        checkVDNN(vdnn_memcpy_d2h(ctx, host, dev, count * sizeof(float)));
    }
}

void Network::setInput(const float* host) {
    M_ASSERT(inputResident && inputData, "input block is not resident");
    if (options.planOnly) return;
    inputHost.assign(host, host + getInputSize());
    uploadActivations(inputData, host, getInputSize());
}

void Network::getInput(float* host) {
    M_ASSERT(inputResident && inputData, "input block is not resident");
    downloadActivations(host, inputData, getInputSize());
}

void Network::setLabels(const int32_t* labels) {
    const int classes = c_out * h_out * w_out;
    std::vector<float> dense((size_t)n_out * classes, 0.0f);
    for (int i = 0; i < n_out; i++) {
        M_ASSERT(labels[i] >= 0 && labels[i] < classes, "label out of range");
        dense[(size_t)i * classes + labels[i]] = 1.0f;
    }
    setLabelTensor(dense.data());
}

void Network::setLabelTensor(const float* host) {
    if (options.planOnly) return;
    uploadActivations(labelData, host, getOutputSize());
}

int Network::setLayerParams(int l, const float* filter, const float* bias) {
    if (l < 0 || l >= numLayers || !layer[l]->hasParams()) return -1;
    if (filter) checkVDNN(vdnn_memcpy_h2d(ctx, layer[l]->FilterData(), filter, layer[l]->FilterDataSize() * sizeof(float)));
    if (bias) checkVDNN(vdnn_memcpy_h2d(ctx, layer[l]->BiasData(), bias, layer[l]->BiasDataSize() * sizeof(float)));
    return 0;
}

int Network::getLayerParams(int l, float* filter, float* bias) {
    if (l < 0 || l >= numLayers || !layer[l]->hasParams()) return -1;
    if (filter) checkVDNN(vdnn_memcpy_d2h(ctx, filter, layer[l]->FilterData(), layer[l]->FilterDataSize() * sizeof(float)));
    if (bias) checkVDNN(vdnn_memcpy_d2h(ctx, bias, layer[l]->BiasData(), layer[l]->BiasDataSize() * sizeof(float)));
    return 0;
}

float Network::loss() {
    float v = 0.0f;
    if (options.planOnly) return v;
    checkVDNN(vdnn_memcpy_d2h(ctx, &v, lossData, sizeof(float)));
    return v;
}

void Network::synchronize() { checkVDNN(vdnn_device_synchronize(ctx)); }

NetworkStats Network::stats() {
    NetworkStats s = lastStats;
    vdnn_pool_peak(ctx, &s.peakBytesInUse, &s.peakExtent);
    size_t freeB = 0;
    vdnn_pool_info(ctx, &freeB, &s.poolBytes);
    s.weightBytes = 0;
    for (int l = 0; l < numLayers; l++) s.weightBytes += (layer[l]->FilterDataSize() + layer[l]->BiasDataSize()) * sizeof(float);
    return s;
}

void Network::resetPeak() { vdnn_pool_reset_peak(ctx); }
