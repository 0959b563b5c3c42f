// Command-line front end: vdnn MODEL POLICY ALGO [--steps N] [--warmup N] [--batch N] [--seed N]
//                                               [--cap-gb X] [--host-sync] [--plan] [--verbose] [--refined] [--fuse]
//                                               [--zvc] [--keep-packed] [--hbm-budget-gb X] [--plan-link-gb X] [--packed-fraction F] [--in-place] [--recompute-first] ...
// The three positional words are the reference's grammar (vdnn.cu:8-54, README.md:18-60). The
// reference times one unsynchronised iteration and prints microseconds labelled "ms"
// (vdnn.cu:72-79); here the device is synchronised on both sides of the timed region and the
// figures are printed as one JSON line after the human-readable banner.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>

#include "network.h"
#include "vdnn_capi.h"

using namespace std;
using namespace std::chrono;

/* vdnn.cu:8-54 */
static void parseVdnnInputs(char** argv, CNN_t* _cnnType, vdnn_t* _vdnnType, vdnnAlgoMode_t* _algoMode) {
    int v = 0;
    if (vdnn_parse_cnn(argv[1], &v) != 0)
        M_ASSERT(0, "CNN type must be one of ALEXNET, OVERFEAT, VGG16_64, VGG16_128, VGG16_256, VGG16_512, ALEXNET_LRN");
    *_cnnType = (CNN_t)v;
    if (vdnn_parse_policy(argv[2], &v) != 0)
        M_ASSERT(0, "VDNN type must be one of BASELINE, VDNN_NONE, VDNN_ALL, VDNN_CONV");
    *_vdnnType = (vdnn_t)v;
    if (vdnn_parse_algo(argv[3], &v) != 0)
        M_ASSERT(0, "Algorithm type must be one of VDNN_MEMORY_OPT_ALGO, VDNN_PERF_OPT_ALGO, VDNN_DYNAMIC_ALGO");
    *_algoMode = (vdnnAlgoMode_t)v;

    printf("################# VDNN Configurations #################\n");
    printf("CNN Model Type: %s\n", argv[1]);
    printf("VDNN Mode: %s\n", argv[2]);
    printf("Convolution Algorithm: %s\n", argv[3]);
    printf("#######################################################\n\n");
}

int main(int argc, char** argv) {
    M_ASSERT(argc >= 4, "Need to specify CNN model, VDNN mode, and Algorithm choice");
    CNN_t cnnType;
    vdnn_t vdnnType;
    vdnnAlgoMode_t algoMode;
    parseVdnnInputs(argv, &cnnType, &vdnnType, &algoMode);

    NetworkOptions opt;
    int steps = 1, warmup = 0, batch = DEFAULT_BATCH_SIZE;
    for (int i = 4; i < argc; i++) {
        auto need = [&](const char* flag) { M_ASSERT(i + 1 < argc, flag); return argv[++i]; };
        if (!strcmp(argv[i], "--steps")) steps = atoi(need("--steps needs a value"));
        else if (!strcmp(argv[i], "--warmup")) warmup = atoi(need("--warmup needs a value"));
        else if (!strcmp(argv[i], "--batch")) batch = atoi(need("--batch needs a value"));
        else if (!strcmp(argv[i], "--seed")) opt.seed = strtoull(need("--seed needs a value"), nullptr, 10);
        else if (!strcmp(argv[i], "--cap-gb")) opt.capBytes = (size_t)(atof(need("--cap-gb needs a value")) * 1e9);
        else if (!strcmp(argv[i], "--host-sync")) opt.hostSync = true;
        else if (!strcmp(argv[i], "--plan")) opt.planOnly = true;
        else if (!strcmp(argv[i], "--refined")) opt.refinedLifetimes = true;
        else if (!strcmp(argv[i], "--fuse")) opt.fuseActivations = true;
        else if (!strcmp(argv[i], "--zvc")) opt.compressOffload = true;
        else if (!strcmp(argv[i], "--keep-packed")) opt.keepPackedOnDevice = true;
        else if (!strcmp(argv[i], "--prefetch-within-peak")) opt.prefetchWithinPeak = true;
        else if (!strcmp(argv[i], "--keep-tail-gb")) opt.keepTailBytes = (size_t)(atof(need("--keep-tail-gb needs a value")) * 1e9);
        else if (!strcmp(argv[i], "--hbm-budget-gb")) opt.hbmBudgetBytes = (size_t)(atof(need("--hbm-budget-gb needs a value")) * 1e9);
        else if (!strcmp(argv[i], "--plan-link-gb")) opt.planLinkBytes = (size_t)(atof(need("--plan-link-gb needs a value")) * 1e9);
        else if (!strcmp(argv[i], "--packed-fraction")) opt.planPackedFraction = atof(need("--packed-fraction needs a value"));
        else if (!strcmp(argv[i], "--in-place")) opt.inPlaceBackward = true;
        else if (!strcmp(argv[i], "--recompute-first")) opt.recomputeFirstLayer = true;
        else if (!strcmp(argv[i], "--unfused")) opt.unfusedOptimizer = true;
        else if (!strcmp(argv[i], "--bf16")) opt.dataType = VDNN_DTYPE_BF16;
        else if (!strcmp(argv[i], "--offload-lag")) opt.offloadLag = atoi(need("--offload-lag needs a value"));
        else if (!strcmp(argv[i], "--prefetch-depth")) opt.prefetchDepth = atoi(need("--prefetch-depth needs a value"));
        else if (!strcmp(argv[i], "--winograd")) vdnn_conv_perf_variant(1); /* VDNN_PERF_OPT_ALGO: Winograd where the default variant and it both apply */
        else if (!strcmp(argv[i], "--verbose")) opt.verbose = true;
        else M_ASSERT(0, "unknown flag");
    }

    /* Initialize network */
    Network network(cnnType, vdnnType, algoMode, batch, opt);

    /* A step that runs out of pool memory returns -1 when asked to (layer.h:110-128 of the reference: dynamic mode);
     * under an artificial cap or a budget that is the expected failure, so the steps are run that way and the
     * program says so and exits non-zero instead of printing a throughput. Without either, a failed request
     * aborts as in the reference. */
    const bool soft = opt.capBytes != 0 || opt.hbmBudgetBytes != 0;
    auto step = [&](const char* phase, int i) {
        int rc = network.forwardPropagation(soft);
        const char* pass = "forward";
        if (rc >= 0) { rc = network.backwardPropagation(soft); pass = "backward"; }
        if (rc < 0) {
            const NetworkStats st = network.stats();
            fprintf(stderr, "vdnn: %s step %d: %sPropagation returned %d (out of pool memory: %zu bytes in use at the peak, cap %zu, "
                            "budget %zu, plan_feasible %s, plan_peak_bytes %zu); no throughput to report\n",
                    phase, i, pass, rc, st.peakBytesInUse, opt.capBytes, opt.hbmBudgetBytes, network.planFeasible() ? "true" : "false",
                    network.planPeakBytes());
            printf("{\"model\": \"%s\", \"policy\": \"%s\", \"algo\": \"%s\", \"batch\": %d, \"error\": \"out of memory\", \"failed_in\": \"%s\", "
                   "\"plan_only\": %s, \"plan_feasible\": %s, \"plan_peak_bytes\": %zu}\n",
                   argv[1], argv[2], argv[3], network.batch(), pass, opt.planOnly ? "true" : "false",
                   network.planFeasible() ? "true" : "false", network.planPeakBytes());
            fflush(stdout);
            exit(3);
        }
    };

    for (int i = 0; i < warmup; i++) step("warm-up", i);
    network.synchronize();
    network.resetPeak();

    /* Perform `steps` iterations of fwd/bwd propagation */
    auto t1 = high_resolution_clock::now();
    for (int i = 0; i < steps; i++) step("timed", i);
    network.synchronize();
    auto t2 = high_resolution_clock::now();

    const double us = (double)duration_cast<microseconds>(t2 - t1).count();
    const NetworkStats st = network.stats();
    cout << "Elapsed Time: " << us / 1000.0 << " ms for " << steps << " step(s)" << endl;
    printf("{\"model\": \"%s\", \"policy\": \"%s\", \"algo\": \"%s\", \"batch\": %d, \"steps\": %d, \"ms_per_step\": %.3f, "
           "\"images_per_s\": %.2f, \"loss\": %.6f, \"peak_bytes\": %zu, \"peak_extent\": %zu, \"offload_bytes\": %zu, "
           "\"prefetch_bytes\": %zu, \"pinned_bytes\": %zu, \"plan_only\": %s, \"plan_feasible\": %s, \"plan_peak_bytes\": %zu}\n",
           argv[1], argv[2], argv[3], network.batch(), steps, us / 1000.0 / steps,
           opt.planOnly ? 0.0 : network.batch() * steps / (us * 1e-6), network.loss(), st.peakBytesInUse, st.peakExtent,
           st.offloadBytes, st.prefetchBytes, st.pinnedBytes, opt.planOnly ? "true" : "false",
           network.planFeasible() ? "true" : "false", network.planPeakBytes());
    return 0;
}
