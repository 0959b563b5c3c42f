// A main of the shape of the reference's (vdnn.cu:56-83): three words -> enums, a Network, one forward and one
// backward pass, the elapsed time. It includes only the public headers under include/ and is compiled by
// tests/test_host_logic.py with the host compiler against libvdnn_amd.so. With --plan as a fourth argument
// the network replays its allocation schedule without a device, which is how the test runs it on a machine
// without a GPU; without it the constructor is the reference's four-argument one.
#include <chrono>
#include <cstdio>
#include <cstring>
#include <iostream>

#include "network.h"
#include "vdnn_capi.h"

using namespace std;
using namespace std::chrono;

static void parseVdnnInputs(char** argv, CNN_t* _cnnType, vdnn_t* _vdnnType, vdnnAlgoMode_t* _algoMode) {
    int cnn = 0, policy = 0, algo = 0;
    M_ASSERT(vdnn_parse_cnn(argv[1], &cnn) == 0, "unknown CNN type");
    M_ASSERT(vdnn_parse_policy(argv[2], &policy) == 0, "unknown VDNN type");
    M_ASSERT(vdnn_parse_algo(argv[3], &algo) == 0, "unknown algorithm type");
    *_cnnType = (CNN_t)cnn;
    *_vdnnType = (vdnn_t)policy;
    *_algoMode = (vdnnAlgoMode_t)algo;
}

int main(int argc, char** argv) {
    M_ASSERT(argc >= 4, "Need to specify CNN model, VDNN mode, and Algorithm choice");
    CNN_t cnnType;
    vdnn_t vdnnType;
    vdnnAlgoMode_t algoMode;
    parseVdnnInputs(argv, &cnnType, &vdnnType, &algoMode);

    const bool plan = argc > 4 && strcmp(argv[4], "--plan") == 0;
    NetworkOptions options;
    options.planOnly = plan;
    Network* network = plan ? new Network(cnnType, vdnnType, algoMode, DEFAULT_BATCH_SIZE, options)
                            : new Network(cnnType, vdnnType, algoMode);

    auto t1 = high_resolution_clock::now();
    const int fwd = network->forwardPropagation();
    const int bwd = network->backwardPropagation();
    network->synchronize();
    auto t2 = high_resolution_clock::now();

    Layer** layers = network->layerArray();
    size_t offloaded = 0;
    for (int l = 0; l < network->numLayersCount(); l++)
        if (network->offloadedSrcDataArray()[l] != NULL) offloaded += layers[l]->SrcDataSize() * sizeof(DATATYPE);
    cout << "Elapsed Time: " << duration_cast<microseconds>(t2 - t1).count() << " us" << endl;
    printf("status %d %d layers %d batch %d input %zu output %zu offloaded %zu prefetched %zu dxdy %zu\n", fwd, bwd,
           network->numLayersCount(), network->batch(), network->getInputSize(), network->getOutputSize(), offloaded,
           network->stats().prefetchBytes, network->findMaxDxDySize());
    delete network;
    return fwd == 0 && bwd == 0 ? 0 : 1;
}
