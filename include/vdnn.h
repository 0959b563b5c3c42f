/* Public parameters and enums of the vDNN engine.
 *
 * Names and numeric values follow the reference's vdnn.h (vdnn.h:5-61) so that code written against
 * it keeps compiling; additions are appended after the reference's last value and marked.
 */
#ifndef VDNN_AMD_VDNN_H_
#define VDNN_AMD_VDNN_H_

/* Parameters (vdnn.h:5-12) */
#define DEFAULT_DEVICE 0
#define DEFAULT_NUM_LAYER 40
#define DEFAULT_BATCH_SIZE 128
#define LEARNING_RATE 1e-5
#define BLOCK_SIZE 256
#define RANDOM_VALUE_LIMIT 1e-2
#define DATATYPE float

/* Memory policy (vdnn.h:23-29) */
typedef enum {
    BASELINE  = 0, /* every layer output resident; dx/dy ping-pong pair and one shared workspace */
    VDNN_NONE = 1, /* per-layer allocation, nothing offloaded */
    VDNN_ALL  = 2, /* srcData of every layer but the last is offloaded, then prefetched in backward */
    VDNN_CONV = 3, /* srcData of convolution layers only */
} vdnn_t;

/* Convolution algorithm mode (vdnn.h:31-36) */
typedef enum {
    VDNN_MEMORY_OPT_ALGO = 0, /* implicit GEMM, im2col tiles staged in LDS only, zero workspace */
    VDNN_PERF_OPT_ALGO   = 1, /* workspace-using variants (packed filters, wide split-K) */
    VDNN_DYNAMIC_ALGO    = 2, /* fall-back ladder driven by out-of-memory results */
} vdnnAlgoMode_t;

/* Layer kinds (vdnn.h:38-50); LRN is an addition (the reference has no normalisation layer). */
typedef enum {
    FC_GEMM         = 0,
    CONV            = 1,
    FC_CONV         = 2,
    RELU            = 3,
    TANH            = 4,
    SIGMOID         = 5,
    SOFTMAX         = 6,
    POOL            = 7,
    CONCATENATE     = 8,
    NUM_LAYER_TYPES = 9,
    LRN             = 10, /* addition: cross-channel local response normalisation */
} Layer_t;

/* Networks (vdnn.h:52-61); ALEXNET_LRN and VGG16_512 are additions. */
typedef enum {
    ALEXNET     = 0, /* the reference's 19-layer table (network.cu:156-323), no LRN */
    OVERFEAT    = 1,
    GOOGLENET   = 2, /* empty in the reference (network.cu:497-499); rejected here */
    VGG16_64    = 3,
    VGG16_128   = 4,
    VGG16_256   = 5,
    CUSTOM_CNN  = 6, /* empty in the reference (network.cu:815-817); rejected here */
    ALEXNET_LRN = 7, /* addition: AlexNet with the two LRN layers, conv-ReLU-LRN-pool (21 layers) */
    VGG16_512   = 8, /* addition: VGG16 at batch 512 */
} CNN_t;

#endif
