// bf16 GEMM with direct global->LDS loads, NN layout (see gemm_bf16_dma.inc).
#define DMA_AKM false
#define DMA_BKM true
#define DMA_ENTRY gemm_bf16_dma_nn
#define DMA_GROUPED_ENTRY gemm_bf16_dma_nn_grouped
#include "gemm_bf16_dma.inc"
