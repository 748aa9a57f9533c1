// bf16 GEMM with direct global->LDS loads, TN layout (see gemm_bf16_dma.inc).
#define DMA_AKM true
#define DMA_BKM true
#define DMA_ENTRY gemm_bf16_dma_tn
#define DMA_GROUPED_ENTRY gemm_bf16_dma_tn_grouped
#include "gemm_bf16_dma.inc"
