// bf16 GEMM with direct global->LDS loads, NT layout (see gemm_bf16_dma.inc).
#define DMA_AKM false
#define DMA_BKM false
#define DMA_ENTRY gemm_bf16_dma_nt
#define DMA_GROUPED_ENTRY gemm_bf16_dma_nt_grouped
#include "gemm_bf16_dma.inc"
