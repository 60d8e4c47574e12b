#define BERTH_GEMM_CB 2
#include "exl3_gemm_inst.cuh"
