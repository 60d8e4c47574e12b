#define BERTH_GEMM_CB 1
#include "exl3_gemm_inst.cuh"
