#define BERTH_GEMM_CB 0
#include "exl3_gemm_inst.cuh"
