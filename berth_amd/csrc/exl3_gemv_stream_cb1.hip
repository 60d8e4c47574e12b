#define BERTH_GEMV_CB 1
#include "exl3_gemv_stream_inst.cuh"
