#define BERTH_GEMV_CB 0
#include "exl3_gemv_stream_inst.cuh"
