#define BERTH_GEMV_CB 2
#include "exl3_gemv_stream_inst.cuh"
