// The tiled kernels of one (operation, epilogue) pair: GEMM, DQ8_EPI_REQUANT_CPU.
#include "qgemm_launch.h"

DQ8_INSTANTIATE_LAUNCH(false, DQ8_EPI_REQUANT_CPU)
