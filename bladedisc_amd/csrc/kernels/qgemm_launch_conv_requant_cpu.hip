// The tiled kernels of one (operation, epilogue) pair: implicit-GEMM convolution, DQ8_EPI_REQUANT_CPU.
#include "qgemm_launch.h"

DQ8_INSTANTIATE_LAUNCH(true, DQ8_EPI_REQUANT_CPU)
