// The 3-, 5- and 6-bit instantiations of the 128-column-tile GEMM (qmm_mid.hip):
// MLX's 3- and 5-byte packs, a row's codes as one little-endian bit stream.
#define MFQ_MID_STREAM 1
#include "qmm_mid.hip"
