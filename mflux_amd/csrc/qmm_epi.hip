// The instantiations of the 256 x 256-tile GEMM (qmm.hip) whose results pass
// through an epilogue (epilogue.h) on their way to y.
#define MFQ_QMM_EPI 1
#include "qmm.hip"
