// TEST INFRASTRUCTURE ONLY: portable build of the oracle kernels (software f16 conversions)
#define ORC_NS orc_soft
#define ORC_HW_F16 0
#include "orc_kernels.inc"
