// TEST INFRASTRUCTURE ONLY: -mf16c build of the oracle kernels (hardware f16 conversions)
#define ORC_NS orc_hw
#define ORC_HW_F16 1
#include "orc_kernels.inc"
