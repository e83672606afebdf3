// One translation unit per (element type, direction) of the softmax kernels:
// compiled with -DOSLO_SM_TYPE=<float|_Float16|__bf16> and -DOSLO_SM_PART=<0|1>
// (0: forward launchers, 1: backward launchers), see the Makefile.
#include "softmax_kernels.hip.h"

namespace oslo {

#if OSLO_SM_PART == 0
OSLO_SM_FWD_INSTANCES(, OSLO_SM_TYPE)
#else
OSLO_SM_BWD_INSTANCES(, OSLO_SM_TYPE)
#endif

}  // namespace oslo
