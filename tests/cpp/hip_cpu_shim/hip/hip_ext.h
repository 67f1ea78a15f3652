// Part of the CPU stand-in for the HIP runtime (test infrastructure only):
// hipExtLaunchKernelGGL is defined in hip_runtime.h.
#include "hip_runtime.h"
