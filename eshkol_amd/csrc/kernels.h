/* Internal alias: every launcher is declared in the public tier header, the
 * switches and read-outs for tests in the testing header. */
#ifndef ESHKOL_HIP_KERNELS_H
#define ESHKOL_HIP_KERNELS_H
#include "eshkol/backend/gpu/gpu_hip_tiers.h"
#include "eshkol/backend/gpu/gpu_hip_testing.h"
#endif
