/* Internal alias: every launcher is declared in the public tier header. */
#ifndef ESHKOL_HIP_KERNELS_H
#define ESHKOL_HIP_KERNELS_H
#include "eshkol/backend/gpu/gpu_hip_tiers.h"
#endif
