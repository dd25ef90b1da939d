/* Internal alias: every launcher is declared in the public tier header. */
#ifndef ESHKOL_HIP_TIERS_INTERNAL_H
#define ESHKOL_HIP_TIERS_INTERNAL_H
#include "eshkol/backend/gpu/gpu_hip_tiers.h"
#endif
