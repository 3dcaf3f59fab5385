// Host-side helpers shared by the C-ABI launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../../include/gpuk_amd.h"

namespace gpuk {

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
inline int round_up(int v, int m) { return (v + m - 1) / m * m; }
inline int hip_status(hipError_t e) { return e == hipSuccess ? GPUK_OK : GPUK_ERR_LAUNCH; }

void set_norm_quant_tuning(int key, int value);  // add_rmsnorm_quant.hip
void set_rope_tuning(int key, int value);  // rope_rms.hip

}  // namespace gpuk
