// Internal interface between the C ABI (gmm_api.hip) and the kernel families.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/grouped_mm_hip.h"
#include "gmm_sched.h"

// Each returns 0 on success, 1 if the launch failed, -1 if the dtype pair is unsupported.
int gmm_launch_generic(GmmParams p, int in_dtype, int out_dtype, int num_cus, hipStream_t stream);

// Operand layout facts the host derived from strides.
struct GmmLayout {
  bool a_kc;  // A contiguous along K (row-major); otherwise contiguous along M
  bool b_kc;  // B contiguous along K (column-major); otherwise contiguous along N
};

// Tile configurations of the MFMA family.
// REG: tiles staged through registers, compiler-scheduled (takes every aligned layout and the
//      jagged-column / unaligned jagged-contraction cases).
// ASM: generated assembly tile with direct-to-LDS copies (the fast one).
enum GmmMfmaConfig : int { GMM_CFG_REG_256x256 = 0, GMM_CFG_ASM_256x256 = 1, GMM_CFG_COUNT };

// bf16 inputs only; out_dtype bf16 or fp32.  Returns like gmm_launch_generic.
int gmm_launch_mfma(GmmParams p, GmmLayout lay, int in_dtype, int out_dtype, int config, int num_cus, hipStream_t stream);
