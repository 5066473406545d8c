// ABI bookkeeping of libomni_moe_hip.so: version and error strings.
#include "omni_moe_hip.h"
#include "common.h"

extern "C" OMNI_API int32_t omni_abi_version(void) { return OMNI_ABI_VERSION; }

extern "C" OMNI_API int32_t omni_init(void) {
  for (omni::LdsKernel* k = omni::lds_kernel_list(); k; k = k->next)
    if (hipError_t e = k->ensure(); e != hipSuccess) return OMNI_ERR_HIP_BASE + (int)e;
  return omni::schedule_scratch_prepare();
}

extern "C" OMNI_API const char* omni_error_string(int32_t code) {
  switch (code) {
    case OMNI_OK: return "ok";
    case OMNI_ERR_NULL: return "a required pointer is NULL";
    case OMNI_ERR_SHAPE: return "a size is negative, misaligned or out of range";
    case OMNI_ERR_DTYPE: return "unknown dtype code";
    case OMNI_ERR_TOPK: return "num_experts_per_token must be even, <= 128 and <= num_expert_sqrt^2";
    case OMNI_ERR_UNSUPPORTED: return "valid request that no kernel of this library covers";
    case OMNI_ERR_WORKSPACE: return "workspace is NULL or too small";
    case OMNI_ERR_SCRATCH: return "the request needs more than the fixed device scratch of the entry point that allocates nothing";
    default: return code >= OMNI_ERR_HIP_BASE ? "the HIP runtime refused a launch (code - 1000 is the hipError_t)" : "unknown error code";
  }
}
