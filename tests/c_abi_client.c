/* A plain C caller of libomni_moe_hip.so: what a host program in another language binds.
 * Only host-side entry points are called (version, error strings, workspace sizes, argument
 * checks), so it runs without a GPU.  Built and run by tests/test_abi.py. */
#include <stdio.h>
#include <string.h>

#include "omni_moe_hip.h"

int main(void) {
  if (omni_abi_version() != 1) return 1;
  if (strcmp(omni_error_string(OMNI_OK), "ok") != 0) return 2;
  /* README shape: 4096 tokens, hidden 1024, intermediate 4096, 4096 experts (64 x 64), top-16, bf16 */
  const size_t layer = omni_moe_workspace_bytes(4096, 1024, 4096, 4096, 64, 16, OMNI_BF16);
  const size_t mlp = omni_mlp_workspace_bytes(4096, 1024, 4096, OMNI_BF16);
  if (mlp != (size_t)4096 * 4096 * 2 || layer <= mlp) return 3;
  if (omni_expert_workspace_bytes(4096, 1024, 4096, 16, OMNI_BF16, OMNI_EXPERT_ALGO_GATHER) != 0) return 4;
  if (omni_expert_bwd_workspace_bytes(4096, 1024, 4096, 16, OMNI_BF16) == 0) return 5;
  /* rejected before anything touches a device */
  if (omni_router_select(NULL, NULL, NULL, NULL, 8, 4, 3, OMNI_BF16, NULL) != OMNI_ERR_TOPK) return 6;
  if (omni_expert_fwd(NULL, NULL, NULL, NULL, NULL, NULL, 8, 64, 16, 2, 7, 0, NULL, NULL) >= 0) return 7;   /* dtype 7 */
  if (omni_add_inplace(NULL, NULL, 3, OMNI_BF16, NULL) >= 0) return 8;                                      /* 3 elements */
  printf("c abi ok: layer workspace %zu bytes\n", layer);
  return 0;
}
