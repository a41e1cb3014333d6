/* A C99 client of the C ABI: the header must compile as plain C, the library must
 * link without any C++ or torch symbol leaking into the interface, and argument
 * errors must come back as status codes (no GPU is touched on these paths). */
#include <stdio.h>
#include <string.h>

#include "kinetics_amd.h"

int main(void) {
  int fails = 0;
  const int version = kin_version();
  printf("version %d\n", version);
  if (version < 10000) ++fails;
  if (kin_sel_list_capacity(128, 0, 1) != 129) ++fails;
  if (strcmp(kin_status_string(KIN_OK), "KIN_OK") != 0) ++fails;
  /* null pointers: rejected before anything is launched */
  int st = kin_rms_norm(NULL, NULL, NULL, NULL, 4, 4096, 4096, 4096, 1e-6f, NULL);
  printf("kin_rms_norm(NULL...) -> %s: %s\n", kin_status_string(st), kin_last_error());
  if (st != KIN_ERR_NULL_POINTER || strlen(kin_last_error()) == 0) ++fails;
  st = kin_blocktopk_decode_step(NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, 8, 0, 1, NULL, NULL, NULL, NULL, 2, 4, 1,
                                 128, 16, 8, 4, 0, 0, 0.0f, NULL, 0, NULL, 0, NULL, NULL);
  printf("kin_blocktopk_decode_step(NULL...) -> %s\n", kin_status_string(st));
  if (st != KIN_ERR_NULL_POINTER) ++fails;
  if (kin_step_workspace_bytes(4096, 1, 2048) != 0) ++fails;
  if (kin_step_workspace_bytes(2, 1, 4096) == 0) ++fails;
  if (kin_token_topk_workspace_bytes(2, 1, 4) != 256 + 2 * 4 * 16 * 4) ++fails;
  printf("%s\n", fails ? "FAILED" : "ok");
  return fails;
}
