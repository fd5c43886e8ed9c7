/* Compiled as C (not C++) by tests/test_c_abi.py: shows that include/helix_a2a.h is a C header and that a
 * plain C host can drive the device-free part of the library -- sizes for a given CU count and argument
 * validation -- through it. Prints one line per check; exit status 0 when all hold. */
#include <stdio.h>
#include <string.h>

#include "helix_a2a.h"

static int failures = 0;
#define CHECK(cond)                                        \
  do {                                                     \
    if (!(cond)) {                                         \
      printf("FAILED: %s (line %d)\n", #cond, __LINE__);   \
      failures++;                                          \
    }                                                      \
  } while (0)

int main(void) {
  helix_a2a_params_t p;
  static uint64_t dummy[4];

  CHECK(helix_a2a_max_channel_count(8, 256) == 128);
  CHECK(helix_a2a_max_channel_count(16, 256) == 64);
  CHECK(helix_a2a_max_channel_count(8, 132) == 66);
  CHECK(helix_a2a_workspace_size_per_rank(8, 256) == 537395200LL);
  CHECK(helix_a2a_workspace_size_per_rank(2, 256) == 134348800LL);
  CHECK(helix_a2a_auto_channel_count(8, 256, 256) == 128);
  CHECK(helix_a2a_auto_channel_count(8, 5, 256) == 5);
  CHECK(helix_a2a_max_channel_count(32, 256) == 32);
  CHECK(helix_a2a_max_channel_count(33, 256) < 0);
  CHECK(strstr(helix_a2a_last_error(), "cp_size") != NULL);

  memset(&p, 0, sizeof(p));
  CHECK(helix_a2a_alltoall(NULL, NULL) == HELIX_A2A_ERR_INVALID_ARGUMENT);
  p.cp_size = 4;
  p.cp_rank = 0;
  p.entry_count = 2;
  CHECK(helix_a2a_alltoall(&p, NULL) == HELIX_A2A_ERR_INVALID_ARGUMENT); /* null workspace */
  CHECK(strstr(helix_a2a_last_error(), "workspace") != NULL);
  p.workspace = dummy;
  p.workspace_stride_u64 = 2;
  p.send_fields[0].data = dummy;
  p.send_fields[0].element_count = 64;
  p.send_fields[0].element_size = 4; /* partial_o must be 2-byte elements */
  p.send_fields[0].stride_bytes = 256;
  CHECK(helix_a2a_alltoall(&p, NULL) == HELIX_A2A_ERR_INVALID_ARGUMENT);
  CHECK(strstr(helix_a2a_last_error(), "element size") != NULL);
  CHECK(helix_a2a_init_workspace(NULL, 4, 256, NULL) == HELIX_A2A_ERR_INVALID_ARGUMENT);
  CHECK(strlen(helix_a2a_version()) > 0);

  printf("%s: %d failure(s)\n", failures ? "c_abi_smoke FAILED" : "c_abi_smoke ok", failures);
  return failures ? 1 : 0;
}
