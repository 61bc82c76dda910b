/* A plain C99 client of the C ABI: includes the public header, links against
 * libatex_norms_hip.so and calls only the host-side entry points (no GPU needed).
 * Built and run by tests/test_host_semantics.py. Exit code 0 = every check passed. */
#include <stdio.h>
#include <string.h>

#include "atex_norms.h"

#define CHECK(cond)                                                  \
  do {                                                               \
    if (!(cond)) {                                                   \
      fprintf(stderr, "line %d: %s failed (%s)\n", __LINE__, #cond,  \
              atexn_last_error());                                   \
      return 1;                                                      \
    }                                                                \
  } while (0)

int main(void) {
  int64_t dims[4] = {2, 3, 4, 5};
  int axis[2] = {-1, 2};
  int64_t N = 0, D = 0, C = 0;
  int layout = -1;

  CHECK(atexn_abi_version() >= 1);
  CHECK(strcmp(atexn_status_string(ATEXN_OK), atexn_status_string(ATEXN_INVALID_ARGUMENT)) != 0);

  /* axes {-1, 2} of a rank-4 tensor: packed up to the last dim -> N = 2*3, D = 4*5 */
  CHECK(atexn_layer_norm_resolve_axes(4, dims, axis, 2, &N, &D) == ATEXN_OK);
  CHECK(N == 6 && D == 20);
  /* axis {1} alone is not packed up to the last dim */
  axis[0] = 1;
  CHECK(atexn_layer_norm_resolve_axes(4, dims, axis, 1, &N, &D) == ATEXN_INVALID_ARGUMENT);
  CHECK(strlen(atexn_last_error()) > 0);

  CHECK(atexn_instance_norm_resolve_format(4, dims, "NCHW", &layout, &N, &C, &D) == ATEXN_OK);
  CHECK(layout == ATEXN_LAYOUT_NC_ && N == 2 && C == 3 && D == 20);
  CHECK(atexn_instance_norm_resolve_format(4, dims, NULL, &layout, &N, &C, &D) == ATEXN_OK);
  CHECK(layout == ATEXN_LAYOUT_N_C && N == 2 && C == 5 && D == 12);
  CHECK(atexn_instance_norm_resolve_format(4, dims, "HWNC", &layout, &N, &C, &D) ==
        ATEXN_INVALID_ARGUMENT);

  /* a null data pointer is rejected before anything touches a device */
  CHECK(atexn_layer_norm_fwd(ATEXN_F16, NULL, NULL, NULL, 4, 8, 1e-3f, NULL, NULL, NULL, NULL, 0,
                             NULL) == ATEXN_INVALID_ARGUMENT);
  /* empty input: success, nothing read */
  CHECK(atexn_layer_norm_fwd(ATEXN_F16, NULL, NULL, NULL, 0, 8, 1e-3f, NULL, NULL, NULL, NULL, 0,
                             NULL) == ATEXN_OK);
  printf("capi host check ok\n");
  return 0;
}
