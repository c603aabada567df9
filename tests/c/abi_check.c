/* Plain C99 client of libmoe_i8.so: the header must compile as C, every call below must behave as
 * documented without a GPU (sizes, argument errors), and the error text must be retrievable. */
#include <stdio.h>
#include <string.h>

#include "moe_i8.h"

#define CHECK(cond)                                      \
  do {                                                   \
    if (!(cond)) {                                       \
      printf("FAILED line %d: %s\n", __LINE__, #cond);   \
      return 1;                                          \
    }                                                    \
  } while (0)

int main(void) {
  static int32_t buf[1024];
  CHECK(moe_i8_version() >= 1);
  CHECK(moe_i8_sorted_capacity(128, 128, 64) == 128 + 128 * 63);
  CHECK(moe_i8_sorted_capacity(2, 128, 64) == 2 * 64);
  CHECK(moe_i8_workspace_bytes(16, 8, 128, 2048, 768, 64) % 256 == 0);
  CHECK(moe_i8_workspace_bytes(16, 8, 128, 2048, 768, 48) == -1);
  CHECK(moe_i8_dense_workspace_bytes(100, 2048, 768) > moe_i8_dense_workspace_bytes(100, 2048, 0));
  CHECK(moe_i8_align_block_size(buf, 8, 4, 48, buf, 260, buf, 5, buf, NULL, 0, NULL) == MOE_I8_EINVAL);
  CHECK(strstr(moe_i8_last_error(), "block_size") != NULL);
  CHECK(moe_i8_quant_rows(buf, 7, 4, 64, 64, NULL, 1, 4, (int8_t*)buf, (float*)buf, NULL) == MOE_I8_EUNSUPPORTED);
  CHECK(moe_i8_route_topk((const float*)buf, 4, 128, 65, MOE_I8_SCORE_SOFTMAX, NULL, 1, 1, 0, 1, 1.0f, (float*)buf, buf,
                          NULL, 0, 0, 0, NULL) == MOE_I8_EINVAL);
  CHECK(moe_i8_fused_experts(buf, (const int8_t*)buf, (const int8_t*)buf, (const float*)buf, buf, (const float*)buf,
                             (const float*)buf, buf, 0, 8, 128, 2048, 768, 64, buf, 0, MOE_I8_GEMM_AUTO, NULL) ==
        MOE_I8_OK); /* zero tokens: nothing to do */
  CHECK(moe_i8_fused_experts(buf, (const int8_t*)buf, (const int8_t*)buf, (const float*)buf, buf, (const float*)buf,
                             (const float*)buf, buf, 4, 8, 128, 2000, 768, 64, buf, 1 << 20, MOE_I8_GEMM_AUTO,
                             NULL) == MOE_I8_EINVAL);
  printf("ok\n");
  return 0;
}
