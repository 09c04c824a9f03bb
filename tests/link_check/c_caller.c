/* A plain C99 caller of the C ABI: proves that include/amem.h and include/amem_testing.h are valid C
 * and that the symbols link. */
#include <stdio.h>
#include <stdlib.h>

#include "amem.h"
#include "amem_testing.h"

int main(void) {
  amem_counters c;
  amem_region_info info;
  int gid = -1;
  if (amem_set_enabled(1) != 0) return 1;
  if (amem_set_group_id(77) != 0) return 2;
  if (amem_add_alloc_info(0x7f0000000000ull, 2u << 20, AMEM_TYPE_LOCAL, 0, 0xabcull, -1, 0, NULL, AMEM_CALLER_P2P) != 0) return 3;
  if (amem_set_group_id(78) != 1) return 4; /* too late */
  amem_get_group_id(&gid);
  if (gid != 77) return 5;
  if (amem_region_count(0) != 1 || amem_region_at(0, 0, &info) != 0 || info.handle != 0xabcull) return 6;
  if (info.state != AMEM_STATE_ALLOC || info.tags != AMEM_CALLER_P2P) return 7;
  amem_get_counters(&c);
  if (c.alloc_bytes[AMEM_CALLER_P2P] != (2u << 20) || c.group_id != 77) return 8;
  if (ncclMemStats() != 0 || ncclGetGroupID(&gid) != 0) return 9;
  if (amem_del_alloc_info(0x7f0000000000ull, 0xabcull, 0) != 0 || amem_region_count(0) != 0) return 10;
  if (amem_shutdown() != 0) return 11;
  if (amem_device_count() < 0) return 12; /* a helper of amem_testing.h: 0 without a GPU */
  printf("c caller ok\n");
  return 0;
}
