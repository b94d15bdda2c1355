// placeholder until the backward kernels land
#include "chunk_common.h"
extern "C" int lnx_chunk_bwd(const lnx_scan_args* a, void* s) {
  (void)s;
  int rc = lnx_chunk_check(a, true);
  if (rc != LNX_OK) return rc;
  return lnx_set_error(LNX_ERR_SHAPE, "chunk backward not built");
}
