// placeholder until the MFMA chunk kernels land
#include "lnx_common.h"
extern "C" uint64_t lnx_chunk_workspace_bytes(const lnx_scan_args* a) { (void)a; return 0; }
extern "C" int lnx_chunk_fwd(const lnx_scan_args* a, void* s) { (void)a; (void)s; return lnx_set_error(LNX_ERR_SHAPE, "chunk forward not built"); }
extern "C" int lnx_chunk_bwd(const lnx_scan_args* a, void* s) { (void)a; (void)s; return lnx_set_error(LNX_ERR_SHAPE, "chunk backward not built"); }
