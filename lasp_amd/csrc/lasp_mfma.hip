// placeholder until the MFMA kernels land: route to the generic kernels
#include "lasp_common.h"
namespace lasp {
int mfma_fwd(const FwdArgs &a, const Geom &g, hipStream_t st) { return generic_fwd(a, g, LASP_DTYPE_BF16, st); }
int mfma_bwd(const BwdArgs &a, const Geom &g, hipStream_t st) { return generic_bwd(a, g, LASP_DTYPE_BF16, st); }
}
