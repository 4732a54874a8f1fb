// MFMA (matrix-core) NA1D kernels for gfx950.
#include "na1d_common.h"

namespace na1d {
namespace mfma {

int qk(float *, const void *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int av(void *, const float *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int gather(void *, const float *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int fused_fwd(void *, float *, const void *, const void *, const void *, const float *, const int32_t *,
              const Geom &, float, int, hipStream_t) {
    return NA1D_ERR_UNSUPPORTED;
}
int fused_bwd(void *, void *, void *, float *, const void *, const void *, const void *, const void *, const void *,
              const float *, const float *, const int32_t *, const Geom &, float, int, hipStream_t) {
    return NA1D_ERR_UNSUPPORTED;
}

}  // namespace mfma
}  // namespace na1d
