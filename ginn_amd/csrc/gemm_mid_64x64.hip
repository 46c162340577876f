// Instantiates the 64 x 64 tile shape of the 128 x 128 product kernel family.
#include "gemm_mid.h"

namespace ginn_hip {
namespace mid {
template int launch_shape<1, 1>(ginn_hip_ctx*, const MidParams&, int, int, int, int, bool, bool);
}  // namespace mid
}  // namespace ginn_hip
