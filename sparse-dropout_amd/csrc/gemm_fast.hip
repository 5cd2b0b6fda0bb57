// Specialised kernels for tile-aligned shapes (placeholder dispatch: nothing specialised yet).
#include "common.h"

namespace sd {

int launch_fast(const GemmArgs&, int, int, hipStream_t) { return SD_ERR_UNSUPPORTED; }

}  // namespace sd
