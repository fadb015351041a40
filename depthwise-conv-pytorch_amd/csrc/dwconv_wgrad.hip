// fp32 grad-weight with LDS tiles (placeholder until the tiled kernel lands).
#include "dwconv_common.hpp"

namespace dwconv {

size_t wgrad_tiled_workspace(const WgradGeometry &) { return 0; }

int try_launch_wgrad_tiled(const float *, const float *, float *, void *, size_t, const WgradGeometry &,
                           hipStream_t)
{
    return -1;
}

}  // namespace dwconv
