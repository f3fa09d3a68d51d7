// MFMA kernel family (placeholder until the tiled kernels land): declines every problem.
#include "wm_common.hpp"

namespace wm {
bool mfma_supports(int, int64_t, int64_t, int64_t, int64_t, int) { return false; }
bool try_launch_mfma_p1(const Problem &, const View &, const View &, const View &, hipError_t *) { return false; }
bool try_launch_mfma_p2(const Problem &, const View &, const View &, const View &, hipError_t *) { return false; }
bool try_launch_mfma_p3(const Problem &, const View &, const View &, const View &, hipError_t *) { return false; }
}  // namespace wm
