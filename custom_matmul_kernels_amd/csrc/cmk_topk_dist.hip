// topk_bmm for the distances that run on the vector unit ((x-y)^2 and |x-y|,
// reference kernels/bmm_helpers.cu:28-35, 46-52): the same kernel template as
// the inner product, instantiated here so that the two compile side by side.
#include "cmk_topk_kernel.hpp"

namespace cmk {

void launch_topk_dist(int distance, int xk, int yk, bool multi, dim3 grid, dim3 block, hipStream_t st,
                      const TopkArgs& a) {
  if (distance == kL2) launch_topk_kernel<kL2>(xk, yk, multi, grid, block, st, a);
  else launch_topk_kernel<kL1>(xk, yk, multi, grid, block, st, a);
}

}  // namespace cmk
