// Row-resident backward (dq + dk + dv in one pass), bfloat16 instantiations.
#include "tri_bwd_row_inst.hpp"

namespace tri {

hipError_t bwd_row_launch_bf16(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry) {
  return bwd_row_dispatch_d<__bf16>(a, bh, d, tile, st, dry);
}

}  // namespace tri
