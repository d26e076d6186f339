// Row-resident backward (dq + dk + dv in one pass), float16 instantiations.
#include "tri_bwd_row_inst.hpp"

namespace tri {

hipError_t bwd_row_launch_f16(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry) {
  return bwd_row_dispatch_d<_Float16>(a, bh, d, tile, st, dry);
}

}  // namespace tri
