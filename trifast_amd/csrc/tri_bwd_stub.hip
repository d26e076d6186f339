#include "tri_launch.hpp"
namespace tri {
#define STUB(name) \
int name##_num_tiles() { return 1; } \
TileInfo name##_tile_info(int) { return TileInfo{32,32,4}; } \
bool name##_supports(int, int64_t, int, int) { return false; } \
hipError_t name##_launch(const BwdArgs&, int, int, int, int, hipStream_t) { return hipErrorNotSupported; }
STUB(bwd_q) STUB(bwd_kv) STUB(bwd_b)
}
