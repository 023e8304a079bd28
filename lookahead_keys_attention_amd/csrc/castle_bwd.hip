// placeholder until the backward kernels land
#include "castle_tiles.h"
#include "castle_params.h"
namespace castle {
int launch_bwd(const BwdArgs&, int, hipStream_t) { return -2; }
}  // namespace castle
