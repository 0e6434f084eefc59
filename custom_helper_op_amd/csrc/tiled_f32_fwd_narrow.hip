// Tiled cost-volume kernels instantiated for float storage: forward, 1 to 4 lanes per
// pixel, and the public entry points of this direction.
#define CHOP_S float
#define CHOP_TILED_FORWARD
#define CHOP_LPP_PART 0
#include "tiled_launch.inc"
