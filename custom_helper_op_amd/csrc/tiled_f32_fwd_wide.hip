// Tiled cost-volume kernels instantiated for float storage: forward, 8 and 16 lanes per
// pixel.
#define CHOP_S float
#define CHOP_TILED_FORWARD
#define CHOP_LPP_PART 1
#include "tiled_launch.inc"
