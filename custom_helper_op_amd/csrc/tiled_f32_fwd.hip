// Tiled cost-volume kernels instantiated for float storage: forward.
#define CHOP_S float
#define CHOP_TILED_FORWARD
#include "tiled_launch.inc"
