// Tiled cost-volume kernels instantiated for float storage: backward.
#define CHOP_S float
#define CHOP_TILED_BACKWARD
#include "tiled_launch.inc"
