// Tiled cost-volume kernels instantiated for __half storage: backward.
#define CHOP_S __half
#define CHOP_TILED_BACKWARD
#include "tiled_launch.inc"
