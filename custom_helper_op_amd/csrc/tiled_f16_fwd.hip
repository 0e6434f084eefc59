// Tiled cost-volume kernels instantiated for __half storage: forward.
#define CHOP_S __half
#define CHOP_TILED_FORWARD
#include "tiled_launch.inc"
