// Tiled cost-volume kernels instantiated for __half storage.
#define CHOP_S __half
#include "tiled_launch.inc"
