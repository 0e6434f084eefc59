// Tiled cost-volume kernels instantiated for float storage.
#define CHOP_S float
#include "tiled_launch.inc"
