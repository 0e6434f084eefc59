// Tiled cost-volume kernels instantiated for bf16_t storage: backward.
#define CHOP_S bf16_t
#define CHOP_TILED_BACKWARD
#include "tiled_launch.inc"
