// Tiled cost-volume kernels instantiated for bf16_t storage.
#define CHOP_S bf16_t
#include "tiled_launch.inc"
