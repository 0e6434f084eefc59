// Tiled cost-volume kernels instantiated for bf16_t storage: forward.
#define CHOP_S bf16_t
#define CHOP_TILED_FORWARD
#include "tiled_launch.inc"
