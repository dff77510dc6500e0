// placeholder until the LDS-tiled prefill kernels land
#include "tppx_common.h"
