// Matrix-core decode kernels for packed rows of 2 bits.
#define TQ_WIDTH_HERE 2
#include "tq_width_inst.h"
