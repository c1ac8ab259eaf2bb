// Matrix-core decode kernels for packed rows of 4 bits.
#define TQ_WIDTH_HERE 4
#include "tq_width_inst.h"
