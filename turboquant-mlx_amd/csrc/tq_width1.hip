// Matrix-core decode kernels for packed rows of 1 bit.
#define TQ_WIDTH_HERE 1
#include "tq_width_inst.h"
