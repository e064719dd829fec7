// Backward kernels and their dispatch for one dtype (TraitsC64).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_c64, TraitsC64, true)
