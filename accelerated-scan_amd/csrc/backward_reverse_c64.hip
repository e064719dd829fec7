// Backward kernels of reverse scans and their dispatch for one dtype (TraitsC64).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_reverse_c64, TraitsC64, false)
