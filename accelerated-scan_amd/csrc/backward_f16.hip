// Backward kernels and their dispatch for one dtype (TraitsF16).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_f16, TraitsF16, true)
