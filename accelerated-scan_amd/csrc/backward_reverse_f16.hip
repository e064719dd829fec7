// Backward kernels of reverse scans and their dispatch for one dtype (TraitsF16).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_reverse_f16, TraitsF16, false)
