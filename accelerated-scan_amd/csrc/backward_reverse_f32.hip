// Backward kernels of reverse scans and their dispatch for one dtype (TraitsF32).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_reverse_f32, TraitsF32, false)
