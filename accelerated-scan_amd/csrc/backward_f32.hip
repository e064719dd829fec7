// Backward kernels and their dispatch for one dtype (TraitsF32).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_f32, TraitsF32, true)
