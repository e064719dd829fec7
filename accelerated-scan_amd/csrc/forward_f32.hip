// Forward kernels and their dispatch for one dtype (TraitsF32).
#include "forward_dispatch.h"

ASCAN_DEFINE_FORWARD(forward_f32, TraitsF32)
