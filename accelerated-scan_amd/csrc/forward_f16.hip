// Forward kernels and their dispatch for one dtype (TraitsF16).
#include "forward_dispatch.h"

ASCAN_DEFINE_FORWARD(forward_f16, TraitsF16)
