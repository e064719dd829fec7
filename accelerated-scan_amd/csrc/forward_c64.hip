// Forward kernels and their dispatch for one dtype (TraitsC64).
#include "forward_dispatch.h"

ASCAN_DEFINE_FORWARD(forward_c64, TraitsC64)
