// Forward kernels and their dispatch for one dtype (TraitsC64RealTokens).
#include "forward_dispatch.h"

ASCAN_DEFINE_FORWARD(forward_c64_real_tokens, TraitsC64RealTokens)
