// Backward kernels and their dispatch for one dtype (TraitsC64RealTokens).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_c64_real_tokens, TraitsC64RealTokens, true)
