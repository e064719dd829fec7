// Backward kernels and their dispatch for one dtype (TraitsBF16).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_bf16, TraitsBF16, true)
