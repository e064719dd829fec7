// Forward kernels and their dispatch for one dtype (TraitsBF16).
#include "forward_dispatch.h"

ASCAN_DEFINE_FORWARD(forward_bf16, TraitsBF16)
