// Backward kernels of reverse scans and their dispatch for one dtype (TraitsBF16).
#include "backward_dispatch.h"

ASCAN_DEFINE_BACKWARD(backward_reverse_bf16, TraitsBF16, false)
