// Causal prefill attention on f16 MFMA for gfx950 (placeholder until the kernel lands: the plan table routes
// every prefill chunk to the split-K kernel in column groups, so this launcher is never reached).
#include "pa_internal.h"

hipError_t pa_launch_prefill(const AttnParams&, uint32_t, uint32_t, uint32_t, hipStream_t) { return hipErrorNotSupported; }
