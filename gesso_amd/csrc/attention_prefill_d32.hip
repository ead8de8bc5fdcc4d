// Prompt attention for heads 32 wide.
#include "attention_prefill_impl.h"

int gs_attention_prefill_d32(const PrefillCall& c) { return prefill_for_width<32>(c); }
