// Prompt attention for heads 64 wide.
#include "attention_prefill_impl.h"

int gs_attention_prefill_d64(const PrefillCall& c) { return prefill_for_width<64>(c); }
