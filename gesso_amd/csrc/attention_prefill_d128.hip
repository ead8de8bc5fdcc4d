// Prompt attention for heads 128 wide.
#include "attention_prefill_impl.h"

int gs_attention_prefill_d128(const PrefillCall& c) { return prefill_for_width<128>(c); }
