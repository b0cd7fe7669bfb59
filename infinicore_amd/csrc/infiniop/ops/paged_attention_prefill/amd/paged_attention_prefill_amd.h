#ifndef INFINICORE_AMD_PAGED_ATTENTION_PREFILL_AMD_H
#define INFINICORE_AMD_PAGED_ATTENTION_PREFILL_AMD_H

#include "../paged_attention_prefill.h"

DESCRIPTOR(amd)

#endif
