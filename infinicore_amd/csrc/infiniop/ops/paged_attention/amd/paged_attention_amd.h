#ifndef INFINICORE_AMD_PAGED_ATTENTION_AMD_H
#define INFINICORE_AMD_PAGED_ATTENTION_AMD_H

#include "../paged_attention.h"

DESCRIPTOR(amd)

#endif
