#ifndef INFINICORE_AMD_ROPE_PAGED_CACHING_AMD_H
#define INFINICORE_AMD_ROPE_PAGED_CACHING_AMD_H

#include "../rope_paged_caching.h"

DESCRIPTOR(amd)

#endif
