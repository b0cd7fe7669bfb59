#ifndef INFINICORE_AMD_PAGED_CACHING_AMD_H
#define INFINICORE_AMD_PAGED_CACHING_AMD_H

#include "../paged_caching.h"

DESCRIPTOR(amd)

#endif
