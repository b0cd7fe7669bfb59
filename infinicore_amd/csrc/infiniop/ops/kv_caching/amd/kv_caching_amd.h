#ifndef INFINICORE_AMD_KV_CACHING_AMD_H
#define INFINICORE_AMD_KV_CACHING_AMD_H

#include "../kv_caching.h"

DESCRIPTOR(amd)

#endif
