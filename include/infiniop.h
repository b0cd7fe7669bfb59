/* Umbrella header of libinfiniop.so as built here: the context objects and the paged-KV operators. */
#ifndef INFINICORE_AMD_INFINIOP_H
#define INFINICORE_AMD_INFINIOP_H

#include "infiniop/handle.h"
#include "infiniop/operator_descriptor.h"
#include "infiniop/ops/kv_caching.h"
#include "infiniop/ops/paged_attention.h"
#include "infiniop/ops/paged_attention_prefill.h"
#include "infiniop/ops/paged_caching.h"
#include "infiniop/ops/rope_paged_caching.h"
#include "infiniop/tensor_descriptor.h"

#endif
