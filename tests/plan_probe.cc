// Test-only view of the decode launch plan (infinicore_amd/csrc/infiniop/ops/paged_attention/amd/decode_plan.h):
// compiled with the host compiler by tests/test_decode_plan.py, no GPU and no HIP needed.
#include "infiniop/ops/paged_attention/amd/decode_plan.h"

// in:  {num_seqs, num_heads, num_kv_heads, head_size, value_size, block_size, max_blocks_per_seq, num_blocks, compute_units}
// out: {tiled, balanced, latent_wide, partition_tokens, max_partitions, fallback_partition_tokens,
//       fallback_max_partitions, waves_per_stream, workspace_bytes, launchable, acc_bytes, ml_bytes, latent_chunks, latent_roles}
extern "C" void planProbe(const long long *in, long long *out) {
    using namespace op::paged_attention;
    PagedAttentionInfo info{};
    info.dtype = INFINI_DTYPE_BF16;
    info.index_dtype = INFINI_DTYPE_I64;
    info.num_seqs = in[0];
    info.num_heads = in[1];
    info.num_kv_heads = in[2];
    info.head_size = in[3];
    info.value_size = in[4];
    info.page_block_size = in[5];
    info.max_num_blocks_per_seq = in[6];
    info.num_blocks = in[7];
    // packed tensors
    info.q_head_stride = in[3];
    info.q_stride = in[1] * in[3];
    info.o_head_stride = in[4];
    info.o_stride = in[1] * in[4];
    info.k_row_stride = in[3];
    info.k_head_stride = in[5] * in[3];
    info.k_batch_stride = in[2] * in[5] * in[3];
    info.v_row_stride = in[4];
    info.v_head_stride = in[5] * in[4];
    info.v_batch_stride = in[2] * in[5] * in[4];
    info.block_table_batch_stride = in[6];
    info.cache_lens_stride = 1;
    const device::amd::DeviceInfo dev{static_cast<int>(in[8]), 64, false};
    const amd::Plan plan = amd::makePlan(info, dev);
    out[0] = plan.tiled;
    out[1] = plan.balanced;
    out[2] = plan.latent_wide;
    out[3] = plan.partition_tokens;
    out[4] = plan.max_partitions;
    out[5] = plan.fallback_partition_tokens;
    out[6] = plan.fallback_max_partitions;
    out[7] = plan.waves_per_stream;
    out[8] = static_cast<long long>(plan.workspaceBytes());
    out[9] = amd::launchable(info);
    out[10] = static_cast<long long>(plan.acc_bytes);
    out[11] = static_cast<long long>(plan.ml_bytes);
    out[12] = plan.latent_chunks;
    out[13] = plan.latent_roles ? 1 : 0;
}
