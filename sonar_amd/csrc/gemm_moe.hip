// Grouped (mixture-of-experts) W4A16 GEMM entry points.
#include "common.hpp"

using namespace sonar;

extern "C" size_t sonar_moe_marlin_gemm_scratch_bytes(int64_t sorted_len, int64_t moe_block_size,
                                                      int64_t size_n, int64_t size_k) {
  (void)sorted_len; (void)moe_block_size; (void)size_n; (void)size_k;
  return 0;
}

extern "C" int sonar_moe_wna16_marlin_gemm(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout, const void* b_bias,
    const void* b_scales, const uint32_t* b_zeros, const int32_t* g_idx, const int32_t* perm,
    int32_t* workspace, int64_t workspace_len, void* scratch, size_t scratch_bytes,
    const int32_t* sorted_token_ids, int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights, int64_t moe_block_size,
    int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, int is_k_full,
    int use_atomic_add, int use_fp32_reduce, void* stream) {
  return fail(SONAR_E_UNSUPPORTED, "moe_wna16_marlin_gemm is not built yet");
}
