// Entry points whose kernels are not built yet report PipelineCreation, the
// reference's answer for a missing optional pipeline (kernels.rs:125-218).
#include "common.hpp"
#define LH_PENDING(name, ...) int name(__VA_ARGS__) { return lh_fail(LH_ERR_PIPELINE_CREATION, #name " pipeline not available"); }
extern "C" {
LH_PENDING(lh_matmul_nt_q4_0_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_matmul_nt_tq2_0_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_multivec_nt_q4_0_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_multivec_nt_tq2_0_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_matmul_nt_quant_typed_into, lh_batch*, lh_quant, const lh_buffer*, lh_dtype, const lh_buffer*, lh_buffer*, lh_dtype, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_matmul_nt_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_dequant_q4_0_into, lh_batch*, const lh_buffer*, size_t, lh_buffer*, size_t)
LH_PENDING(lh_dequant_tq2_0_into, lh_batch*, const lh_buffer*, size_t, lh_buffer*, size_t)
LH_PENDING(lh_tq2_dequant, lh_context*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t)
LH_PENDING(lh_encode_kv_turboquant, lh_context*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_encode_kv_turboquant_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_encode_kv_turboquant_batched_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, lh_buffer*, const lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_dequantize_kv_turboquant, lh_context*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_dequantize_kv_turboquant_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_hadamard_rotate_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, int, int)
LH_PENDING(lh_hadamard_rotate_hf_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, int, int)
LH_PENDING(lh_hadamard_rotate_fh_into, lh_batch*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, int, int)
LH_PENDING(lh_flash_attention_tq_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_flash_attention_tq_prefill_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_flash_attention_tq_prefill_tiled_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_flash_attention_tq_batched_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, const lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_flash_decoding_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
LH_PENDING(lh_flash_attention_windowed_split_into, lh_batch*, const lh_buffer*, const lh_buffer*, const lh_buffer*, lh_buffer*, lh_buffer*, lh_buffer*, lh_buffer*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t)
uint32_t lh_flash_split_count(uint32_t eff) { uint32_t s = (eff + 15) / 16; return s < 1 ? 1 : (s > 16 ? 16 : s); }
int lh_turboquant_levels(uint32_t, uint32_t, float*) { return lh_fail(LH_ERR_PIPELINE_CREATION, "pending"); }
int lh_turboquant_signs(uint32_t, uint64_t, float*) { return lh_fail(LH_ERR_PIPELINE_CREATION, "pending"); }
uint32_t lh_turboquant_code_bytes(uint32_t dim, uint32_t bits) { return (dim * bits + 7) / 8; }
size_t lh_swa_ring_capacity(size_t, size_t) { return 0; }
uint32_t lh_kv_bits_from_env(void) { return 2; }
}
