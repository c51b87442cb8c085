// Matrix-core attention for head sizes 80, 96, 112 and 128 (see attention_mfma.inc).
#define RV_ATTN_ENTRY rv_attn_mfma_g1
#define RV_ATTN_SLOTS_ENTRY rv_attn_mfma_wave_slots_g1
#define RV_ATTN_CASES RV_ATTN_CASE(80) RV_ATTN_CASE(96) RV_ATTN_CASE(112) RV_ATTN_CASE(128)
#define RV_PREFILL_ENTRY rv_attn_prefill_g1
#define RV_PREFILL_SLOTS_ENTRY rv_attn_prefill_block_slots_g1
#define RV_PREFILL_CASES RV_PREFILL_CASE(80) RV_PREFILL_CASE(96) RV_PREFILL_CASE(112) RV_PREFILL_CASE(128)
#include "attention_mfma.inc"
