// Matrix-core attention for head sizes 16, 32, 48 and 64 (see attention_mfma.inc).
#define RV_ATTN_ENTRY rv_attn_mfma_g0
#define RV_ATTN_SLOTS_ENTRY rv_attn_mfma_wave_slots_g0
#define RV_ATTN_CASES RV_ATTN_CASE(16) RV_ATTN_CASE(32) RV_ATTN_CASE(48) RV_ATTN_CASE(64)
#define RV_PREFILL_ENTRY rv_attn_prefill_g0
#define RV_PREFILL_SLOTS_ENTRY rv_attn_prefill_block_slots_g0
#define RV_PREFILL_CASES RV_PREFILL_CASE(16) RV_PREFILL_CASE(32) RV_PREFILL_CASE(48) RV_PREFILL_CASE(64)
#include "attention_mfma.inc"
