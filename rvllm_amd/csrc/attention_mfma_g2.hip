// Matrix-core attention for head sizes 144, 160, 176 and 192 (see attention_mfma.inc).
#define RV_ATTN_ENTRY rv_attn_mfma_g2
#define RV_ATTN_SLOTS_ENTRY rv_attn_mfma_wave_slots_g2
#define RV_ATTN_CASES RV_ATTN_CASE(144) RV_ATTN_CASE(160) RV_ATTN_CASE(176) RV_ATTN_CASE(192)
#define RV_PREFILL_ENTRY rv_attn_prefill_g2
#define RV_PREFILL_SLOTS_ENTRY rv_attn_prefill_block_slots_g2
#define RV_PREFILL_CASES RV_PREFILL_CASE(144) RV_PREFILL_CASE(160) RV_PREFILL_CASE(176) RV_PREFILL_CASE(192)
#include "attention_mfma.inc"
