// Matrix-core attention for head sizes 208, 224, 240 and 256 (see attention_mfma.inc).
#define RV_ATTN_ENTRY rv_attn_mfma_g3
#define RV_ATTN_SLOTS_ENTRY rv_attn_mfma_wave_slots_g3
#define RV_ATTN_CASES RV_ATTN_CASE(208) RV_ATTN_CASE(224) RV_ATTN_CASE(240) RV_ATTN_CASE(256)
#define RV_PREFILL_ENTRY rv_attn_prefill_g3
#define RV_PREFILL_SLOTS_ENTRY rv_attn_prefill_block_slots_g3
#define RV_PREFILL_CASES RV_PREFILL_CASE(208) RV_PREFILL_CASE(224) RV_PREFILL_CASE(240) RV_PREFILL_CASE(256)
#include "attention_mfma.inc"
