// The single translation unit of the gfx950 code object: hipcc --genco builds this file into
// singe_attention_gfx950.hsaco, which the C-ABI library loads with hipModuleLoadData.
#include "paged_decode.hip"
#include "fmha_prefill.hip"
#include "fmha_prefill_f32.hip"
#include "paged_attention.hip"
#include "splitk_reduce.hip"
#include "attention_rows_f32.hip"
#include "general_attention.hip"
#include "latent_attention.hip"
#include "latent_attention_mfma.hip"
#include "cache_ops.hip"
