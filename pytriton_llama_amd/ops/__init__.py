from . import library
from .library import KernelLibraryError
from .kernels import (PROBE_MFMA_FLOPS_PER_ITER, ROWS_MIN, KernelError, RowScale, add_rmsnorm, argmax, attention_decode,
                      attention_decode_mfma_fits, attention_generic, attention_prefill_mfma,
                      attention_prefill_mfma_fits, attention_prefill_mfma_plan, blocked_weight, compute_units, embedding, gate_up_silu, gate_up_silu_fits,
                      gemm_library, gemm_library_fits, timed_library_products, library_product_choice, gemm_nt, gemm_rows, gemm_rows_add_rmsnorm, gemm_rows_add_rmsnorm_fits, gemm_rows_fits, gemm_rows_splits, sum_add_rmsnorm, gemm_skinny, gemm_skinny_add_norm, gemm_skinny_add_norm_fits,
                      gemm_skinny_fits, probe_mfma, probe_stream_read, qkv_rope_store, qkv_rope_store_fits,
                      rope_store, row_scale,
                      sample_top_p, silu_mul, stage_step, to_device, token_logprob,
                      ACT_CLAMPED, ACT_SILU, Routing, dyt, embedding_scaled, gated_act, gelu_gather_mul,
                      gemm_heads_nt, latent_prepare, moe_experts, moe_route, stream_add_dyt,
                      stream_add_rmsnorm,
                      NORM_NONE, NORM_HEAD, NORM_WHOLE, GATE_NONE, GATE_SIGMOID, GATE_SILU,
                      attention_generic_kv, attention_decode_kv, attention_decode_kv_fits, attention_prefill_mfma_kv,
                      attention_prefill_mfma_kv_fits, qkv_prepare, head_norm_gate, stream_add_rmsnorm_sum,
                      stream_rmsnorm, recurrent_block_floats, recurrent_state_floats, conv_prepare,
                      conv_tail_update, delta_scan, memory_scan, MEMORY_SEGMENT, MEMORY_SEGMENTS_FROM,
                      DELTA_SEGMENTS_FROM, delta_segment)
