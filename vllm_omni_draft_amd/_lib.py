"""ctypes binding of libsd_amd.so (the C ABI declared in include/sd_amd.h).

There is no fallback: if the library is missing or a call fails, an exception
is raised.  Tensors cross the boundary as raw device pointers only.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_LIB_NAME = "libsd_amd.so"
# The sources that layer-list models need, built alone (`make seq`): loaded where the whole
# library has not been built (a first run in a fresh checkout); it exports a subset of the ABI.
_SEQ_LIB_NAME = "libsd_seq.so"
_lib: Optional[C.CDLL] = None
_partial = False

c_i32p = C.POINTER(C.c_int32)
vp = C.c_void_p
i64 = C.c_int64
i32 = C.c_int


class SdError(RuntimeError):
    pass


class LayerWeights(C.Structure):
    _fields_ = [(n, vp) for n in (
        "attn_norm_w", "attn_norm_b", "qkv_w", "qkv_b", "o_w", "o_b", "mlp_norm_w", "mlp_norm_b",
        "up_w", "up_b", "down_w", "down_b", "qkv_s", "o_s", "up_s", "down_s", "down_w_km")]


class ModelDesc(C.Structure):
    _fields_ = [
        ("arch", i32), ("n_layers", i32), ("hidden", i32), ("n_heads", i32), ("n_kv_heads", i32),
        ("head_dim", i32), ("ffn", i32), ("vocab", i32), ("max_pos", i32), ("pos_bias", i32),
        ("norm_eps", C.c_float), ("attn_scale", C.c_float),
        ("embed", vp), ("embed_tiled", i32), ("pos_table", vp), ("rope_cs", vp), ("final_norm_w", vp),
        ("final_norm_b", vp), ("lm_head", vp), ("layers", C.POINTER(LayerWeights)),
        ("tp_rank", i32), ("allreduce", vp), ("allreduce_ctx", vp),
        ("weight_fp8", i32), ("lm_head_s", vp), ("lm_vocab", i32),
        ("mrope_section_t", i32), ("mrope_section_h", i32),
    ]


# int (*sd_allreduce_fn)(void* buf, size_t n_bf16, void* ctx, sd_stream_t stream)
ALLREDUCE_FN = C.CFUNCTYPE(i32, vp, C.c_size_t, vp, vp)


class KvCacheDesc(C.Structure):
    _fields_ = [("k_cache", vp), ("v_cache", vp), ("layer_stride_bytes", i64),
                ("block_tables", vp), ("max_blocks_per_seq", i32)]


class ForwardArgs(C.Structure):
    _fields_ = [("B", i32), ("q_len", i32), ("token_ids", vp), ("tok_stride", i64),
                ("tok_offset", i64), ("seq_lens", vp), ("pos_offset", i32), ("max_ctx", i32),
                ("split_tokens", i32), ("logits", vp), ("wide", i32),
                ("input_embeds", vp), ("rope_pos", vp), ("rope_delta", vp), ("tree_mask", vp),
                ("chain_state", vp), ("draft_fused", i32), ("read_ahead_mb", i32),
                ("wide_a8", i32), ("argmax_val", vp), ("argmax_idx", vp)]


class UniformRegion(C.Structure):
    _fields_ = [("offset", i64), ("n", i32), ("stride_j", i64), ("stride_b", i64)]


class RowAdds(C.Structure):
    _fields_ = [("add", vp), ("ld_add", i64), ("x_out", vp)]


class RopePositions(C.Structure):
    _fields_ = [("pos", vp), ("delta", vp), ("section_t", i32), ("section_h", i32)]


class SeqLayer(C.Structure):
    """sd_seq_layer"""
    _fields_ = [("kind", i32), ("heads", i32), ("kv_heads", i32), ("dim", i32), ("vdim", i32), ("ff", i32),
                ("rot_dims", i32), ("rot_layout", i32), ("inv_freq", vp), ("qk_unit_norm", i32),
                ("q_scale", C.c_float), ("k_scale", C.c_float), ("score_scale", C.c_float),
                ("window", i32), ("pool", i32), ("rank", i32), ("tau", C.c_float),
                ("norm_w", vp), ("w_in", vp), ("w_in_tiled", vp), ("r1_bias", vp), ("r2_bias", vp), ("w_o", vp),
                ("w_o_tiled", vp), ("w_down", vp), ("w_down_tiled", vp), ("w_a2", vp),
                ("b_a2", vp), ("head_decay", vp), ("head_bias", vp), ("head_norm_w", vp), ("state", vp),
                ("k_cache", vp), ("v_cache", vp), ("pk_cache", vp), ("pv_cache", vp),
                ("block", i32), ("keep_first", i32), ("norm2_w", vp),
                ("q_rank", i32), ("kv_rank", i32), ("rot_dim", i32), ("rot_mag", C.c_float),
                ("dq_norm_w", vp), ("dkv_norm_w", vp), ("w_uq", vp), ("w_uq_tiled", vp), ("w_uk_t", vp), ("w_uv", vp),
                ("q_norm_w", vp), ("k_norm_w", vp), ("left_scale", C.c_float), ("right_scale", C.c_float),
                ("s_heads", i32), ("s_vdim", i32), ("s_state", i32), ("s_groups", i32), ("s_taps", i32),
                ("s_norm_groups", i32), ("conv_w", vp), ("conv_b", vp), ("dt_bias", vp), ("a_log", vp),
                ("skip_d", vp), ("s_norm_w", vp), ("w_o2", vp), ("w_o2_tiled", vp), ("conv_state", vp),
                ("n_experts", i32), ("top", i32), ("expert_ff", i32), ("w_router", vp), ("w_gate_up", vp),
                ("w_down_e", vp),
                ("post_norm_w", vp), ("post_norm2_w", vp), ("pre_add", vp), ("chunk", i32), ("softcap", C.c_float),
                ("sinks", vp), ("head_gate", i32), ("qk_head_norm", i32), ("w_ff_in", vp), ("w_ff_in_tiled", vp),
                ("ff_act", i32), ("expert_act", i32), ("route_score", i32), ("route_renorm", i32),
                ("expert_scale_input", i32), ("route_renorm_eps", C.c_float), ("route_scale", C.c_float),
                ("shared_ff", i32), ("shared_act", i32), ("w_shared_in", vp), ("w_shared_in_tiled", vp),
                ("w_shared_down", vp), ("w_shared_down_tiled", vp), ("w_shared_gate", vp),
                ("maps", i32), ("diff_lambda", C.c_float), ("diff_scale", C.c_float), ("qk_full_norm", i32),
                ("value_from_key", i32), ("kv_shared", i32), ("w_in_bias", vp), ("w_o_bias", vp),
                ("router_bias", vp), ("residual_mult", C.c_float)]


class SeqModelDesc(C.Structure):
    _fields_ = [("n_layers", i32), ("width", i32), ("vocab", i32), ("weights_f32", i32),
                ("norm_eps", C.c_float), ("embed", vp), ("head_tiled", vp), ("final_norm_w", vp),
                ("layers", C.POINTER(SeqLayer)),
                ("plain_norm", i32), ("embed_scale", C.c_float), ("bigram", vp), ("buckets", i32),
                ("mul_prev", i32), ("mul_cur", i32), ("head", vp), ("logit_scale", C.c_float)]


class SeqBatch(C.Structure):
    _fields_ = [("n_rows", i32), ("n_entries", i32), ("tokens", vp), ("row_pos", vp), ("row_slot", vp),
                ("entries", vp), ("block_tables", vp), ("max_blocks", i32), ("page", i32), ("n_out", i32),
                ("out_rows", vp), ("logits", vp), ("layer_out", vp), ("prev_tokens", vp)]


# name -> (restype, argtypes); every symbol include/sd_amd.h declares.
SIGNATURES = {
    "sd_version": (i32, []),
    "sd_last_error": (i32, [C.c_char_p, C.c_size_t]),
    "sd_device_info": (i32, [C.POINTER(i32), C.c_char_p, C.c_size_t]),
    "sd_rejection_sample": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "sd_typical_acceptance": (i32, [vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, i32, i32, i32, vp]),
    "sd_greedy_verify": (i32, [vp, vp, vp, vp, vp, i32, i32, vp]),
    "sd_argmax_rows": (i32, [vp, i64, vp, i32, i32, vp]),
    "sd_softmax_rows": (i32, [vp, i64, C.c_float, vp, i64, i32, i32, vp]),
    "sd_filter_probs_seq": (i32, [vp, i64, vp, vp, vp, i32, i32, i32, vp]),
    "sd_add_logit_bias": (i32, [vp, i64, vp, i64, vp, i32, i32, i32, vp]),
    "sd_token_logprobs": (i32, [vp, i64, vp, i32, i32, i32, vp, vp, vp, vp]),
    "sd_softmax_rows_seq": (i32, [vp, i64, vp, i32, vp, i64, i32, i32, vp, vp]),
    "sd_sample_rows": (i32, [vp, i64, vp, vp, i32, i32, vp]),
    "sd_rope_append": (i32, [vp, vp, i32, vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, i32, vp]),
    "sd_paged_attention_workspace_bytes": (C.c_size_t, [i32, i32, i32, i32, i32, i32]),
    "sd_paged_attention": (i32, [vp, i64, vp, vp, vp, i32, vp, i32, vp, i64, i32, i32, i32, i32,
                                 i32, C.c_float, i32, i32, vp, C.c_size_t, vp]),
    "sd_paged_attention_blocked": (i32, [vp, i64, vp, vp, vp, i32, vp, i32, vp, i64, i32, i32, i32,
                                         i32, i32, i32, C.c_float, i32, i32, vp, C.c_size_t, vp]),
    "sd_paged_attention_static": (i32, [vp, i64, vp, vp, vp, i32, vp, i32, vp, i64, i32, i32, i32,
                                        i32, i32, C.c_float, i32, i32, vp]),
    "sd_paged_attention_tree": (i32, [vp, i64, vp, vp, vp, i32, vp, i32, vp, vp, i64, i32, i32, i32,
                                      i32, i32, C.c_float, i32, i32, vp, C.c_size_t, vp]),
    "sd_map_tokens": (i32, [vp, i64, i32, vp, i32, i32, vp]),
    "sd_tree_prepare": (i32, [vp, i64, i32, vp, vp, vp, i32, vp, i32, i32, vp]),
    "sd_tree_accept_greedy": (i32, [vp, vp, vp, vp, i32, i32, vp, vp, vp, vp, i32, vp]),
    "sd_tree_accept_sample": (i32, [vp, i64, vp, vp, vp, i32, i32, vp, vp, vp, vp, vp, vp, i32, i32, vp]),
    "sd_kv_compact": (i32, [vp, vp, i64, i32, vp, i32, vp, i32, vp, vp, i32, i32, i32, i32, vp]),
    "sd_linear": (i32, [vp, vp, vp, i64, vp, vp, vp, i64, i32, i32, i32, i32, vp]),
    "sd_norm_linear": (i32, [vp, vp, vp, i64, vp, vp, C.c_float, i32, vp, vp, i64, i32, i32, i32, i32, vp]),
    "sd_norm_qkv_rope": (i32, [vp, vp, vp, i64, vp, vp, C.c_float, i32, vp, vp, i64, vp, i32, vp, vp, vp,
                               i32, vp, i32, i32, i32, i32, i32, i32, i32,
                               C.POINTER(RopePositions), vp]),
    "sd_norm_linear_adds": (i32, [vp, vp, vp, i64, vp, vp, C.c_float, i32, vp, vp, i64, i32, i32, i32, i32,
                                  C.POINTER(RowAdds), vp]),
    "sd_norm_qkv_rope_adds": (i32, [vp, vp, vp, i64, vp, vp, C.c_float, i32, vp, vp, i64, vp, i32, vp, vp, vp,
                                    i32, vp, i32, i32, i32, i32, i32, i32, i32,
                                    C.POINTER(RopePositions), C.POINTER(RowAdds), vp]),
    "sd_draft_layer_supported": (i32, [i32, i32, i32, i32, i32, i32, i32, i32]),
    "sd_draft_attn_oproj": (i32, [vp, i64, vp, vp, vp, i32, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32,
                                  i32, i32, C.c_float, i32, vp]),
    "sd_draft_mlp": (i32, [vp, i64, vp, i32, vp, vp, C.c_float, vp, vp, vp, i32, i32, i32, vp]),
    "sd_rmsnorm": (i32, [vp, i64, vp, vp, i64, i32, i32, C.c_float, vp]),
    "sd_layernorm": (i32, [vp, i64, vp, vp, vp, i64, i32, i32, C.c_float, vp]),
    "sd_embed": (i32, [vp, i64, i64, vp, i32, vp, i32, vp, i32, vp, i32, i32, i32, i32, vp]),
    "sd_tiled_weight_elems": (C.c_size_t, [i32, i32, i32]),
    "sd_tile_weights": (i32, [vp, vp, i32, i32, i32, i32, vp]),
    "sd_argmax_combine": (i32, [vp, vp, i32, i32, i32, i64, vp, vp, vp]),
    "sd_argmax_from_partials": (i32, [vp, vp, vp, i32, vp]),
    "sd_tp_allgather": (i32, [vp, vp, C.c_size_t, vp, vp]),
    "sd_tile_weights_fp8": (i32, [vp, vp, i32, i32, i32, i32, vp]),
    "sd_model_create": (vp, [C.POINTER(ModelDesc)]),
    "sd_model_destroy": (None, [vp]),
    "sd_model_workspace_bytes": (C.c_size_t, [vp, i32, i32, i32]),
    "sd_model_forward": (i32, [vp, C.POINTER(KvCacheDesc), C.POINTER(ForwardArgs), vp,
                               C.c_size_t, vp]),
    "sd_store_proposal": (i32, [vp, vp, i32, i32, i32, vp]),
    "sd_debug_force_proposals": (i32, [vp, i32, vp, vp, i64, C.c_char_p, i32, vp, i32, i32, vp]),
    "sd_gather_proposals": (i32, [vp, vp, i32, i32, vp]),
    "sd_set_proposals": (i32, [vp, vp, i32, i32, vp]),
    "sd_advance_state": (i32, [vp, vp, vp, vp, i64, i32, vp, vp, i32, i32, vp]),
    "sd_linear_wide_workspace_bytes": (C.c_size_t, [i32, i32, i32, i32]),
    "sd_linear_wide": (i32, [vp, vp, vp, i64, vp, vp, vp, i64, i32, i32, i32, i32, vp, C.c_size_t, vp]),
    "sd_qkv_rope_wide": (i32, [vp, vp, vp, i64, vp, vp, i64, vp, i32, vp, vp, vp, i32, vp, i32, i32,
                               i32, i32, i32, i32, i32, C.POINTER(RopePositions), vp, C.c_size_t, vp]),
    "sd_row_scales_fp8": (i32, [vp, i64, i32, i32, vp, vp]),
    "sd_topk_tokens": (i32, [vp, i64, i32, i32, i32, i32, i32, vp, i64, i32, i32, vp]),
    "sd_norm_linear_argmax": (i32, [vp, vp, vp, i64, vp, vp, C.c_float, i32, vp, vp, i32, i32, i32, vp]),
    "sd_linear_wide_a8": (i32, [vp, vp, vp, vp, i64, vp, vp, vp, i64, i32, i32, i32, i32, vp, C.c_size_t, vp]),
    "sd_qkv_rope_wide_a8": (i32, [vp, vp, vp, vp, i64, vp, vp, i64, vp, i32, vp, vp, vp, i32, vp, i32, i32,
                               i32, i32, i32, i32, i32, C.POINTER(RopePositions), vp, C.c_size_t, vp]),
    "sd_linear_attn_merge": (i32, [vp, vp, vp, C.c_size_t, vp, i32, i32, i32, i32, i32, i32, i32, i32,
                                   vp, vp, vp, i64, i32, i32, vp]),
    "sd_tp_unique_id": (i32, [vp]),
    "sd_tp_comm_create": (vp, [vp, i32, i32]),
    "sd_tp_comm_destroy": (None, [vp]),
    "sd_tp_allreduce": (i32, [vp, C.c_size_t, vp, vp]),
    "sd_sampling_scratch_bytes": (C.c_size_t, [i32]),
    "sd_softmax_rows_split": (i32, [vp, i64, C.c_float, vp, i64, i32, i32, vp, vp]),
    "sd_sample_rows_split": (i32, [vp, i64, vp, vp, i32, i32, vp, vp]),
    "sd_rejection_sample_split": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, vp]),
    "sd_ipc_buffer_bytes": (C.c_size_t, [C.c_size_t]),
    "sd_ipc_buffer_create": (i32, [C.c_size_t, C.POINTER(vp), vp]),
    "sd_ipc_buffer_open": (i32, [vp, C.POINTER(vp)]),
    "sd_ipc_buffer_close": (i32, [vp]),
    "sd_ipc_buffer_destroy": (i32, [vp]),
    "sd_ipc_comm_create": (vp, [i32, i32, C.POINTER(vp), C.c_size_t]),
    "sd_ipc_comm_destroy": (None, [vp]),
    "sd_ipc_comm_errors": (i32, [vp, C.POINTER(i32)]),
    "sd_ipc_comm_set_timeout_ms": (i32, [vp, i32]),
    "sd_ipc_allreduce": (i32, [vp, C.c_size_t, vp, vp]),
    "sd_ipc_allgather": (i32, [vp, vp, C.c_size_t, vp, vp]),
    "sd_fill_uniforms": (i32, [vp, i32, C.c_uint64, vp, vp]),
    "sd_fill_uniforms_seq": (i32, [vp, vp, i32, vp, vp, i32, vp]),
    "sd_argmax_partial": (i32, [vp, i64, vp, vp, i32, i32, vp]),
    "sd_propose_from_partials": (i32, [vp, vp, i32, i32, vp, i32, i32, i32, vp]),
    "sd_verify_from_partials": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, vp, vp, i32, i32,
                                      vp]),
    "sd_chain_state_bytes": (C.c_size_t, [i32]),
    "sd_chain_state_init": (i32, [vp, C.c_size_t, i32, vp]),
    "sd_chain_errors": (i32, [vp, C.POINTER(i32)]),
    "sd_chain_supported": (i32, [i32, i32, i32, i32]),
    "sd_chain_o_up": (i32, [vp, vp, vp, vp, vp, i64, vp, C.c_size_t, vp, i32, i32, i32, i32, i32, i32,
                            i32, i32, vp, i32, vp, C.c_float, vp, vp, vp, vp, i64, i32, vp]),
    "sd_chain_down_qkv": (i32, [vp, vp, vp, vp, vp, i64, i32, vp, i32, vp, C.c_float, vp, vp, vp, vp,
                                i64, vp, i32, vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, i32, vp]),
    "sd_graph_begin": (i32, [vp]),
    "sd_graph_end": (i32, [vp, C.POINTER(vp)]),
    "sd_graph_launch": (i32, [vp, vp]),
    "sd_matmul_rows": (i32, [vp, vp, i64, vp, i32, vp, vp, i64, i32, i32, i32, vp]),
    "sd_rmsnorm_rows": (i32, [vp, vp, vp, i32, C.c_float, C.c_float, vp, vp, i32, i32, vp]),
    "sd_head_prep": (i32, [vp, vp, vp, i64, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp, i32, C.c_float,
                           C.c_float, C.c_float, vp, vp, i32, vp, i32, i32, vp]),
    "sd_sigmoid_power": (i32, [vp, i64, C.c_float, vp, i32, i32, vp]),
    "sd_decay_scan": (i32, [vp, vp, vp, i64, vp, i32, vp, vp, i32, vp, i32, i32, i32, vp]),
    "sd_head_post": (i32, [vp, vp, i64, vp, i32, i32, C.c_float, i32, vp, vp, i32, i32, i32, i32, vp]),
    "sd_pooled_slots_per_page": (i32, [i32, i32]),
    "sd_window_pool_attention_scratch_bytes": (C.c_size_t, [i32, i32, i32, i32, i32, i32]),
    "sd_window_pool_attention": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32,
                                       i32, i32, i32, C.c_float, vp, vp, vp, C.c_size_t, vp]),
    "sd_gated_residual": (i32, [vp, vp, vp, i64, vp, vp, vp, vp, i32, i32, vp]),
    "sd_gated_residual_norm": (i32, [vp, vp, vp, i64, vp, vp, vp, vp, i32, i32, vp, i32, C.c_float, C.c_float,
                                     vp, vp, vp]),
    "sd_relu_mul_rows": (i32, [vp, vp, i64, vp, i32, i32, vp]),
    "sd_embed_hashed": (i32, [vp, vp, vp, vp, i32, C.c_float, i32, i32, i32, vp, vp, i32, i32, i32, vp]),
    "sd_rmsnorm_parts": (i32, [vp, i64, vp, i64, vp, i32, C.c_float, vp, i64, vp, i64, i32, i32, i32, i32, vp]),
    "sd_rope_rows": (i32, [vp, i64, vp, i32, i32, i32, i32, i32, i32, vp, C.c_float, vp]),
    "sd_rope_copy_rows": (i32, [vp, i64, i32, i32, vp, i64, i32, i32, vp, i32, i32, i32, i32, i32, vp, C.c_float, vp]),
    "sd_latent_prep": (i32, [vp, i32, vp, vp, i64, vp, i32, i32, vp, i64, i32, C.c_float, i32, i32, vp, C.c_float, vp,
                             vp, vp, vp, i32, i32, i32, vp]),
    "sd_qk_norm_append": (i32, [vp, i32, vp, vp, i32, i32, vp, vp, i32, i64, i32, C.c_float, vp, vp, vp, vp, vp, i32,
                                i32, i32, vp]),
    "sd_cache_append": (i32, [vp, i64, vp, i64, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]),
    "sd_window_softmax_attention_scratch_bytes": (C.c_size_t, [i32, i32, i32, i32, i32, i32]),
    "sd_window_softmax_attention": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32,
                                          i32, C.c_float, vp, vp, vp, C.c_size_t, vp]),
    "sd_matmul_rows_batched": (i32, [vp, i64, i64, vp, i32, i64, vp, i64, i64, vp, i32, i32, i32, i32, vp]),
    "sd_causal_conv_rows": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, vp, i32, vp, i64, i32, i32, i32, i32, vp]),
    "sd_ssd_steps": (i32, [vp, i64, vp, vp, i32, vp, vp, i32, i32, vp]),
    "sd_decay_scan_rows": (i32, [vp, vp, i64, vp, i64, vp, vp, vp, i32, vp, vp, i32, vp, i32, i32, i32, i32, vp]),
    "sd_moe_route": (i32, [vp, i64, vp, vp, i32, i32, i32, i32, i32, vp]),
    "sd_moe_route_rows": (i32, [vp, i64, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]),
    "sd_moe_experts_scratch_bytes": (C.c_size_t, [i32, i32, i32, i32, i32]),
    "sd_moe_experts": (i32, [vp, vp, i64, vp, vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, i32, i32, vp, C.c_size_t, vp]),
    "sd_postnorm_residual": (i32, [vp, vp, i32, C.c_float, vp, C.c_float, vp, i32, C.c_float, vp, i32, i32, vp]),
    "sd_scale_rows": (i32, [vp, i64, C.c_float, i32, i32, vp]),
    "sd_masked_softmax_attention_scratch_bytes": (C.c_size_t, [i32, i32, i32, i32, i32, i32, i32]),
    "sd_masked_softmax_attention": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32,
                                          i32, i32, C.c_float, C.c_float, vp, vp, vp, vp, C.c_size_t, vp]),
    "sd_qk_head_norm_append": (i32, [vp, i32, vp, vp, i32, i32, vp, vp, i32, i64, i32, C.c_float, vp, vp, vp, vp, vp,
                                     i32, i32, i32, vp]),
    "sd_head_gate_rows": (i32, [vp, i64, vp, i64, vp, i64, i32, i32, i32, i32, vp]),
    "sd_act_rows": (i32, [vp, vp, i64, vp, i64, vp, i64, i32, i32, i32, i32, vp]),
    "sd_moe_route_rows_gated": (i32, [vp, i64, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, C.c_float, C.c_float,
                                      vp, i32, vp, vp]),
    "sd_residual_norm": (i32, [vp, vp, i32, vp, vp, i64, vp, vp, vp, i32, C.c_float, vp, vp, vp, i32, i32, vp]),
    "sd_multimap_softmax_attention_scratch_bytes": (C.c_size_t, [i32, i32, i32, i32, i32, i32, i32, i32]),
    "sd_multimap_softmax_attention": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32,
                                            i32, i32, i32, C.c_float, C.c_float, vp, vp, vp, vp, C.c_size_t, vp]),
    "sd_attn_prep": (i32, [vp, i32, vp, i32, i32, vp, i32, i32, i32, i64, vp, vp, i32, vp, vp, i32, C.c_float, i32,
                           i32, vp, C.c_float, vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "sd_diff_combine_rows": (i32, [vp, C.c_float, C.c_float, C.c_float, vp, vp, i32, i32, i32, i32, vp]),
    "sd_moe_route_rows_biased": (i32, [vp, i64, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, C.c_float,
                                       C.c_float, vp, i32, vp, vp]),
    "sd_residual_norm_scaled": (i32, [vp, vp, i32, vp, vp, vp, i64, vp, C.c_float, vp, vp, i32, C.c_float, vp, vp,
                                      vp, i32, i32, vp]),
    "sd_seq_model_create": (vp, [C.POINTER(SeqModelDesc)]),
    "sd_seq_model_destroy": (None, [vp]),
    "sd_seq_model_workspace_bytes": (C.c_size_t, [vp, i32, i32, i32]),
    "sd_seq_model_forward": (i32, [vp, C.POINTER(SeqBatch), vp, C.c_size_t, vp]),
    "sd_graph_destroy": (None, [vp]),
}


def backend() -> str:
    """"gpu" (libsd_amd.so, gfx950; the default) or "cpu" (libsd_cpu.so, the C++/OpenMP build of
    the same ABI for hosts without a GPU), chosen for the whole process by SD_AMD_BACKEND before
    the first call.  The choice is explicit: a missing GPU library is an error, never a reason
    to load the other one."""
    b = os.environ.get("SD_AMD_BACKEND", "gpu").lower()
    if b not in ("gpu", "cpu"):
        raise SdError(f"SD_AMD_BACKEND must be 'gpu' or 'cpu', not {b!r}")
    return b


def lib_path() -> str:
    """The in-tree library of the chosen backend; SD_AMD_LIB names another build of the GPU
    sources (the timestamp-instrumented one of `make stamps`, for experiments/)."""
    here = os.path.dirname(os.path.abspath(__file__))
    if backend() == "cpu":
        return os.path.join(here, "libsd_cpu.so")
    override = os.environ.get("SD_AMD_LIB")
    if override:
        return os.path.abspath(override)
    full, seq = os.path.join(here, _LIB_NAME), os.path.join(here, _SEQ_LIB_NAME)
    return seq if (not os.path.exists(full) and os.path.exists(seq)) else full


def load() -> C.CDLL:
    """Loads the in-tree library and declares every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise SdError(f"{path} is missing: build it with `make` (hipcc --offload-arch=gfx950; "
                      "g++ for the CPU build); nothing falls back to another library or to PyTorch")
    global _partial
    lib = C.CDLL(path)
    _partial = os.path.basename(path) == _SEQ_LIB_NAME
    for name, (res, args) in SIGNATURES.items():
        if _partial and not hasattr(lib, name):
            continue             # the subset build: calling such an entry point raises AttributeError
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def ensure_built(seq_only: bool = False) -> str:
    """Builds the GPU library in-tree if no build of it is there (hipcc, gfx950) and returns the
    path that load() will open.  seq_only: only what layer-list models need, unless the whole
    library exists already."""
    here = os.path.dirname(os.path.abspath(__file__))
    if backend() == "gpu" and not os.environ.get("SD_AMD_LIB"):
        full, seq = os.path.join(here, _LIB_NAME), os.path.join(here, _SEQ_LIB_NAME)
        if not os.path.exists(full) and not (seq_only and os.path.exists(seq)):
            import subprocess
            jobs = str(min(16, os.cpu_count() or 4))
            subprocess.run(["make", "-C", os.path.dirname(here), "-j" + jobs,
                            os.path.relpath(seq if seq_only else full, os.path.dirname(here))],
                           check=True, stdout=subprocess.DEVNULL)
    return lib_path()


def last_error() -> str:
    buf = C.create_string_buffer(512)
    load().sd_last_error(buf, 512)
    return buf.value.decode(errors="replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise SdError(f"{what} failed ({rc}): {last_error()}")
