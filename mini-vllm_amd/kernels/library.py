"""Loads the HIP kernel libraries and declares their C entry points.

There is no fall-back: when a library is missing it is compiled once (hipcc, a few seconds
per file); when that is impossible the import of an operation fails with the reason.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Dict

from ..csrc import build as _build

c_int = ctypes.c_int
c_long = ctypes.c_long
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p

DTYPE_F32 = 0
DTYPE_BF16 = 1

_SIGNATURES = {
    "mv_last_error": (ctypes.c_char_p, []),
    "mv_built_dtypes": (c_int, []),
    "mv_abi_version": (c_int, []),
    "mv_graph_census": (c_int, [c_void_p, c_void_p]),
    # logits, ld, M, V, temperature, top_k, top_p, rng, out, stream (no workspace: see csrc/mv_noalloc.h)
    "mv_sample_noalloc": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p]),
    "mv_embedding": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "mv_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                               c_int, c_int, c_int, c_void_p]),
    "mv_rmsnorm": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_int, c_void_p, c_long, c_int, c_int,
                           c_int, c_void_p]),
    "mv_rope_table": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mv_qk_norm_rope_store": (c_int, [c_void_p, c_long, c_int, c_int, c_int,            # qkv, stride, offsets
                                      c_void_p, c_void_p, c_void_p, c_int, c_int,      # pos, seq, bt, width, page
                                      c_void_p, c_void_p, c_int, c_int, c_int, c_int,  # k, v pages, n, H, Hkv, D
                                      c_void_p, c_void_p, c_int, c_float, c_int,       # qw, kw, wdtype, eps, unit
                                      c_void_p, c_int, c_int, c_int, c_int, c_void_p]),  # table, rot, inter, store, dtype
    "mv_store_v_pages": (c_int, [c_void_p, c_long, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                 c_int, c_int, c_int, c_int, c_void_p]),
    "mv_swiglu": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_ref": (c_int, [c_void_p, c_long, c_int, c_void_p, c_long, c_int, c_void_p, c_void_p, c_long, c_int,
                            c_int, c_int, c_int, c_void_p]),
    # q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size, positions, token_seq, n, H, Hkv, D,
    # Dv, scale, window, first, gate, gate_stride, dtype, stream
    "mv_attention_ref": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_long,
                                 c_int, c_void_p]),
    # qkv, stride, q_off, k_off, v_off, positions, token_seq, block_table, bt_width, page_size, k_pages, v_pages, n, H, Hkv, D,
    # Dv, q_weight, k_weight, weight_dtype, unit_norm, eps, table, rot_dim, interleaved, mix_rows, mix_stride, mix_weight,
    # mix_weight_dtype, dtype, stream
    "mv_qkv_rotate_norm_store": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int,
                                         c_float, c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_int, c_int, c_void_p]),
    # lanes, plane, first, S, n, W, y, ldy, w_mix, w_out, w_in, w_norm, norm_dtype, eps, h, ldh, total, dtype, stream
    "mv_hyper_step": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_int, c_float, c_void_p, c_long, c_void_p, c_int, c_void_p]),
    # tokens, table, rows, n, E, top, dense, ld_dense, ids, weights, stream
    "mv_moe_table_route": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                   c_void_p]),
    # resid, x, ldx, delta, weight, weight_dtype, eps, groups, out, ldo, rows, n_out, h, dtype, stream
    "mv_group_norm_rows": (c_int, [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_long,
                                   c_void_p, c_int, c_int, c_int, c_void_p]),
    # y, ldy, wa, wa_dtype, eps_a, resid, wb, wb_dtype, eps_b, groups, out, n, h, conv_taps, conv_w, conv_wt, conv_w_dtype,
    # conv_state, token_seq, state_slots, dtype, stream
    "mv_group_norm_add_norm": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_float, c_int,
                                       c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                       c_int, c_void_p]),
    # h, ldh, out, ldo, w, wt, weight_dtype, taps, conv_state, token_seq, cu_seqlens, state_slots, n, n_seqs, C, dtype, stream
    "mv_input_conv": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    # x, ldx, out, ldo, n, cols, a_pos, a_neg, dtype, stream
    "mv_xielu": (c_int, [c_void_p, c_long, c_void_p, c_long, c_int, c_int, c_float, c_float, c_int, c_void_p]),
    # h, ldh, out, ldo, mix, mix_dtype, state, token_seq, cu_seqlens, state_slots, n, width, dtype, stream
    "mv_token_shift": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_int, c_int, c_int, c_void_p]),
    # packed, ld, n, H, D, rank, w2t, w0, a_bias, weight_dtype, decay_rate, key_eps, coef, dtype, stream
    "mv_delta_prepare": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                 c_float, c_float, c_void_p, c_int, c_void_p]),
    # packed, ld, n, H, D, rank, w2t, w0, a_bias, norm_w, weight_dtype, decay_rate, key_eps, eps, state, token_seq,
    # state_slots, out, ldo, dtype, stream
    "mv_delta_step": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                              c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_int, c_void_p]),
    # packed, ld, coef, state, cu_seqlens, state_slots, n_seqs, n, H, D, out, dtype, stream
    "mv_delta_scan": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                              c_void_p, c_int, c_void_p]),
    # raw, packed, ld, weight, weight_dtype, n, H, D, eps, out, ldo, dtype, stream
    "mv_delta_finish": (c_int, [c_void_p, c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p,
                                c_long, c_int, c_void_p]),
    # q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size, positions, token_seq,
    # n, H, Hkv, D, Dv, scale, chunk, window, bias, gate, gate_stride, dtype, stream
    "mv_attention_sigmoid_ref": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                         c_void_p, c_void_p, c_long, c_int, c_void_p]),
    # y, ldy, wa, wa_dtype, eps_a, unit_a, resid, wb, wb_dtype, eps_b, unit_b, out, n, h, shift_mix, shift_mix_dtype,
    # shift_state, token_seq, state_slots, dtype, stream
    "mv_norm_add_norm": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p, c_int, c_float,
                                 c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                 c_void_p]),
    # x, ld, rows, cols, cap, stream
    "mv_soft_cap": (c_int, [c_void_p, c_long, c_int, c_int, c_float, c_void_p]),
    "mv_sample": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_int, c_void_p]),
    # ... as mv_sample up to chunks, then next_ids, positions, context_lens, stream
    "mv_sample_advance": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
}

# entry points that only the bfloat16 library has
_OPTIONAL_SIGNATURES = {
    # x, ldx, ldx_head, w, n, H, IN, OUT, y, ldy, ldy_head, tail, table, positions, gate, ldg, gate_per_head, token_seq, mode, stream
    "mv_head_linear_mfma": (c_int, [c_void_p, c_long, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_long, c_int, c_int,
                                    c_void_p, c_void_p, c_void_p, c_long, c_int, c_void_p, c_int, c_void_p]),
    # q, ldq, out, ldo, pages, pages_t, block_table, bt_width, page_size, positions, token_seq, n, H, R, DR, scale, stream
    "mv_attention_latent_mfma": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                         c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "mv_moe_grouped_ints": (c_long, [c_int, c_int, c_int]),
    # x, ldx, n, hidden, w_gate_up, w_down, n_real, identity, F, ids, weights, top, dense, ld_dense, ints, act, out, y, ldy,
    # limit, slope, stream
    "mv_moe_grouped": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int,
                               c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_float, c_float, c_void_p]),
    "mv_gemm_skinny": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_long, c_int,
                               c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_swiglu": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_fold_parts": (c_int, [c_int, c_int, c_int]),
    # A, lda, W, bias, resid, ldr, norm_weight, norm_weight_dtype, unit_offset, weighted, ldw, partial, P, M, N, K, stream
    "mv_gemm_skinny_fold": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_int, c_int,
                                    c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, partial, P, eps, M, N, K, swiglu, stream
    "mv_gemm_skinny_scaled": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_int, c_float,
                                      c_int, c_int, c_int, c_int, c_void_p]),
    # weighted, ldw, partial, P, eps, out, ldo, dtype, M, width, stream
    "mv_scale_rows": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_long, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                                    c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_lt_workspace": (c_long, []),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, workspace, workspace_bytes, stream
    "mv_gemm_lt": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p,
                           c_long, c_void_p]),
    "mv_gemm_mid_workspace": (c_long, [c_int, c_int, c_int]),
    "mv_gemm_mid_splits": (c_int, [c_int, c_int]),
    # A, lda, W, M, N, K, work, work_floats, stream
    "mv_gemm_mid_sums": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_void_p]),
    # work, bias, C, ldc, c_dtype, M, N, F, swiglu, stream
    "mv_gemm_mid_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    # resid, part, F, plane, bias, weight, weight_dtype, eps, unit_offset, out, rows, n_out, h, dtype, stream
    "mv_add_rmsnorm_split": (c_int, [c_void_p, c_void_p, c_int, c_long, c_void_p, c_void_p, c_int, c_float, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, swiglu, work, work_floats, stream
    "mv_gemm_mid": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int,
                            c_void_p, c_long, c_void_p]),
    "mv_device_compute_units": (c_int, []),
    "mv_gemm_tile_workspace": (c_long, [c_int, c_int, c_int, c_int, c_int]),
    "mv_gemm_tile_splits": (c_int, [c_int, c_int, c_int, c_int, c_int]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, work, work_floats, force, stream
    "mv_gemm_tile": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int,
                             c_void_p, c_long, c_int, c_void_p]),
    # A, lda, W, M, N, K, work, work_floats, force, stream
    "mv_gemm_tile_sums": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, partial, P, eps, stream
    "mv_gemm_tile_scaled": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int,
                                    c_int, c_void_p, c_int, c_float, c_void_p]),
    # q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size, positions, cu_seqlens, n_seqs, H, Hkv,
    # D, scale, window, partials, counters, nsplit, max_pages, waves, token_seq, first, gate, gate_stride, stream
    "mv_attention_decode": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                    c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int,
                                    c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_long, c_void_p]),
    # qkv, stride, q_off, k_off, v_off, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size,
    # positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, q_weight, k_weight, weight_dtype, eps, unit_offset,
    # table, rows, store_kv, partials, counters, nsplit, max_pages, waves, token_seq, stream
    "mv_attention_decode_fused": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p,
                                          c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                          c_float, c_int, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                                          c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    # ids, table, table_dtype, resid, n, h, vocab, scale, ids2, table2, out2, h2, rows2, stream
    "mv_embedding_gather": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_void_p]),
    # ..., positions, cu_seqlens, n_seqs, n_units, n_busy, nt, kw, H, Hkv, D, scale, window, first, gate, gate_stride, stream
    "mv_attention_prefill": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_float, c_int, c_int, c_void_p, c_long, c_void_p]),
    "mv_attention_prefill_unit_tokens": (c_int, [c_int, c_int]),
    # as mv_attention_prefill up to window, then chunk, bias, gate, gate_stride, stream
    "mv_attention_prefill_sigmoid": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                             c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                             c_float, c_int, c_int, c_void_p, c_void_p, c_long, c_void_p]),
    # packed, ld, n, n_seqs, H, G, DK, DV, taps, conv_w, a_log, dt_bias, weight_dtype, conv_state, unit_eps, token_seq,
    # cu_seqlens, state_slots, qk, vals, gates, dtype, stream
    "mv_gdelta_prepare": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p]),
    # packed, ld, n, n_seqs, H, DK, DV, i_bias, f_bias, weight_dtype, cap, max_state, token_seq, cu_seqlens, state_slots,
    # qk, vals, gates, dtype, stream
    "mv_mlstm_prepare": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    # qk, vals, gates, state, cu_seqlens, state_slots, n_seqs, n, H, G, DK, DV, read, out, stream
    "mv_state_scan": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                              c_int, c_int, c_void_p, c_void_p]),
    # mode, packed, ld, n, n_seqs, H, G, DK, DV, taps, conv_w, a_log, dt_bias, i_bias, f_bias, norm_w, weight_dtype, conv_state,
    # max_state, state, unit_eps, cap, denom_eps, eps, token_seq, cu_seqlens, state_slots, out, ldo, dtype, stream
    "mv_state_step": (c_int, [c_int, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float, c_float,
                              c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_int, c_void_p]),
    # raw, gates, packed, ld, g_off, weight, weight_dtype, shared_weight, silu_gate, normaliser, denom_eps, n, H, DV, eps,
    # token_seq, out, ldo, dtype, stream
    "mv_state_finish": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_long, c_void_p, c_int, c_int, c_int, c_int, c_float,
                                c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_long, c_int, c_void_p]),
    # packed, ld, n, QR, R, DR, wq, wkv, weight_dtype, eps, table, table_rows, positions, token_seq, block_table, bt_width,
    # page_size, cq, ldq, pages, pages_t, dtype, stream
    "mv_latent_prepare": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p,
                                  c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_int,
                                  c_void_p]),
    # x, ldx, ldx_head, w, weight_dtype, n, H, IN, OUT, y, ldy, ldy_head, tail, table, positions, gate, ldg, token_seq, mode,
    # dtype, stream
    "mv_head_linear": (c_int, [c_void_p, c_long, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_long, c_int,
                               c_int, c_void_p, c_void_p, c_void_p, c_long, c_int, c_void_p, c_int, c_int, c_void_p]),
    # q, ldq, out, ldo, pages, block_table, bt_width, page_size, positions, token_seq, n, H, R, DR, scale, dtype, stream
    "mv_attention_latent": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p,
                                    c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "mv_attention_latent_split_workspace": (c_long, [c_int, c_int, c_int, c_int]),
    # as mv_attention_latent up to scale, then max_context, work, work_floats, dtype, stream
    "mv_attention_latent_split": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                          c_void_p, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_long, c_int,
                                          c_void_p]),
    # logits, ld, n, E, correction, weight_dtype, groups, keep, top, sum_eps, flags, dense, ids, weights, stream
    "mv_moe_route": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p,
                             c_void_p, c_void_p, c_void_p]),
    # gate_up, ld, dense, ld_dense, n, E, F, act, limit, slope, dtype, stream
    # gate_up, ld, dense, ld_dense, n, E, F, FS, act, limit, slope, tokens, table, table_rows, top, dtype, stream
    "mv_moe_swiglu_scale": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_float,
                                    c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    # y, ldy, h, ldh, dense, ld_dense, first, count, n, width, set, dtype, stream
    "mv_moe_identity_add": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_void_p]),
    "mv_scale_f32": (c_int, [c_void_p, c_long, c_int, c_int, c_float, c_void_p]),
    # y, ldy, x, ldx, rows, cols, dtype, stream
    "mv_add_rows": (c_int, [c_void_p, c_long, c_void_p, c_long, c_int, c_int, c_int, c_void_p]),
    "mv_launch_empty": (c_int, [c_int, c_int, c_void_p, c_void_p]),
}


class KernelLibraryError(RuntimeError):
    pass


class KernelLibrary:
    """One loaded ``libmvk_<variant>.so``."""

    def __init__(self, variant: str, path: str):
        self.variant = variant
        self.path = path
        try:
            self.dll = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load the HIP kernel library {path}: {e}") from e
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(self.dll, name)
            except AttributeError as e:
                raise KernelLibraryError(f"{path} lacks the entry point {name}; rebuild it") from e
            fn.restype = res
            fn.argtypes = args
        self.optional = set()
        for name, (res, args) in _OPTIONAL_SIGNATURES.items():
            fn = getattr(self.dll, name, None)
            if fn is not None:
                fn.restype = res
                fn.argtypes = args
                self.optional.add(name)

    def has(self, name: str) -> bool:
        return name in self.optional or name in _SIGNATURES

    def call(self, name: str, *args) -> None:
        rc = getattr(self.dll, name)(*args)
        if rc != 0:
            msg = self.dll.mv_last_error()
            raise KernelLibraryError(msg.decode("utf-8", "replace") if msg else f"{name} failed")

    def offer(self, name: str, *args) -> bool:
        """Calls an entry point that may decline its arguments (return code 2, nothing done):
        False then, True when it ran; any other failure raises."""
        rc = getattr(self.dll, name)(*args)
        if rc == 0:
            return True
        if rc == 2:
            return False
        msg = self.dll.mv_last_error()
        raise KernelLibraryError(msg.decode("utf-8", "replace") if msg else f"{name} failed")


_LOCK = threading.Lock()
_LOADED: Dict[str, KernelLibrary] = {}


def variant_of(dtype_name: str) -> str:
    if dtype_name in ("float32", "f32"):
        return "f32"
    if dtype_name in ("bfloat16", "bf16"):
        return "bf16"
    raise ValueError(f"no kernel library for dtype {dtype_name!r}")


def load(variant: str) -> KernelLibrary:
    """The library of ``variant`` ("f32" or "bf16"), building it first if it is not there."""
    with _LOCK:
        lib = _LOADED.get(variant)
        if lib is not None:
            return lib
        path = _build.find_library(variant)
        if path is None:
            try:
                path = _build.build(variant)
            except Exception as e:
                stale = _build.find_library(variant, require_fresh=False)
                hint = f" (a library built from other sources is at {stale})" if stale else ""
                raise KernelLibraryError(
                    f"the HIP kernel library '{variant}' is not built and building it failed{hint}: {e}") from e
        lib = KernelLibrary(variant, path)
        _LOADED[variant] = lib
        return lib
