"""`torch.ops.nvx.*`: the C-ABI kernels as PyTorch custom ops (device key only, no CPU kernels).

Importing this module registers the ops.  Every op is a thin call into `nano_vllm_x_amd.ops` (argument checks,
output allocation, one launch through the C ABI on the current stream).  The paged-attention wrappers of
`layers/attention.py` -- the objects that stand where the reference's third-party attention wrappers stood
(nanovllmx/layers/attention.py:360-369) -- launch their kernels through these operators, so the attention path of
the engine is "custom ops over a C ABI" end to end; workspaces are ordinary tensors passed in and mutated.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops

_LIB = torch.library.Library("nvx", "DEF")
_DEFS = {
    "store_kvcache": "(Tensor k, Tensor v, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor kv_indices) -> ()",
    "rmsnorm": "(Tensor x, Tensor weight, float eps) -> Tensor",
    "rmsnorm_residual": "(Tensor x, Tensor residual, Tensor weight, float eps) -> (Tensor, Tensor)",
    "rope": "(Tensor positions, Tensor q, Tensor k, Tensor cos_sin) -> (Tensor, Tensor)",
    "silu_mul": "(Tensor x) -> Tensor",
    "sample": "(Tensor logits, Tensor temperatures, Tensor top_ks, Tensor top_ps, Tensor min_ps, int seed, int offset) -> Tensor",
    "sampler_probs": "(Tensor logits, Tensor temperatures, Tensor top_ks, Tensor top_ps, Tensor min_ps) -> Tensor",
    "sample_shard": "(Tensor logits, Tensor temperatures, int vocab_offset, int vocab, int seed, int offset) -> Tensor",
    "sample_pick": "(Tensor winners) -> Tensor",
    "lmhead_pack": "(Tensor weight) -> Tensor",
    "linear_stream": "(Tensor x, Tensor packed, int n) -> Tensor",
    "linear_block": "(Tensor x, Tensor packed, int n, int mode, int k_slices) -> Tensor",
    "splitk_sum": "(Tensor partials, bool half, bool silu_mul) -> Tensor",
    "lmhead_sample": "(Tensor packed, int n_rows, Tensor x, Tensor temperatures, int vocab_offset, int vocab, int seed, int offset, "
                     "bool keys) -> Tensor",
    "qknorm_rope_store": "(Tensor qkv, Tensor positions, Tensor cos_sin, Tensor q_weight, Tensor k_weight, float eps, Tensor slots, "
                         "Tensor(a!) k_cache, Tensor(b!) v_cache, int n_q_heads, int n_kv_heads) -> Tensor",
    # paged attention, decode: plan once per step, then one call per layer
    "decode_plan": "(Tensor kv_len, Tensor kv_start, Tensor? out_slots, int n_kv_heads, Tensor(a!) plan_ws) -> ()",
    "paged_decode": "(Tensor q, Tensor k_cache, Tensor v_cache, Tensor kv_indices, Tensor plan_ws, Tensor(a!) partial_ws, "
                    "int n_q_heads, int n_kv_heads, float sm_scale) -> Tensor",
    "paged_decode_qkv": "(Tensor qkv, Tensor positions, Tensor cos_sin, Tensor q_weight, Tensor k_weight, float eps, "
                        "Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor kv_indices, Tensor plan_ws, Tensor(c!) partial_ws, "
                        "int n_q_heads, int n_kv_heads, float sm_scale) -> Tensor",
    "paged_decode_noalloc": "(Tensor q, Tensor k_cache, Tensor v_cache, Tensor kv_indices, Tensor kv_len, Tensor kv_start, "
                            "int n_q_heads, int n_kv_heads, float sm_scale) -> Tensor",
    # paged attention, prefill
    "prefill_plan": "(Tensor qo_indptr, Tensor(a!) plan_ws) -> ()",
    "paged_prefill": "(Tensor q, Tensor k_cache, Tensor v_cache, Tensor qo_indptr, Tensor kv_indptr, Tensor kv_indices, "
                     "Tensor plan_ws, int n_q_heads, int n_kv_heads, float sm_scale) -> Tensor",
    # projections of a decode step and the norm that sums their K-split partials
    "linear_decode": "(Tensor x, Tensor w, int mode, int k_splits) -> Tensor",
    "rmsnorm_splitk": "(Tensor partials, Tensor weight, float eps) -> Tensor",
    "rmsnorm_splitk_residual": "(Tensor partials, Tensor residual, Tensor weight, float eps) -> (Tensor, Tensor)",
    # direct-peer all-reduce of a tensor-parallel group (`group`: the integer ops.PeerGroup.comm), alone or with the norm
    "peer_allreduce": "(int group, Tensor(a!) x) -> ()",
    "peer_allreduce_norm": "(int group, Tensor x, Tensor? residual, Tensor weight, float eps) -> (Tensor, Tensor)",
    # device-resident block table
    "block_table_write_rows": "(Tensor kv_indices, Tensor kv_indptr, Tensor rows, Tensor(a!) table) -> ()",
    "decode_step_setup": "(Tensor step, int stride, int padded_batch, Tensor(a!) table, int pad_start, Tensor(b!) kv_start, "
                         "Tensor(c!) kv_len, Tensor(d!) out_slots, Tensor(e!) positions, Tensor(f!) input_ids, Tensor? prev_ids) -> ()",
    # layers with a float32 residual stream, per-sequence state and latent attention; the step's layout travels as its four
    # tensors (qo_indptr and tok_seq absent: one token per sequence)
    "boundary_norm": "(Tensor m, Tensor w_post, float eps, Tensor? res, Tensor(a!)? hist, int hist_slot, Tensor? mix, Tensor? w_pre, "
                     "bool pre_f32, Tensor? taps, Tensor(b!)? state, Tensor? pos0, Tensor? state_slot) -> (Tensor, Tensor?)",
    "canon_conv": "(Tensor h, Tensor taps, Tensor(a!) state, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq, "
                  "ScalarType dtype) -> Tensor",
    "relu2": "(Tensor x) -> Tensor",
    "mingru_scan": "(Tensor zxg, Tensor(a!) state, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq) -> Tensor",
    "latent_prep": "(Tensor x, Tensor w_q, Tensor w_kv, float eps, Tensor slots, Tensor(a!) cache, int heads) -> (Tensor, Tensor)",
    "latent_attn": "(Tensor q, Tensor cache, Tensor kv_indices, Tensor kv_start, Tensor kv_len, Tensor pos0, Tensor state_slot, "
                   "Tensor? qo_indptr, Tensor? tok_seq, float scale, Tensor? gate) -> Tensor",
    # gated residuals with grouped norms, matrix-memory recurrences, capped attention, mixtures of experts
    "gated_residual_norm": "(Tensor(a!) x, Tensor? y, Tensor? gate, Tensor? gate_bias, float mult, Tensor? w_norm, int groups, float eps, "
                           "Tensor? y2, Tensor? w_y, Tensor? w_y2, ScalarType dtype) -> Tensor?",
    "head_norm_gate": "(Tensor o, Tensor w, float eps, Tensor? gate, str kind, ScalarType dtype) -> Tensor",
    "short_conv_silu": "(Tensor x, Tensor w, Tensor(a!)? state, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq) -> Tensor",
    "token_shift_mix": "(Tensor h, Tensor mu, Tensor(a!) state, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq) -> Tensor",
    "mlstm_scan": "(Tensor x, int q_off, int k_off, int v_off, Tensor gates, Tensor gate_bias, float cap, Tensor(a!) mem, Tensor(b!) norm, "
                  "Tensor(c!) peak, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq, int heads, int dim, int vdim) -> Tensor",
    "delta_scan": "(Tensor x, int q_off, int k_off, int v_off, Tensor ab, Tensor a_log, Tensor dt_bias, Tensor(a!) mem, Tensor pos0, "
                  "Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq, int heads, int kv_heads, int dim, int vdim) -> Tensor",
    "rwkv_scan": "(Tensor r, Tensor k, Tensor v, Tensor wlog, Tensor w0, Tensor bonus, Tensor(a!) mem, Tensor pos0, Tensor state_slot, "
                 "Tensor? qo_indptr, Tensor? tok_seq, int heads, int dim) -> Tensor",
    "rope_vnorm_store": "(Tensor qkv, Tensor positions, Tensor? freq, float mag, int rot_dims, float eps, Tensor slots, Tensor(a!) k_cache, "
                        "Tensor(b!) v_cache, int heads, int kv_heads, int dim, int vdim) -> Tensor",
    "softcap_attn": "(Tensor q, Tensor k_cache, Tensor v_cache, Tensor kv_indices, Tensor kv_start, Tensor kv_len, Tensor pos0, "
                    "Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq, float scale, float cap, int heads, int kv_heads, int dim, int vdim, "
                    "int window=0, Tensor? r1=None, Tensor? r2=None, Tensor? v_turn=None, bool v_interleaved=False, Tensor? gate=None, "
                    "float? sink_score=None) -> Tensor",
    # post-normed stream, query/key norms with rotated values, decayed linear attention, experts with weights on their outputs
    "attn_prep_store": "(Tensor x, int q_off, int k_off, int v_off, Tensor positions, Tensor? q_w, Tensor? k_w, str norm_mode, float eps, "
                       "Tensor? freq, int rot_dims, bool interleaved, Tensor? vfreq, Tensor? slots, Tensor(a!)? k_cache, Tensor(b!)? v_cache, "
                       "int heads, int kv_heads, int dim, int vdim) -> (Tensor, Tensor?)",
    "decay_scan": "(Tensor x, int q_off, int k_off, int v_off, Tensor decay, Tensor(a!) mem, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, "
                  "Tensor? tok_seq, int heads, int dim, int vdim, str act) -> Tensor",
    "postnorm_residual": "(Tensor(a!) x, Tensor? y, Tensor? w_post, float eps, Tensor? y2, float a, float b, Tensor? w_next, ScalarType dtype) -> Tensor",
    "embed_scale": "(Tensor ids, Tensor table, float scale) -> (Tensor, Tensor)",
    "tanh_cap": "(Tensor z, float cap) -> Tensor",
    "moe_route": "(Tensor logits, int top) -> (Tensor, Tensor)",
    "moe_expert_rows": "(Tensor h, Tensor idx, Tensor wts, Tensor w_gu, Tensor w_d, float limit, float alpha, float shift=1.0, "
                       "bool weight_out=False) -> Tensor",
    "moe_order": "(Tensor idx, int n_exp) -> (Tensor, Tensor)",
    "moe_scatter_rows": "(Tensor h, Tensor? wts, Tensor dst) -> Tensor",
    "moe_glu": "(Tensor gu, float limit, float alpha, float shift=1.0) -> Tensor",
    "moe_gather_rows": "(Tensor ys, Tensor dst, Tensor? wts=None) -> Tensor",
    "skinny_proj": "(Tensor x, Tensor w, str in_act) -> Tensor",
    # several residual streams, the real-gated recurrence, a latent with a rotated key part, the softmax router with groups
    "hyper_mix": "(Tensor(a!) x, Tensor? y, Tensor? scale, Tensor? mix, Tensor? w_out, Tensor? w_in, Tensor? w_norm, float eps, ScalarType out_dtype) "
                 "-> Tensor",
    "hyper_start": "(Tensor x, int n_streams, Tensor? w_in, Tensor? w_norm, float eps, ScalarType out_dtype) -> (Tensor, Tensor)",
    "short_conv": "(Tensor x, Tensor w, Tensor(a!)? state, Tensor pos0, Tensor state_slot, Tensor? qo_indptr, Tensor? tok_seq, Tensor? bias, "
                  "str act) -> Tensor",
    "rglru_scan": "(Tensor y, Tensor u, Tensor gates, Tensor gate_bias, Tensor rate, Tensor(a!) state, Tensor pos0, Tensor state_slot, "
                  "Tensor? qo_indptr, Tensor? tok_seq) -> Tensor",
    "latent_rope_prep": "(Tensor x, int q_off, int kv_off, int g_off, Tensor positions, Tensor? freq, float mag, Tensor w_kv, float eps, "
                        "Tensor slots, Tensor(a!) cache, int heads, int dim, int rot) -> (Tensor, Tensor)",
    "moe_route_softmax": "(Tensor logits, int top, int n_groups, int keep_groups, float norm_eps) -> (Tensor, Tensor)",
}
for _name, _sig in _DEFS.items():
    _LIB.define(_name + _sig)


def _ws(plan_ws, partial_ws, n_q_heads, n_kv_heads):
    return ops.DecodeWorkspace.from_tensors(plan_ws, partial_ws, n_q_heads, n_kv_heads)


def _store_kvcache(k, v, k_cache, v_cache, kv_indices):
    ops.store_kvcache(k, v, k_cache, v_cache, kv_indices)


def _rmsnorm(x, weight, eps):
    return ops.rmsnorm(x, weight, eps)


def _rmsnorm_residual(x, residual, weight, eps):
    return ops.rmsnorm(x, weight, eps, residual=residual)


def _rope(positions, q, k, cos_sin):
    return ops.rope(positions, q, k, cos_sin)


def _silu_mul(x):
    return ops.silu_mul(x)


def _sample(logits, temperatures, top_ks, top_ps, min_ps, seed, offset):
    return ops.sample(logits, temperatures, top_ks, top_ps, min_ps, seed, offset)


def _sampler_probs(logits, temperatures, top_ks, top_ps, min_ps):
    return ops.sampler_probs(logits, temperatures, top_ks, top_ps, min_ps)


def _sample_shard(logits, temperatures, vocab_offset, vocab, seed, offset):
    return ops.sample_shard(logits, temperatures, vocab_offset, vocab, seed, offset)


def _sample_pick(winners):
    return ops.sample_pick(winners)


def _linear_stream(x, packed, n):
    return ops.linear_stream(x, packed, n)


def _linear_block(x, packed, n, mode, k_slices):
    return ops.linear_block(x, packed, n, mode=mode, k_slices=k_slices)


def _splitk_sum(partials, half, silu_mul):
    return ops.splitk_sum(partials, torch.float16 if half else torch.bfloat16, silu_mul)


def _lmhead_pack(weight):
    return ops.lmhead_pack(weight)


def _lmhead_sample(packed, n_rows, x, temperatures, vocab_offset, vocab, seed, offset, keys):
    return ops.lmhead_sample(packed, n_rows, x, temperatures, vocab_offset, vocab, seed, offset, keys=keys)


def _qknorm_rope_store(qkv, positions, cos_sin, q_weight, k_weight, eps, slots, k_cache, v_cache, n_q_heads, n_kv_heads):
    return ops.qknorm_rope_store(qkv, positions, cos_sin, q_weight, k_weight, eps, slots, k_cache, v_cache, n_q_heads, n_kv_heads)


def _decode_plan(kv_len, kv_start, out_slots: Optional[torch.Tensor], n_kv_heads, plan_ws):
    ops.decode_plan(kv_len, kv_start, ops.DecodeWorkspace.from_tensors(plan_ws, None, 0, n_kv_heads), out_slots=out_slots)


def _paged_decode(q, k_cache, v_cache, kv_indices, plan_ws, partial_ws, n_q_heads, n_kv_heads, sm_scale):
    return ops.paged_decode(q, k_cache, v_cache, kv_indices, q.shape[0], _ws(plan_ws, partial_ws, n_q_heads, n_kv_heads), sm_scale)


def _paged_decode_qkv(qkv, positions, cos_sin, q_weight, k_weight, eps, k_cache, v_cache, kv_indices, plan_ws, partial_ws,
                      n_q_heads, n_kv_heads, sm_scale):
    return ops.paged_decode_qkv(qkv, positions, cos_sin, q_weight, k_weight, eps, k_cache, v_cache, kv_indices, qkv.shape[0],
                                _ws(plan_ws, partial_ws, n_q_heads, n_kv_heads), sm_scale)


def _paged_decode_noalloc(q, k_cache, v_cache, kv_indices, kv_len, kv_start, n_q_heads, n_kv_heads, sm_scale):
    return ops.paged_decode_noalloc(q, k_cache, v_cache, kv_indices, kv_len, kv_start, n_q_heads, n_kv_heads, sm_scale)


def _prefill_plan(qo_indptr, plan_ws):
    ops.prefill_plan(qo_indptr, plan_ws)


def _paged_prefill(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, plan_ws, n_q_heads, n_kv_heads, sm_scale):
    return ops.paged_prefill(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, plan_ws, n_q_heads, n_kv_heads, sm_scale)


def _linear_decode(x, w, mode, k_splits):
    return ops.linear_decode(x, w, mode=mode, k_splits=k_splits)


def _rmsnorm_splitk(partials, weight, eps):
    return ops.rmsnorm_splitk(partials, weight, eps)


def _rmsnorm_splitk_residual(partials, residual, weight, eps):
    return ops.rmsnorm_splitk(partials, weight, eps, residual=residual)


def _peer_allreduce(group, x):
    ops.peer_allreduce_norm(ops.PeerGroup._registry[group], x)


def _peer_allreduce_norm(group, x, residual: Optional[torch.Tensor], weight, eps):
    g = ops.PeerGroup._registry[group]
    if residual is None:
        return ops.peer_allreduce_norm(g, x, weight, eps), x.new_empty(0)
    return ops.peer_allreduce_norm(g, x, weight, eps, residual=residual)


def _block_table_write_rows(kv_indices, kv_indptr, rows, table):
    ops.block_table_write_rows(kv_indices, kv_indptr, rows, table)


def _decode_step_setup(step, stride, padded_batch, table, pad_start, kv_start, kv_len, out_slots, positions, input_ids,
                       prev_ids: Optional[torch.Tensor]):
    ops.decode_step_setup(step, stride, padded_batch, table, pad_start, kv_start, kv_len, out_slots, positions, input_ids,
                          prev_ids=prev_ids)


def _layout(n_tok, pos0, state_slot, qo_indptr, tok_seq):
    n_seq = n_tok if qo_indptr is None else qo_indptr.numel() - 1
    return ops.StepLayout(n_tok, n_seq, pos0, state_slot, qo_indptr, tok_seq)


def _boundary_norm(m, w_post, eps, res, hist, hist_slot, mix, w_pre, pre_f32, taps, state, pos0, state_slot):
    canon = None if taps is None else (taps, state, _layout(m.shape[0], pos0, state_slot, None, None))
    return ops.boundary_norm(m, w_post, eps, res=res, hist=hist, hist_slot=hist_slot, mix=mix, w_pre=w_pre, pre_f32=pre_f32, canon=canon)


def _canon_conv(h, taps, state, pos0, state_slot, qo_indptr, tok_seq, dtype):
    return ops.canon_conv(h, taps, state, _layout(h.shape[0], pos0, state_slot, qo_indptr, tok_seq), dtype)


def _relu2(x):
    return ops.relu2(x)


def _mingru_scan(zxg, state, pos0, state_slot, qo_indptr, tok_seq):
    return ops.mingru_scan(zxg, state, _layout(zxg.shape[0], pos0, state_slot, qo_indptr, tok_seq))


def _latent_prep(x, w_q, w_kv, eps, slots, cache, heads):
    return ops.latent_prep(x, w_q, w_kv, eps, slots, cache, heads)


def _latent_attn(q, cache, kv_indices, kv_start, kv_len, pos0, state_slot, qo_indptr, tok_seq, scale, gate):
    return ops.latent_attn(q, cache, kv_indices, kv_start, kv_len, _layout(q.shape[1], pos0, state_slot, qo_indptr, tok_seq), scale, gate)


def _gated_residual_norm(x, y, gate, gate_bias, mult, w_norm, groups, eps, y2, w_y, w_y2, dtype):
    return ops.gated_residual_norm(x, y=y, gate=gate, gate_bias=gate_bias, mult=mult, w_norm=w_norm, groups=groups, eps=eps, y2=y2, w_y=w_y,
                                   w_y2=w_y2, dtype=dtype)


def _head_norm_gate(o, w, eps, gate, kind, dtype):
    return ops.head_norm_gate(o, w, eps, gate=gate, kind=kind, dtype=dtype)


def _short_conv_silu(x, w, state, pos0, state_slot, qo_indptr, tok_seq):
    return ops.short_conv_silu(x, w, state, _layout(x.shape[0], pos0, state_slot, qo_indptr, tok_seq))


def _token_shift_mix(h, mu, state, pos0, state_slot, qo_indptr, tok_seq):
    return ops.token_shift_mix(h, mu, state, _layout(h.shape[0], pos0, state_slot, qo_indptr, tok_seq))


def _mlstm_scan(x, q_off, k_off, v_off, gates, gate_bias, cap, mem, norm, peak, pos0, state_slot, qo_indptr, tok_seq, heads, dim, vdim):
    return ops.mlstm_scan(x, (q_off, k_off, v_off), gates, gate_bias, cap, mem, norm, peak, _layout(x.shape[0], pos0, state_slot, qo_indptr, tok_seq),
                          heads, dim, vdim)


def _delta_scan(x, q_off, k_off, v_off, ab, a_log, dt_bias, mem, pos0, state_slot, qo_indptr, tok_seq, heads, kv_heads, dim, vdim):
    return ops.delta_scan(x, (q_off, k_off, v_off), ab, a_log, dt_bias, mem, _layout(x.shape[0], pos0, state_slot, qo_indptr, tok_seq), heads,
                          kv_heads, dim, vdim)


def _rwkv_scan(r, k, v, wlog, w0, bonus, mem, pos0, state_slot, qo_indptr, tok_seq, heads, dim):
    return ops.rwkv_scan(r, k, v, wlog, w0, bonus, mem, _layout(r.shape[0], pos0, state_slot, qo_indptr, tok_seq), heads, dim)


def _rope_vnorm_store(qkv, positions, freq, mag, rot_dims, eps, slots, k_cache, v_cache, heads, kv_heads, dim, vdim):
    return ops.rope_vnorm_store(qkv, positions, freq, mag, rot_dims, eps, slots, k_cache, v_cache, heads, kv_heads, dim, vdim)


def _softcap_attn(q, k_cache, v_cache, kv_indices, kv_start, kv_len, pos0, state_slot, qo_indptr, tok_seq, scale, cap, heads, kv_heads, dim, vdim,
                  window=0, r1=None, r2=None, v_turn=None, v_interleaved=False, gate=None, sink_score=None):
    return ops.softcap_attn(q, k_cache, v_cache, kv_indices, kv_start, kv_len, _layout(q.shape[0], pos0, state_slot, qo_indptr, tok_seq), scale, cap,
                            heads, kv_heads, dim, vdim, window=window, r1=r1, r2=r2, v_turn=v_turn, v_interleaved=v_interleaved, gate=gate,
                            sink_score=sink_score)


def _attn_prep_store(x, q_off, k_off, v_off, positions, q_w, k_w, norm_mode, eps, freq, rot_dims, interleaved, vfreq, slots, k_cache, v_cache,
                     heads, kv_heads, dim, vdim):
    return ops.attn_prep_store(x, (q_off, k_off, v_off), positions, q_w, k_w, norm_mode, eps, freq, rot_dims, interleaved, vfreq, slots, k_cache,
                               v_cache, heads, kv_heads, dim, vdim)


def _decay_scan(x, q_off, k_off, v_off, decay, mem, pos0, state_slot, qo_indptr, tok_seq, heads, dim, vdim, act):
    return ops.decay_scan(x, (q_off, k_off, v_off), decay, mem, _layout(x.shape[0], pos0, state_slot, qo_indptr, tok_seq), heads, dim, vdim, act=act)


def _postnorm_residual(x, y, w_post, eps, y2, a, b, w_next, dtype):
    return ops.postnorm_residual(x, y=y, w_post=w_post, eps=eps, y2=y2, a=a, b=b, w_next=w_next, out_dtype=dtype)


def _embed_scale(ids, table, scale):
    return ops.embed_scale(ids, table, scale)


def _tanh_cap(z, cap):
    return ops.tanh_cap(z, cap)


def _moe_route(logits, top):
    return ops.moe_route(logits, top)


def _moe_expert_rows(h, idx, wts, w_gu, w_d, limit, alpha, shift=1.0, weight_out=False):
    return ops.moe_expert_rows(h, idx, wts, w_gu, w_d, limit, alpha, shift, weight_out)


def _moe_order(idx, n_exp):
    return ops.moe_order(idx, n_exp)


def _moe_scatter_rows(h, wts, dst):
    return ops.moe_scatter_rows(h, wts, dst)


def _moe_glu(gu, limit, alpha, shift=1.0):
    return ops.moe_glu(gu, limit, alpha, shift)


def _moe_gather_rows(ys, dst, wts=None):
    return ops.moe_gather_rows(ys, dst, wts)


def _skinny_proj(x, w, in_act):
    return ops.skinny_proj(x, w, in_act)


def _hyper_mix(x, y, scale, mix, w_out, w_in, w_norm, eps, out_dtype):
    return ops.hyper_mix(x, y, scale, mix, w_out, w_in, w_norm, eps, out_dtype=out_dtype)[1]


def _hyper_start(x, n_streams, w_in, w_norm, eps, out_dtype):
    return ops.hyper_mix(x, w_in=w_in, w_norm=w_norm, eps=eps, n_streams=n_streams, out_dtype=out_dtype)


def _short_conv(x, w, state, pos0, state_slot, qo_indptr, tok_seq, bias, act):
    return ops.short_conv(x, w, state, _layout(x.shape[0], pos0, state_slot, qo_indptr, tok_seq), bias=bias, act=act)


def _rglru_scan(y, u, gates, gate_bias, rate, state, pos0, state_slot, qo_indptr, tok_seq):
    return ops.rglru_scan(y, u, gates, gate_bias, rate, state, _layout(u.shape[0], pos0, state_slot, qo_indptr, tok_seq))


def _latent_rope_prep(x, q_off, kv_off, g_off, positions, freq, mag, w_kv, eps, slots, cache, heads, dim, rot):
    return ops.latent_rope_prep(x, (q_off, kv_off, g_off), positions, freq, mag, w_kv, eps, slots, cache, heads, dim, rot)


def _moe_route_softmax(logits, top, n_groups, keep_groups, norm_eps):
    return ops.moe_route_softmax(logits, top, n_groups, keep_groups, norm_eps)


for _name in _DEFS:
    _LIB.impl(_name, globals()["_" + _name], "CUDA")   # PyTorch-ROCm's device key is spelled CUDA
