"""Tensor-level wrappers over the C ABI (include/nvx.h).

PyTorch is used here only as the owner of device memory and of the current HIP stream; every
function validates shapes on the host (a kernel that is handed a wrong shape faults the GPU), then
makes exactly one call into libnvx_hip.so on `torch.cuda.current_stream()`, which makes all of them
capturable into a hipGraph.  `nano_vllm_x_amd.torch_ops` registers the stateless ones as
`torch.ops.nvx.*` custom ops.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib

BF16 = torch.bfloat16
F16 = torch.float16
H16 = (BF16, F16)   # the 16-bit formats the library is built for: the kernels of a call all run in the format of its activations


def _fn(lib, name: str, dtype):
    """Entry point `name` in the build for `dtype`: bfloat16 is the unsuffixed symbol, float16 `name_f16`."""
    return getattr(lib, name + "_f16" if dtype == F16 else name)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "nvx ops need device tensors (the HIP path has no CPU fallback)")


def _ptr(t):
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------------------------
def store_kvcache(k, v, k_cache, v_cache, kv_indices):
    """Same contract as nanovllmx.core.kv_cache.store_kvcache (kv_cache.py:36-44)."""
    _dev(k, v, k_cache, v_cache, kv_indices)
    num_tokens, num_heads, head_dim = k.shape
    row = num_heads * head_dim
    assert k.stride(-1) == 1 and v.stride(-1) == 1
    assert k.stride(-2) == head_dim and v.stride(-2) == head_dim
    assert k_cache.stride(-3) == row and v_cache.stride(-3) == row
    assert kv_indices.numel() == num_tokens
    _need(k.dtype == v.dtype == k_cache.dtype == v_cache.dtype and k.element_size() == 2, "store_kvcache: 16-bit dtypes only")
    _need(kv_indices.dtype == torch.int64 and kv_indices.is_contiguous(), "store_kvcache: kv_indices must be contiguous int64")
    lib = _lib.load()
    _lib.check(lib.nvx_store_kv(_ptr(k), _ptr(v), k.stride(0), v.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(kv_indices),
                                num_tokens, row, k_cache.shape[-3], _stream()), "nvx_store_kv")


def rmsnorm(x, weight, eps, residual=None):
    """RMSNorm.forward (layernorm.py:17-36): returns y, or (y, new_residual) when residual is given."""
    _dev(x, weight, residual)
    _need(x.dtype in H16, "rmsnorm: bfloat16 or float16 activations")
    hidden = x.shape[-1]
    if x.dim() == 2 and x.stride(1) == 1:
        x2 = x  # rows may be strided (a split view of a fused projection)
    else:
        x = x.contiguous()
        x2 = x.view(-1, hidden)
    rows = x2.shape[0]
    _need(weight.numel() == hidden and weight.is_contiguous(), "rmsnorm: weight shape")
    _need(weight.dtype in (x.dtype, torch.float32), "rmsnorm: weight must have the activations' dtype or be fp32")
    y = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    res_out = None
    if residual is not None:
        _need(residual.dtype == x.dtype and residual.shape == x.shape, "rmsnorm: residual shape/dtype")
        residual = residual.contiguous()
        res_out = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_rmsnorm", x.dtype)(_ptr(x2), x2.stride(0), _ptr(residual), _ptr(weight), int(weight.dtype == torch.float32),
                               _ptr(y), _ptr(res_out), rows, hidden, float(eps), _stream()), "nvx_rmsnorm")
    y = y.view(x.shape)
    if residual is None:
        return y
    return y, res_out.view(x.shape)


def rope(positions, q, k, cos_sin_cache, head_size=128):
    """RotaryEmbedding.forward (rotary_embedding.py:74-102), rotary_dim == head_size == 128."""
    _dev(positions, q, k, cos_sin_cache)
    _need(head_size == 128 and cos_sin_cache.shape[-1] == 128 and cos_sin_cache.dtype == torch.float32 and
          cos_sin_cache.is_contiguous(), "rope: needs an fp32 (max_pos, 128) table")
    _need(q.dtype in H16 and k.dtype == q.dtype, "rope: bfloat16 or float16, q and k alike")
    positions = positions.flatten()
    _need(positions.dtype == torch.int64 and positions.is_contiguous(), "rope: positions must be int64")
    t = positions.numel()
    q2, k2 = q.reshape(t, -1) if q.is_contiguous() else q.view(t, -1), k.reshape(t, -1) if k.is_contiguous() else k.view(t, -1)
    _need(q2.stride(1) == 1 and k2.stride(1) == 1 and q2.shape[1] % 128 == 0 and k2.shape[1] % 128 == 0, "rope: row layout")
    q_out = torch.empty((t, q2.shape[1]), dtype=q.dtype, device=q.device)
    k_out = torch.empty((t, k2.shape[1]), dtype=k.dtype, device=k.device)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_rope", q.dtype)(_ptr(positions), _ptr(cos_sin_cache), cos_sin_cache.shape[0], _ptr(q2), q2.stride(0), _ptr(k2),
                            k2.stride(0), _ptr(q_out), _ptr(k_out), t, q2.shape[1] // 128, k2.shape[1] // 128, _stream()),
               "nvx_rope")
    return q_out.view(q.shape), k_out.view(k.shape)


def qknorm_rope_store(qkv, positions, cos_sin_cache, q_norm_weight, k_norm_weight, eps, slots, k_cache, v_cache,
                      n_q_heads, n_kv_heads, q_out=None):
    """qwen3.py:123-133 + attention.py:344-352 in one launch.  Returns q (T, n_q_heads*128)."""
    _dev(qkv, positions, cos_sin_cache, q_norm_weight, k_norm_weight, slots, k_cache, v_cache)
    t = qkv.shape[0]
    width = (n_q_heads + 2 * n_kv_heads) * 128
    _need(qkv.dim() == 2 and qkv.shape[1] == width and qkv.stride(1) == 1 and qkv.dtype in H16, "qknorm_rope_store: qkv layout")
    _need(positions.dtype == torch.int64 and positions.numel() >= t and positions.is_contiguous(), "qknorm_rope_store: positions")
    _need(slots.dtype == torch.int64 and slots.numel() >= t and slots.is_contiguous(), "qknorm_rope_store: slots")
    _need(k_cache.shape[-2:] == (n_kv_heads, 128) and v_cache.shape == k_cache.shape and k_cache.is_contiguous() and
          v_cache.is_contiguous() and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "qknorm_rope_store: cache layout")
    _need(q_norm_weight.dtype == qkv.dtype and k_norm_weight.dtype == qkv.dtype and q_norm_weight.numel() == 128 and
          k_norm_weight.numel() == 128, "qknorm_rope_store: norm weights must be bf16 (128)")
    _need(cos_sin_cache.dtype == torch.float32 and cos_sin_cache.shape[-1] == 128 and cos_sin_cache.is_contiguous(), "qknorm_rope_store: table")
    if q_out is None:
        q_out = torch.empty((t, n_q_heads * 128), dtype=qkv.dtype, device=qkv.device)
    else:
        _need(q_out.shape == (t, n_q_heads * 128) and q_out.is_contiguous() and q_out.dtype == qkv.dtype, "qknorm_rope_store: q_out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_qknorm_rope_store", qkv.dtype)(_ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(cos_sin_cache), cos_sin_cache.shape[0],
                                         _ptr(q_norm_weight), _ptr(k_norm_weight), float(eps), _ptr(slots), _ptr(q_out),
                                         _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], t, n_q_heads, n_kv_heads, _stream()),
               "nvx_qknorm_rope_store")
    return q_out


def linear_decode_splits(n: int, k: int) -> int:
    return int(_lib.load().nvx_linear_decode_splits(n, k))


def linear_decode(x, w, mode: int = 0, k_splits: int = 1, out=None):
    """x (m <= 256, k) bf16 times w (n, k)^T.  mode 0 -> bf16 (m, n); mode 1 -> SiluAndMul of the
    [gate; up] projection, bf16 (m, n/2); mode 2 -> fp32 partials (k_splits, m, n) for rmsnorm_splitk."""
    _dev(x, w, out)
    _need(x.dim() == 2 and w.dim() == 2 and x.dtype in H16 and w.dtype == x.dtype, "linear_decode: 2-D bfloat16 or float16 operands")
    _need(x.stride(1) == 1 and w.is_contiguous() and x.shape[1] == w.shape[1], "linear_decode: layouts")
    m, k = x.shape
    n = w.shape[0]
    if mode == 0:
        shape, dtype = (m, n), x.dtype
    elif mode == 1:
        shape, dtype = (m, n // 2), x.dtype
    else:
        shape, dtype = (k_splits, m, n), torch.float32
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=x.device)
    else:
        _need(out.dtype == dtype and out.is_contiguous() and out.numel() >= shape[0] * shape[1] * (shape[2] if len(shape) == 3 else 1),
              "linear_decode: out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_linear_decode", x.dtype)(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, mode, k_splits, _stream()), "nvx_linear_decode")
    return out


def rmsnorm_splitk(partials, weight, eps, residual=None):
    """RMSNorm over bf16(sum of fp32 partials (splits, rows, hidden)); returns y or (y, new_residual)."""
    _dev(partials, weight, residual)
    _need(partials.dim() == 3 and partials.dtype == torch.float32 and partials.is_contiguous(), "rmsnorm_splitk: partials")
    _need(weight.dtype in H16 and weight.is_contiguous(), "rmsnorm_splitk: bfloat16 or float16 weight (it sets the output format)")
    s, rows, hidden = partials.shape
    y = torch.empty((rows, hidden), dtype=weight.dtype, device=partials.device)
    res_out = None
    if residual is not None:
        _need(residual.dtype == weight.dtype and residual.is_contiguous() and residual.shape == (rows, hidden), "rmsnorm_splitk: residual")
        res_out = torch.empty_like(residual)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_rmsnorm_splitk", weight.dtype)(_ptr(partials), s, _ptr(residual), _ptr(weight), _ptr(y), _ptr(res_out), rows, hidden,
                                      float(eps), _stream()), "nvx_rmsnorm_splitk")
    return y if residual is None else (y, res_out)


def silu_mul(x, out=None):
    """SiluAndMul.forward (activation.py:15-18)."""
    _dev(x)
    _need(x.dtype in H16 and x.is_contiguous(), "silu_mul: contiguous bfloat16 or float16")
    d = x.shape[-1] // 2
    rows = x.numel() // (2 * d)
    if out is None:
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
    else:
        _need(out.is_contiguous() and out.numel() == rows * d and out.dtype == x.dtype, "silu_mul: out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_silu_mul", x.dtype)(_ptr(x), _ptr(out), rows, d, _stream()), "nvx_silu_mul")
    return out


# ---------------------------------------------------------------------------------------------
class DecodeWorkspace:
    """Caller-owned scratch of the decode attention (plan list + split partials), sized once."""

    def __init__(self, max_batch: int, n_q_heads: int, n_kv_heads: int, device):
        lib = _lib.load()
        self.max_batch, self.n_q_heads, self.n_kv_heads = max_batch, n_q_heads, n_kv_heads
        self.plan = torch.zeros(lib.nvx_decode_plan_ws_ints(max_batch, n_kv_heads), dtype=torch.int32, device=device)
        self.partial = torch.empty(lib.nvx_decode_partial_ws_floats(max_batch, n_q_heads, n_kv_heads), dtype=torch.float32,
                                   device=device)

    @classmethod
    def from_tensors(cls, plan: torch.Tensor, partial, n_q_heads: int, n_kv_heads: int) -> "DecodeWorkspace":
        """A workspace over tensors the caller already holds (how the custom ops receive it).  The batch it can
        serve is what both tensors have room for, by the library's own sizing rules."""
        lib = _lib.load()
        _need(plan.dtype == torch.int32 and plan.is_contiguous(), "decode workspace: plan must be contiguous int32")
        self = cls.__new__(cls)
        self.n_q_heads, self.n_kv_heads, self.plan, self.partial = n_q_heads, n_kv_heads, plan, partial
        # nvx_decode_plan_ws_ints(b, hkv) = 8 + 8 * (b + 2048 / hkv + 8) + 2 * b, nvx_decode_partial_ws_floats likewise linear in b
        fixed = int(lib.nvx_decode_plan_ws_ints(0, n_kv_heads))
        mb = (plan.numel() - fixed) // 10
        if partial is not None:
            _need(partial.dtype == torch.float32 and partial.is_contiguous(), "decode workspace: partials must be contiguous fp32")
            per = int(lib.nvx_decode_partial_ws_floats(1, n_q_heads, n_kv_heads)) - int(lib.nvx_decode_partial_ws_floats(0, n_q_heads, n_kv_heads))
            mb = min(mb, (partial.numel() - int(lib.nvx_decode_partial_ws_floats(0, n_q_heads, n_kv_heads))) // max(1, per))
        self.max_batch = max(0, int(mb))
        return self


def decode_plan(kv_len, kv_start, ws: DecodeWorkspace, out_slots=None):
    """Cut the batch's sequences into chunks (device side); must precede paged_decode of the same step.
    `out_slots` (int64 per sequence, -1 = none) is needed by paged_decode_qkv: the slot the step's new
    K/V row goes to."""
    _dev(kv_len, kv_start, out_slots, ws.plan)
    b = kv_len.numel()
    if out_slots is not None:
        _need(out_slots.dtype == torch.int64 and out_slots.is_contiguous() and out_slots.numel() == b, "decode_plan: out_slots")
    _need(kv_len.dtype == torch.int32 and kv_len.is_contiguous() and 0 < b <= ws.max_batch, "decode_plan: kv_len")
    _need(kv_start.dtype == torch.int64 and kv_start.is_contiguous() and kv_start.numel() == b, "decode_plan: kv_start")
    lib = _lib.load()
    _lib.check(lib.nvx_decode_plan(_ptr(kv_len), _ptr(kv_start), _ptr(out_slots), b, ws.n_kv_heads, _ptr(ws.plan), ws.plan.numel(),
                                   _stream()), "nvx_decode_plan")


def paged_decode_qkv(qkv, positions, cos_sin_cache, q_weight, k_weight, eps, k_cache, v_cache, kv_indices, batch: int,
                     ws: DecodeWorkspace, sm_scale, out=None):
    """Decode attention fed with the raw fused projection (B, (Hq + 2*Hkv)*128): per-head RMSNorm + rotary
    of q and of the new k, scatter of the new k/v row (to the slots given to decode_plan) and attention,
    in one launch.  Equivalent to qknorm_rope_store followed by paged_decode."""
    _dev(qkv, positions, cos_sin_cache, q_weight, k_weight, k_cache, v_cache, kv_indices)
    b = batch
    hq, hkv = ws.n_q_heads, ws.n_kv_heads
    _need(qkv.dim() == 2 and qkv.shape[0] == b and qkv.shape[1] == (hq + 2 * hkv) * 128 and qkv.dtype in H16 and qkv.stride(1) == 1,
          "paged_decode_qkv: qkv layout")
    _need(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == b, "paged_decode_qkv: positions")
    _need(cos_sin_cache.dtype == torch.float32 and cos_sin_cache.is_contiguous() and cos_sin_cache.shape[-1] == 128,
          "paged_decode_qkv: cos/sin table")
    _need(q_weight.dtype == qkv.dtype and k_weight.dtype == qkv.dtype and q_weight.numel() == 128 and k_weight.numel() == 128,
          "paged_decode_qkv: norm weights")
    _need(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          tuple(k_cache.shape[-2:]) == (hkv, 128) and v_cache.shape == k_cache.shape, "paged_decode_qkv: cache layout")
    _need(kv_indices.dtype == torch.int32 and kv_indices.is_contiguous(), "paged_decode_qkv: kv_indices must be int32")
    _need(0 < b <= ws.max_batch, "paged_decode_qkv: batch exceeds the workspace")
    if out is None:
        out = torch.empty((b, hq * 128), dtype=qkv.dtype, device=qkv.device)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_paged_decode_qkv", qkv.dtype)(_ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(cos_sin_cache), cos_sin_cache.shape[0],
                                        _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(k_cache), _ptr(v_cache), k_cache.shape[-3],
                                        _ptr(kv_indices), _ptr(ws.plan), _ptr(ws.partial), _ptr(out), b, hq, hkv, float(sm_scale),
                                        _stream()), "nvx_paged_decode_qkv")
    return out


def paged_decode(q, k_cache, v_cache, kv_indices, batch: int, ws: DecodeWorkspace, sm_scale, out=None):
    """q (B, Hq*128) or (B, Hq, 128); caches (slots, Hkv, 128) of one layer; ws.plan must hold the plan
    of this step (decode_plan with the same kv_indices layout)."""
    _dev(q, k_cache, v_cache, kv_indices)
    b = batch
    hq, hkv = ws.n_q_heads, ws.n_kv_heads
    q2 = q.view(b, hq * 128)
    _need(q2.dtype in H16 and q2.stride(1) == 1, "paged_decode: q layout")
    _need(k_cache.dtype == q2.dtype and v_cache.dtype == q2.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          tuple(k_cache.shape[-2:]) == (hkv, 128) and v_cache.shape == k_cache.shape, "paged_decode: cache layout")
    _need(kv_indices.dtype == torch.int32 and kv_indices.is_contiguous(), "paged_decode: kv_indices must be int32")
    _need(0 < b <= ws.max_batch, "paged_decode: batch exceeds the workspace")
    if out is None:
        out = torch.empty((b, hq * 128), dtype=q2.dtype, device=q.device)
    else:
        _need(out.is_contiguous() and out.numel() == b * hq * 128 and out.dtype == q2.dtype, "paged_decode: out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_paged_decode", q2.dtype)(_ptr(q2), q2.stride(0), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], _ptr(kv_indices),
                                    _ptr(ws.plan), _ptr(ws.partial), _ptr(out), b, hq, hkv, float(sm_scale), _stream()),
               "nvx_paged_decode")
    return out


def paged_decode_noalloc(q, k_cache, v_cache, kv_indices, kv_len, kv_start, n_q_heads: int, n_kv_heads: int, sm_scale, out=None):
    """decode_plan + paged_decode without a workspace: plan and partials live in an array built into the library
    (one per GPU; batch <= 256; calls that overlap on one GPU race).  For callers that cannot allocate."""
    _dev(q, k_cache, v_cache, kv_indices, kv_len, kv_start)
    b = kv_len.numel()
    q2 = q.view(b, n_q_heads * 128)
    _need(q2.dtype == BF16 and q2.stride(1) == 1, "paged_decode_noalloc: q layout")
    _need(k_cache.dtype == q2.dtype and v_cache.dtype == q2.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          tuple(k_cache.shape[-2:]) == (n_kv_heads, 128) and v_cache.shape == k_cache.shape, "paged_decode_noalloc: cache layout")
    _need(kv_indices.dtype == torch.int32 and kv_indices.is_contiguous(), "paged_decode_noalloc: kv_indices must be int32")
    _need(kv_len.dtype == torch.int32 and kv_len.is_contiguous() and kv_start.dtype == torch.int64 and kv_start.is_contiguous()
          and kv_start.numel() == b, "paged_decode_noalloc: kv_len int32 / kv_start int64, one per sequence")
    if out is None:
        out = torch.empty((b, n_q_heads * 128), dtype=BF16, device=q.device)
    lib = _lib.load()
    _lib.check(lib.nvx_paged_decode_noalloc(_ptr(q2), q2.stride(0), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], _ptr(kv_indices),
                                            _ptr(kv_len), _ptr(kv_start), _ptr(out), b, n_q_heads, n_kv_heads, float(sm_scale),
                                            _stream()), "nvx_paged_decode_noalloc")
    return out


def prefill_plan_ws(batch: int, device):
    lib = _lib.load()
    return torch.zeros(lib.nvx_prefill_plan_ws_ints(batch), dtype=torch.int32, device=device)


def prefill_plan(qo_indptr, plan_ws):
    _dev(qo_indptr, plan_ws)
    b = qo_indptr.numel() - 1
    _need(qo_indptr.dtype == torch.int32 and qo_indptr.is_contiguous() and b > 0, "prefill_plan: qo_indptr")
    lib = _lib.load()
    _lib.check(lib.nvx_prefill_plan(_ptr(qo_indptr), b, _ptr(plan_ws), plan_ws.numel(), _stream()), "nvx_prefill_plan")


def paged_prefill(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, plan_ws, n_q_heads, n_kv_heads, sm_scale, out=None):
    """q (T, Hq*128); causal varlen attention over paged K/V (attention.py:360-364)."""
    _dev(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, plan_ws)
    t = q.shape[0]
    b = qo_indptr.numel() - 1
    q2 = q.view(t, n_q_heads * 128)
    _need(q2.dtype in H16 and q2.stride(1) == 1, "paged_prefill: q layout")
    _need(k_cache.dtype == q2.dtype and v_cache.dtype == q2.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          tuple(k_cache.shape[-2:]) == (n_kv_heads, 128) and v_cache.shape == k_cache.shape, "paged_prefill: cache layout")
    for name, x in (("qo_indptr", qo_indptr), ("kv_indptr", kv_indptr), ("kv_indices", kv_indices)):
        _need(x.dtype == torch.int32 and x.is_contiguous(), f"paged_prefill: {name} must be contiguous int32")
    _need(kv_indptr.numel() == b + 1, "paged_prefill: indptr lengths differ")
    if out is None:
        out = torch.empty((t, n_q_heads * 128), dtype=q2.dtype, device=q.device)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_paged_prefill", q2.dtype)(_ptr(q2), q2.stride(0), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], _ptr(qo_indptr),
                                     _ptr(kv_indptr), _ptr(kv_indices), _ptr(plan_ws), _ptr(out), t, b, n_q_heads, n_kv_heads,
                                     float(sm_scale), _stream()), "nvx_paged_prefill")
    return out


# ---------------------------------------------------------------------------------------------
def _sampler_args(logits, temperatures, top_ks, top_ps, min_ps):
    _dev(logits, temperatures, top_ks, top_ps, min_ps)
    _need(logits.dim() == 2 and logits.stride(1) == 1 and logits.dtype in (BF16, torch.float32), "sampler: logits layout")
    b, v = logits.shape
    _need(temperatures.dtype == torch.float32 and top_ps.dtype == torch.float32 and min_ps.dtype == torch.float32 and
          top_ks.dtype == torch.int64, "sampler: parameter dtypes (float32, int64)")
    for x in (temperatures, top_ks, top_ps, min_ps):
        _need(x.numel() == b and x.is_contiguous(), "sampler: one parameter per row")
    return b, v


_SAMPLE_WS: dict = {}   # device -> int64 workspace (slices' winners), grown on demand outside graph capture


def sample_workspace(batch: int, device) -> torch.Tensor:
    """Workspace that lets nvx_sample cut rows into slices.  Allocate it before capturing a graph that
    samples: the captured launch keeps the pointer."""
    lib = _lib.load()
    need = int(lib.nvx_sample_ws_bytes(batch)) // 8
    key = torch.device(device)
    ws = _SAMPLE_WS.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, int(lib.nvx_sample_ws_bytes(256)) // 8), dtype=torch.int64, device=device)
        _SAMPLE_WS[key] = ws
    return ws


def sample(logits, temperatures, top_ks, top_ps, min_ps, seed: int, offset: int, out=None, ws=None):
    """Sampler.forward (sampler.py:39-55): one token id per row, Philox(seed, offset) Gumbel-max draw."""
    b, v = _sampler_args(logits, temperatures, top_ks, top_ps, min_ps)
    if ws is None:
        ws = sample_workspace(b, logits.device)
    if out is None:
        out = torch.empty((b,), dtype=torch.int64, device=logits.device)
    else:
        _need(out.dtype == torch.int64 and out.numel() >= b and out.is_contiguous(), "sample: out")
    lib = _lib.load()
    _lib.check(lib.nvx_sample(_ptr(logits), int(logits.dtype == torch.float32), logits.stride(0), _ptr(temperatures),
                              _ptr(top_ks), _ptr(top_ps), _ptr(min_ps), b, v, seed & (2**64 - 1), offset & (2**64 - 1),
                              _ptr(out), _ptr(ws), ws.numel() * 8, _stream()), "nvx_sample")
    return out


def sample_shard(logits, temperatures, vocab_offset: int, vocab: int, seed: int, offset: int, out=None, ws=None):
    """One tensor-parallel rank's part of an unfiltered sampling step: the draw over its shard of the vocabulary
    (logits (B, shard), token j = token vocab_offset + j of the whole row), one 64-bit (score, token) key per row."""
    _dev(logits, temperatures)
    _need(logits.dim() == 2 and logits.stride(1) == 1 and logits.dtype in (BF16, torch.float32), "sample_shard: logits layout")
    b, v = logits.shape
    _need(temperatures.dtype == torch.float32 and temperatures.numel() == b and temperatures.is_contiguous(), "sample_shard: temperatures")
    _need(vocab_offset >= 0 and vocab_offset % 4 == 0 and vocab > 0, "sample_shard: the shard must start at a multiple of 4 tokens")
    if ws is None:
        ws = sample_workspace(b, logits.device)
    if out is None:
        out = torch.empty((b,), dtype=torch.int64, device=logits.device)
    else:
        _need(out.dtype == torch.int64 and out.numel() >= b and out.is_contiguous(), "sample_shard: out")
    lib = _lib.load()
    _lib.check(lib.nvx_sample_shard(_ptr(logits), int(logits.dtype == torch.float32), logits.stride(0), _ptr(temperatures), b, v,
                                    vocab_offset, vocab, seed & (2**64 - 1), offset & (2**64 - 1), _ptr(out), _ptr(ws), ws.numel() * 8,
                                    _stream()), "nvx_sample_shard")
    return out


def lmhead_max_rows() -> int:
    return int(_lib.load().nvx_lmhead_max_rows())


def lmhead_pack(weight):
    """LM-head weight (rows, k) 16-bit -> the tiled copy lmhead_sample streams (built once, when the model is loaded)."""
    _dev(weight)
    _need(weight.dim() == 2 and weight.is_contiguous() and weight.dtype in H16 and weight.shape[1] % 32 == 0, "lmhead_pack: weight layout")
    lib = _lib.load()
    n, k = weight.shape
    packed = torch.empty(int(lib.nvx_lmhead_packed_elems(n, k)), dtype=weight.dtype, device=weight.device)
    _lib.check(lib.nvx_lmhead_pack(_ptr(weight), n, k, _ptr(packed), _stream()), "nvx_lmhead_pack")
    return packed


def lmhead_workspace(batch: int, device):
    return torch.empty(int(_lib.load().nvx_lmhead_ws_bytes(batch)) // 8, dtype=torch.int64, device=device)


def lmhead_sample(packed, n_rows: int, x, temperatures, vocab_offset: int, vocab: int, seed: int, offset: int, ws=None, keys=False,
                  out=None, logits_out=None):
    """hidden states x (B, k) -> one token per row (or, `keys`, the 64-bit (score, token) keys as int64 bit patterns, for
    sample_pick over tensor-parallel ranks): the LM head and the unfiltered Gumbel-max draw in one pass over the packed
    weight.  `logits_out` (B, >= n_rows padded to 16) receives the 16-bit logits if given."""
    _dev(packed, x, temperatures, logits_out)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.dtype in H16 and packed.dtype == x.dtype, "lmhead_sample: x layout")
    b, k = x.shape
    _need(0 < b <= lmhead_max_rows(), "lmhead_sample: batch exceeds what the kernel keeps on a compute unit")
    _need(temperatures.dtype == torch.float32 and temperatures.numel() == b and temperatures.is_contiguous(), "lmhead_sample: temperatures")
    _need(packed.is_contiguous() and packed.numel() == ((n_rows + 15) // 16) * 16 * k, "lmhead_sample: packed weight size")
    if ws is None:
        ws = lmhead_workspace(b, x.device)
    if out is None:
        out = torch.empty((b,), dtype=torch.int64, device=x.device)
    else:
        _need(out.dtype == torch.int64 and out.numel() >= b and out.is_contiguous(), "lmhead_sample: out")
    if logits_out is not None:
        _need(logits_out.dim() == 2 and logits_out.dtype == x.dtype and logits_out.shape[0] >= b and logits_out.stride(1) == 1 and
              logits_out.shape[1] >= ((n_rows + 15) // 16) * 16, "lmhead_sample: logits_out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_lmhead_sample", x.dtype)(_ptr(packed), n_rows, k, _ptr(x), x.stride(0), b, _ptr(temperatures), vocab_offset, vocab,
                                                     seed & (2**64 - 1), offset & (2**64 - 1), _ptr(ws), ws.numel() * 8,
                                                     _ptr(out) if keys else None, None if keys else _ptr(out), _ptr(logits_out),
                                                     logits_out.stride(0) if logits_out is not None else 0, _stream()), "nvx_lmhead_sample")
    return out


def linear_stream(x, packed, n: int, out=None):
    """x (m, k) 16-bit, m <= 64, k a multiple of 1024; `packed` = lmhead_pack of the (n, k) weight -> fp32 partial products
    (k / 1024, m, n), one per 1024-wide slice of k, for rmsnorm_splitk or splitk_sum to add up."""
    _dev(x, packed, out)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.dtype in H16 and packed.dtype == x.dtype and packed.is_contiguous(), "linear_stream: x / packed layout")
    m, k = x.shape
    _need(0 < m <= lmhead_rows_per_pass() and k % 1024 == 0, "linear_stream: at most 64 rows, k a multiple of 1024")
    _need(packed.numel() == ((n + 15) // 16) * 16 * k, "linear_stream: packed weight size")
    s = k // 1024
    if out is None:
        out = torch.empty((s, m, n), dtype=torch.float32, device=x.device)
    else:
        _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (s, m, n), "linear_stream: out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_linear_stream", x.dtype)(_ptr(packed), n, k, _ptr(x), x.stride(0), m, _ptr(out), _stream()), "nvx_linear_stream")
    return out


def linear_block_max_rows() -> int:
    return int(_lib.load().nvx_linear_block_max_rows())


def linear_block_slices(n: int, k: int, mode: int) -> int:
    """k-slices linear_block cuts a weight of n rows over k into (mode 2), 1 for modes 0 / 1; 0 = shape not supported."""
    return int(_lib.load().nvx_linear_block_slices(n, k, mode))


def linear_block(x, packed, n: int, mode: int = 0, k_slices: int = 1, out=None):
    """x (m, k) 16-bit, m <= 256; `packed` = lmhead_pack of the (n, k) weight.  mode 0: y (m, n); mode 1: the weight is
    [gate rows; up rows], y (m, n / 2) = SiluAndMul of the 16-bit-rounded projection; mode 2: fp32 partial products
    (k_slices, m, n) for rmsnorm_splitk / splitk_sum to add up."""
    _dev(x, packed, out)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.dtype in H16 and packed.dtype == x.dtype and packed.is_contiguous(), "linear_block: x / packed layout")
    m, k = x.shape
    _need(0 < m <= linear_block_max_rows(), "linear_block: 1..256 rows")
    _need(n % 16 == 0 and packed.numel() == n * k, "linear_block: packed weight size")
    _need(mode in (0, 1, 2) and k_slices >= 1 and (mode == 2 or k_slices == 1), "linear_block: mode / k_slices")
    shape = (k_slices, m, n) if mode == 2 else (m, n // 2 if mode == 1 else n)
    dtype = torch.float32 if mode == 2 else x.dtype
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=x.device)
    else:
        _need(out.dtype == dtype and out.is_contiguous() and tuple(out.shape) == shape, "linear_block: out")
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_linear_block", x.dtype)(_ptr(packed), n, k, _ptr(x), x.stride(0), m, mode, k_slices, _ptr(out), _stream()),
               "nvx_linear_block")
    return out


def lmhead_rows_per_pass() -> int:
    return int(_lib.load().nvx_lmhead_rows_per_pass())


def splitk_sum(partials, dtype, silu_mul: bool = False):
    """(splits, rows, n) fp32 -> (rows, n) in `dtype`, or SiluAndMul of the summed [gate | up] projection, (rows, n / 2)."""
    _dev(partials)
    _need(partials.dim() == 3 and partials.dtype == torch.float32 and partials.is_contiguous() and dtype in H16, "splitk_sum: partials")
    s, rows, n = partials.shape
    y = torch.empty((rows, n // 2 if silu_mul else n), dtype=dtype, device=partials.device)
    lib = _lib.load()
    _lib.check(_fn(lib, "nvx_splitk_sum", dtype)(_ptr(partials), s, rows, n, int(silu_mul), _ptr(y), _stream()), "nvx_splitk_sum")
    return y


def sample_pick(winners, out=None):
    """Token ids from the ranks' keys: winners (n_sets, B) int64 (bit patterns of the 64-bit keys) -> (B,) int64."""
    _dev(winners)
    _need(winners.dim() == 2 and winners.dtype == torch.int64 and winners.is_contiguous(), "sample_pick: winners must be contiguous int64 (sets, B)")
    n, b = winners.shape
    if out is None:
        out = torch.empty((b,), dtype=torch.int64, device=winners.device)
    else:
        _need(out.dtype == torch.int64 and out.numel() >= b and out.is_contiguous(), "sample_pick: out")
    lib = _lib.load()
    _lib.check(lib.nvx_sample_pick(_ptr(winners), n, b, _ptr(out), _stream()), "nvx_sample_pick")
    return out


def sampler_probs(logits, temperatures, top_ks, top_ps, min_ps):
    """The distribution the sampler draws from (after temperature, top-k, top-p, min-p), fp32 (B, V)."""
    b, v = _sampler_args(logits, temperatures, top_ks, top_ps, min_ps)
    probs = torch.empty((b, v), dtype=torch.float32, device=logits.device)
    lib = _lib.load()
    _lib.check(lib.nvx_sampler_probs(_ptr(logits), int(logits.dtype == torch.float32), logits.stride(0), _ptr(temperatures),
                                     _ptr(top_ks), _ptr(top_ps), _ptr(min_ps), b, v, _ptr(probs), _stream()),
               "nvx_sampler_probs")
    return probs


# ---------------------------------------------------------------------------------------------
def block_table_write_rows(kv_indices, kv_indptr, rows, table):
    _dev(kv_indices, kv_indptr, rows, table)
    b = rows.numel()
    _need(table.dim() == 2 and table.is_contiguous() and table.dtype == torch.int32, "block_table_write_rows: table")
    for x in (kv_indices, kv_indptr, rows):
        _need(x.dtype == torch.int32 and x.is_contiguous(), "block_table_write_rows: int32 inputs")
    _need(kv_indptr.numel() == b + 1, "block_table_write_rows: indptr length")
    lib = _lib.load()
    _lib.check(lib.nvx_block_table_write_rows(_ptr(kv_indices), _ptr(kv_indptr), _ptr(rows), b, _ptr(table), table.shape[0],
                                              table.shape[1], _stream()), "nvx_block_table_write_rows")


def decode_step_setup(step, stride, padded_batch, table, pad_start, kv_start, kv_len, out_slots, positions, input_ids,
                      prev_ids=None):
    """`prev_ids` (int64, at least `stride` entries): where a negative token -1-j of the step buffer is looked up."""
    _dev(step, table, kv_start, kv_len, out_slots, positions, input_ids)
    if prev_ids is not None:
        _dev(prev_ids)
        _need(prev_ids.dtype == torch.int64 and prev_ids.numel() >= stride and prev_ids.is_contiguous(), "decode_step_setup: prev_ids")
    _need(step.dtype == torch.int32 and step.numel() >= 4 + 4 * stride and step.is_contiguous(), "decode_step_setup: step buffer")
    _need(table.dim() == 2 and table.is_contiguous() and table.dtype == torch.int32, "decode_step_setup: table")
    _need(kv_len.dtype == torch.int32 and all(x.dtype == torch.int64 for x in (kv_start, out_slots, positions, input_ids)),
          "decode_step_setup: output dtypes")
    for x in (kv_start, kv_len, out_slots, positions, input_ids):
        _need(x.numel() >= padded_batch and x.is_contiguous(), "decode_step_setup: output sizes")
    lib = _lib.load()
    _lib.check(lib.nvx_decode_step_setup(_ptr(step), stride, padded_batch, _ptr(table), table.shape[0], table.shape[1], pad_start,
                                         _ptr(kv_start), _ptr(kv_len), _ptr(out_slots), _ptr(positions), _ptr(input_ids),
                                         _ptr(prev_ids) if prev_ids is not None else None, _stream()), "nvx_decode_step_setup")


# ---------------------------------------------------------------------------------------------
class PeerGroup:
    """One rank's end of the direct-peer all-reduce of a tensor-parallel group (include/nvx.h, nvx_peer_*): a landing
    buffer in uncached device memory that every peer has mapped, into which the peers' kernels write their rows.
    Created once at start-up; `export_handle` / `import_handle` carry the 64-byte inter-process handles, which the
    caller exchanges by its own means.  `_registry` lets the custom ops address a group by an integer."""

    _registry: dict = {}

    def __init__(self, tp_size: int, rank: int, max_rows: int, hidden: int, timeout_ms: int = 0):
        import ctypes
        lib = _lib.load()
        comm = ctypes.c_void_p()
        _lib.check(lib.nvx_peer_create(tp_size, rank, max_rows, hidden, timeout_ms, ctypes.byref(comm)), "nvx_peer_create")
        self.comm, self.tp_size, self.rank, self.max_rows, self.hidden = comm.value, tp_size, rank, max_rows, hidden
        self.exchange_bytes = int(lib.nvx_peer_exchange_bytes(tp_size, max_rows, hidden))
        PeerGroup._registry[self.comm] = self

    def export_handle(self) -> bytes:
        import ctypes
        buf = ctypes.create_string_buffer(64)
        _lib.check(_lib.load().nvx_peer_export(self.comm, buf), "nvx_peer_export")
        return buf.raw

    def import_handle(self, peer_rank: int, handle: bytes):
        _need(len(handle) == 64, "PeerGroup.import_handle: a handle is 64 bytes")
        _lib.check(_lib.load().nvx_peer_import(self.comm, peer_rank, handle), "nvx_peer_import")

    def status(self) -> int:
        """0, or 1 once a wait inside an exchange ran out (a peer died or fell behind by more than the time-out)."""
        return int(_lib.load().nvx_peer_status(self.comm)) if self.comm else -1

    def close(self):
        if self.comm:
            PeerGroup._registry.pop(self.comm, None)
            _lib.check(_lib.load().nvx_peer_destroy(self.comm), "nvx_peer_destroy")
            self.comm = None

    # Every rank writes its whole tensor to every peer (one hop, no second exchange): the latency of one posted write,
    # but (tp - 1) x rows x hidden x 4 bytes leave each GPU (2 bytes of tag beside every 2 bytes of data), against
    # 2 x (tp - 1) / tp x rows x hidden x 2 for a reduce-scatter + all-gather.  Past a few MiB per exchange the links'
    # time outweighs the saved hops and launches, and the library's bandwidth-oriented all-reduce takes over.
    # This is a ROUTING policy (`prefer`), not a limit of the kernel (`accepts`); the ranks of a group must route alike,
    # so distributed.init_peer_allreduce agrees on one value for all of them (`max_push_bytes`).
    MAX_PUSH_BYTES = int(__import__("os").environ.get("NVX_PEER_MAX_PUSH_BYTES", str(4 << 20)))

    @staticmethod
    def rows_within_push_cap(tp_size: int, hidden: int, max_push_bytes: int) -> int:
        """Most rows of one exchange whose pushes stay within `max_push_bytes` per GPU (at least one)."""
        return max(1, max_push_bytes // (max(tp_size - 1, 1) * hidden * 4))

    max_push_bytes = MAX_PUSH_BYTES

    def accepts(self, x) -> bool:
        """What the kernel can take at all: the group's row width and format, at most the rows its landing buffer holds."""
        return self.comm is not None and x.dim() == 2 and x.shape[0] <= self.max_rows and x.shape[1] == self.hidden and x.dtype in H16 \
            and x.stride(1) == 1

    def prefer(self, x) -> bool:
        """Whether this exchange should go peer to peer rather than through the library all-reduce."""
        return self.accepts(x) and (self.tp_size - 1) * x.shape[0] * self.hidden * 4 <= self.max_push_bytes

    fits = prefer     # (older name)


def peer_allreduce_norm(group: PeerGroup, x, weight=None, eps: float = 0.0, residual=None):
    """Sum of the ranks' `x` (rows, hidden), rounded to the 16-bit format; then, with `weight`, RMSNorm of it (of it plus
    `residual`).  Returns the sum written over `x` (weight None), y, or (y, new_residual).  Every rank of the group
    must make the same calls in the same order."""
    _dev(x, weight, residual)
    _need(group.accepts(x), f"peer_allreduce_norm: x {tuple(x.shape)} {x.dtype} does not fit the group ({group.max_rows} rows x {group.hidden})")
    rows, hidden = x.shape
    lib = _lib.load()
    if weight is None:
        _need(residual is None, "peer_allreduce_norm: a residual needs the norm")
        _need(x.stride(0) == hidden, "peer_allreduce_norm: the in-place sum needs contiguous rows")
        _lib.check(_fn(lib, "nvx_peer_allreduce_norm", x.dtype)(group.comm, _ptr(x), x.stride(0), None, None, _ptr(x), None, rows, hidden, 0.0,
                                                                 _stream()), "nvx_peer_allreduce_norm")
        return x
    _need(weight.dtype == x.dtype and weight.is_contiguous() and weight.numel() == hidden, "peer_allreduce_norm: weight")
    y = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    res_out = None
    if residual is not None:
        _need(residual.dtype == x.dtype and residual.is_contiguous() and residual.shape == (rows, hidden), "peer_allreduce_norm: residual")
        res_out = torch.empty_like(residual)
    _lib.check(_fn(lib, "nvx_peer_allreduce_norm", x.dtype)(group.comm, _ptr(x), x.stride(0), _ptr(residual), _ptr(weight), _ptr(y), _ptr(res_out),
                                                             rows, hidden, float(eps), _stream()), "nvx_peer_allreduce_norm")
    return y if residual is None else (y, res_out)


# ---------------------------------------------------------------------------------------------
# layers with a float32 residual stream, per-sequence state and latent attention
# ---------------------------------------------------------------------------------------------
F32 = torch.float32
_FMT = {BF16: 0, F16: 1, F32: 2}


def _fmt(t) -> int:
    _need(t.dtype in _FMT, "activations must be bfloat16, float16 or float32")
    return _FMT[t.dtype]


def _f32c(t, what: str):
    _need(t.dtype == F32 and t.is_contiguous(), f"{what} must be contiguous float32")


class StepLayout:
    """Where the tokens of a step belong: `qo_indptr` (int32, B+1) and `tok_seq` (int32, T) give each token its sequence
    (both None: one token per sequence, a decode step), `pos0` (int64, B) the position of each sequence's first token of
    the step, `state_slot` (int32, B) its slot in the state tensors (negative: a padding row)."""

    def __init__(self, n_tok: int, n_seq: int, pos0, state_slot, qo_indptr=None, tok_seq=None, max_q=None):
        _dev(pos0, state_slot, qo_indptr, tok_seq)
        _need(pos0.dtype == torch.int64 and pos0.is_contiguous() and pos0.numel() >= n_seq, "StepLayout: pos0 must be int64 (B)")
        _need(state_slot.dtype == torch.int32 and state_slot.is_contiguous() and state_slot.numel() >= n_seq,
              "StepLayout: state_slot must be int32 (B)")
        _need((qo_indptr is None) == (tok_seq is None), "StepLayout: qo_indptr and tok_seq go together")
        if qo_indptr is None:
            _need(n_tok == n_seq, "StepLayout: without qo_indptr every sequence has one token")
        else:
            _need(qo_indptr.dtype == torch.int32 and qo_indptr.is_contiguous() and qo_indptr.numel() == n_seq + 1, "StepLayout: qo_indptr")
            _need(tok_seq.dtype == torch.int32 and tok_seq.is_contiguous() and tok_seq.numel() == n_tok, "StepLayout: tok_seq")
        self.n_tok, self.n_seq = n_tok, n_seq
        self.pos0, self.state_slot, self.qo_indptr, self.tok_seq = pos0, state_slot, qo_indptr, tok_seq
        # tokens of the step's longest portion, where the host knows it (it sizes launches that cut portions into chunks); else n_tok bounds it
        self.max_q = int(max_q) if max_q else n_tok


def boundary_canon_fits(width: int) -> bool:
    """Whether boundary_norm can apply the convolution of a decode step in the same launch for rows of this width."""
    return width % 4 == 0 and width <= 8192


def boundary_norm(m, w_post, eps: float, res=None, hist=None, hist_slot: int = -1, mix=None, w_pre=None, pre_f32: bool = True,
                  x_out=None, canon=None):
    """Post-norm of a sublayer's output `m` (T, width) + residual `res` (float32) [+ weighted sum `mix` over the results
    kept in `hist` (slots, T, width), this one stored at `hist_slot`] [+ pre-norm `w_pre` of what follows].  Both norms
    are RMS norms whose stored weight is the deviation from one.  Returns (x, y): the new stream (float32) and the
    pre-normed rows (float32 if `pre_f32`, else in m's format; None without `w_pre`).
    `canon` = (taps, state, layout), for a step with one token per sequence: the convolution of canon_conv is applied to
    the pre-normed rows in the same launch (state read and shifted); y is then its result, in m's format."""
    _dev(m, w_post, res, hist, mix, w_pre)
    _need(m.dim() == 2 and m.stride(1) == 1, "boundary_norm: m must be (T, width) with unit inner stride")
    t, width = m.shape
    _f32c(w_post, "boundary_norm: w_post")
    _need(w_post.numel() == width, "boundary_norm: w_post size")
    if res is not None:
        _f32c(res, "boundary_norm: res")
        _need(res.shape == (t, width), "boundary_norm: res shape")
    n_mix, hist_stride = 0, 0
    if hist is not None:
        _f32c(hist, "boundary_norm: hist")
        _need(hist.dim() == 3 and hist.shape[1:] == (t, width) and 0 <= hist_slot < hist.shape[0], "boundary_norm: hist shape / slot")
        hist_stride = hist.stride(0)
        if mix is not None:
            _f32c(mix, "boundary_norm: mix")
            n_mix = mix.numel()
            _need(hist_slot < n_mix <= hist.shape[0], "boundary_norm: mix longer than the history, or without this result")
    else:
        _need(mix is None and hist_slot < 0, "boundary_norm: mix / hist_slot need hist")
    if x_out is None:
        x_out = torch.empty((t, width), dtype=F32, device=m.device)
    else:
        _f32c(x_out, "boundary_norm: x_out")
        _need(x_out.shape == (t, width), "boundary_norm: x_out shape")
    y = None
    taps = state = pos0 = state_slot = None
    taps_n = n_slots = 0
    if canon is not None:
        taps, state, layout = canon
        _need(w_pre is not None and layout.qo_indptr is None and layout.n_tok == t and boundary_canon_fits(width),
              "boundary_norm: the fused convolution is for one token per sequence, a pre-norm, and a width that fits")
        _dev(taps, state)
        _f32c(taps, "boundary_norm: taps")
        taps_n = taps.shape[0]
        _need(taps.dim() == 2 and taps.shape[1] == width, "boundary_norm: taps shape")
        if taps_n > 1:
            _f32c(state, "boundary_norm: state")
            _need(state.dim() == 3 and state.shape[1:] == (taps_n - 1, width), "boundary_norm: state shape")
            n_slots = state.shape[0]
        else:
            state = None
        pos0, state_slot, pre_f32 = layout.pos0, layout.state_slot, False
    if w_pre is not None:
        _f32c(w_pre, "boundary_norm: w_pre")
        _need(w_pre.numel() == width, "boundary_norm: w_pre size")
        y = torch.empty((t, width), dtype=F32 if pre_f32 else m.dtype, device=m.device)
    lib = _lib.load()
    _lib.check(lib.nvx_boundary_norm(_ptr(m), m.stride(0), _fmt(m), _ptr(res), _ptr(w_post), _ptr(hist), hist_stride, hist_slot, n_mix,
                                     _ptr(mix), _ptr(x_out), _ptr(w_pre), _ptr(y) if (y is not None and pre_f32) else None,
                                     _ptr(y) if (y is not None and not pre_f32) else None, t, width, float(eps), _ptr(taps), taps_n,
                                     _ptr(state), n_slots, _ptr(pos0), _ptr(state_slot), _stream()),
               "nvx_boundary_norm")
    return x_out, y


def canon_conv(h, taps, state, layout: StepLayout, dtype):
    """h + causal convolution over time per channel.  h (T, width) float32; taps (taps_n, width) float32, row j multiplying
    the input taps_n - 1 - j tokens back; state
    (slots, taps_n - 1, width) float32, read for the inputs before this step and replaced by each sequence's last ones.
    Returns (T, width) in `dtype`."""
    _dev(h, taps, state)
    _f32c(h, "canon_conv: h")
    _f32c(taps, "canon_conv: taps")
    t, width = h.shape
    taps_n = taps.shape[0]
    _need(t == layout.n_tok and taps.dim() == 2 and taps.shape[1] == width, "canon_conv: shapes")
    n_slots = 0
    if taps_n > 1:
        _f32c(state, "canon_conv: state")
        _need(state.dim() == 3 and state.shape[1:] == (taps_n - 1, width), "canon_conv: state shape")
        n_slots = state.shape[0]
    out = torch.empty((t, width), dtype=dtype, device=h.device)
    lib = _lib.load()
    _lib.check(lib.nvx_canon_conv(_ptr(h), _ptr(taps), taps_n, _ptr(state) if taps_n > 1 else None, n_slots, _ptr(layout.tok_seq),
                                  _ptr(layout.qo_indptr), _ptr(layout.pos0), _ptr(layout.state_slot), _ptr(out), _fmt(out), t,
                                  layout.n_seq, width, _stream()), "nvx_canon_conv")
    return out


def relu2(x):
    """max(x, 0)^2."""
    _dev(x)
    x = x.contiguous()
    y = torch.empty_like(x)
    lib = _lib.load()
    _lib.check(lib.nvx_relu2(_ptr(x), _ptr(y), _fmt(x), x.numel(), _stream()), "nvx_relu2")
    return y


def mingru_scan(zxg, state, layout: StepLayout):
    """Gated recurrence over each sequence's tokens.  zxg (T, 3 * width): update-gate, candidate and output-gate
    pre-activations; state (slots, width) float32, continued and written back.  Returns S * silu(g), (T, width)."""
    _dev(zxg, state)
    _need(zxg.dim() == 2 and zxg.stride(1) == 1 and zxg.shape[1] % 3 == 0, "mingru_scan: zxg must be (T, 3 * width)")
    t, width = zxg.shape[0], zxg.shape[1] // 3
    _f32c(state, "mingru_scan: state")
    _need(t == layout.n_tok and state.dim() == 2 and state.shape[1] == width, "mingru_scan: shapes")
    out = torch.empty((t, width), dtype=zxg.dtype, device=zxg.device)
    lib = _lib.load()
    _lib.check(lib.nvx_mingru_scan(_ptr(zxg), zxg.stride(0), _fmt(zxg), _ptr(state), state.shape[0], _ptr(layout.qo_indptr),
                                   _ptr(layout.pos0), _ptr(layout.state_slot), _ptr(out), t, layout.n_seq, width, _stream()),
               "nvx_mingru_scan")
    return out


def latent_prep(x, w_q, w_kv, eps: float, slots, cache, heads: int):
    """After the down projections of latent attention: x (T, q_rank + kv_rank + heads).  Returns (cq, gate): the
    RMS-normed query latent (T, q_rank) in x's format and sigmoid of the per-head gates (T, heads) float32; the RMS-normed
    key/value latent of token t is stored at cache[slots[t]] (cache: (slots, kv_rank) in x's format)."""
    _dev(x, w_q, w_kv, slots, cache)
    _f32c(w_q, "latent_prep: w_q")
    _f32c(w_kv, "latent_prep: w_kv")
    q_rank, kv_rank = w_q.numel(), w_kv.numel()
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] == q_rank + kv_rank + heads, "latent_prep: x shape")
    t = x.shape[0]
    _need(cache.dtype == x.dtype and cache.is_contiguous() and cache.dim() == 2 and cache.shape[1] == kv_rank, "latent_prep: cache")
    _need(slots.dtype == torch.int64 and slots.is_contiguous() and slots.numel() == t, "latent_prep: slots must be int64 (T)")
    cq = torch.empty((t, q_rank), dtype=x.dtype, device=x.device)
    gate = torch.empty((t, heads), dtype=F32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_latent_prep(_ptr(x), x.stride(0), _fmt(x), _ptr(w_q), _ptr(w_kv), float(eps), _ptr(slots), _ptr(cq), _ptr(cache),
                                   cache.shape[0], _ptr(gate), t, q_rank, kv_rank, heads, _stream()), "nvx_latent_prep")
    return cq, gate


def latent_attn(q, cache, kv_indices, kv_start, kv_len, layout: StepLayout, scale: float, gate=None):
    """Attention over cached latents: q (heads, T, rank) folded queries, cache (slots, rank).  Sequence b's tokens are
    at slots kv_indices[kv_start[b] : kv_start[b] + kv_len[b]]; causal.  Returns (heads, T, rank) in q's format, each
    head's rows multiplied by gate[t][h] if given."""
    _dev(q, cache, kv_indices, kv_start, kv_len, gate)
    _need(q.dim() == 3 and q.is_contiguous(), "latent_attn: q must be contiguous (heads, T, rank)")
    heads, t, rank = q.shape
    _need(t == layout.n_tok, "latent_attn: token count")
    _need(cache.dtype == q.dtype and cache.is_contiguous() and cache.dim() == 2 and cache.shape[1] == rank, "latent_attn: cache")
    _need(kv_indices.dtype == torch.int32 and kv_indices.is_contiguous(), "latent_attn: kv_indices must be int32")
    _need(kv_start.dtype == torch.int64 and kv_start.numel() >= layout.n_seq, "latent_attn: kv_start must be int64 (B)")
    _need(kv_len.dtype == torch.int32 and kv_len.numel() >= layout.n_seq, "latent_attn: kv_len must be int32 (B)")
    if gate is not None:
        _f32c(gate, "latent_attn: gate")
        _need(gate.shape == (t, heads), "latent_attn: gate shape")
    out = torch.empty_like(q)
    lib = _lib.load()
    _lib.check(lib.nvx_latent_attn(_ptr(q), _ptr(cache), _fmt(q), _ptr(kv_indices), _ptr(kv_start), _ptr(kv_len), _ptr(layout.qo_indptr),
                                   _ptr(layout.tok_seq), _ptr(gate), _ptr(out), heads, rank, t, float(scale), _stream()), "nvx_latent_attn")
    return out


# ---------------------------------------------------------------------------------------------
# gated residuals with grouped norms, matrix-memory recurrences, capped attention, mixtures of experts
# ---------------------------------------------------------------------------------------------
def gated_residual_norm(x, y=None, gate=None, gate_bias=None, mult: float = 1.0, w_norm=None, groups: int = 1, eps: float = 0.0,
                        y2=None, w_y=None, w_y2=None, dtype=None):
    """x (T, width) float32, updated in place: x += mult * r with r = y, or the mean of y and y2 after each was divided by its
    root mean square and multiplied by w_y / w_y2; r passes sigmoid(gate + gate_bias) first if a gate is given.  With
    `w_norm`, returns the grouped RMS norm of the new x (each of `groups` slices of a row by its own root mean square) times
    w_norm, in `dtype` (default: y's)."""
    _dev(x, y, gate, gate_bias, w_norm, y2, w_y, w_y2)
    _f32c(x, "gated_residual_norm: x")
    _need(x.dim() == 2, "gated_residual_norm: x must be (T, width)")
    t, width = x.shape
    for name, a in (("y", y), ("y2", y2), ("gate", gate)):
        if a is not None:
            _need(a.shape == (t, width) and a.stride(1) == 1, f"gated_residual_norm: {name} must be (T, width) with unit inner stride")
    acts = [a for a in (y, y2, gate) if a is not None]
    dtype = dtype or (acts[0].dtype if acts else None)
    _need(dtype in _FMT and all(a.dtype == dtype for a in acts), "gated_residual_norm: y, y2, gate and the output share one format")
    for name, a in (("gate_bias", gate_bias), ("w_norm", w_norm), ("w_y", w_y), ("w_y2", w_y2)):
        if a is not None:
            _f32c(a, "gated_residual_norm: " + name)
            _need(a.numel() == width, f"gated_residual_norm: {name} size")
    _need(width % groups == 0, "gated_residual_norm: the width must be a multiple of the groups")
    h = torch.empty((t, width), dtype=dtype, device=x.device) if w_norm is not None else None
    lib = _lib.load()
    _lib.check(lib.nvx_gated_residual_norm(_ptr(y), y.stride(0) if y is not None else 0, _ptr(y2), y2.stride(0) if y2 is not None else 0,
                                           _ptr(w_y), _ptr(w_y2), _ptr(gate), gate.stride(0) if gate is not None else 0, _ptr(gate_bias),
                                           _FMT[dtype], float(mult), _ptr(x), _ptr(w_norm), groups, float(eps), _ptr(h), t, width, _stream()),
               "nvx_gated_residual_norm")
    return h


def head_norm_gate(o, w, eps: float, gate=None, kind: str = "none", dtype=None):
    """o (T, heads, vdim) float32: every head's row divided by its root mean square, times w ((heads, vdim), or (vdim,) shared
    by the heads), times the output gate: kind "sigmoid" or "silu" of `gate` (T, heads * vdim).  Returns (T, heads * vdim)."""
    _dev(o, w, gate)
    _f32c(o, "head_norm_gate: o")
    _f32c(w, "head_norm_gate: w")
    _need(o.dim() == 3, "head_norm_gate: o must be (T, heads, vdim)")
    t, heads, vdim = o.shape
    _need(w.numel() in (vdim, heads * vdim), "head_norm_gate: w size")
    k = {"none": 0, "sigmoid": 1, "silu": 2}[kind]
    if k:
        _need(gate is not None and gate.shape == (t, heads * vdim) and gate.stride(1) == 1, "head_norm_gate: gate shape")
        dtype = dtype or gate.dtype
        _need(gate.dtype == dtype, "head_norm_gate: gate format")
    _need(dtype in _FMT, "head_norm_gate: output format")
    out = torch.empty((t, heads * vdim), dtype=dtype, device=o.device)
    lib = _lib.load()
    _lib.check(lib.nvx_head_norm_gate(_ptr(o), _ptr(w), int(w.numel() == vdim), _ptr(gate) if k else None,
                                      gate.stride(0) if k else 0, k, _FMT[dtype], float(eps), _ptr(out), t, heads, vdim, _stream()),
               "nvx_head_norm_gate")
    return out


def _layout_args(layout: StepLayout):
    return _ptr(layout.qo_indptr), _ptr(layout.pos0), _ptr(layout.state_slot)


def short_conv_silu(x, w, state, layout: StepLayout):
    """silu of a causal convolution over time per channel.  x (T, channels) (rows may be a slice of wider rows); w (taps,
    channels) float32, row j multiplying the input taps - 1 - j tokens back; state (slots, taps - 1, channels) float32, read for
    the inputs before this step and replaced by each sequence's last ones.  Returns (T, channels) in x's format."""
    _dev(x, w, state)
    _need(x.dim() == 2 and x.stride(1) == 1, "short_conv_silu: x must be (T, channels) with unit inner stride")
    t, ch = x.shape
    _f32c(w, "short_conv_silu: w")
    taps = w.shape[0]
    _need(w.dim() == 2 and w.shape[1] == ch and t == layout.n_tok, "short_conv_silu: shapes")
    n_slots = 0
    if taps > 1:
        _f32c(state, "short_conv_silu: state")
        _need(state.dim() == 3 and state.shape[1:] == (taps - 1, ch), "short_conv_silu: state shape")
        n_slots = state.shape[0]
    out = torch.empty((t, ch), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_short_conv_silu(_ptr(x), x.stride(0), _fmt(x), _ptr(w), taps, _ptr(state) if taps > 1 else None, n_slots,
                                       _ptr(layout.tok_seq), *_layout_args(layout), _ptr(out), t, layout.n_seq, ch, _stream()),
               "nvx_short_conv_silu")
    return out


def token_shift_mix(h, mu, state, layout: StepLayout):
    """out[m] = h + (previous token's h - h) * mu[m].  h (T, width); mu (n_mix, width) float32; state (slots, width) float32:
    the row before each sequence's first token of this step (zeros at position 0), replaced by its last row.
    Returns (n_mix, T, width) in h's format."""
    _dev(h, mu, state)
    _need(h.dim() == 2 and h.stride(1) == 1, "token_shift_mix: h must be (T, width) with unit inner stride")
    t, width = h.shape
    _f32c(mu, "token_shift_mix: mu")
    _f32c(state, "token_shift_mix: state")
    _need(mu.dim() == 2 and mu.shape[1] == width and state.dim() == 2 and state.shape[1] == width and t == layout.n_tok, "token_shift_mix: shapes")
    out = torch.empty((mu.shape[0], t, width), dtype=h.dtype, device=h.device)
    lib = _lib.load()
    _lib.check(lib.nvx_token_shift_mix(_ptr(h), h.stride(0), _fmt(h), _ptr(mu), mu.shape[0], _ptr(state), state.shape[0], _ptr(layout.tok_seq),
                                       *_layout_args(layout), _ptr(out), t, layout.n_seq, width, _stream()), "nvx_token_shift_mix")
    return out


def mlstm_scan(x, offsets, gates, gate_bias, cap: float, mem, norm, peak, layout: StepLayout, heads: int, dim: int, vdim: int):
    """Matrix memory with a stabilised exponential input gate.  x (T, >= ...): q, k (heads * dim each) and v (heads * vdim) at the
    three column `offsets`; gates (T, 2 * heads) float32 = input | forget pre-activations, gate_bias (2 * heads); mem (slots,
    heads, dim, vdim), norm (slots, heads, dim), peak (slots, heads) float32, continued and written back.
    Returns the read-out (T, heads, vdim) float32."""
    _dev(x, gates, gate_bias, mem, norm, peak)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[0] == layout.n_tok, "mlstm_scan: x must be (T, columns) with unit inner stride")
    t = x.shape[0]
    for a, what in ((gates, "gates"), (gate_bias, "gate_bias"), (mem, "mem"), (norm, "norm"), (peak, "peak")):
        _f32c(a, "mlstm_scan: " + what)
    _need(gates.shape == (t, 2 * heads) and gate_bias.numel() == 2 * heads, "mlstm_scan: gate shapes")
    n_slots = mem.shape[0]
    _need(mem.shape == (n_slots, heads, dim, vdim) and norm.shape == (n_slots, heads, dim) and peak.shape == (n_slots, heads), "mlstm_scan: state shapes")
    out = torch.empty((t, heads, vdim), dtype=F32, device=x.device)
    lib = _lib.load()
    # a head whose value columns take several workgroups: all of them read the normaliser and the maximum, the first writes them
    # back, so they read from copies (a workgroup that starts late must not see the new values)
    several = lib.nvx_scan_column_blocks(dim, vdim) != 1
    norm_in, peak_in = (norm.clone(), peak.clone()) if several else (norm, peak)
    _lib.check(lib.nvx_mlstm_scan(_ptr(x), x.stride(0), _fmt(x), offsets[0], offsets[1], offsets[2], _ptr(gates), _ptr(gate_bias), float(cap),
                                  _ptr(mem), _ptr(norm_in), _ptr(peak_in), _ptr(norm), _ptr(peak), n_slots, *_layout_args(layout), _ptr(out), t, layout.n_seq, heads, dim, vdim,
                                  _stream()), "nvx_mlstm_scan")
    return out


def delta_scan(x, offsets, ab, a_log, dt_bias, mem, layout: StepLayout, heads: int, kv_heads: int, dim: int, vdim: int):
    """Gated delta rule.  x (T, columns): q, k (kv_heads * dim each) and v (heads * vdim) at the three column `offsets`, after
    their convolution; ab (T, 2 * heads) float32 = decay | write-strength pre-activations; a_log, dt_bias (heads); mem (slots,
    heads, dim, vdim) float32.  Returns the read-out (T, heads, vdim) float32."""
    _dev(x, ab, a_log, dt_bias, mem)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[0] == layout.n_tok, "delta_scan: x must be (T, columns) with unit inner stride")
    t = x.shape[0]
    for a, what in ((ab, "ab"), (a_log, "a_log"), (dt_bias, "dt_bias"), (mem, "mem")):
        _f32c(a, "delta_scan: " + what)
    _need(ab.shape == (t, 2 * heads) and a_log.numel() == heads and dt_bias.numel() == heads, "delta_scan: gate shapes")
    n_slots = mem.shape[0]
    _need(mem.shape == (n_slots, heads, dim, vdim), "delta_scan: state shape")
    out = torch.empty((t, heads, vdim), dtype=F32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_delta_scan(_ptr(x), x.stride(0), _fmt(x), offsets[0], offsets[1], offsets[2], _ptr(ab), _ptr(a_log), _ptr(dt_bias),
                                  _ptr(mem), n_slots, *_layout_args(layout), _ptr(out), t, layout.n_seq, heads, kv_heads, dim, vdim, _stream()),
               "nvx_delta_scan")
    return out


def rwkv_scan(r, k, v, wlog, w0, bonus, mem, layout: StepLayout, heads: int, dim: int):
    """Decayed outer-product memory read with a bonus for the current token.  r, k, v (T, heads * dim) with one common row
    stride; wlog (T, heads * dim) float32 and w0 (heads * dim): decay exp(-exp(wlog + w0)); bonus (heads, dim); mem (slots,
    heads, dim, dim) float32.  Returns the read-out (T, heads, dim) float32."""
    _dev(r, k, v, wlog, w0, bonus, mem)
    t = r.shape[0]
    for a in (r, k, v):
        _need(a.shape == (t, heads * dim) and a.stride(1) == 1 and a.stride(0) == r.stride(0) and a.dtype == r.dtype, "rwkv_scan: r, k, v shapes")
    for a, what in ((wlog, "wlog"), (w0, "w0"), (bonus, "bonus"), (mem, "mem")):
        _f32c(a, "rwkv_scan: " + what)
    n_slots = mem.shape[0]
    _need(t == layout.n_tok and wlog.shape == (t, heads * dim) and w0.numel() == heads * dim and bonus.numel() == heads * dim and
          mem.shape == (n_slots, heads, dim, dim), "rwkv_scan: shapes")
    out = torch.empty((t, heads, dim), dtype=F32, device=r.device)
    lib = _lib.load()
    _lib.check(lib.nvx_rwkv_scan(_ptr(r), _ptr(k), _ptr(v), r.stride(0), _fmt(r), _ptr(wlog), _ptr(w0), _ptr(bonus), _ptr(mem), n_slots,
                                 *_layout_args(layout), _ptr(out), t, layout.n_seq, heads, dim, _stream()), "nvx_rwkv_scan")
    return out


def rope_vnorm_store(qkv, positions, freq, mag: float, rot_dims: int, eps: float, slots, k_cache, v_cache, heads: int, kv_heads: int,
                     dim: int, vdim: int):
    """After the fused projection qkv (T, heads * dim + kv_heads * (dim + vdim)): rotate the first rot_dims of every query and
    key head by positions * freq (freq: rot_dims / 2 float64; cos and sin times `mag`), divide every value head by its root
    mean square, store keys and values at k_cache[slots] / v_cache[slots] ((slots, kv_heads * dim) / (slots, kv_heads * vdim), in
    qkv's format).  Returns the rotated queries (T, heads * dim)."""
    _dev(qkv, positions, freq, slots, k_cache, v_cache)
    t = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == heads * dim + kv_heads * (dim + vdim), "rope_vnorm_store: qkv shape")
    _need(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == t, "rope_vnorm_store: positions must be int64 (T)")
    _need(slots.dtype == torch.int64 and slots.is_contiguous() and slots.numel() == t, "rope_vnorm_store: slots must be int64 (T)")
    _need(rot_dims == 0 or (freq.dtype == torch.float64 and freq.is_contiguous() and freq.numel() == rot_dims // 2), "rope_vnorm_store: freq must be float64 (rot_dims / 2)")
    n_slots = k_cache.shape[0]
    _need(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          k_cache.shape == (n_slots, kv_heads * dim) and v_cache.shape == (n_slots, kv_heads * vdim), "rope_vnorm_store: cache shapes")
    q = torch.empty((t, heads * dim), dtype=qkv.dtype, device=qkv.device)
    lib = _lib.load()
    _lib.check(lib.nvx_rope_vnorm_store(_ptr(qkv), qkv.stride(0), _fmt(qkv), _ptr(positions), _ptr(freq) if rot_dims else None, float(mag), rot_dims,
                                        float(eps), _ptr(slots), _ptr(q), _ptr(k_cache), _ptr(v_cache), n_slots, t, heads, kv_heads, dim, vdim,
                                        _stream()), "nvx_rope_vnorm_store")
    return q


SOFTCAP_SPLIT_BELOW = 1024      # (token, head) pairs of a step below which the keys are split over workgroups too
SOFTCAP_SPLITS = 4


def softcap_attn(q, k_cache, v_cache, kv_indices, kv_start, kv_len, layout: StepLayout, scale: float, cap: float, heads: int,
                 kv_heads: int, dim: int, vdim: int, n_split: Optional[int] = None, window: int = 0, r1=None, r2=None, v_turn=None,
                 v_interleaved: bool = False, gate=None, matrix_cores: bool = True, sink_score: Optional[float] = None):
    """Causal attention of q (T, heads * dim) over cached rows: sequence b's tokens are at slots kv_indices[kv_start[b] :
    kv_start[b] + kv_len[b]]; scores scale * q . k pass cap * tanh(. / cap) (cap <= 0: not) before the softmax.
    `window` > 0: a token sees itself and the window - 1 tokens before it.  `r1`, `r2` (heads, float32): r1 ln(1 + r2 (i - j)) is
    taken off the score of key j for the query at position i.  `v_turn` (T, vdim) float32, every query token's cos | sin as
    attn_prep_store returns them: the read-out's pairs ((m, m + vdim / 2), or (2m, 2m + 1) if `v_interleaved`) are turned back by
    those angles, undoing the turn attn_prep_store gave the values.  `gate`
    (T, heads * vdim), or (T, heads) with one number per head: the read-out times sigmoid(gate).  `sink_score`: the softmax's sum has
    one more term exp(sink_score) that carries no value (0.0: one is added to the denominator).  Steps of many tokens in a 16-bit format, with key and value sizes of 64,
    96 or 128, run on the matrix cores unless `matrix_cores` is False.  Returns (T, heads * vdim) in q's format."""
    _dev(q, k_cache, v_cache, kv_indices, kv_start, kv_len, r1, r2, v_turn, gate)
    _need((r1 is None) == (r2 is None), "softcap_attn: r1 and r2 go together")
    for a in (r1, r2):
        if a is not None:
            _f32c(a, "softcap_attn: r1, r2")
            _need(a.numel() == heads, "softcap_attn: r1 and r2 have one number per head")
    _need(v_turn is None or (v_turn.dtype == F32 and v_turn.is_contiguous() and v_turn.shape == (q.shape[0], vdim) and vdim % 2 == 0),
          "softcap_attn: v_turn must be float32 (T, vdim)")
    _need(gate is None or (gate.dim() == 2 and gate.shape[0] == q.shape[0] and gate.shape[1] in (heads, heads * vdim) and gate.stride(1) == 1 and
                           gate.dtype == q.dtype), "softcap_attn: gate shape / format")
    gate_per_head = gate is not None and gate.shape[1] == heads and vdim != 1
    t = q.shape[0]
    _need(q.shape == (t, heads * dim) and q.is_contiguous() and t == layout.n_tok, "softcap_attn: q must be contiguous (T, heads * dim)")
    n_slots = k_cache.shape[0]
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
          k_cache.shape == (n_slots, kv_heads * dim) and v_cache.shape == (n_slots, kv_heads * vdim), "softcap_attn: cache shapes")
    _need(kv_indices.dtype == torch.int32 and kv_indices.is_contiguous(), "softcap_attn: kv_indices must be int32")
    _need(kv_start.dtype == torch.int64 and kv_start.numel() >= layout.n_seq, "softcap_attn: kv_start must be int64 (B)")
    _need(kv_len.dtype == torch.int32 and kv_len.numel() >= layout.n_seq, "softcap_attn: kv_len must be int32 (B)")
    out = torch.empty((t, heads * vdim), dtype=q.dtype, device=q.device)
    # a step of few tokens is few workgroups, each walking all of its sequence's keys: their keys are dealt out over several
    # workgroups whose partial results a second launch merges (the choice depends on the step's shape only, never on its data)
    if n_split is None:
        n_split = SOFTCAP_SPLITS if t * heads < SOFTCAP_SPLIT_BELOW else 1
    part = torch.empty((t * heads * n_split * (vdim + 2),), dtype=F32, device=q.device) if n_split > 1 else None
    lib = _lib.load()
    _lib.check(lib.nvx_softcap_attn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _fmt(q), _ptr(kv_indices), _ptr(kv_start), _ptr(kv_len),
                                    _ptr(layout.qo_indptr), _ptr(layout.tok_seq), float(scale), float(cap), _ptr(out), t, heads, kv_heads, dim,
                                    vdim, n_split, _ptr(part), int(window or 0), _ptr(r1), _ptr(r2), _ptr(v_turn), int(bool(v_interleaved)),
                                    _ptr(gate), gate.stride(0) if gate is not None else 0, int(gate_per_head), int(sink_score is not None),
                                    float(sink_score or 0.0), layout.n_seq, int(bool(matrix_cores)), _stream()),
               "nvx_softcap_attn")
    return out


def attn_prep_store(x, offsets, positions, q_w, k_w, norm_mode: str, eps: float, freq, rot_dims: int, interleaved: bool, vfreq, slots,
                    k_cache, v_cache, heads: int, kv_heads: int, dim: int, vdim: int):
    """After a fused projection x (T, columns) holding q, k, v at the three column `offsets`: RMS norm of q and k (`norm_mode`
    "head": every head by itself, weights q_w / k_w of `dim` entries shared by the heads; "row": all heads of a token at once,
    weights of heads * dim / kv_heads * dim entries; "none"), rotation of the first rot_dims of every q and k head by positions *
    freq (float64, rot_dims / 2; pairs (m, m + rot_dims / 2), or (2m, 2m + 1) if `interleaved`), rotation of every value head over
    all of vdim by positions * vfreq if vfreq is given, keys and values stored at k_cache[slots] / v_cache[slots].  With kv_heads
    == 0 only the queries are prepared (k_w, slots and the caches may be None).  Returns (queries (T, heads * dim), v_turn): v_turn
    (T, vdim) float32 holds every token's cos | sin of its value rotation (None without vfreq), for softcap_attn to turn back with."""
    _dev(x, positions, q_w, k_w, freq, vfreq, slots, k_cache, v_cache)
    t = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1, "attn_prep_store: x must be (T, columns) with unit inner stride")
    _need(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == t, "attn_prep_store: positions must be int64 (T)")
    mode = {"none": 0, "head": 1, "row": 2}[norm_mode]
    if mode:
        _f32c(q_w, "attn_prep_store: q_w")
        _need(q_w.numel() == (dim if mode == 1 else heads * dim), "attn_prep_store: q_w size")
        if kv_heads:
            _f32c(k_w, "attn_prep_store: k_w")
            _need(k_w.numel() == (dim if mode == 1 else kv_heads * dim), "attn_prep_store: k_w size")
    _need(rot_dims == 0 or (freq.dtype == torch.float64 and freq.is_contiguous() and freq.numel() == rot_dims // 2), "attn_prep_store: freq must be float64 (rot_dims / 2)")
    _need(vfreq is None or (vfreq.dtype == torch.float64 and vfreq.is_contiguous() and vfreq.numel() == vdim // 2 and vdim % 2 == 0),
          "attn_prep_store: vfreq must be float64 (vdim / 2)")
    n_slots = 0
    if kv_heads:
        _need(slots.dtype == torch.int64 and slots.is_contiguous() and slots.numel() == t, "attn_prep_store: slots must be int64 (T)")
        n_slots = k_cache.shape[0]
        _need(k_cache.dtype == x.dtype and v_cache.dtype == x.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
              k_cache.shape == (n_slots, kv_heads * dim) and v_cache.shape == (n_slots, kv_heads * vdim), "attn_prep_store: cache shapes")
    q = torch.empty((t, heads * dim), dtype=x.dtype, device=x.device)
    v_turn = torch.empty((t, vdim), dtype=F32, device=x.device) if vfreq is not None else None
    lib = _lib.load()
    _lib.check(lib.nvx_attn_prep_store(_ptr(x), x.stride(0), _fmt(x), offsets[0], offsets[1], offsets[2], _ptr(positions), _ptr(q_w) if mode else None,
                                       _ptr(k_w) if mode and kv_heads else None, mode, float(eps), _ptr(freq) if rot_dims else None, rot_dims,
                                       int(bool(interleaved)), _ptr(vfreq), _ptr(slots) if kv_heads else None, _ptr(q),
                                       _ptr(k_cache) if kv_heads else None, _ptr(v_cache) if kv_heads else None, n_slots, t, heads, kv_heads, dim,
                                       vdim, _ptr(v_turn), _stream()), "nvx_attn_prep_store")
    return q, v_turn


DECAY_SCAN_CHUNK_FROM = 256       # portions from this length on are cut into chunks that run side by side
DECAY_SCAN_CHUNKS = ((65536, 32), (131072, 64), (None, 128))      # (tokens x heads of a step up to ..., tokens of a chunk): short chunks while
# the step is too small to fill the chip with long ones, long chunks (fewer carried states) from there on (4 x 1 024 tokens, 8
# heads: 895 us in one walk, 301 in chunks of 128, 150 in chunks of 32; 16 x 1 024 tokens: 446 us at 128 and 64, 474 at 32)
DECAY_SCAN_WS_BYTES = 1 << 30     # the chunks' states may take this much; longer chunks otherwise


def decay_scan(x, offsets, decay, mem, layout: StepLayout, heads: int, dim: int, vdim: int, act: str = "none", chunk: Optional[int] = None):
    """Linear attention with one constant decay per head.  x (T, columns): q, k (heads * dim each) and v (heads * vdim) at the
    three column `offsets`, passed through `act` ("none" or "silu") first; decay (heads) float32; mem (slots, heads, dim, vdim)
    float32, continued and written back.  S <- decay S + k v^T, read-out S^T q.  Returns (T, heads, vdim) float32.
    Ragged steps with long portions are cut into chunks of `chunk` tokens (default: by the step's shape; 0: never) that run side by
    side: the result is the same up to the rounding of decay^n against n multiplications."""
    _dev(x, decay, mem)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[0] == layout.n_tok, "decay_scan: x must be (T, columns) with unit inner stride")
    _f32c(decay, "decay_scan: decay")
    _f32c(mem, "decay_scan: mem")
    n_slots = mem.shape[0]
    _need(decay.numel() == heads and mem.shape == (n_slots, heads, dim, vdim), "decay_scan: shapes")
    t = x.shape[0]
    out = torch.empty((t, heads, vdim), dtype=F32, device=x.device)
    if chunk is None:
        chunk = 0
        if layout.qo_indptr is not None and layout.max_q >= DECAY_SCAN_CHUNK_FROM:
            chunk = next(c for upto, c in DECAY_SCAN_CHUNKS if upto is None or t * heads <= upto)
    n_chunks, ws = 0, None
    if chunk and layout.qo_indptr is not None:
        per = heads * dim * vdim * 4
        while layout.n_seq * -(-layout.max_q // chunk) * per > DECAY_SCAN_WS_BYTES or layout.n_seq * -(-layout.max_q // chunk) > 65535:
            chunk *= 2
        n_chunks = -(-layout.max_q // chunk)
        if n_chunks > 1:
            ws = torch.empty((layout.n_seq * n_chunks, heads, dim, vdim), dtype=F32, device=x.device)
    if ws is None:
        chunk = n_chunks = 0
    lib = _lib.load()
    _lib.check(lib.nvx_decay_scan(_ptr(x), x.stride(0), _fmt(x), offsets[0], offsets[1], offsets[2], {"none": 0, "silu": 1}[act], _ptr(decay),
                                  _ptr(mem), n_slots, *_layout_args(layout), _ptr(out), t, layout.n_seq, heads, dim, vdim, chunk, n_chunks,
                                  _ptr(ws), _stream()), "nvx_decay_scan")
    return out


def postnorm_residual(x, y=None, w_post=None, eps: float = 0.0, y2=None, a: float = 1.0, b: float = 1.0, w_next=None, out_dtype=None,
                      want_h: bool = True):
    """x (T, width) float32, updated in place: x += r / rms(r) * w_post with r = a * y (+ b * y2) and w_post one number or one per
    channel (float32).  Returns h (T, width) in `out_dtype` (default: y's): x / rms(x) * w_next if w_next is given (one number or
    one per channel), else x itself; None if not `want_h`."""
    _dev(x, y, y2, w_post, w_next)
    _f32c(x, "postnorm_residual: x")
    _need(x.dim() == 2, "postnorm_residual: x must be (T, width)")
    t, width = x.shape
    for name, r in (("y", y), ("y2", y2)):
        if r is not None:
            _need(r.shape == (t, width) and r.stride(1) == 1, f"postnorm_residual: {name} must be (T, width) with unit inner stride")
    _need(y2 is None or (y is not None and y2.dtype == y.dtype), "postnorm_residual: y2 goes with y, in its format")
    dtype = out_dtype or (y.dtype if y is not None else None)
    _need(dtype in _FMT and (y is None or y.dtype == dtype), "postnorm_residual: y and the output share one format")
    for name, w in (("w_post", w_post), ("w_next", w_next)):
        if w is not None:
            _f32c(w, "postnorm_residual: " + name)
            _need(w.numel() in (1, width), f"postnorm_residual: {name} has one entry or one per channel")
    _need(y is None or w_post is not None, "postnorm_residual: a result needs its norm weight")
    h = torch.empty((t, width), dtype=dtype, device=x.device) if (want_h or w_next is not None) else None
    lib = _lib.load()
    _lib.check(lib.nvx_postnorm_residual(_ptr(y), y.stride(0) if y is not None else 0, _ptr(y2), y2.stride(0) if y2 is not None else 0, float(a),
                                         float(b), _ptr(w_post), w_post.numel() if w_post is not None else 0, _FMT[dtype], _ptr(x), _ptr(w_next),
                                         w_next.numel() if w_next is not None else 0, float(eps), _ptr(h), t, width, _stream()),
               "nvx_postnorm_residual")
    return h


def embed_scale(ids, table, scale: float):
    """(x, h): x = table[ids] * scale in float32 and the same rows in the table's format."""
    _dev(ids, table)
    _need(ids.dtype == torch.int64 and ids.is_contiguous() and ids.dim() == 1, "embed_scale: ids must be int64 (T)")
    _need(table.dim() == 2 and table.is_contiguous(), "embed_scale: table must be contiguous (vocab, width)")
    t, width = ids.numel(), table.shape[1]
    x = torch.empty((t, width), dtype=F32, device=table.device)
    h = torch.empty((t, width), dtype=table.dtype, device=table.device)
    lib = _lib.load()
    _lib.check(lib.nvx_embed_scale(_ptr(ids), _ptr(table), _fmt(table), table.shape[0], float(scale), _ptr(x), _ptr(h), t, width, _stream()),
               "nvx_embed_scale")
    return x, h


def tanh_cap(z, cap: float):
    """cap * tanh(z / cap) in float32 (cap <= 0: z as float32)."""
    _dev(z)
    _need(z.is_contiguous(), "tanh_cap: z must be contiguous")
    out = torch.empty(z.shape, dtype=F32, device=z.device)
    lib = _lib.load()
    _lib.check(lib.nvx_tanh_cap(_ptr(z), _fmt(z), float(cap or 0.0), _ptr(out), z.numel(), _stream()), "nvx_tanh_cap")
    return out


def moe_route(logits, top: int):
    """logits (T, experts) float32 -> (ids (T, top) int32, scores (T, top) float32): the `top` largest logits of every token
    (ties: the lower id) and their sigmoids."""
    _dev(logits)
    _f32c(logits, "moe_route: logits")
    t, n_exp = logits.shape
    idx = torch.empty((t, top), dtype=torch.int32, device=logits.device)
    wts = torch.empty((t, top), dtype=F32, device=logits.device)
    lib = _lib.load()
    _lib.check(lib.nvx_moe_route(_ptr(logits), t, n_exp, top, _ptr(idx), _ptr(wts), _stream()), "nvx_moe_route")
    return idx, wts


def moe_expert_rows_fits(width: int, ff: int) -> bool:
    return width <= _lib.load().nvx_moe_expert_rows_max_width(ff)


def _moe_weights(w_gu, w_d, what: str):
    n_exp, ff2, width = w_gu.shape
    _need(w_gu.is_contiguous() and w_d.is_contiguous() and w_d.shape == (n_exp, width, ff2 // 2) and w_d.dtype == w_gu.dtype, what + ": expert weights")
    return n_exp, ff2 // 2, width


def moe_expert_rows(h, idx, wts, w_gu, w_d, limit: float, alpha: float, shift: float = 1.0, weight_out: bool = False):
    """out[t] = sum over token t's chosen experts of expert(score * h[t]) (or of score * expert(h[t]) if `weight_out`); w_gu
    (experts, 2 * ff, width) = gate | up rows, w_d (experts, width, ff); activation min(g, limit) sigmoid(alpha min(g, limit))
    (clamp(u, +-limit) + shift).  The chosen experts' rows are streamed per (token, choice) pair: the form for steps of few tokens."""
    _dev(h, idx, wts, w_gu, w_d)
    n_exp, ff, width = _moe_weights(w_gu, w_d, "moe_expert_rows")
    t, top = idx.shape
    _need(h.shape == (t, width) and h.stride(1) == 1 and h.dtype == w_gu.dtype, "moe_expert_rows: h shape / format")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and wts.dtype == F32 and wts.is_contiguous() and wts.shape == idx.shape, "moe_expert_rows: choices")
    out = torch.empty((t, width), dtype=h.dtype, device=h.device)
    ws = torch.empty((t, top, ff), dtype=F32, device=h.device)      # the hidden activations between the two launches
    lib = _lib.load()
    _lib.check(lib.nvx_moe_expert_rows(_ptr(h), h.stride(0), _fmt(h), _ptr(idx), _ptr(wts), top, _ptr(w_gu), _ptr(w_d), n_exp, float(limit),
                                       float(alpha), float(shift), int(bool(weight_out)), _ptr(ws), _ptr(out), t, width, ff, _stream()),
               "nvx_moe_expert_rows")
    return out


def moe_order_fits(n_exp: int) -> bool:
    return n_exp <= _lib.load().nvx_moe_order_max_experts()


def moe_order(idx, n_exp: int):
    """idx (T, top) int32 expert ids -> (dst (T, top) int64, counts (n_exp) int32): dst[t][k] is the place of pair (t, k) when all
    pairs are put in expert order (pairs of one expert keep their order), counts[e] the pairs of expert e."""
    _dev(idx)
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and idx.dim() == 2, "moe_order: idx must be contiguous int32 (T, top)")
    dst = torch.empty(idx.shape, dtype=torch.int64, device=idx.device)
    counts = torch.empty((n_exp,), dtype=torch.int32, device=idx.device)
    lib = _lib.load()
    _lib.check(lib.nvx_moe_order(_ptr(idx), idx.numel(), n_exp, _ptr(dst), _ptr(counts), _stream()), "nvx_moe_order")
    return dst, counts


def moe_scatter_rows(h, wts, dst, spare_rows: int = 0):
    """xs[dst[r]] = wts[r] * h[r // top] for every (token, choice) pair r (dst: int64 (T, top), a permutation; wts None: ones).
    `spare_rows` more rows of zeros follow the T * top rows (room for products that run a little past the last pair)."""
    _dev(h, wts, dst)
    t, top = dst.shape
    _need(h.dim() == 2 and h.shape[0] == t and h.stride(1) == 1, "moe_scatter_rows: shapes")
    _need(wts is None or (wts.dtype == F32 and wts.is_contiguous() and wts.shape == dst.shape), "moe_scatter_rows: wts must be float32 (T, top)")
    _need(dst.dtype == torch.int64 and dst.is_contiguous(), "moe_scatter_rows: dst must be int64 (T, top)")
    xs = torch.empty((t * top + spare_rows, h.shape[1]), dtype=h.dtype, device=h.device)
    if spare_rows:
        xs[t * top:].zero_()
    lib = _lib.load()
    _lib.check(lib.nvx_moe_scatter_rows(_ptr(h), h.stride(0), _fmt(h), _ptr(wts), _ptr(dst), top, _ptr(xs), t, h.shape[1], _stream()),
               "nvx_moe_scatter_rows")
    return xs


def moe_glu(gu, limit: float, alpha: float, shift: float = 1.0):
    """gu (rows, 2 * ff) = gate | up pre-activations -> min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + shift)
    (limit = inf, alpha = 1, shift = 0: silu(g) * u)."""
    _dev(gu)
    _need(gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] % 2 == 0, "moe_glu: gu must be contiguous (rows, 2 * ff)")
    y = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
    lib = _lib.load()
    _lib.check(lib.nvx_moe_glu(_ptr(gu), _fmt(gu), float(limit), float(alpha), float(shift), _ptr(y), gu.shape[0], gu.shape[1] // 2, _stream()),
               "nvx_moe_glu")
    return y


def moe_gather_rows(ys, dst, wts=None):
    """out[t] = sum_k wts[t][k] * ys[dst[t][k]] (wts None: ones); ys may have spare rows behind the T * top that dst names."""
    _dev(ys, dst, wts)
    _need(wts is None or (wts.dtype == F32 and wts.is_contiguous() and wts.shape == dst.shape), "moe_gather_rows: wts must be float32 (T, top)")
    t, top = dst.shape
    _need(ys.dim() == 2 and ys.is_contiguous() and ys.shape[0] >= t * top and dst.dtype == torch.int64 and dst.is_contiguous(), "moe_gather_rows: shapes")
    out = torch.empty((t, ys.shape[1]), dtype=ys.dtype, device=ys.device)
    lib = _lib.load()
    _lib.check(lib.nvx_moe_gather_rows(_ptr(ys), _fmt(ys), _ptr(dst), _ptr(wts), top, _ptr(out), t, ys.shape[1], _stream()), "nvx_moe_gather_rows")
    return out


def skinny_proj(x, w, in_act: str = "none"):
    """out = f(x) @ w.T in float32, f = identity or tanh: x (T, k_in) in any activation format (rows may be a slice of wider
    rows), w (n_out, k_in) float32.  For few outputs (gate and router logits) or few inputs; one fixed summation order and
    no workspace, so a captured launch replays to the same bits."""
    _dev(x, w)
    _f32c(w, "skinny_proj: w")
    _need(x.dim() == 2 and x.stride(1) == 1 and w.dim() == 2 and w.shape[1] == x.shape[1], "skinny_proj: x must be (T, k_in), w (n_out, k_in)")
    out = torch.empty((x.shape[0], w.shape[0]), dtype=F32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_skinny_proj(_ptr(x), x.stride(0), _fmt(x), _ptr(w), {"none": 0, "tanh": 1}[in_act], _ptr(out), x.shape[0], w.shape[0],
                                   x.shape[1], _stream()), "nvx_skinny_proj")
    return out


# ---------------------------------------------------------------------------------------------
# several residual streams, the real-gated recurrence, a latent with a rotated key part, the softmax router with groups
# ---------------------------------------------------------------------------------------------
def hyper_mix(x, y=None, scale=None, mix=None, w_out=None, w_in=None, w_norm=None, eps: float = 0.0, n_streams: Optional[int] = None,
              out_dtype=None, want_h: bool = True):
    """Residual streams x (T, streams, width) float32 and a sublayer boundary.  With a result y (T, width): r = y * scale (scale:
    (width) or None) and every stream at once from the old ones, x_j <- sum_s mix[s, j] x_s + w_out[j] r (in place).  x may also be
    (T, width) with `n_streams`: the one row every stream starts from; the streams are then made.  Returns (x, h) with h = u /
    rms(u) * w_norm for u = sum_j w_in[j] x_j (w_in None: the plain sum; w_norm None: ones), in `out_dtype` (default: y's)."""
    _dev(x, y, scale, mix, w_out, w_in, w_norm)
    _f32c(x, "hyper_mix: x")
    if x.dim() == 2:
        _need(n_streams is not None and n_streams >= 1 and y is None, "hyper_mix: one row per token starts n_streams streams, and has no result yet")
        t, width = x.shape
        x_out = torch.empty((t, n_streams, width), dtype=F32, device=x.device)
        tok_stride, stream_stride = width, 0
    else:
        _need(x.dim() == 3, "hyper_mix: x must be (T, streams, width)")
        t, n_streams, width = x.shape
        x_out, tok_stride, stream_stride = x, n_streams * width, width
    if y is not None:
        _need(y.shape == (t, width) and y.stride(1) == 1, "hyper_mix: y must be (T, width) with unit inner stride")
        _need(mix is not None and w_out is not None, "hyper_mix: a result needs the mixing matrix and its output weights")
    for name, a, n in (("scale", scale, width), ("mix", mix, n_streams * n_streams), ("w_out", w_out, n_streams), ("w_in", w_in, n_streams),
                       ("w_norm", w_norm, width)):
        if a is not None:
            _f32c(a, "hyper_mix: " + name)
            _need(a.numel() == n, f"hyper_mix: {name} size")
    dtype = out_dtype or (y.dtype if y is not None else None)
    _need(not want_h or dtype in _FMT, "hyper_mix: output format")
    _need(y is None or dtype is None or y.dtype == dtype, "hyper_mix: y and the output share one format")
    h = torch.empty((t, width), dtype=dtype, device=x.device) if want_h else None
    fmt = _FMT[dtype] if dtype is not None else _fmt(y)
    lib = _lib.load()
    _lib.check(lib.nvx_hyper_mix(_ptr(x), tok_stride, stream_stride, _ptr(y), y.stride(0) if y is not None else 0, fmt, _ptr(scale), _ptr(mix),
                                 _ptr(w_out), _ptr(w_in), _ptr(w_norm), float(eps), _ptr(x_out), _ptr(h), t, n_streams, width, _stream()),
               "nvx_hyper_mix")
    return x_out, h


def short_conv(x, w, state, layout: StepLayout, bias=None, act: str = "none"):
    """act(bias + causal convolution over time per channel): short_conv_silu with an optional bias (channels, float32) and `act`
    "none" or "silu".  x (T, channels) (rows may be a slice of wider rows); w (taps, channels) float32, row j multiplying the input
    taps - 1 - j tokens back; state (slots, taps - 1, channels) float32.  Returns (T, channels) in x's format."""
    _dev(x, w, state, bias)
    _need(x.dim() == 2 and x.stride(1) == 1, "short_conv: x must be (T, channels) with unit inner stride")
    t, ch = x.shape
    _f32c(w, "short_conv: w")
    taps = w.shape[0]
    _need(w.dim() == 2 and w.shape[1] == ch and t == layout.n_tok, "short_conv: shapes")
    if bias is not None:
        _f32c(bias, "short_conv: bias")
        _need(bias.numel() == ch, "short_conv: bias size")
    n_slots = 0
    if taps > 1:
        _f32c(state, "short_conv: state")
        _need(state.dim() == 3 and state.shape[1:] == (taps - 1, ch), "short_conv: state shape")
        n_slots = state.shape[0]
    out = torch.empty((t, ch), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_short_conv(_ptr(x), x.stride(0), _fmt(x), _ptr(w), _ptr(bias), {"none": 0, "silu": 1}[act], taps,
                                  _ptr(state) if taps > 1 else None, n_slots, _ptr(layout.tok_seq), *_layout_args(layout), _ptr(out), t,
                                  layout.n_seq, ch, _stream()), "nvx_short_conv")
    return out


def rglru_scan(y, u, gates, gate_bias, rate, state, layout: StepLayout):
    """Real-gated linear recurrence over each sequence's tokens.  y, u (T, width) (rows may be slices of wider rows): the gelu
    branch's pre-activation and the recurrence's input; gates (blocks, T, 2 * block_width): recurrence-gate | input-gate
    pre-activations of every block of channels; gate_bias (2, width), rate (width) float32; state (slots, width) float32, continued
    and written back.  a = exp(-rate * sigmoid(r)), S <- a S + sqrt(1 - a^2) sigmoid(i) u.  Returns S * gelu_tanh(y), (T, width)."""
    _dev(y, u, gates, gate_bias, rate, state)
    t, width = u.shape
    _need(y.shape == (t, width) and y.stride(1) == 1 and u.stride(1) == 1 and y.dtype == u.dtype == gates.dtype, "rglru_scan: y, u (T, width) in one format")
    _need(gates.dim() == 3 and gates.shape[1] == t and gates.stride(2) == 1 and gates.shape[2] % 2 == 0 and gates.shape[0] * gates.shape[2] == 2 * width,
          "rglru_scan: gates must be (blocks, T, 2 * width / blocks)")
    for a, what, n in ((gate_bias, "gate_bias", 2 * width), (rate, "rate", width)):
        _f32c(a, "rglru_scan: " + what)
        _need(a.numel() == n, f"rglru_scan: {what} size")
    _f32c(state, "rglru_scan: state")
    _need(t == layout.n_tok and state.dim() == 2 and state.shape[1] == width, "rglru_scan: shapes")
    out = torch.empty((t, width), dtype=u.dtype, device=u.device)
    lib = _lib.load()
    _lib.check(lib.nvx_rglru_scan(_ptr(y), y.stride(0), _ptr(u), u.stride(0), _ptr(gates), gates.stride(0), gates.stride(1), gates.shape[2] // 2,
                                  _ptr(gate_bias), _ptr(rate), _fmt(u), _ptr(state), state.shape[0], *_layout_args(layout), _ptr(out), t,
                                  layout.n_seq, width, _stream()), "nvx_rglru_scan")
    return out


def latent_rope_prep(x, offsets, positions, freq, mag: float, w_kv, eps: float, slots, cache, heads: int, dim: int, rot: int):
    """After the fused projection x (T, columns) holding, at the three column `offsets`, the queries (heads x [dim | rot]), the down
    projection [latent (kv_rank) | key part (rot)] and one gate pre-activation per head.  The last `rot` entries of every query head
    and the key part are turned in neighbouring pairs by positions * freq (float64, rot / 2; cos and sin times `mag`); the latent is
    RMS-normed with w_kv (kv_rank, float32); cache[slots[t]] = [latent | key part | zeros] (cache: (slots, row) with row >= kv_rank +
    rot).  Returns (queries (T, heads * (dim + rot)), gate (T, heads) float32 = sigmoid)."""
    _dev(x, positions, freq, w_kv, slots, cache)
    _need(x.dim() == 2 and x.stride(1) == 1, "latent_rope_prep: x must be (T, columns) with unit inner stride")
    t = x.shape[0]
    _f32c(w_kv, "latent_rope_prep: w_kv")
    kv_rank = w_kv.numel()
    _need(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == t, "latent_rope_prep: positions must be int64 (T)")
    _need(slots.dtype == torch.int64 and slots.is_contiguous() and slots.numel() == t, "latent_rope_prep: slots must be int64 (T)")
    _need(rot == 0 or (freq.dtype == torch.float64 and freq.is_contiguous() and freq.numel() == rot // 2), "latent_rope_prep: freq must be float64 (rot / 2)")
    _need(cache.dtype == x.dtype and cache.is_contiguous() and cache.dim() == 2 and cache.shape[1] >= kv_rank + rot, "latent_rope_prep: cache")
    q = torch.empty((t, heads * (dim + rot)), dtype=x.dtype, device=x.device)
    gate = torch.empty((t, heads), dtype=F32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.nvx_latent_rope_prep(_ptr(x), x.stride(0), _fmt(x), offsets[0], offsets[1], offsets[2], _ptr(positions), _ptr(freq) if rot else None,
                                        float(mag), _ptr(w_kv), float(eps), _ptr(slots), _ptr(q), _ptr(cache), cache.shape[0], cache.shape[1],
                                        _ptr(gate), t, heads, dim, rot, kv_rank, _stream()), "nvx_latent_rope_prep")
    return q, gate


def moe_route_softmax(logits, top: int, n_groups: int = 0, keep_groups: int = 0, norm_eps: float = 0.0):
    """logits (T, experts) float32 -> (ids (T, top) int32, weights (T, top) float32).  Scores are the softmax over all experts; with
    n_groups > 1 the experts form equal groups of neighbours, a group counts as its best score, and only experts of the keep_groups
    best groups can be chosen; the `top` largest scores are taken (ties: the lower id) and divided by their sum + norm_eps."""
    _dev(logits)
    _f32c(logits, "moe_route_softmax: logits")
    t, n_exp = logits.shape
    idx = torch.empty((t, top), dtype=torch.int32, device=logits.device)
    wts = torch.empty((t, top), dtype=F32, device=logits.device)
    lib = _lib.load()
    _lib.check(lib.nvx_moe_route_softmax(_ptr(logits), t, n_exp, top, int(n_groups or 0), int(keep_groups or 0), float(norm_eps), _ptr(idx),
                                         _ptr(wts), _stream()), "nvx_moe_route_softmax")
    return idx, wts
