"""The C-ABI library loads on a machine without a GPU and exports every symbol include/nvx.h declares
(no compute call is made here)."""
from __future__ import annotations

import ctypes
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nvx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nvx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_binds():
    from nano_vllm_x_amd import _lib

    names = declared_symbols()
    assert len(names) >= 20
    assert set(_lib.SIGNATURES) | {"nvx_abi_version", "nvx_last_error"} >= set(names), set(names) - set(_lib.SIGNATURES)
    assert set(_lib.SIGNATURES) <= set(names), set(_lib.SIGNATURES) - set(names)


def test_binding_passes_as_many_arguments_as_the_header_declares():
    """A prototype that gains a parameter must gain it in the ctypes table too: a missing trailing argument
    is not an error at the call, the callee just reads a stale register."""
    from nano_vllm_x_amd import _lib

    text = open(os.path.join(ROOT, "include", "nvx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    seen = 0
    for name, args in re.findall(r"\b(nvx_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", text):
        n = 0 if args.strip() in ("", "void") else args.count(",") + 1
        if name in _lib.SIGNATURES:
            assert len(_lib.SIGNATURES[name][1]) == n, f"{name}: header declares {n} parameters, binding passes {len(_lib.SIGNATURES[name][1])}"
            seen += 1
    assert seen == len(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from nano_vllm_x_amd import _lib

    assert os.path.exists(_lib.LIB_PATH), "build first: make -C nano_vllm_x_amd/csrc"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in include/nvx.h but not exported"
    lib.nvx_abi_version.restype = ctypes.c_int
    assert lib.nvx_abi_version() == _lib.header_abi_version(), "library built from another include/nvx.h: rebuild"
    # pure host helpers answer without a device
    lib.nvx_decode_plan_ws_ints.restype = ctypes.c_int64
    lib.nvx_decode_plan_ws_ints.argtypes = [ctypes.c_int64, ctypes.c_int]
    assert lib.nvx_decode_plan_ws_ints(256, 8) > 0
    lib.nvx_linear_decode_splits.argtypes = [ctypes.c_int64, ctypes.c_int64]
    assert lib.nvx_linear_decode_splits(1024, 3072) == 4 and lib.nvx_linear_decode_splits(4096, 1024) == 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from nano_vllm_x_amd import _lib

    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "absent.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    try:
        _lib.load()
    except _lib.NvxLibraryError as e:
        assert "absent.so" in str(e) or "build" in str(e).lower()
    else:
        raise AssertionError("loading a missing library must raise")


def test_build_entry_point_runs_end_to_end():
    """`python __graft_entry__.py` is the documented build command: it must compile (a no-op when the objects
    are current), load the library and agree with it on the ABI version."""
    import __graft_entry__ as g

    g.build()


def test_binding_refuses_a_library_of_another_abi_version(monkeypatch):
    from nano_vllm_x_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "header_abi_version", lambda: 10 ** 6)
    try:
        _lib.load()
    except _lib.NvxLibraryError as e:
        assert "ABI version" in str(e)
    else:
        raise AssertionError("a version mismatch must raise")


def test_every_kernel_entry_point_has_a_custom_op():
    """`torch.ops.nvx.<name>` exists for every launching entry point of the C ABI (size queries and diagnostics
    aside): the operator surface the Python host calls the kernels through."""
    import torch

    import nano_vllm_x_amd.torch_ops  # noqa: F401

    op_of = {"nvx_store_kv": "store_kvcache", "nvx_rmsnorm": "rmsnorm", "nvx_rope": "rope", "nvx_silu_mul": "silu_mul",
             "nvx_qknorm_rope_store": "qknorm_rope_store", "nvx_linear_decode": "linear_decode", "nvx_rmsnorm_splitk": "rmsnorm_splitk",
             "nvx_decode_plan": "decode_plan", "nvx_paged_decode": "paged_decode", "nvx_paged_decode_qkv": "paged_decode_qkv",
             "nvx_paged_decode_noalloc": "paged_decode_noalloc", "nvx_prefill_plan": "prefill_plan", "nvx_paged_prefill": "paged_prefill",
             "nvx_sample": "sample", "nvx_sampler_probs": "sampler_probs", "nvx_block_table_write_rows": "block_table_write_rows",
             "nvx_decode_step_setup": "decode_step_setup", "nvx_peer_allreduce_norm": "peer_allreduce_norm",
             "nvx_sample_shard": "sample_shard", "nvx_sample_pick": "sample_pick", "nvx_lmhead_pack": "lmhead_pack",
             "nvx_lmhead_sample": "lmhead_sample", "nvx_linear_stream": "linear_stream", "nvx_splitk_sum": "splitk_sum",
             "nvx_linear_block": "linear_block", "nvx_boundary_norm": "boundary_norm", "nvx_canon_conv": "canon_conv", "nvx_relu2": "relu2",
             "nvx_mingru_scan": "mingru_scan", "nvx_latent_prep": "latent_prep", "nvx_latent_attn": "latent_attn",
             "nvx_gated_residual_norm": "gated_residual_norm", "nvx_head_norm_gate": "head_norm_gate", "nvx_short_conv_silu": "short_conv_silu",
             "nvx_token_shift_mix": "token_shift_mix", "nvx_mlstm_scan": "mlstm_scan", "nvx_delta_scan": "delta_scan", "nvx_rwkv_scan": "rwkv_scan",
             "nvx_rope_vnorm_store": "rope_vnorm_store", "nvx_softcap_attn": "softcap_attn", "nvx_moe_route": "moe_route",
             "nvx_moe_expert_rows": "moe_expert_rows", "nvx_moe_scatter_rows": "moe_scatter_rows", "nvx_moe_order": "moe_order", "nvx_moe_glu": "moe_glu",
             "nvx_moe_gather_rows": "moe_gather_rows", "nvx_skinny_proj": "skinny_proj", "nvx_attn_prep_store": "attn_prep_store",
             "nvx_decay_scan": "decay_scan", "nvx_postnorm_residual": "postnorm_residual", "nvx_embed_scale": "embed_scale", "nvx_tanh_cap": "tanh_cap",
             "nvx_hyper_mix": "hyper_mix", "nvx_short_conv": "short_conv", "nvx_rglru_scan": "rglru_scan", "nvx_latent_rope_prep": "latent_rope_prep",
             "nvx_moe_route_softmax": "moe_route_softmax"}
    helpers = {"nvx_abi_version", "nvx_last_error", "nvx_linear_decode_splits", "nvx_decode_plan_ws_ints", "nvx_decode_partial_ws_floats",
               "nvx_prefill_plan_ws_ints", "nvx_sample_ws_bytes", "nvx_paged_decode_noalloc_max_batch",
               "nvx_lmhead_max_rows", "nvx_lmhead_rows_per_pass", "nvx_lmhead_packed_elems", "nvx_lmhead_ws_bytes",
               "nvx_linear_block_max_rows", "nvx_linear_block_slices", "nvx_moe_expert_rows_max_width", "nvx_scan_column_blocks", "nvx_moe_order_max_experts", "nvx_softcap_attn_tile_fits",
               # start-up calls of the direct-peer exchange (allocation, handle exchange, status, teardown): host side
               "nvx_peer_exchange_bytes", "nvx_peer_create", "nvx_peer_export", "nvx_peer_import", "nvx_peer_status", "nvx_peer_destroy"}
    # the float16 entry points have no operator of their own: the operator of the bfloat16 one picks them by tensor dtype
    from nano_vllm_x_amd._lib import F16_ENTRY_POINTS
    assert set(F16_ENTRY_POINTS) <= set(op_of)
    half = {name + "_f16" for name in F16_ENTRY_POINTS}
    assert set(declared_symbols()) == set(op_of) | helpers | half, set(declared_symbols()) ^ (set(op_of) | helpers | half)
    for sym, op in op_of.items():
        assert hasattr(torch.ops.nvx, op), f"{sym} has no torch.ops.nvx.{op}"
