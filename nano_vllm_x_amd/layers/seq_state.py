"""Step metadata and cache of models that keep per-sequence state (recurrences, convolution tails) beside a per-token
cache (one latent per token and latent-attention layer).

`SeqStateCache` owns the device tensors, `SeqStateBackend.build_metadata` turns a scheduled batch into what the kernels
read -- the ragged layout of the step, every sequence's state slot and slot list -- and `attention_kv_cache`
(layers/attention.py) hands the result to the modules for one forward pass, as it does for paged attention."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .. import ops
from ..core.common import ForwardBatch, ForwardMode
from ..core.kv_cache import LatentCachePool, RecurrentStatePool


class SeqStateCache:
    """`latent_ranks`: name -> elements a layer caches per token (a latent: the layer's number; keys and values: (layer, "k")
    and (layer, "v")); `state_shapes`: name -> shape of one sequence's entry (names are the model's: (layer, what))."""

    def __init__(self, dtype: torch.dtype, device: torch.device, num_tokens: int, num_slots: int, latent_ranks: dict, state_shapes: dict):
        self.latents = LatentCachePool(dtype, device, num_tokens, latent_ranks)
        self.states = RecurrentStatePool(device, num_slots, state_shapes)
        self.num_tokens, self.num_slots = num_tokens, num_slots

    def latent(self, layer: int) -> torch.Tensor:
        return self.latents.get(layer)

    def state(self, name) -> torch.Tensor:
        return self.states.get(name)


@dataclass
class SeqStateMetadata:
    forward_mode: ForwardMode
    cache: SeqStateCache
    layout: ops.StepLayout          # ragged layout + state slots
    kv_indices: torch.Tensor        # int32: every sequence's token slots, one after the other
    kv_start: torch.Tensor          # int64 (B): where each sequence's list starts in kv_indices
    kv_len: torch.Tensor            # int32 (B): tokens of each sequence, this step's included
    out_slots: torch.Tensor         # int64 (T): slot of every token computed in this step
    kv_indptr: Optional[torch.Tensor] = None     # int32 (B+1): kv_start with the total appended (steps built from a batch)


class SeqStateBackend:
    def __init__(self, cache: SeqStateCache, device: torch.device):
        self.cache, self.device = cache, device

    def _up(self, a: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(a).to(self.device, non_blocking=True)

    def build_metadata(self, batch: ForwardBatch) -> SeqStateMetadata:
        seqs = batch.seqs
        n = len(seqs)
        q_lens = np.fromiter((len(s.token_ids) - s.cached_kv_len for s in seqs), dtype=np.int64, count=n)
        kv_lens = np.fromiter((len(s.token_ids) for s in seqs), dtype=np.int32, count=n)
        for s in seqs:
            if s.state_slot is None or not 0 <= s.state_slot < self.cache.num_slots:
                raise RuntimeError(f"sequence {s.seq_id!r} runs without a state slot")
            if len(s.kv_indices) < len(s.token_ids):
                raise RuntimeError(f"sequence {s.seq_id!r} has fewer slots than tokens")
        pos0 = np.fromiter((s.cached_kv_len for s in seqs), dtype=np.int64, count=n)
        slot = np.fromiter((s.state_slot for s in seqs), dtype=np.int32, count=n)
        kv_start = np.zeros(n, dtype=np.int64)
        np.cumsum(kv_lens[:-1], out=kv_start[1:])
        flat = np.concatenate([np.asarray(s.kv_indices[:len(s.token_ids)], dtype=np.int32) for s in seqs])
        out_slots = np.concatenate([np.asarray(s.kv_indices[s.cached_kv_len:len(s.token_ids)], dtype=np.int64) for s in seqs])
        t = int(q_lens.sum())
        if batch.forward_mode == ForwardMode.DECODE and t == n:
            layout = ops.StepLayout(t, n, self._up(pos0), self._up(slot))
        else:
            qo = np.zeros(n + 1, dtype=np.int32)
            np.cumsum(q_lens, out=qo[1:])
            tok_seq = np.repeat(np.arange(n, dtype=np.int32), q_lens)
            layout = ops.StepLayout(t, n, self._up(pos0), self._up(slot), self._up(qo), self._up(tok_seq), max_q=int(q_lens.max()))
        kv_indptr = np.zeros(n + 1, dtype=np.int32)
        np.cumsum(kv_lens, out=kv_indptr[1:])
        return SeqStateMetadata(forward_mode=batch.forward_mode, cache=self.cache, layout=layout, kv_indices=self._up(flat),
                                kv_start=self._up(kv_start), kv_len=self._up(kv_lens), out_slots=self._up(out_slots),
                                kv_indptr=self._up(kv_indptr))
