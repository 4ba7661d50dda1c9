"""Mixtures of small gated feed-forward experts: behind a sigmoid router whose score scales an expert's input, behind a softmax
router with groups whose renormalised scores weigh the experts' outputs, or chosen by a table of token ids with fixed weights on
the experts' outputs."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops


class ExpertBank(nn.Module):
    """`experts` gated feed-forward layers of one shape, stacked: w_gu (experts, 2 ff, width) = rows gate | up, w_d (experts, width,
    ff).  Expert: g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), W_down (g sigmoid(alpha g) (u + shift)) -- limit =
    inf, alpha = 1, shift = 0 is silu(g) u.  `run` evaluates given choices: idx (T, top) int32 expert ids, wts (T, top) float32
    which scale the experts' inputs, or their outputs if `weight_out`.

    Steps of few tokens (decode steps, which a hipGraph replays: no host decision may depend on the choices) evaluate each
    token's experts in one launch, streaming the chosen experts' rows.  Steps of many tokens put the inputs into expert order
    (ops.moe_order: a counting sort, which also gives the per-expert counts) and run one pair of matrix products per expert
    that received tokens; the counts are the one host read of that path.  An expert's product runs over its row count rounded up
    to a multiple of ROW_STEP: the rows past its own are the next experts', whose products come later on the same stream and
    write them anew (the buffers end in ROW_STEP spare rows), so every row ends as its own expert's.  The library then sees a
    handful of row counts instead of a new one per expert, layer and step, which halves what a product's launch costs the host."""

    ROWS_PATH_TOKENS = 32
    ROW_STEP = 64

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, alpha: float, shift: float):
        super().__init__()
        self.width, self.experts, self.top, self.ff = width, experts, top, ff
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        self.w_gu = nn.Parameter(torch.empty(experts, 2 * ff, width))      # rows of an expert: gate | up
        self.w_d = nn.Parameter(torch.empty(experts, width, ff))
        self._rows_fit = None

    def by_rows(self, t: int, decode_step: bool) -> bool:
        """Whether a step of t tokens streams the chosen experts' rows (else: per-expert products over the expert order)."""
        if self._rows_fit is None:
            self._rows_fit = ops.moe_expert_rows_fits(self.width, self.ff)
            self._order_fit = ops.moe_order_fits(self.experts)      # more experts than the ordering kernel holds: pair by pair
            if not (self._rows_fit or self._order_fit):
                raise NotImplementedError(f"{self.experts} experts of {self.ff} x {self.width}: neither expert path is built for these sizes")
        return self._rows_fit and (decode_step or t <= self.ROWS_PATH_TOKENS or not self._order_fit)

    def run(self, h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, decode_step: bool, weight_out: bool, order=None) -> torch.Tensor:
        """`order` = (dst, counts as a list): the expert order of idx where the caller has it already (ops.moe_order)."""
        t = h.shape[0]
        if self.by_rows(t, decode_step):
            return ops.moe_expert_rows(h, idx, wts, self.w_gu, self.w_d, self.limit, self.alpha, self.shift, weight_out)
        if order is None:
            dst, counts = ops.moe_order(idx, self.experts)
            counts = counts.tolist()
        else:
            dst, counts = order
        step = self.ROW_STEP
        xs = ops.moe_scatter_rows(h, None if weight_out else wts, dst, spare_rows=step)
        spans, a = [], 0
        for e, n in enumerate(counts):            # (expert, first row, rows of the product): a + m never passes the spare rows
            if n:
                spans.append((e, a, -(-n // step) * step))
                a += n
        assert a + step == xs.shape[0]
        gu = torch.empty((xs.shape[0], 2 * self.ff), dtype=h.dtype, device=h.device)
        for e, a, m in spans:
            torch.mm(xs[a:a + m], self.w_gu[e].t(), out=gu[a:a + m])
        y = ops.moe_glu(gu, self.limit, self.alpha, self.shift)
        ys = torch.empty((xs.shape[0], self.width), dtype=h.dtype, device=h.device)
        for e, a, m in spans:
            torch.mm(y[a:a + m], self.w_d[e].t(), out=ys[a:a + m])
        return ops.moe_gather_rows(ys, dst, wts if weight_out else None)


class SigmoidInputMoE(ExpertBank):
    """scores = sigmoid(W_router h) (float32); every token takes the `top` experts with the largest scores, and a score
    scales its expert's INPUT (no renormalisation): out = sum_e expert_e(score_e * h).  Expert: g = min(W_gate x, limit),
    u = clamp(W_up x, -limit, limit), W_down (g * sigmoid(alpha * g) * (u + 1))."""

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, alpha: float):
        super().__init__(width, experts, top, ff, limit, alpha, 1.0)
        self.router = nn.Parameter(torch.zeros(experts, width, dtype=torch.float32))

    def forward(self, h: torch.Tensor, decode_step: bool = False) -> torch.Tensor:
        idx, wts = ops.moe_route(ops.skinny_proj(h, self.router), self.top)
        return self.run(h, idx, wts, decode_step, weight_out=False)


class TableMoE(ExpertBank):
    """No router: `table` (vocab, top) int32 names the experts of every token id (the entries of a row differ); each chosen expert
    weighs 1 / top and the weights apply to the experts' OUTPUTS.  Expert: W_down (silu(W_gate x) * (W_up x))."""

    def __init__(self, width: int, experts: int, top: int, ff: int, vocab: int):
        super().__init__(width, experts, top, ff, float("inf"), 1.0, 0.0)
        self.register_buffer("table", torch.zeros(vocab, top, dtype=torch.int32), persistent=False)
        self.register_buffer("share", torch.full((1, top), 1.0 / top, dtype=torch.float32), persistent=False)

    def choices(self, input_ids: torch.Tensor):
        """(idx, wts) of a step's tokens: they depend on the token ids alone."""
        idx = self.table.index_select(0, input_ids)
        return idx, self.share.expand(idx.shape[0], self.top).contiguous()

    @staticmethod
    def plan_step(layers, input_ids: torch.Tensor, decode_step: bool) -> list:
        """What every TableMoE of `layers` (None where a layer has none) needs for this step, made before the first layer runs: the
        choices, and for steps of many tokens the expert order with its counts -- ONE host read for all layers instead of one per
        layer in the middle of the step, so the host can queue the whole step without waiting for the device."""
        plans, pending = [], []
        for moe in layers:
            if moe is None:
                plans.append(None)
                continue
            idx, wts = moe.choices(input_ids)
            plan = {"idx": idx, "wts": wts, "order": None}
            if not moe.by_rows(idx.shape[0], decode_step):
                dst, counts = ops.moe_order(idx, moe.experts)
                pending.append((plan, dst, counts))
            plans.append(plan)
        if pending:
            flat = torch.cat([c for _, _, c in pending]).tolist()
            at = 0
            for plan, dst, counts in pending:
                plan["order"] = (dst, flat[at:at + counts.numel()])
                at += counts.numel()
        return plans

    def forward(self, h: torch.Tensor, input_ids: torch.Tensor, decode_step: bool = False, plan=None) -> torch.Tensor:
        if plan is None:
            idx, wts = self.choices(input_ids)
            return self.run(h, idx, wts, decode_step, weight_out=True)
        return self.run(h, plan["idx"], plan["wts"], decode_step, weight_out=True, order=plan["order"])


class GroupedSoftmaxMoE(ExpertBank):
    """scores = softmax(W_router h) over all experts (float32).  The experts form `groups` equal groups of neighbours; a group counts
    as its best score and only experts of the `keep` best groups can be chosen (groups None or 1: no such limit).  Every token takes
    the `top` largest scores among those, the weights are these scores divided by their sum + norm_eps, and they weigh the experts'
    OUTPUTS.  Expert: g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), W_down (g * sigmoid(alpha * g) * (u + shift))."""

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, alpha: float, shift: float = 1.0, groups=None, keep=None,
                 norm_eps: float = 1e-20):
        super().__init__(width, experts, top, ff, limit, alpha, shift)
        self.groups, self.keep = int(groups or 0), int(keep or 0)
        if self.groups > 1:
            if experts % self.groups or not 1 <= self.keep <= self.groups or self.keep * (experts // self.groups) < top:
                raise ValueError("groups must divide the experts and the kept groups must hold `top` experts")
        self.norm_eps = float(norm_eps)
        self.router = nn.Parameter(torch.zeros(experts, width, dtype=torch.float32))

    def forward(self, h: torch.Tensor, decode_step: bool = False) -> torch.Tensor:
        idx, wts = ops.moe_route_softmax(ops.skinny_proj(h, self.router), self.top, self.groups, self.keep, self.norm_eps)
        return self.run(h, idx, wts, decode_step, weight_out=True)
