"""Feed-forward parts.  A feed-forward adds its output into the residual stream."""

from __future__ import annotations

from typing import Dict

import torch

from ..ops import kernels, residual
from ..ops.linear import LazyNorm, as_tensor, linear, linear_add, linear_xielu, packed_weight, plain_residual
from .base import MATRIX, Part, StepContext, TABLE, VECTOR, WeightRequest, register_feed_forward

# activations of the dense feed-forward: an epilogue of the product kernels, or (None) one that brings coefficients
# (ops.linear.linear_xielu: the tiled kernel's epilogue, elsewhere a kernel of its own behind the product)
_ACTIVATIONS = {"gelu_tanh": kernels.EPI_GELU, "xielu": None}


class FeedForward(Part):
    category = "feed_forward"

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        """x[:n_rows] += ff(h[:n_rows]); h is a tensor or an ops.linear.LazyNorm (see Mixer.forward_add)."""
        raise NotImplementedError


@register_feed_forward("dense_mlp")
class DenseMLP(FeedForward):
    """u = h Wfc^T (+ b); g = 0.5 u (1 + tanh(sqrt(2/pi)(u + 0.044715 u^3))); m = g Wproj^T (+ b)
    (reference: src/minigpt_infer/model.py:96-101; there the hidden size is 4*n_embd, here it is
    a parameter).  With activation "xielu" g is instead, from two stored numbers (p, q) (the tensor `act`),
    softplus(p) u^2 + u / 2 for u > 0 and (1/2 + softplus(q)) (exp(u) - 1 - u) + u / 2 for u <= 0."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True

    def __init__(self, width: int, hidden: int, bias: bool, activation: str = "gelu_tanh") -> None:
        if activation not in _ACTIVATIONS:
            raise ValueError(f"activation {activation!r} has no kernel epilogue; known: {sorted(_ACTIVATIONS)}")
        self.width, self.hidden, self.has_bias = int(width), int(hidden), bool(bias)
        self.activation = activation
        self.fc_weight = self.fc_bias = self.proj_weight = self.proj_bias = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = {"fc_weight": WeightRequest((self.hidden, self.width), MATRIX),
               "proj_weight": WeightRequest((self.width, self.hidden), MATRIX)}
        if self.has_bias:
            req["fc_bias"] = WeightRequest((self.hidden,), VECTOR)
            req["proj_bias"] = WeightRequest((self.width,), VECTOR)
        if self.activation == "xielu":
            req["act"] = WeightRequest((2,), VECTOR)
        return req

    def bind(self, tensors):
        super().bind(tensors)
        if self.activation == "xielu":
            # the two branches' coefficients, made once: softplus(p) and 1/2 + softplus(q)
            sp = torch.nn.functional.softplus(tensors["act"].to(torch.float32))
            self.act_coef = torch.stack([sp[0], sp[1] + 0.5]).contiguous()
        return None

    def _forward_add_fused(self, ctx: StepContext, h, x: torch.Tensor) -> bool:
        """A decode-only step of few rows: one kernel from the residual (a sum, as the kernels
        before left it) through LayerNorm, both products and the activation to this part's addition
        to the residual, left as one partial sum per 64 hidden units.  False, with nothing launched,
        where that kernel does not apply."""
        parts_n = kernels.fused_mlp_parts(self.hidden)
        if not (isinstance(h, LazyNorm) and h._tensor is None and h.rows is None and h.x is x
                and getattr(h.norm, "fusable_layer_norm", False) and parts_n and residual.usable(ctx, self.width, parts_n)
                and self.activation == "gelu_tanh" and self.fc_weight.dtype == torch.bfloat16
                and self.proj_weight.dtype == torch.bfloat16):
            return False
        wfc, wproj = packed_weight(self.fc_weight, ctx), packed_weight(self.proj_weight, ctx)
        if wfc is None or wproj is None:
            return False
        n = ctx.n_rows
        if ctx.pending is not None and ctx.pending.base is None:
            residual.settle(ctx, x, n)      # table rows: this kernel reads residual rows only
        pending, settled = residual.take(ctx, x)
        parts = residual.parts_buffer(ctx, "feed_forward_parts", parts_n, n, self.width)
        if not kernels.fused_mlp_decode(pending, settled, h.norm.weight, h.norm.bias, h.norm.eps, wfc, self.fc_bias,
                                        wproj, self.proj_bias, parts, n, self.hidden):
            return False
        ctx.pending = residual.PendingSums(settled, parts, parts_n)
        return True

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        if self._forward_add_fused(ctx, h, x):
            return
        plain_residual(ctx, h, x)
        n = ctx.n_rows
        u = ctx.workspace.get("ff_hidden", n, self.hidden, ctx.dtype)
        if self.activation == "xielu":
            linear_xielu(ctx, h, self.fc_weight, self.fc_bias, u, n, self.act_coef)
        else:
            linear(ctx, h, self.fc_weight, self.fc_bias, u, n, _ACTIVATIONS[self.activation])
        # (a caller that hands over a LazyNorm of x itself knows that x may be left as a sum)
        linear_add(ctx, u, self.proj_weight, self.proj_bias, x, n,
                   may_leave_parts=isinstance(h, LazyNorm) and h.x is x)


def _gated(ctx: StepContext, h, in_weight: torch.Tensor, down_weight: torch.Tensor, x: torch.Tensor, n: int,
           hidden: int, activation: str = "silu") -> None:
    """x += (act(h Wgate^T) * (h Wup^T)) Wdown^T with the gate and up matrices stacked in in_weight."""
    z = ctx.workspace.get("gated_z", n, 2 * hidden, ctx.dtype)
    linear(ctx, h, in_weight, None, z, n)
    act = ctx.workspace.get("gated_act", n, hidden, ctx.dtype)
    kernels.gated_unit(z, act, n, hidden, fast=not ctx.exact, activation=activation)
    linear_add(ctx, act, down_weight, None, x, n)


def _stack_gate_up(part: Part, tensors, gate: str, up: str):
    """One matrix [2 * hidden, width] from a gate and an up matrix; the two names become views of it."""
    joint = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
    hidden = tensors[gate].shape[0]
    views = {gate: joint[:hidden], up: joint[hidden:]}
    for name, view in views.items():
        setattr(part, name, view)
    return joint, views


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    """m = (act(h Wgate^T) * (h Wup^T)) Wdown^T, no biases; act is silu(v) = v sigmoid(v) unless
    `activation` names relu or gelu_tanh; the unit's nonlinearity and product in float32."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, hidden: int, activation: str = "silu") -> None:
        self.width, self.hidden = int(width), int(hidden)
        if activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"gated unit: activation {activation!r} is none of {sorted(kernels.GATE_ACTIVATIONS)}")
        self.activation = activation
        self.in_weight = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"gate_weight": WeightRequest((self.hidden, self.width), MATRIX),
                "up_weight": WeightRequest((self.hidden, self.width), MATRIX),
                "down_weight": WeightRequest((self.width, self.hidden), MATRIX)}

    def bind(self, tensors):
        super().bind(tensors)
        self.in_weight, views = _stack_gate_up(self, tensors, "gate_weight", "up_weight")
        return views

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor) -> None:
        plain_residual(ctx, h, x)
        _gated(ctx, h, self.in_weight, self.down_weight, x, ctx.n_rows, self.hidden, self.activation)


@register_feed_forward("table_experts")
class TableExperts(FeedForward):
    """A mixture of gated feed-forwards without a router: row id_t of an integer table [vocab, top]
    names the experts of token t, each weighted 1 / top; a shared expert (shared_hidden > 0) takes
    every token and is added.

    The (token, choice) pairs are sorted by expert on the device, every expert multiplies its run
    of pairs by its own matrices (csrc/hip/experts.hip), and the pairs' outputs are added up per
    token in the order of the table's columns."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, hidden: int, n_experts: int, top: int, vocab_size: int,
                 shared_hidden: int = 0) -> None:
        self.width, self.hidden, self.n_experts, self.top = int(width), int(hidden), int(n_experts), int(top)
        self.vocab_size, self.shared_hidden = int(vocab_size), int(shared_hidden)
        if not 0 < self.top <= self.n_experts <= kernels.MAX_EXPERTS:
            raise ValueError(f"top {self.top} of {self.n_experts} experts: need 0 < top <= experts <= {kernels.MAX_EXPERTS}")
        self.in_weights = self.down_weights = self.shared_in_weight = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = {"table": WeightRequest((self.vocab_size, self.top), TABLE)}
        for e in range(self.n_experts):
            req[f"e{e}_gate"] = WeightRequest((self.hidden, self.width), MATRIX)
            req[f"e{e}_up"] = WeightRequest((self.hidden, self.width), MATRIX)
            req[f"e{e}_down"] = WeightRequest((self.width, self.hidden), MATRIX)
        if self.shared_hidden:
            req["shared_gate"] = WeightRequest((self.shared_hidden, self.width), MATRIX)
            req["shared_up"] = WeightRequest((self.shared_hidden, self.width), MATRIX)
            req["shared_down"] = WeightRequest((self.width, self.shared_hidden), MATRIX)
        return req

    def bind(self, tensors):
        self.table = tensors["table"]
        if self.table.dtype != torch.int32:
            raise ValueError("the experts' table must hold integers")
        return self._bind_experts(tensors)

    def _bind_experts(self, tensors):
        f, views = self.hidden, {}
        # [experts, 2 * hidden, width] and [experts, width, hidden]: an expert's matrices lie together
        self.in_weights = torch.stack([torch.cat([tensors[f"e{e}_gate"], tensors[f"e{e}_up"]], dim=0)
                                       for e in range(self.n_experts)]).contiguous()
        self.down_weights = torch.stack([tensors[f"e{e}_down"] for e in range(self.n_experts)]).contiguous()
        for e in range(self.n_experts):
            views[f"e{e}_gate"], views[f"e{e}_up"] = self.in_weights[e, :f], self.in_weights[e, f:]
            views[f"e{e}_down"] = self.down_weights[e]
        if self.shared_hidden:
            self.shared_down = tensors["shared_down"]
            self.shared_in_weight, shared = _stack_gate_up(self, tensors, "shared_gate", "shared_up")
            views.update(shared)
        return views

    def token_matrix_elements(self) -> int:
        """Matrix elements one token goes through: its `top` experts and the shared one."""
        return 3 * self.width * (self.top * self.hidden + self.shared_hidden)

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor) -> None:
        plain_residual(ctx, h, x)
        hn = as_tensor(ctx, h)
        self._experts_add(ctx, hn, x, ctx.n_rows, ctx.token_ids, self.table, None, 1.0 / self.top)

    def _experts_add(self, ctx: StepContext, hn: torch.Tensor, x: torch.Tensor, n: int, ids, table: torch.Tensor,
                     pair_weight, combine_weight: float) -> None:
        """x += combine_weight * sum over token n's experts (row ids[n] of the table, or row n without ids) of
        expert(w h), w = pair_weight[n][choice] (None: 1), plus the shared expert."""
        ws = ctx.workspace
        fast = not ctx.exact and ctx.dtype == torch.bfloat16
        if fast and n * self.top >= self.TILED_FROM_PAIRS and self.width % 16 == 0 and self.hidden % 16 == 0 \
                and self._forward_tiled(ctx, hn, x, n, ids, table, pair_weight, combine_weight):
            return
        # tiles of 64 slots for the MFMA kernel of few rows, of 16 for the general one, and for the MFMA kernel too
        # where an expert gets 16 pairs at most on average (a decode step): a tile's empty slots are loaded and
        # multiplied like the used ones
        tile = 64 if fast and n * self.top > 16 * self.n_experts else 16
        slots = kernels.expert_slots(n, self.top, self.n_experts, tile)
        slot_token = ws.get("expert_slot_token", slots, 1, torch.int32).view(-1)
        slot_pair = ws.get("expert_slot_pair", slots, 1, torch.int32).view(-1)
        tile_expert = ws.get("expert_tile", slots // tile, 1, torch.int32).view(-1)
        kernels.expert_route(ids, ctx.q_req, table, n, self.n_experts, slot_token, slot_pair, tile_expert, tile)
        z = ws.get("expert_z", slots, 2 * self.hidden, ctx.dtype)
        if pair_weight is None:
            kernels.grouped_linear(hn, slot_token, self.in_weights, tile_expert, slot_token, z, None, slots, tile, fast)
        else:
            # the weight multiplies the expert's input: every pair's row is made first, scaled, in the experts' order
            rows = ws.get("expert_rows", slots, self.width, ctx.dtype)
            kernels.gather_scale_rows(hn, slot_token, slot_pair, pair_weight, rows, slots)
            kernels.grouped_linear(rows, None, self.in_weights, tile_expert, slot_token, z, None, slots, tile, fast)
        act = ws.get("expert_act", slots, self.hidden, ctx.dtype)
        kernels.gated_unit(z, act, slots, self.hidden, fast=not ctx.exact)
        pair_out = ws.get("expert_pair_out", n * self.top, self.width, torch.float32)
        kernels.grouped_linear(act, None, self.down_weights, tile_expert, slot_token, pair_out, slot_pair, slots,
                               tile, fast)
        if self.shared_hidden:
            _gated(ctx, hn, self.shared_in_weight, self.shared_down, x, n, self.shared_hidden)
        kernels.expert_combine(pair_out, x, n, self.top, combine_weight, q_req=ctx.q_req)

    # From this many (token, choice) pairs on, the experts' products go through the tiled MFMA kernel
    # of the dense layers: the pairs' rows are copied into the experts' order first, every expert's
    # run padded to whole tiles of 256 slots, so that a tile of that kernel multiplies one expert's
    # matrix.  Below it a step is a decode step or a short portion, and padding every expert to 256
    # rows would be most of the work.
    TILED_FROM_PAIRS = 512

    def _forward_tiled(self, ctx: StepContext, hn: torch.Tensor, x: torch.Tensor, n: int, ids, table: torch.Tensor,
                       pair_weight, combine_weight: float) -> bool:
        ws, tile = ctx.workspace, 256
        slots = kernels.expert_slots(n, self.top, self.n_experts, tile)
        slot_token = ws.get("expert_slot_token", slots, 1, torch.int32).view(-1)
        slot_pair = ws.get("expert_slot_pair", slots, 1, torch.int32).view(-1)
        pair_slot = ws.get("expert_pair_slot", n * self.top, 1, torch.int32).view(-1)
        tile_expert = ws.get("expert_tile", slots // tile, 1, torch.int32).view(-1)
        sorted_rows = ws.get("expert_rows", slots, self.width, ctx.dtype)
        if hn.stride(0) % 8 or hn.data_ptr() % 16 or sorted_rows.data_ptr() % 16 or self.width % 8:
            return False
        kernels.expert_route(ids, ctx.q_req, table, n, self.n_experts, slot_token, slot_pair,
                             tile_expert, tile, pair_slot=pair_slot)
        if pair_weight is not None:
            kernels.gather_scale_rows(hn, slot_token, slot_pair, pair_weight, sorted_rows, slots)
        elif not kernels.gather_rows(hn, slot_token, sorted_rows, slots):
            return False
        z = ws.get("expert_z", slots, 2 * self.hidden, ctx.dtype)
        if not kernels.grouped_linear_tiled(sorted_rows, self.in_weights, tile_expert, slot_token, z, slots):
            return False
        act = ws.get("expert_act", slots, self.hidden, ctx.dtype)
        kernels.gated_unit(z, act, slots, self.hidden, fast=True)
        slot_out = ws.get("expert_slot_out", slots, self.width, torch.float32)
        if not kernels.grouped_linear_tiled(act, self.down_weights, tile_expert, slot_token, slot_out, slots):
            return False
        if self.shared_hidden:
            _gated(ctx, hn, self.shared_in_weight, self.shared_down, x, n, self.shared_hidden)
        kernels.expert_combine(slot_out, x, n, self.top, combine_weight, pair_slot=pair_slot, q_req=ctx.q_req)
        return True


@register_feed_forward("routed_experts")
class RoutedExperts(TableExperts):
    """A mixture of gated feed-forwards chosen by a router: scores s = sigmoid(h Wr^T), computed in
    float32; a token uses the `top` experts with the largest scores; the output is the sum over them of
    expert_e(s_e h), expert(u) = (silu(u Wgate^T) * (u Wup^T)) Wdown^T: the score multiplies the expert's
    input and is not renormalised.  A shared expert (shared_hidden > 0) takes every token unweighted.

    The router kernel writes the step's own table of experts and scores; from there on the experts run as
    those chosen by a stored table do."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, hidden: int, n_experts: int, top: int, shared_hidden: int = 0,
                 score: str = "sigmoid") -> None:
        super().__init__(width, hidden, n_experts, top, vocab_size=0, shared_hidden=shared_hidden)
        if score not in kernels.ROUTER_SCORES:
            raise ValueError(f"router score {score!r} is none of {sorted(kernels.ROUTER_SCORES)}")
        self.score = score

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = super().weight_requests()
        del req["table"]
        req["router_weight"] = WeightRequest((self.n_experts, self.width), MATRIX)
        return req

    def bind(self, tensors):
        self.router_weight = tensors["router_weight"]
        return self._bind_experts(tensors)

    def token_matrix_elements(self) -> int:
        return super().token_matrix_elements() + self.n_experts * self.width

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor) -> None:
        plain_residual(ctx, h, x)
        n, ws = ctx.n_rows, ctx.workspace
        hn = as_tensor(ctx, h)
        chosen = ws.get("router_chosen", n, self.top, torch.int32)
        weight = ws.get("router_weight", n, self.top, torch.float32)
        kernels.router_topk(hn, self.router_weight, n, self.top, chosen, weight, q_req=ctx.q_req, score=self.score)
        self._experts_add(ctx, hn, x, n, None, chosen, weight.view(-1), 1.0)
