"""Arrangements: how a layer's norm, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

from typing import Dict, Mapping, Optional, Tuple

import torch

from ..ops import kernels, residual
from ..ops.linear import LazyNorm
from .base import CacheBinding, Part, StepContext, VECTOR, WeightRequest, register_arrangement
from .feedforward import FeedForward
from .mixers import Mixer
from .positions import PositionEncoding


class Arrangement(Part):
    """How a layer's parts sit around the residual stream.  `roles` names the parts it arranges (the
    model refuses a layer whose parts are others); run() gets them by role, and for every mixer role
    the binding of this run's cache."""

    category = "arrangement"
    roles: Optional[Tuple[str, ...]] = None     # None: whatever the layer brings

    def run(self, ctx: StepContext, x: torch.Tensor, parts: Mapping[str, Part],
            bindings: Mapping[str, CacheBinding], position: PositionEncoding) -> None:
        raise NotImplementedError


@register_arrangement("pre_norm")
class PreNorm(Arrangement):
    """x = x + mixer(norm1(x)); x = x + ff(norm2(x)) (reference: src/minigpt_infer/model.py:112-115)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True
    roles = ("norm1", "mixer", "norm2", "feed_forward")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        norm1, mixer, norm2, feed_forward = (parts[r] for r in self.roles)
        binding = bindings["mixer"]
        # the norms are handed on uncomputed: a linear layer that can normalise in its prologue
        # does, everything else calls .tensor(ctx) and gets the normed rows.  A part that does not
        # know of a residual whose sums are still pending gets a plain one.
        n = ctx.n_rows
        if not mixer.takes_pending_residual:
            residual.settle(ctx, x, n)
        mixer.forward_add(ctx, LazyNorm(norm1, x, n), x, binding, position)
        if not feed_forward.takes_pending_residual:
            residual.settle(ctx, x, n)
        feed_forward.forward_add(ctx, LazyNorm(norm2, x, n), x)


@register_arrangement("pre_norm_mixer")
class PreNormMixerOnly(Arrangement):
    """x = x + mixer(norm1(x)): a pre-norm layer that has no feed-forward."""

    graph_safe = True
    plan_safe = True
    takes_pending_residual = True
    roles = ("norm1", "mixer")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        mixer = parts["mixer"]
        if not mixer.takes_pending_residual:
            residual.settle(ctx, x, ctx.n_rows)
        mixer.forward_add(ctx, LazyNorm(parts["norm1"], x, ctx.n_rows), x, bindings["mixer"], position)


def flush_streams(ctx: StepContext, x: torch.Tensor, streams: int) -> None:
    """Makes the write into the residual streams that a sublayer has left pending, if any."""
    if ctx.pending_streams is not None:
        mix, out, y = ctx.pending_streams
        ctx.pending_streams = None
        kernels.streams_write(x, mix, out, y, ctx.n_rows, streams)


@register_arrangement("hyper_connections")
class HyperConnections(Arrangement):
    """A pre-norm layer over several residual streams.  A token's residual is S rows x_1 .. x_S.
    For sublayer q (1: the mixer, 2: the feed-forward, which a layer may lack) with its own
    a_q [S], M_q [S, S] and b_q [S]:

        u = sum_s a_q[s] x_s;  y = sublayer_q(norm_q(u));  x_t <- sum_s M_q[s, t] x_s + b_q[t] y

    every new stream from the old ones, all in float32.  With S = 1, a = b = 1 and M = 1 this is
    the plain pre-norm layer.  The sublayers are the framework's ordinary parts: they add their
    output into a cleared buffer that stands for y.  A sublayer's write is left pending
    (ctx.pending_streams) and made by the kernel that reads the streams next: the next sublayer's
    read and LayerNorm, or the model before the final norm."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, streams: int, feed_forward: bool = True) -> None:
        self.width, self.streams = int(width), int(streams)
        if not 1 <= self.streams <= kernels.MAX_STREAMS:
            raise ValueError(f"{self.streams} residual streams: the kernels take 1 to {kernels.MAX_STREAMS}")
        self.has_feed_forward = bool(feed_forward)
        self.roles = ("norm1", "mixer", "norm2", "feed_forward") if self.has_feed_forward else ("norm1", "mixer")

    def weight_requests(self) -> Dict[str, WeightRequest]:
        s, req = self.streams, {}
        for q in ("1", "2") if self.has_feed_forward else ("1",):
            req["in" + q] = WeightRequest((s,), VECTOR)
            req["out" + q] = WeightRequest((s,), VECTOR)
            req["mix" + q] = WeightRequest((s, s), VECTOR)
        return req

    # the arrangement reads ctx.pending_streams: a write that the sublayer before (of this layer or of
    # the one before) has left to be made together with this sublayer's read
    takes_pending_streams = True

    def _sublayer(self, ctx: StepContext, x: torch.Tensor, q: str, norm: Part, call) -> None:
        n, ws = ctx.n_rows, ctx.workspace
        u = ws.get("streams_read", n, self.width, torch.float32)
        y = ws.get("streams_update", n, self.width, torch.float32)
        if getattr(norm, "fusable_layer_norm", False):
            # one kernel: the write left over from the sublayer before, y cleared, this sublayer's
            # read and its LayerNorm
            h = ws.get("normed", n, self.width, ctx.dtype)
            kernels.streams_step(x, ctx.pending_streams, getattr(self, "in" + q), u, norm.weight, norm.bias, norm.eps,
                                 h, n, self.streams, zero=y)
            ctx.pending_streams = None
        else:
            flush_streams(ctx, x, self.streams)
            kernels.streams_read(x, getattr(self, "in" + q), u, n, self.streams, zero=y)
            h = LazyNorm(norm, u, n)
        call(h, y)
        ctx.pending_streams = (getattr(self, "mix" + q), getattr(self, "out" + q), y)

    def run(self, ctx, x, parts, bindings, position) -> None:
        mixer = parts["mixer"]
        self._sublayer(ctx, x, "1", parts["norm1"],
                       lambda h, y: mixer.forward_add(ctx, h, y, bindings["mixer"], position))
        if self.has_feed_forward:
            feed_forward = parts["feed_forward"]
            self._sublayer(ctx, x, "2", parts["norm2"], lambda h, y: feed_forward.forward_add(ctx, h, y))


@register_arrangement("sandwich_norm")
class SandwichNorm(Arrangement):
    """A layer whose sublayers are normed on both sides and whose additions to the residual are scaled:

        x <- x + m * norm1b(mixer(norm1(x)));   x <- x + m * norm2b(ff(norm2(x)))

    with m = `residual_mult`; the feed-forward half is optional.  With `branches` = B > 1 the mixer is
    B mixers side by side that read the same norm1(x) (roles mixer0 .. mixer{B-1}), and what norm1b
    sees is the mean of their outputs, each first normed with a gain of its own (roles join0 ..):
    (1 / B) * sum_b join_b(mixer_b(h)); with `join_weights` = (c_0, .., c_(B-1)) it is the weighted sum
    sum_b c_b mixer_b(h) instead, and there are no join norms.  With `layer_scale` each sublayer's normed
    output is multiplied channel by channel by a vector of the layer's own (`scale1`, `scale2`) before
    it is added.  All norms are RMS norms (kind "rms_norm"); the norms around the sublayers share one
    eps and one way of storing the gain, the joins have plain gains.

    The sublayers are the framework's ordinary parts: they add their output into a cleared float32
    buffer.  One kernel stands between two sublayers: it joins the branches, norms the sum, adds it
    to the residual, computes the next sublayer's input norm and clears the buffers again."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, residual_mult: float = 1.0, feed_forward: bool = True, branches: int = 1,
                 join_weights=None, layer_scale: bool = False) -> None:
        self.width, self.mult = int(width), float(residual_mult)
        self.has_feed_forward, self.branches = bool(feed_forward), int(branches)
        if not 1 <= self.branches <= kernels.MAX_NORM_BRANCHES:
            raise ValueError(f"{self.branches} parallel mixers: the kernels take 1 to {kernels.MAX_NORM_BRANCHES}")
        self.join_weights = None if join_weights is None else tuple(float(c) for c in join_weights)
        if self.join_weights is not None and (self.branches < 2 or len(self.join_weights) != self.branches):
            raise ValueError("join_weights gives one weight per parallel mixer")
        self.has_layer_scale = bool(layer_scale)
        if self.branches == 1:
            self.mixer_roles, self.join_roles = ("mixer",), ()
        else:
            self.mixer_roles = tuple(f"mixer{b}" for b in range(self.branches))
            self.join_roles = () if self.join_weights is not None else tuple(f"join{b}" for b in range(self.branches))
        self.roles = ("norm1",) + self.mixer_roles + self.join_roles + ("norm1b",)
        if self.has_feed_forward:
            self.roles += ("norm2", "feed_forward", "norm2b")
        self._checked = False
        self.scale1 = self.scale2 = None
        self._join_gains = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        if not self.has_layer_scale:
            return {}
        req = {"scale1": WeightRequest((self.width,), VECTOR)}
        if self.has_feed_forward:
            req["scale2"] = WeightRequest((self.width,), VECTOR)
        return req

    def bind(self, tensors):
        super().bind(tensors)
        first = next(iter(tensors.values()), None)
        if first is not None and self.join_weights is not None:      # made here, not inside a step
            self._join_gains = [torch.full((self.width,), c, dtype=torch.float32, device=first.device)
                                for c in self.join_weights]
        return None

    def _joins(self, ys, parts):
        """Per branch: its buffer and the vector that multiplies it in the join (a join norm's gain, or the
        branch's constant weight on every channel)."""
        if self.branches == 1:
            return [(ys[0], None)]
        if self.join_weights is None:
            return [(ys[b], parts[self.join_roles[b]].weight) for b in range(self.branches)]
        if self._join_gains is None or self._join_gains[0].device != ys.device:
            self._join_gains = [torch.full((self.width,), c, dtype=torch.float32, device=ys.device)
                                for c in self.join_weights]
        return [(ys[b], self._join_gains[b]) for b in range(self.branches)]

    def _check(self, parts) -> None:
        around = [parts[r] for r in self.roles if r.startswith("norm")]
        for p in around + [parts[r] for r in self.join_roles]:
            if not (hasattr(p, "offset") and getattr(p, "has_weight", False) and p.width == self.width):
                raise ValueError("a sandwich-norm layer takes RMS norms with gains as wide as the model")
        if len({(p.eps, p.offset) for p in around}) != 1 or any(parts[r].eps != around[0].eps for r in self.join_roles):
            raise ValueError("the norms of a sandwich-norm layer share one eps and one way of storing the gain")
        if any(parts[r].offset != 0.0 for r in self.join_roles):
            raise ValueError("the norms that join parallel mixers have plain gains")
        self._checked = True

    # the arrangement reads ctx.pending_update: the addition that the layer before has left to be made
    # together with this layer's first norm
    takes_pending_update = True

    def _buffers(self, ctx) -> torch.Tensor:
        """[branches, rows, width] float32, zero: what the sublayers add their outputs into.  A buffer per number of
        branches (one that grew from layer to layer inside a step would move); cleared when it is made, and by
        the kernel that takes the sums out of it ever after."""
        ws, n, B = ctx.workspace, ctx.n_rows, self.branches
        made = ws.generation
        flat = ws.get(f"sublayer_sums_{B}", B * n, self.width, torch.float32)
        if ws.generation != made:
            flat.zero_()
        return flat[:B * n].view(B, n, self.width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        if not self._checked:
            self._check(parts)
        n, B = ctx.n_rows, self.branches
        norm1 = parts["norm1"]
        ys = self._buffers(ctx)
        h = ctx.workspace.get("normed", n, self.width, ctx.dtype)
        left, ctx.pending_update = ctx.pending_update, None
        if left is not None and left.goes_with(norm1, x, n):
            left.run(norm1.weight, h)       # the layer before's last addition and this layer's first norm in one kernel
        else:
            if left is not None:
                left.run(None, None)
            norm1.forward(ctx, x, h, n)
        for b, role in enumerate(self.mixer_roles):
            parts[role].forward_add(ctx, h, ys[b], bindings[role], position)
        joins = self._joins(ys, parts)
        join_unit = self.join_weights is None
        if not self.has_feed_forward:
            ctx.pending_update = PendingSandwich(joins, x, parts["norm1b"], self.mult, n, join_unit, self.scale1)
            return
        norm1b = parts["norm1b"]
        kernels.rms_post_norm(joins, x, norm1b.weight, n, norm1b.eps, norm1b.offset, self.mult,
                              gain_next=parts["norm2"].weight, h=h, join_unit=join_unit, scale_post=self.scale1)
        parts["feed_forward"].forward_add(ctx, h, ys[0])
        ctx.pending_update = PendingSandwich([(ys[0], None)], x, parts["norm2b"], self.mult, n, True, self.scale2)


@register_arrangement("parallel_shift")
class ParallelShift(Arrangement):
    """A layer with one norm whose sublayers all read it and are added together:

        h = norm1(x);   x <- x + m * (mixer(shifted(h)) + ff(h))

    with m = `residual_mult`; the feed-forward is optional.  With `token_shift` the mixer (not the feed-forward)
    reads h blended with the previous token's: shifted(h)_t = h_t + (h_(t-1) - h_t) * shift, channel by channel,
    `shift` a vector of the layer, h_(-1) = 0.  The h of a request's last token is kept per request in a
    state pool of the arrangement's own.  norm1 is an RMS norm (kind "rms_norm") with a gain.

    The sublayers are the framework's ordinary parts: they add their output into one cleared float32 buffer.
    The addition to the residual is left pending and made by the next layer's norm kernel (or by whoever
    reads the residual next)."""

    graph_safe = True
    plan_safe = True
    takes_pending_update = True

    def __init__(self, width: int, residual_mult: float = 1.0, feed_forward: bool = True, token_shift: bool = False) -> None:
        self.width, self.mult = int(width), float(residual_mult)
        self.has_feed_forward, self.has_shift = bool(feed_forward), bool(token_shift)
        self.roles = ("norm1", "mixer") + (("feed_forward",) if self.has_feed_forward else ())
        self.shift = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"shift": WeightRequest((self.width,), VECTOR)} if self.has_shift else {}

    def state_numel(self) -> int:
        """float32 values kept per request: the last token's normed row."""
        return self.width if self.has_shift else 0

    def run(self, ctx, x, parts, bindings, position) -> None:
        norm1 = parts["norm1"]
        if not (hasattr(norm1, "offset") and getattr(norm1, "has_weight", False) and norm1.width == self.width):
            raise ValueError("a parallel layer takes an RMS norm with a gain as wide as the model")
        n, ws = ctx.n_rows, ctx.workspace
        made = ws.generation
        y = ws.get("parallel_sums", n, self.width, torch.float32)
        if ws.generation != made:
            y.zero_()       # cleared when it is made, and by the kernel that takes the sums out of it ever after
        h = ws.get("normed", n, self.width, ctx.dtype)
        hs = ws.get("normed_shifted", n, self.width, ctx.dtype) if self.has_shift else None
        left, ctx.pending_update = ctx.pending_update, None
        y_before, mult_before = None, 0.0
        if isinstance(left, PendingParallel) and left.goes_with(x, n):
            y_before, mult_before = left.y, left.mult     # the layer before's addition and this layer's norm in one kernel
        elif left is not None:
            left.run(None, None)
        state = ctx.state_pools[bindings[STATE_ROLE].index] if self.has_shift else None
        # every request brings one token: a row's neighbour in time is its request's kept row, and the same kernel
        # shifts and keeps; else the shift reads the step's rows and runs behind the norm
        single = self.has_shift and ctx.decode_only
        kernels.parallel_norm(x, y_before, mult_before, n, gain=norm1.weight, offset=norm1.offset, eps=norm1.eps, h=h,
                              hs=hs if single else None, shift=self.shift, state=state, state_slots=ctx.state_slots,
                              q_req=ctx.q_req, positions=ctx.positions)
        if self.has_shift and not single:
            kernels.token_shift(h, hs, self.shift, state, ctx.state_slots, ctx.q_req, ctx.cu_q, ctx.positions, n,
                                ctx.cu_q.numel() - 1)
        parts["mixer"].forward_add(ctx, hs if self.has_shift else h, y, bindings["mixer"], position)
        if self.has_feed_forward:
            parts["feed_forward"].forward_add(ctx, h, y)
        ctx.pending_update = PendingParallel(x, y, self.mult, n)


STATE_ROLE = "arrangement"     # the name under which a run's bindings hold an arrangement's own state pool


class PendingParallel:
    """The sum of a parallel layer's sublayers that is still to be added to the residual: x += mult * y, y = 0."""

    def __init__(self, x: torch.Tensor, y: torch.Tensor, mult: float, n_rows: int) -> None:
        self.x, self.y, self.mult, self.n_rows = x, y, mult, n_rows

    def goes_with(self, *args) -> bool:
        """(x, n_rows): whether a parallel layer over these rows may make the addition in its norm kernel; asked
        with anything else (another arrangement's norm), no."""
        return len(args) == 2 and args[0] is self.x and args[1] == self.n_rows

    def run(self, gain_next=None, h=None) -> None:
        kernels.parallel_norm(self.x, self.y, self.mult, self.n_rows)


class PendingSandwich:
    """A sublayer's output that is still to be normed and added to the residual: x += mult * norm(y).  Whoever
    reads x next makes the addition: a layer of the same kind together with its first norm (run(gain, h) also
    leaves h = norm_next(x)), anyone else through flush_update."""

    def __init__(self, joins, x: torch.Tensor, norm: Part, mult: float, n_rows: int, join_unit: bool = True,
                 scale: Optional[torch.Tensor] = None) -> None:
        self.joins, self.x, self.norm, self.mult, self.n_rows = joins, x, norm, mult, n_rows
        self.join_unit, self.scale = join_unit, scale      # how several branches meet; the layer's scale per channel

    def goes_with(self, norm_next: Part, x: torch.Tensor, n_rows: int) -> bool:
        return (x is self.x and n_rows == self.n_rows and norm_next.eps == self.norm.eps
                and norm_next.offset == self.norm.offset)

    def run(self, gain_next: Optional[torch.Tensor], h: Optional[torch.Tensor]) -> None:
        kernels.rms_post_norm(self.joins, self.x, self.norm.weight, self.n_rows, self.norm.eps, self.norm.offset,
                              self.mult, gain_next=gain_next, h=h, join_unit=self.join_unit, scale_post=self.scale)


def flush_update(ctx: StepContext) -> None:
    """Makes the addition to the residual that a layer has left pending, if any."""
    if ctx.pending_update is not None:
        left, ctx.pending_update = ctx.pending_update, None
        left.run(None, None)
