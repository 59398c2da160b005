"""Sequence mixers.  A mixer adds its output into the residual stream."""

from __future__ import annotations

from typing import Dict, Optional, Union

import torch

from ..ops import attention as attention_ops
from ..ops import kernels, residual
from ..ops.linear import LazyNorm, as_tensor, linear, linear_add, packed_weight, plain_residual
from .base import (CacheBinding, KVNeed, MATRIX, POSITIONS, Part, PartSpec, StateNeed, StepContext, VECTOR,
                   WeightRequest, register_mixer)
from .positions import PositionEncoding


class Mixer(Part):
    category = "mixer"

    def cache_need(self) -> Union[KVNeed, StateNeed, None]:
        return None

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        """x[:n_rows] += mixer(h[:n_rows]).  x is the float32 residual stream; h is the normed input,
        either a tensor in the compute dtype or an ops.linear.LazyNorm, which linear() takes as it
        is and as_tensor(ctx, h) turns into a tensor."""
        raise NotImplementedError


@register_mixer("paged_causal_attention")
class PagedCausalAttention(Mixer):
    """Multi-head causal self-attention over the paged cache.

    qkv = h Wqkv^T (+ b); q = columns [0, H*D), k = the next Hkv*D, v = the last Hkv*D, head i of
    each = columns i*D..(i+1)*D (reference: src/minigpt_infer/model.py:43,49-53).  New keys and
    values are stored unscaled before attention reads everything up to and including them
    (model.py:55-59).  S = q k^T * scale with scale = 1/sqrt(D) unless given (SDPA's default,
    model.py:87); a query sees the keys of its own request at positions <= its own (and, with a
    window, only the last `window` of them); softmax in float32; y = P v; heads concatenated
    head-major; out = y Wproj^T (+ b) (model.py:89-90), added into the residual (model.py:113)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True

    def __init__(self, width: int, n_head: int, head_dim: int, bias: bool, n_kv_head: Optional[int] = None,
                 scale: Optional[float] = None, window: int = 0) -> None:
        self.width, self.n_head, self.head_dim = int(width), int(n_head), int(head_dim)
        self.n_kv_head = int(n_kv_head) if n_kv_head is not None else self.n_head
        self.has_bias = bool(bias)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window = int(window)
        if not 0 < self.head_dim <= 256:
            raise ValueError(f"head size {self.head_dim}: the kernels take head sizes up to 256")
        if self.n_head % self.n_kv_head != 0:
            raise ValueError("n_head must be a multiple of n_kv_head")
        self.q_width = self.n_head * self.head_dim
        self.kv_width = self.n_kv_head * self.head_dim
        self.qkv_weight = self.qkv_bias = self.proj_weight = self.proj_bias = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        total = self.q_width + 2 * self.kv_width
        req = {"qkv_weight": WeightRequest((total, self.width), MATRIX),
               "proj_weight": WeightRequest((self.width, self.q_width), MATRIX)}
        if self.has_bias:
            req["qkv_bias"] = WeightRequest((total,), VECTOR)
            req["proj_bias"] = WeightRequest((self.width,), VECTOR)
        return req

    def cache_need(self) -> KVNeed:
        return KVNeed(self.n_kv_head, self.head_dim, self.window)

    def _forward_add_fused(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                           position: PositionEncoding) -> bool:
        """A decode-only step of few rows: one kernel from the residual (as the kernels before left
        it: a sum) through LayerNorm, projections, cache write and attention to this mixer's
        addition to the residual, left as one partial sum per head.  False where that kernel does
        not apply (with nothing launched but, in a step of many rows, the LayerNorm that the other
        path needs as well)."""
        if not (isinstance(h, LazyNorm) and h._tensor is None and h.rows is None and h.x is x
                and getattr(h.norm, "fusable_layer_norm", False) and residual.usable(ctx, self.width, self.n_head)
                and binding.writes and not position.rotates and self.window == 0
                and self.n_kv_head == self.n_head and self.qkv_weight.dtype == torch.bfloat16
                and self.proj_weight.dtype == torch.bfloat16):
            return False
        wqkv, wproj = packed_weight(self.qkv_weight, ctx), packed_weight(self.proj_weight, ctx)
        if wqkv is None or wproj is None:
            return False
        n = ctx.n_rows
        group = ctx.groups[binding.group]
        # In a step of so many rows that a workgroup takes several tokens, every head's workgroup
        # adding up its tokens' pending parts would be most of the kernel's traffic: the LayerNorm
        # kernel adds them up once (x is plain after it) and hands the rows over normed.
        normed = None
        table_rows = ctx.pending is not None and ctx.pending.base is None
        tokens = kernels.fused_attention_tokens(n, self.n_head, self.head_dim)
        if tokens == 0:
            return False
        if not table_rows and tokens > 1:
            normed = h.tensor(ctx)
            if ctx.pending is not None:
                return False
        pending, settled = residual.take(ctx, x)
        parts = residual.parts_buffer(ctx, "attention_parts", self.n_head, n, self.width)
        if not kernels.fused_attention_decode(
                pending, settled, h.norm.weight, h.norm.bias, h.norm.eps, wqkv, self.qkv_bias, wproj, self.proj_bias,
                parts, group.k_pools[binding.index], group.v_pools[binding.index], group.slot_mapping,
                group.block_tables, ctx.positions, ctx.q_req, n, self.n_head, self.scale, normed=normed):
            return False
        ctx.pending = residual.PendingSums(x if normed is not None else settled, parts, self.n_head)
        return True

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if self._forward_add_fused(ctx, h, x, binding, position):
            return
        plain_residual(ctx, h, x)
        n = ctx.n_rows
        total = self.q_width + 2 * self.kv_width
        qkv = ctx.workspace.get("qkv", n, total, ctx.dtype)
        group = ctx.groups[binding.group]
        k_pool, v_pool = group.k_pools[binding.index], group.v_pools[binding.index]
        # a position encoding that rotates queries and keys must act before the keys are stored;
        # only without one may the projection kernel store them itself
        scatter = None
        if binding.writes and not position.rotates:
            scatter = (k_pool, v_pool, group.slot_mapping, self.q_width, self.kv_width)
        stored = linear(ctx, h, self.qkv_weight, self.qkv_bias, qkv, n, scatter=scatter)
        position.rotate(ctx, qkv[:, :self.q_width], qkv[:, self.q_width:self.q_width + self.kv_width], n)
        if binding.writes and not stored:
            kernels.kv_write(qkv, self.q_width, self.q_width + self.kv_width, k_pool, v_pool,
                             group.slot_mapping, n)
        y = ctx.workspace.get("attn_out", n, self.q_width, ctx.dtype)
        attention_ops.paged_attention(ctx, qkv, y, k_pool, v_pool, group, self.n_head, self.scale, self.window)
        linear_add(ctx, y, self.proj_weight, self.proj_bias, x, n,
                   may_leave_parts=isinstance(h, LazyNorm) and h.x is x)


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Attention whose keys and values are made from one small latent per token, which is all the
    cache keeps (one joint tensor per page).

    c = rms_norm(h Wdkv^T) * gain, [rank], stored into the pages.  Per head a: q_a = h Wq_a^T [D],
    k_a = Wuk_a c [D], v_a = Wuv_a c [E]; S = (q_a . k_a) * scale over the keys at positions
    p - window < j <= p (window 0: all j <= p); softmax in float32 with one more term exp(sink_a) in
    the denominator that has no value; y = concat_a(P v_a) * sigmoid(h Wg^T); out = y Wo^T, added
    into the residual.  The gate is a number per channel of y (`gate` "channel", Wg [H * E, W]) or a
    number per head ("head", Wg [H, W]).

    With `rot_dim` = P > 0 a position signal rides beside the latent: a query head is [D plain | P rotated]
    channels (Wq has H (D + P) rows), Wdkv has rank + P rows of which the last P, not normed, are one key part
    kr that all heads share, and S = (q_plain . k_a + rot(q_rot) . rot(kr)) * scale with `rotary` (the mixer's
    own rotation over P channels).  The cache then keeps [c | rot(kr)] per token.

    The kernels never make k_a and v_a: (q_a . Wuk_a c) = (Wuk_a^T q_a) . c, so the queries are
    folded onto the latent basis (one product per head, which passes the rotated part through), attention
    runs with one key/value head of the cached row's size that every query head shares, and its output
    sum_j P_j c_j is unfolded by Wuv_a afterwards (which has no columns for the rotated part).  A layer with
    makes_latent=False has no Wdkv: it reads the pages that another run
    of the same step wrote (LayerRun.reads_cache_of), with its own Wuk, Wuv, window and the rest."""

    graph_safe = True
    plan_safe = True
    # up to this many rows queries, gate and latent come from one product with the matrices stacked
    # (one launch less in a decode step); beyond it from two
    JOINT_PRODUCT_MAX_ROWS = 128
    JOINT_PRODUCT_MAX_WORK = 4 << 20     # rows x (query + gate columns); a smaller product has no full round to lose

    def __init__(self, width: int, n_head: int, head_dim: int, value_dim: int, rank: int, scale: float,
                 window: int = 0, eps: float = 1e-6, makes_latent: bool = True, rot_dim: int = 0,
                 rotary: Optional[dict] = None, gate: str = "channel") -> None:
        self.width, self.n_head, self.head_dim = int(width), int(n_head), int(head_dim)
        self.value_dim, self.rank = int(value_dim), int(rank)
        self.scale, self.window, self.eps = float(scale), int(window), float(eps)
        self.makes_latent = bool(makes_latent)
        self.rot_dim = int(rot_dim or 0)
        self.rotation = _own_rotation(rotary) if self.rot_dim else None
        if self.rot_dim and (self.rotation is None or self.rotation.dims != self.rot_dim):
            raise ValueError("a latent with a rotated part needs a rotation over exactly rot_dim channels")
        if gate not in ("channel", "head"):
            raise ValueError(f"gate {gate!r} is neither 'channel' nor 'head'")
        self.head_gate = gate == "head"
        # what a cached row holds: the latent alone, or the latent and the rotated key part (rows then
        # start 16 bytes apart in bfloat16 too)
        self.row = self.rank if not self.rot_dim else -(-(self.rank + self.rot_dim) // 8) * 8
        if not 0 < self.row <= 1024:
            raise ValueError(f"latent size {self.row}: the attention kernels take up to 1024")
        self.q_head = self.head_dim + self.rot_dim
        self.q_width = self.n_head * self.q_head
        self.y_width = self.n_head * self.value_dim
        self.g_width = self.n_head if self.head_gate else self.y_width
        self.in_weight = self.uk_folded = self.uv_heads = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = {"q_weight": WeightRequest((self.q_width, self.width), MATRIX),
               "gate_weight": WeightRequest((self.g_width, self.width), MATRIX),
               "uk_weight": WeightRequest((self.n_head * self.head_dim, self.rank), MATRIX),
               "uv_weight": WeightRequest((self.y_width, self.rank), MATRIX),
               "sink": WeightRequest((self.n_head,), VECTOR),
               "out_weight": WeightRequest((self.width, self.y_width), MATRIX)}
        if self.makes_latent:
            req["dkv_weight"] = WeightRequest((self.rank + self.rot_dim, self.width), MATRIX)
            req["dkv_norm"] = WeightRequest((self.rank,), VECTOR)
        return req

    def token_matrix_elements(self) -> int:
        if self.in_weight is None:
            return 0
        return self.in_weight.numel() + self.uk_folded.numel() + self.uv_heads.numel() + self.out_weight.numel()

    def bind(self, tensors):
        super().bind(tensors)
        # the products that read h as one: queries, gate and (where this layer makes it) the latent
        names = ["q_weight", "gate_weight"] + (["dkv_weight"] if self.makes_latent else [])
        stacked = [tensors[n] for n in names]
        rows = sum(t.shape[0] for t in stacked)
        if self.rot_dim and rows % 16:      # rows of the products' output start 16 bytes apart
            stacked.append(torch.zeros((16 - rows % 16, self.width), dtype=stacked[0].dtype, device=stacked[0].device))
        self.in_weight = torch.cat(stacked, dim=0).contiguous()
        views, at = {}, 0
        for n in names:
            rows = tensors[n].shape[0]
            views[n] = self.in_weight[at:at + rows]
            setattr(self, n, views[n])
            at += rows
        # per head: Wuk_a^T as [row, D (+ P)] (so that folding a query is a product with a matrix stored
        # [out, in]; the rotated part of a query passes through an identity block) and Wuv_a as [E, row]
        H, D, P, R = self.n_head, self.head_dim, self.rot_dim, self.rank
        uk_t = self.uk_weight.view(H, D, R).transpose(1, 2)
        if P:
            folded = torch.zeros((H, self.row, D + P), dtype=uk_t.dtype, device=uk_t.device)
            folded[:, :R, :D] = uk_t
            folded[:, R:R + P, D:] = torch.eye(P, dtype=uk_t.dtype, device=uk_t.device)
            self.uk_folded = folded
            uv = torch.zeros((H, self.value_dim, self.row), dtype=uk_t.dtype, device=uk_t.device)
            uv[:, :, :R] = self.uv_weight.view(H, self.value_dim, R)
            self.uv_heads = uv
            self.uk_weight = folded[:, :R, :D].transpose(1, 2)
            views["uv_weight"] = uv[:, :, :R]
            self.uv_weight = views["uv_weight"]
        else:
            self.uk_folded = uk_t.contiguous()
            self.uv_heads = self.uv_weight.view(H, self.value_dim, R)
            self.uk_weight = self.uk_folded.transpose(1, 2)
        views["uk_weight"] = self.uk_weight
        return views

    def cache_need(self) -> KVNeed:
        return KVNeed(1, self.row, self.window, joint=True)

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if binding.writes != self.makes_latent:
            raise ValueError("a latent-attention layer writes the latent cache exactly when it has the matrix that makes it")
        plain_residual(ctx, h, x)
        n, ws = ctx.n_rows, ctx.workspace
        fast = not ctx.exact
        z = ws.get("latent_in", n, self.in_weight.shape[0], ctx.dtype)
        split = self.q_width + self.g_width
        if (self.makes_latent and not self.rot_dim and n > self.JOINT_PRODUCT_MAX_ROWS
                and n * split > self.JOINT_PRODUCT_MAX_WORK):
            # many rows: the few latent columns on top of queries and gate would start another
            # round of the tiled kernel's tiles (17 x 16 tiles of 128 x 256 on 256 compute units
            # where 16 x 16 fit), so the latent gets a small product of its own
            hn = as_tensor(ctx, h)
            linear(ctx, hn, self.in_weight[:split], None, z[:, :split], n)
            linear(ctx, hn, self.in_weight[split:], None, z[:, split:], n)
        else:
            linear(ctx, h, self.in_weight, None, z, n)
        group = ctx.groups[binding.group]
        pool = group.k_pools[binding.index]
        if self.rot_dim:
            # the queries' rotated parts in place; the normed latent and the rotated key part into the pages
            kernels.latent_prepare(z, 0, self.n_head, self.head_dim, self.rot_dim, ctx.positions,
                                   self.rotation.frequencies(z.device), n, getattr(self.rotation, "magnitude", 1.0),
                                   c_off=split, rank=self.rank, gain=self.dkv_norm if self.makes_latent else None,
                                   eps=self.eps, pool=pool if self.makes_latent else None,
                                   slot_mapping=group.slot_mapping if self.makes_latent else None)
        elif self.makes_latent:
            kernels.rms_norm_store(z[:, split:], self.dkv_norm, self.eps, pool, group.slot_mapping, n)
        q_lat = ws.get("latent_q", n, self.n_head * self.row, ctx.dtype)
        kernels.heads_linear(z, self.uk_folded, q_lat, n, fast=fast)
        o_lat = ws.get("latent_o", n, self.n_head * self.row, ctx.dtype)
        gate = z[:, self.q_width:split]
        attention_ops.paged_attention(ctx, q_lat, o_lat, pool, pool, group, self.n_head, self.scale, self.window,
                                      sinks=self.sink, gate=gate if self.head_gate else None)
        y = ws.get("attn_out", n, self.y_width, ctx.dtype)
        kernels.heads_linear(o_lat, self.uv_heads, y, n, gate=None if self.head_gate else gate, fast=fast)
        linear_add(ctx, y, self.out_weight, None, x, n)


def _own_rotation(rotary: Optional[dict]) -> Optional[PositionEncoding]:
    """A mixer's own position encoding from its parameters ({"kind": ..., constants}), through the
    registry of position encodings; None: the mixer does not rotate."""
    if not rotary:
        return None
    params = dict(rotary)
    part = POSITIONS.build(PartSpec(params.pop("kind", "rotary_half"), params))
    if not hasattr(part, "frequencies"):
        raise ValueError("a mixer's own rotation must give a frequency table (frequencies(device))")
    return part


@register_mixer("gated_attention")
class GatedAttention(Mixer):
    """Causal softmax attention over the paged cache with grouped key/value heads, a query/key size
    D that may differ from the value size E, and these optional steps, each a parameter:

    q = h Wq^T (+ b), k = h Wk^T (+ b), v = h Wv^T (+ b);  q, k rotated by position (`rotary`: the
    mixer's own rotation);  q, k divided by their root mean square per head (`qk_norm_eps`);
    v <- (1 - lambda) v + lambda v_other with v_other the values that the layer with
    value_mix="keep" made for the same token (value_mix="mix"; lambda is the tensor `mix`); what is
    cached is the rotated, normed key and the mixed value.  S = (q . k) * scale, capped as
    cap * tanh(S / cap) (`softcap`), softmax in float32 over the keys at positions <= the query's;
    head a's output times sigmoid(h Wg^T)_a, one number per head (`head_gate`); out = y Wo^T, added
    into the residual.  With `conv_taps` = J > 1 the projected q, k and v pass a causal convolution over
    time first, channel by channel (weights [channels, J], the last tap on the current token, zeros
    before the sequence's start), whose last J - 1 inputs are kept per request beside the pages.  With
    `window` = w > 0 a query sees only the keys at the last w positions, its own included, and with
    `keep_first` = f also those at positions below f (which keep their true positions).  Further options:
    `qk_norm_weights` "head" or "whole": instead of the unit norm behind the rotation, an RMS norm with weights
    (eps `qk_norm_eps`) *before* the rotation, head by head with one weight vector [D] that the query heads share
    and one for the key heads, or over all of a token's query channels at once (and all of its key channels) with
    weights as long as the projection; `values_from_keys`: there is no Wv, a key head's values are its keys as
    projected (before norm and rotation), so E = D; `score_bias`: no softmax, a visible key's weight is
    sigmoid(score + b_a) with a number per head (the tensor `score_bias`), not normalised over the keys;
    `out_bias`: the output projection has a bias.

    The cache keeps keys and values in pages of one head size, so both are laid out with
    max(D, E) channels a head (rounded up to what the bfloat16 attention kernels take), the
    channels beyond a head's own being zeros that the stacked projection matrix makes by itself."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, n_head: int, n_kv_head: int, head_dim: int, value_dim: int, scale: float,
                 bias: bool = False, rotary: Optional[dict] = None, qk_norm_eps: Optional[float] = None,
                 softcap: float = 0.0, head_gate: bool = False, value_mix: Optional[str] = None,
                 share: str = "values", conv_taps: int = 0, window: int = 0, keep_first: int = 0,
                 qk_norm_weights: Optional[str] = None, values_from_keys: bool = False, score_bias: bool = False,
                 out_bias: bool = False) -> None:
        self.width, self.n_head, self.n_kv_head = int(width), int(n_head), int(n_kv_head)
        self.head_dim, self.value_dim, self.scale = int(head_dim), int(value_dim), float(scale)
        self.has_bias, self.has_gate = bool(bias), bool(head_gate)
        self.rotation = _own_rotation(rotary)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.softcap = float(softcap or 0.0)
        if value_mix not in (None, "keep", "mix"):
            raise ValueError(f"value_mix {value_mix!r} is none of None, 'keep', 'mix'")
        self.value_mix, self.share = value_mix, str(share)
        self.conv_taps, self.window = int(conv_taps or 0), int(window or 0)
        if not 0 <= self.conv_taps <= kernels.MAX_CONV_TAPS or self.window < 0:
            raise ValueError(f"{conv_taps} taps, window {window}: the convolution takes up to {kernels.MAX_CONV_TAPS} taps")
        if self.n_head % self.n_kv_head != 0:
            raise ValueError("n_head must be a multiple of n_kv_head")
        if self.rotation is not None and self.rotation.dims > self.head_dim:
            raise ValueError(f"rotation over {self.rotation.dims} channels of heads of {self.head_dim}")
        self.keep_first = int(keep_first or 0) if self.window else 0
        if int(keep_first or 0) < 0:
            raise ValueError("keep_first must not be negative")
        if qk_norm_weights not in (None, "head", "whole") or (qk_norm_weights and self.qk_norm_eps is None):
            raise ValueError("qk_norm_weights is None, 'head' or 'whole', and needs qk_norm_eps")
        self.qk_norm_weights = qk_norm_weights
        self.values_from_keys, self.has_score_bias, self.has_out_bias = bool(values_from_keys), bool(score_bias), bool(out_bias)
        if self.values_from_keys and (self.value_dim != self.head_dim or self.value_mix is not None or self.conv_taps > 1):
            raise ValueError("values that are the keys have the keys' size, and are neither mixed nor convolved")
        if self.has_score_bias and self.softcap > 0.0:
            raise ValueError("sigmoid weights take no score cap")
        size = max(self.head_dim, self.value_dim)
        self.head_stride = -(-size // 32) * 32 if size <= 128 else -(-size // 8) * 8
        if self.head_stride > 512:
            raise ValueError(f"head size {size}: the attention kernels take up to 512")
        s = self.head_stride
        self.q_off, self.k_off = 0, self.n_head * s
        self.v_off = self.k_off + self.n_kv_head * s
        self.g_off = self.v_off + (0 if self.values_from_keys else self.n_kv_head * s)
        self.in_rows = -(-(self.g_off + (self.n_head if self.has_gate else 0)) // 16) * 16
        self.in_weight = self.in_bias = self.out_padded = self.conv_weight = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        H, G, D, E, W = self.n_head, self.n_kv_head, self.head_dim, self.value_dim, self.width
        req = {"q_weight": WeightRequest((H * D, W), MATRIX), "k_weight": WeightRequest((G * D, W), MATRIX),
               "out_weight": WeightRequest((W, H * E), MATRIX)}
        if not self.values_from_keys:
            req["v_weight"] = WeightRequest((G * E, W), MATRIX)
        if self.qk_norm_weights is not None:
            whole = self.qk_norm_weights == "whole"
            req.update(q_norm=WeightRequest((H * D if whole else D,), VECTOR), k_norm=WeightRequest((G * D if whole else D,), VECTOR))
        if self.has_score_bias:
            req["score_bias"] = WeightRequest((H,), VECTOR)
        if self.has_out_bias:
            req["out_bias"] = WeightRequest((W,), VECTOR)
        if self.conv_taps > 1:
            J = self.conv_taps
            req.update(q_conv=WeightRequest((H * D, J), VECTOR), k_conv=WeightRequest((G * D, J), VECTOR),
                       v_conv=WeightRequest((G * E, J), VECTOR))
        if self.has_bias:
            req.update(q_bias=WeightRequest((H * D,), VECTOR), k_bias=WeightRequest((G * D,), VECTOR))
            if not self.values_from_keys:
                req["v_bias"] = WeightRequest((G * E,), VECTOR)
        if self.has_gate:
            req["gate_weight"] = WeightRequest((H, W), MATRIX)
        if self.value_mix is not None:
            req["mix"] = WeightRequest((), VECTOR)
        return req

    def bind(self, tensors):
        super().bind(tensors)
        H, G, D, E, W, s = self.n_head, self.n_kv_head, self.head_dim, self.value_dim, self.width, self.head_stride
        q = tensors["q_weight"]
        joint = torch.zeros((self.in_rows, W), dtype=q.dtype, device=q.device)
        views = {}

        def place(name: str, at: int, heads: int, size: int) -> None:
            block = joint[at:at + heads * s].view(heads, s, W)[:, :size]
            block.copy_(tensors[name].view(heads, size, W))
            views[name] = block

        place("q_weight", self.q_off, H, D)
        place("k_weight", self.k_off, G, D)
        if not self.values_from_keys:
            place("v_weight", self.v_off, G, E)
        if self.has_gate:
            joint[self.g_off:self.g_off + H].copy_(tensors["gate_weight"])
            views["gate_weight"] = joint[self.g_off:self.g_off + H]
        self.in_weight = joint
        if self.has_bias:
            bias = torch.zeros(self.in_rows, dtype=torch.float32, device=q.device)
            for name, at, heads, size in (("q_bias", self.q_off, H, D), ("k_bias", self.k_off, G, D),
                                          ("v_bias", self.v_off, G, E)):
                if name not in tensors:
                    continue
                bias[at:at + heads * s].view(heads, s)[:, :size].copy_(tensors[name].view(heads, size))
            self.in_bias = bias
        if self.conv_taps > 1:
            # the taps of the padded layout's channels (zeros for the channels a head does not have)
            taps = torch.zeros((self.g_off, self.conv_taps), dtype=torch.float32, device=q.device)
            for name, at, heads, size in (("q_conv", self.q_off, H, D), ("k_conv", self.k_off, G, D),
                                          ("v_conv", self.v_off, G, E)):
                taps[at:at + heads * s].view(heads, s, -1)[:, :size].copy_(tensors[name].view(heads, size, -1))
            self.conv_weight = taps
        out = tensors["out_weight"]
        padded = torch.zeros((W, H * s), dtype=out.dtype, device=out.device)
        padded.view(W, H, s)[:, :, :E].copy_(out.view(W, H, E))
        self.out_padded = padded
        views["out_weight"] = padded.view(W, H, s)[:, :, :E]
        for name, view in views.items():
            setattr(self, name, view)
        return views

    def cache_need(self) -> KVNeed:
        return KVNeed(self.n_kv_head, self.head_stride, self.window, keep_first=self.keep_first,
                      state_numel=(self.conv_taps - 1) * self.g_off if self.conv_taps > 1 else 0)

    def token_matrix_elements(self) -> int:
        return self.in_weight.numel() + self.out_padded.numel() if self.in_weight is not None else 0

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if not binding.writes:
            raise ValueError("gated attention keeps its own keys and values")
        plain_residual(ctx, h, x)
        n, ws, s = ctx.n_rows, ctx.workspace, self.head_stride
        z = ws.get("gated_attention_in", n, self.in_rows, ctx.dtype)
        linear(ctx, h, self.in_weight, self.in_bias, z, n)
        if self.conv_taps > 1:
            # q, k and v through their short convolution into a second buffer (a token reads the inputs of the
            # tokens before it); the gate's columns, if any, stay where they are
            zc = ws.get("gated_attention_conv", n, self.in_rows, ctx.dtype)
            kernels.short_conv(z, 0, self.conv_weight, None, ctx.state_pools[binding.state], ctx.state_slots, ctx.cu_q,
                               ctx.q_req, ctx.positions, ctx.cu_q.numel() - 1, zc, 0, n)
            gate_rows, z = z, zc
        else:
            gate_rows = z
        group = ctx.groups[binding.group]
        k_pool, v_pool = group.k_pools[binding.index], group.v_pools[binding.index]
        other, mode = None, 0
        if self.value_mix is not None:
            other = ws.get("shared_" + self.share, n, self.n_kv_head * self.value_dim, ctx.dtype)
            mode = 1 if self.value_mix == "keep" else 2
        kernels.qk_prepare(z, self.q_off, self.k_off, self.v_off, self.n_head, self.n_kv_head, self.head_dim, self.value_dim, s, n,
                           positions=ctx.positions,
                           freq=self.rotation.frequencies(z.device) if self.rotation is not None else None,
                           norm_eps=self.qk_norm_eps, mix_lambda=self.mix if mode == 2 else None, v_other=other,
                           mix_mode=mode, k_pool=k_pool, v_pool=v_pool, slot_mapping=group.slot_mapping,
                           norm=self.qk_norm_weights, q_norm_weight=self.q_norm if self.qk_norm_weights else None,
                           k_norm_weight=self.k_norm if self.qk_norm_weights else None,
                           values_from_keys=self.values_from_keys,
                           rot_magnitude=getattr(self.rotation, "magnitude", 1.0))
        y = ws.get("attn_out", n, self.n_head * s, ctx.dtype)
        # (the gate per head is applied by the attention kernel as it stores a head's output)
        attention_ops.paged_attention(ctx, z, y, k_pool, v_pool, group, self.n_head, self.scale, self.window,
                                      softcap=self.softcap, gate=gate_rows[:, self.g_off:] if self.has_gate else None,
                                      keep_first=self.keep_first, score_bias=self.score_bias if self.has_score_bias else None)
        linear_add(ctx, y, self.out_padded, self.out_bias if self.has_out_bias else None, x, n)


@register_mixer("decay_state")
class DecayStateMixer(Mixer):
    """Linear attention with a fixed decay per head: no softmax, no denominator, and instead of a
    cache one float32 matrix per request and head.

    q = f(h Wq^T), k = f(h Wk^T) [H, D], v = f(h Wv^T) [H, E] with f the identity or silu
    (`input_activation`); q and k rotated by position (`rotary`); k times `k_scale`;
    S_t = decay_a S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head a, S zero before the first token.
    Then either each head's o divided by its root mean square (`head_norm_eps`) and the heads
    multiplied by silu(h Wg^T), or (`out_norm_eps`) the concatenated heads RMS-normed with the
    weight `norm_weight` and multiplied by sigmoid(h Wg^T); out = y Wo^T, added into the residual.
    From the rotation on everything is float32 up to y."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, n_head: int, head_dim: int, value_dim: int, decay, rotary: Optional[dict] = None,
                 k_scale: float = 1.0, input_activation: Optional[str] = None, head_norm_eps: Optional[float] = None,
                 out_norm_eps: Optional[float] = None) -> None:
        self.width, self.n_head, self.head_dim, self.value_dim = int(width), int(n_head), int(head_dim), int(value_dim)
        self.decay_values = [float(d) for d in decay]
        if len(self.decay_values) != self.n_head:
            raise ValueError(f"{len(self.decay_values)} decays for {self.n_head} heads")
        if input_activation not in (None, "silu"):
            raise ValueError(f"input activation {input_activation!r} is neither None nor 'silu'")
        if (head_norm_eps is None) == (out_norm_eps is None):
            raise ValueError("exactly one of head_norm_eps and out_norm_eps says how the heads' outputs are normed")
        if not (0 < self.head_dim <= 256 and 0 < self.value_dim <= 256):
            raise ValueError("the state kernel takes head sizes up to 256")
        self.rotation = _own_rotation(rotary)
        if self.rotation is not None and self.rotation.dims > self.head_dim:
            raise ValueError(f"rotation over {self.rotation.dims} channels of heads of {self.head_dim}")
        self.k_scale, self.silu_inputs = float(k_scale), input_activation == "silu"
        self.head_norm_eps = None if head_norm_eps is None else float(head_norm_eps)
        self.out_norm_eps = None if out_norm_eps is None else float(out_norm_eps)
        self.qk_width, self.v_width = self.n_head * self.head_dim, self.n_head * self.value_dim
        self.k_off, self.v_off, self.g_off = self.qk_width, 2 * self.qk_width, 2 * self.qk_width + self.v_width
        self.in_weight = None
        self._decay: Dict[torch.device, torch.Tensor] = {}

    def weight_requests(self) -> Dict[str, WeightRequest]:
        W = self.width
        req = {"q_weight": WeightRequest((self.qk_width, W), MATRIX), "k_weight": WeightRequest((self.qk_width, W), MATRIX),
               "v_weight": WeightRequest((self.v_width, W), MATRIX), "gate_weight": WeightRequest((self.v_width, W), MATRIX),
               "out_weight": WeightRequest((W, self.v_width), MATRIX)}
        if self.out_norm_eps is not None:
            req["norm_weight"] = WeightRequest((self.v_width,), VECTOR)
        return req

    def bind(self, tensors):
        super().bind(tensors)
        names = ["q_weight", "k_weight", "v_weight", "gate_weight"]
        self.in_weight = torch.cat([tensors[n] for n in names], dim=0).contiguous()
        views, at = {}, 0
        for n in names:
            rows = tensors[n].shape[0]
            views[n] = self.in_weight[at:at + rows]
            setattr(self, n, views[n])
            at += rows
        return views

    def cache_need(self) -> StateNeed:
        return StateNeed(self.n_head * self.head_dim * self.value_dim)

    def _decays(self, device: torch.device) -> torch.Tensor:
        d = self._decay.get(device)
        if d is None:
            d = self._decay[device] = torch.tensor(self.decay_values, dtype=torch.float32, device=device)
        return d

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if binding.kind != "state":
            raise ValueError("a decaying-state mixer needs a state pool")
        plain_residual(ctx, h, x)
        n, ws = ctx.n_rows, ctx.workspace
        z = ws.get("decay_state_in", n, self.in_weight.shape[0], ctx.dtype)
        linear(ctx, h, self.in_weight, None, z, n)
        y = ws.get("decay_state_out", n, self.v_width, ctx.dtype)
        freq = self.rotation.frequencies(z.device) if self.rotation is not None else None
        state, n_req = ctx.state_pools[binding.index], ctx.cu_q.numel() - 1
        # a step with prompt portions: the recurrence a chunk of tokens at a time on the matrix cores, the
        # heads' norm and gate in a kernel behind it; single tokens: token by token, norm and gate inside
        chunked = False
        if not ctx.decode_only and self.head_dim <= kernels.CHUNKED_STATE_MAX_DIM:
            sums = ws.get("decay_state_sums", n, self.v_width, torch.float32)
            qk = ws.get("decay_state_qk", n, 2 * self.qk_width, torch.float32)
            chunked = kernels.decay_state_chunked(z, 0, self.k_off, self.v_off, self.n_head, self.head_dim, self.value_dim,
                                                  self._decays(z.device), state, ctx.state_slots, ctx.cu_q, n_req, n,
                                                  ctx.positions, qk, sums, silu_inputs=self.silu_inputs, freq=freq,
                                                  k_scale=self.k_scale)
        gated_inside = self.head_norm_eps is not None and not chunked
        if not chunked:
            sums = y if gated_inside else ws.get("decay_state_sums", n, self.v_width, torch.float32)
            kernels.decay_state(z, 0, self.k_off, self.v_off, self.g_off if gated_inside else -1, self.n_head,
                                self.head_dim, self.value_dim, self._decays(z.device), state, ctx.state_slots, ctx.cu_q,
                                n_req, ctx.positions, sums, silu_inputs=self.silu_inputs, freq=freq, k_scale=self.k_scale,
                                norm_eps=self.head_norm_eps)
        if self.head_norm_eps is not None and not gated_inside:
            kernels.rms_norm(sums, None, y, n, self.head_norm_eps, self.value_dim, groups=self.n_head,
                             gate=z[:, self.g_off:], gate_act="silu")
        elif self.head_norm_eps is None:
            kernels.rms_norm(sums, self.norm_weight, y, n, self.out_norm_eps, self.v_width, gate=z[:, self.g_off:],
                             gate_act="sigmoid")
        linear_add(ctx, y, self.out_weight, None, x, n)


@register_mixer("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Linear attention whose state decays channel by channel at a rate made from the token: no softmax,
    and instead of a cache one float32 matrix per request and head.

    q = h Wq^T * q_scale, k = h Wk^T [H, D], v = h Wv^T [H, E]; u = (h Wa1^T) Wa2^T + b [H, D] through a narrow
    middle; decay_t = sigmoid(u)^(1/tau) per key channel; S_t = diag(decay_t) S_(t-1) + k_t v_t^T,
    o_t = S_t^T q_t per head, S zero before the first token.  Each head's o is divided by its root mean
    square and multiplied by `norm_weight` [E] (one weight for all heads), the heads by silu(h Wg^T);
    out = y Wo^T, added into the residual.  From the decay's logit on everything is float32 up to y."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, n_head: int, head_dim: int, value_dim: int, tau: float, norm_eps: float,
                 decay_rank: Optional[int] = None, q_scale: Optional[float] = None) -> None:
        self.width, self.n_head, self.head_dim, self.value_dim = int(width), int(n_head), int(head_dim), int(value_dim)
        # the narrow middle of the decay's projection: given, or (None) whatever the stored tensors have
        self.decay_rank = -1 if decay_rank is None else int(decay_rank)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.q_scale = self.head_dim ** -0.5 if q_scale is None else float(q_scale)
        if not (0 < self.head_dim <= 256 and 0 < self.value_dim <= 256):
            raise ValueError("the state kernel takes head sizes up to 256")
        if not self.tau > 0.0 or self.decay_rank == 0 or self.decay_rank < -1:
            raise ValueError(f"tau {tau} and decay rank {decay_rank} must be positive")
        self.qk_width, self.v_width = self.n_head * self.head_dim, self.n_head * self.value_dim
        self.k_off, self.v_off = self.qk_width, 2 * self.qk_width
        self.g_off = self.v_off + self.v_width
        self.a_off = self.g_off + self.v_width
        self.in_weight = self.head_gain = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        W = self.width
        return {"q_weight": WeightRequest((self.qk_width, W), MATRIX), "k_weight": WeightRequest((self.qk_width, W), MATRIX),
                "v_weight": WeightRequest((self.v_width, W), MATRIX), "gate_weight": WeightRequest((self.v_width, W), MATRIX),
                "decay_in_weight": WeightRequest((self.decay_rank, W), MATRIX),
                "decay_out_weight": WeightRequest((self.qk_width, self.decay_rank), MATRIX),
                "decay_out_bias": WeightRequest((self.qk_width,), VECTOR),
                "norm_weight": WeightRequest((self.value_dim,), VECTOR),
                "out_weight": WeightRequest((W, self.v_width), MATRIX)}

    def token_matrix_elements(self) -> int:
        if self.in_weight is None:
            return 0
        return self.in_weight.numel() + self.decay_out_weight.numel() + self.out_weight.numel()

    def bind(self, tensors):
        super().bind(tensors)
        if tensors["decay_in_weight"].shape[0] != tensors["decay_out_weight"].shape[1]:
            raise ValueError("the two steps of the decay's projection do not fit each other")
        self.decay_rank = int(tensors["decay_in_weight"].shape[0])
        names = ["q_weight", "k_weight", "v_weight", "gate_weight", "decay_in_weight"]
        self.in_weight = torch.cat([tensors[n] for n in names], dim=0).contiguous()
        views, at = {}, 0
        for n in names:
            rows = tensors[n].shape[0]
            views[n] = self.in_weight[at:at + rows]
            setattr(self, n, views[n])
            at += rows
        self.head_gain = self.norm_weight.repeat(self.n_head).contiguous()    # the heads' one weight, head by head
        return views

    def cache_need(self) -> StateNeed:
        return StateNeed(self.n_head * self.head_dim * self.value_dim)

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if binding.kind != "state":
            raise ValueError("gated linear attention needs a state pool")
        plain_residual(ctx, h, x)
        n, ws = ctx.n_rows, ctx.workspace
        z = ws.get("gla_in", n, self.in_weight.shape[0], ctx.dtype)
        linear(ctx, h, self.in_weight, None, z, n)
        u = ws.get("gla_decay", n, self.qk_width, ctx.dtype)
        linear(ctx, z[:, self.a_off:], self.decay_out_weight, self.decay_out_bias, u, n)
        sums = ws.get("gla_sums", n, self.v_width, torch.float32)
        state, n_req = ctx.state_pools[binding.index], ctx.cu_q.numel() - 1
        # a step with prompt portions: the recurrence a chunk of tokens at a time on the matrix cores; single
        # tokens: token by token
        chunked = False
        if not ctx.decode_only and self.head_dim <= kernels.CHUNKED_STATE_MAX_DIM:
            qkg = ws.get("gated_state_qkg", n, 3 * self.qk_width, torch.float32)
            chunked = kernels.gated_state_chunked(z, 0, self.k_off, self.v_off, self.n_head, self.n_head, self.head_dim,
                                                  self.value_dim, u, 0, "channel_sigmoid", state, ctx.state_slots, ctx.cu_q,
                                                  n_req, n, ctx.positions, qkg, sums, q_scale=self.q_scale, tau=self.tau)
        if not chunked:
            kernels.gated_state(z, 0, self.k_off, self.v_off, self.n_head, self.n_head, self.head_dim, self.value_dim, u, 0,
                                "channel_sigmoid", state, ctx.state_slots, ctx.cu_q, n_req, ctx.positions, sums,
                                q_scale=self.q_scale, tau=self.tau)
        y = ws.get("gla_out", n, self.v_width, ctx.dtype)
        kernels.rms_norm(sums, self.head_gain, y, n, self.norm_eps, self.value_dim, groups=self.n_head,
                         gate=z[:, self.g_off:], gate_act="silu")
        linear_add(ctx, y, self.out_weight, None, x, n)


@register_mixer("state_space")
class StateSpaceMixer(Mixer):
    """A selective state-space mixer in its scalar-decay (state-space duality) form: per head a float32
    state [N, E] per request, whose decay and input step come from the token.

    h Win^T is laid out [z: H*E | x: H*E | B: G*N | C: G*N | dt: H].  x, B and C together pass a causal
    convolution over time, channel by channel (`conv_weight` [channels, J], bias, the last tap on the
    current token, zeros before the sequence's start), then silu.  dt = softplus(dt + dt_bias); head a
    (which reads B and C of group a // (H / G)): S_t = exp(-exp(A_log_a) dt) S_(t-1) + dt B_t x_t^T,
    y_t = S_t^T C_t + D_a x_t.  The heads' y times silu(z), then divided by its root mean square in
    `norm_groups` equal parts and multiplied by `norm_weight`; out = y Wo^T, added into the residual.
    Kept per request: the state and the convolution's last J - 1 inputs.  Float32 from dt's softplus on up to
    the normed y."""

    graph_safe = True
    plan_safe = True

    def __init__(self, width: int, n_head: int, value_dim: int, state_dim: int, n_group: int, conv_taps: int,
                 norm_groups: int, norm_eps: float) -> None:
        self.width, self.n_head, self.value_dim = int(width), int(n_head), int(value_dim)
        self.state_dim, self.n_group, self.conv_taps = int(state_dim), int(n_group), int(conv_taps)
        self.norm_groups, self.norm_eps = int(norm_groups), float(norm_eps)
        self.inner = self.n_head * self.value_dim
        if self.n_head % self.n_group or self.inner % self.norm_groups:
            raise ValueError("heads must be a multiple of groups, and heads * vdim of the norm's parts")
        if not (0 < self.state_dim <= 256 and 0 < self.value_dim <= 256):
            raise ValueError("the state kernel takes head sizes up to 256")
        if not 1 <= self.conv_taps <= kernels.MAX_CONV_TAPS:
            raise ValueError(f"the convolution takes 1 to {kernels.MAX_CONV_TAPS} taps")
        self.conv_width = self.inner + 2 * self.n_group * self.state_dim
        self.dt_off = self.inner + self.conv_width
        self.in_rows = self.dt_off + self.n_head
        self.state_numel = self.n_head * self.state_dim * self.value_dim
        self.conv_numel = (self.conv_taps - 1) * self.conv_width

    def weight_requests(self) -> Dict[str, WeightRequest]:
        H = self.n_head
        return {"in_weight": WeightRequest((self.in_rows, self.width), MATRIX),
                "conv_weight": WeightRequest((self.conv_width, self.conv_taps), VECTOR),
                "conv_bias": WeightRequest((self.conv_width,), VECTOR),
                "dt_bias": WeightRequest((H,), VECTOR), "a_log": WeightRequest((H,), VECTOR),
                "skip": WeightRequest((H,), VECTOR), "norm_weight": WeightRequest((self.inner,), VECTOR),
                "out_weight": WeightRequest((self.width, self.inner), MATRIX)}

    def cache_need(self) -> StateNeed:
        return StateNeed(self.state_numel + self.conv_numel)

    def forward_add(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if binding.kind != "state":
            raise ValueError("a state-space mixer needs a state pool")
        plain_residual(ctx, h, x)
        n, ws = ctx.n_rows, ctx.workspace
        n_req = ctx.cu_q.numel() - 1
        pool = ctx.state_pools[binding.index]
        u = ws.get("state_space_in", n, self.in_rows, ctx.dtype)
        linear(ctx, h, self.in_weight, None, u, n)
        xbc = ws.get("state_space_conv", n, self.conv_width, ctx.dtype)
        kernels.short_conv(u, self.inner, self.conv_weight, self.conv_bias, pool[:, self.state_numel:], ctx.state_slots,
                           ctx.cu_q, ctx.q_req, ctx.positions, n_req, xbc, 0, n, activation="silu")
        sums = ws.get("state_space_sums", n, self.inner, torch.float32)
        gn = self.n_group * self.state_dim
        state = pool[:, :self.state_numel]
        chunked = False
        if not ctx.decode_only and self.state_dim <= kernels.CHUNKED_STATE_MAX_DIM:
            qkg = ws.get("gated_state_qkg", n, 3 * self.n_head * self.state_dim, torch.float32)
            chunked = kernels.gated_state_chunked(xbc, self.inner + gn, self.inner, 0, self.n_head, self.n_group,
                                                  self.state_dim, self.value_dim, u, self.dt_off, "head_softplus", state,
                                                  ctx.state_slots, ctx.cu_q, n_req, n, ctx.positions, qkg, sums,
                                                  dt_bias=self.dt_bias, a_log=self.a_log, skip=self.skip)
        if not chunked:
            kernels.gated_state(xbc, self.inner + gn, self.inner, 0, self.n_head, self.n_group, self.state_dim,
                                self.value_dim, u, self.dt_off, "head_softplus", state, ctx.state_slots, ctx.cu_q, n_req,
                                ctx.positions, sums, dt_bias=self.dt_bias, a_log=self.a_log, skip=self.skip)
        y = ws.get("state_space_out", n, self.inner, ctx.dtype)
        kernels.rms_norm(sums, self.norm_weight, y, n, self.norm_eps, self.inner // self.norm_groups,
                         groups=self.norm_groups, gate=u, gate_act="silu_first")
        linear_add(ctx, y, self.out_weight, None, x, n)
