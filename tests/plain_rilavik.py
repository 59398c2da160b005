"""A plain, slow implementation of the Rilavik decoder: one function per mechanism, whole sequences
at once on the CPU, no cache and no state carried between calls.  It shares nothing with the engine:
it reads the raw config.json dictionary and a dictionary of tensors by name.

Notation: T tokens of one sequence at positions 0 .. T-1, W the model width, H heads, G key/value
heads (or groups), D the query/key size of a head, E its value size, N the size of a state-space
head's state, J the taps of a short convolution.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Tuple

import torch
from safetensors import safe_open

DTYPE = torch.float64       # what the functions compute in


def read_model_folder(path: str) -> Tuple[dict, Dict[str, torch.Tensor]]:
    with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    tensors: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as fh:
        for name in fh.keys():
            t = fh.get_tensor(name)
            tensors[name] = t.to(DTYPE) if t.is_floating_point() else t.to(torch.int64)
    return cfg, tensors


# With ROUNDING set to torch.bfloat16 every matrix product and short convolution takes operands
# rounded to that format and its result is rounded to it too, as a kernel that computes "in bfloat16
# with 32-bit accumulation" does.  The difference between the two modes is the size of what
# rounding alone does to the logits: the tests' bound for the engine's bfloat16 path is a multiple
# of it.
ROUNDING = None


def _r(x: torch.Tensor) -> torch.Tensor:
    return x if ROUNDING is None else x.to(ROUNDING).to(DTYPE)


def lin(h: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """w h (+ b) for every row of h, w stored [out, in]."""
    y = _r(h) @ _r(w).T
    return _r(y if b is None else y + b)


# ---------------------------------------------------------------- norms and activations
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * gain


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    """log(1 + exp(z)), without overflow for large z."""
    return torch.clamp(z, min=0.0) + torch.log1p(torch.exp(-z.abs()))


# ---------------------------------------------------------------- short convolution
def short_conv(u: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C], w [C, J]: y_t = sum_j w[:, j] u_(t - J + 1 + j) (+ b), with zeros before the first token:
    the last column of w multiplies the current token."""
    T, J = u.shape[0], w.shape[1]
    u, w = _r(u), _r(w)
    y = torch.zeros_like(u)
    for j in range(J):
        back = J - 1 - j
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return _r(y if b is None else y + b)


# ---------------------------------------------------------------- rotation
def rotate_half(x: torch.Tensor, dims: int, base: float, factor: float = 1.0) -> torch.Tensor:
    """x [T, heads, D]: the first `dims` channels of every head are rotated in pairs (i, i + dims/2)
    by the angle t * base^(-2i/dims) / factor at position t; the other channels pass."""
    T, half = x.shape[0], dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=DTYPE)
    angle = torch.arange(T, dtype=DTYPE)[:, None] * freq[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- gated linear attention
def gla_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """q, k, alpha [T, H, D], v [T, H, E].  Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T with S [D, E] zero
    before the first token, o_t = S_t^T q_t.  Returns o [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[2]
    S = torch.zeros(H, D, E, dtype=DTYPE)
    out = torch.zeros(T, H, E, dtype=DTYPE)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out


def gla_mixer(h: torch.Tensor, tensors: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The mixer of a layer of type `gla` (tensors p + q, k, v, g, o, norm, a1, a2, a2.b)."""
    T, H, D, E = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = lin(h, tensors[p + "q"]).view(T, H, D) * D ** -0.5
    k = lin(h, tensors[p + "k"]).view(T, H, D)
    v = lin(h, tensors[p + "v"]).view(T, H, E)
    z = lin(lin(h, tensors[p + "a1"]), tensors[p + "a2"], tensors[p + "a2.b"]).view(T, H, D)
    alpha = sigmoid(z) ** (1.0 / float(m["tau"]))
    o = gla_recurrence(q, k, v, alpha)
    o = unit_rms(o, eps) * tensors[p + "norm"]
    y = o.reshape(T, H * E) * silu(lin(h, tensors[p + "g"]))
    return lin(y, tensors[p + "o"])


# ---------------------------------------------------------------- softmax attention behind a window
def window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, E]; query head a uses key/value head a // (H / G); the query at i sees
    the keys at j with 0 <= i - j < window (window 0 or None: every j <= i).  Returns [T, H, E]."""
    T, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(T)
    seen = (i[:, None] >= i[None, :])
    if window:
        seen &= (i[:, None] - i[None, :]) < window
    out = torch.zeros(T, H, v.shape[2], dtype=DTYPE)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        out[:, a] = _r(torch.softmax(s, dim=-1)) @ v[:, g]
    return out


def left_mixer(h: torch.Tensor, tensors: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    """The attention half of a `parallel` layer (tensors p + q, k, v, q.conv, k.conv, v.conv, o)."""
    T, H, G, D, E = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = (lin(h, tensors[p + n]) for n in ("q", "k", "v"))
    if m.get("conv"):
        q, k, v = (short_conv(u, tensors[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, E)
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = _r(rotate_half(q, rot["dims"], float(rot["base"]), factor))
        k = _r(rotate_half(k, rot["dims"], float(rot["base"]), factor))
    window = int((m.get("mask") or {}).get("size", 0))
    y = _r(window_attention(q, k, v, float(m["scale"]), window))
    return lin(y.reshape(T, H * E), tensors[p + "o"])


# ---------------------------------------------------------------- state-space mixer
def ssd_recurrence(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt: torch.Tensor, A: torch.Tensor,
                   skip: torch.Tensor) -> torch.Tensor:
    """x [T, H, E], B, C [T, G, N], dt [T, H] (positive), A [H] (positive), skip [H].  Head a uses group
    a // (H / G): S_t = exp(-A dt_t) S_(t-1) + dt_t B_t x_t^T with S [N, E] zero before the first token,
    y_t = S_t^T C_t + skip x_t.  Returns [T, H, E]."""
    T, H, E = x.shape
    G, N = B.shape[1], B.shape[2]
    rep = H // G
    S = torch.zeros(H, N, E, dtype=DTYPE)
    out = torch.zeros(T, H, E, dtype=DTYPE)
    for t in range(T):
        Bt, Ct = B[t].repeat_interleave(rep, dim=0), C[t].repeat_interleave(rep, dim=0)      # [H, N]
        S = torch.exp(-A * dt[t])[:, None, None] * S + (dt[t][:, None] * Bt)[:, :, None] * x[t][:, None, :]
        out[t] = torch.einsum("hne,hn->he", S, Ct) + skip[:, None] * x[t]
    return out


def right_mixer(h: torch.Tensor, tensors: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The state-space half of a `parallel` layer (tensors p + in, conv, conv.b, dt_bias, A_log, D, norm, o)."""
    T, H, E, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * E
    u = lin(h, tensors[p + "in"])
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = _r(silu(short_conv(xbc, tensors[p + "conv"], tensors[p + "conv.b"])))
    x = xbc[:, :inner].reshape(T, H, E)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + tensors[p + "dt_bias"])
    y = ssd_recurrence(x, B, C, dt, torch.exp(tensors[p + "A_log"]), tensors[p + "D"]).reshape(T, inner)
    y = y * silu(z)
    parts = int(m.get("norm_groups", 1))
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * tensors[p + "norm"]
    return lin(y, tensors[p + "o"])


# ---------------------------------------------------------------- feed-forward
# With ROUTER_GAPS a list, every call of routed_experts appends one number per token: by how much the router's
# choice is decided.  A test that compares with reduced precision leaves out the tokens whose choice hangs on
# less than that precision can tell.
ROUTER_GAPS: Optional[list] = None


def routed_experts(h: torch.Tensor, tensors: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    """Scores s = sigmoid(router h); a token's `top` experts are those with the largest scores; the output is
    the sum over them of expert(s_e h), expert(u) = down (silu(gate u) * (up u))."""
    n, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    logits = _r(h) @ tensors[p + "router"].T
    if ROUTER_GAPS is not None:
        # how decided each token's choice is: the last chosen logit minus the first one left out
        srt = torch.sort(logits, dim=-1, descending=True).values
        ROUTER_GAPS.append(srt[:, top - 1] - srt[:, top] if top < n else torch.full((h.shape[0],), math.inf, dtype=DTYPE))
    scores = sigmoid(logits)
    chosen = torch.topk(scores, top, dim=-1).indices
    out = torch.zeros_like(h)
    for e in range(n):
        for c in range(top):
            rows = (chosen[:, c] == e).nonzero().flatten()
            if rows.numel() == 0:
                continue
            u = _r(scores[rows, e][:, None] * h[rows])
            act = _r(silu(lin(u, tensors[f"{p}e{e}.gate"])) * lin(u, tensors[f"{p}e{e}.up"]))
            out[rows] += lin(act, tensors[f"{p}e{e}.down"])
    return out


# ---------------------------------------------------------------- the model
def layer_forward(x: torch.Tensor, tensors: Dict[str, torch.Tensor], i: int, layer: dict, eps: float) -> torch.Tensor:
    p = f"l{i}."
    h = _r(rms_norm(x, tensors[p + "norm1"], eps))
    m = layer["mixer"]
    if layer["type"] == "gla":
        y = gla_mixer(h, tensors, p + "mix.", m, eps)
    elif layer["type"] == "parallel":
        y = float(m["left_scale"]) * left_mixer(h, tensors, p + "mix.left.", m["left"]) \
            + float(m["right_scale"]) * right_mixer(h, tensors, p + "mix.right.", m["right"], eps)
    else:
        raise ValueError(f"unknown layer type {layer['type']!r}")
    x = x + rms_norm(y, tensors[p + "norm1b"], eps) * tensors[p + "ls1"]
    if layer.get("mlp") is not None:
        h = _r(rms_norm(x, tensors[p + "norm2"], eps))
        y = routed_experts(h, tensors, p + "mlp.", layer["mlp"])
        x = x + rms_norm(y, tensors[p + "norm2b"], eps) * tensors[p + "ls2"]
    return x


def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int],
            residuals: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  With `residuals` a list, the residual stream after every
    layer is appended to it."""
    eps = float(cfg["norm"]["eps"])
    x = tensors["embed"][torch.tensor(tokens, dtype=torch.long)].to(DTYPE)
    for i, layer in enumerate(cfg["layers"]):
        x = layer_forward(x, tensors, i, layer, eps)
        if residuals is not None:
            residuals.append(x.clone())
    return lin(_r(rms_norm(x, tensors["final.norm"], eps)), tensors["head"])


def greedy(cfg: dict, tensors: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(cfg, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
