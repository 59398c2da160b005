"""A plain, slow implementation of the Nutitar decoder: one function per mechanism, whole sequences
at once on the CPU, no cache and no state carried between calls.  It shares nothing with the engine:
it reads the raw config.json dictionary and a dictionary of tensors by name.

Notation: T tokens of one sequence at positions 0 .. T-1, W the model width, H query heads, G
key/value heads, D the query/key size of a head, E its value size, R the size of a latent, P the
number of rotated channels of a latent-attention head.
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


# With ROUNDING set to torch.bfloat16 every matrix product takes operands rounded to that format and
# its result is rounded to it too, as a kernel that computes "in bfloat16 with 32-bit accumulation"
# does.  The difference between the two modes is the size of what rounding alone does to the
# logits: the tests' bound for the engine's bfloat16 path is a multiple of it.
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


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_ff(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act: torch.Tensor) -> torch.Tensor:
    return lin(_r(xielu(lin(h, up), act[0], act[1])), down)


def token_shift(h: torch.Tensor, shift: torch.Tensor) -> torch.Tensor:
    """h_t + (h_(t-1) - h_t) * shift channel by channel, with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * shift


# ---------------------------------------------------------------- rotation
def plain_frequencies(dims: int, base: float) -> List[float]:
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def stretched_frequencies(dims: int, base: float, factor: float, low: float, high: float, original: float) -> List[float]:
    """Long wavelengths (beyond original / low) are divided by `factor`, short ones (below original /
    high) stay, those between move from one to the other linearly in original / wavelength."""
    out = []
    for f in plain_frequencies(dims, base):
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


def ramped_frequencies(dims: int, base: float, factor: float, original: float, fast: float, slow: float) -> Tuple[List[float], float]:
    """Pair i keeps its frequency below the ramp's start, has it divided by `factor` above the ramp's end and
    is blended between; also the number that multiplies every cosine and sine."""
    def where(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(where(fast)), 0), min(math.ceil(where(slow)), dims - 1)
    out = []
    for i, f in enumerate(plain_frequencies(dims, base)):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotation_of(rot: dict) -> Tuple[int, List[float], float]:
    """(dims, frequencies, magnitude) of a mixer's `rot` entry; which scaling it is shows in its keys."""
    dims, base, scaling = rot["dims"], rot["base"], rot.get("scaling")
    if not scaling:
        return dims, plain_frequencies(dims, base), 1.0
    if "fast" in scaling:
        f, mag = ramped_frequencies(dims, base, scaling["factor"], scaling["original"], scaling["fast"], scaling["slow"])
        return dims, f, mag
    return dims, stretched_frequencies(dims, base, scaling["factor"], scaling["low"], scaling["high"], scaling["original"]), 1.0


def rotate_half(x: torch.Tensor, dims: int, freq: List[float], magnitude: float = 1.0) -> torch.Tensor:
    """x [T, heads, D]: the first `dims` channels of every head are rotated in pairs (i, i + dims/2) by the
    angle t * freq[i] at position t, cosine and sine both times `magnitude`; the other channels pass."""
    T, half = x.shape[0], dims // 2
    angle = torch.arange(T, dtype=DTYPE)[:, None] * torch.tensor(freq, dtype=DTYPE)[None, :]
    cos, sin = (torch.cos(angle) * magnitude)[:, None, :], (torch.sin(angle) * magnitude)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- mixers
def causal(T: int) -> torch.Tensor:
    i = torch.arange(T)
    return i[None, :] <= i[:, None]


def window_with_first(T: int, size: int, keep_first: int) -> torch.Tensor:
    """Query i sees key j if j <= i and (i - j < size or j < keep_first)."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, seen: torch.Tensor,
           score_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q, k [T, H, D], v [T, H, E], seen [T, T] (query i sees key j).  Weights: a softmax of the scaled scores over
    the keys seen, or with score_bias [H] sigmoid(score + score_bias[h]) for every key seen, not normalised.
    Returns [T, H, E]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if score_bias is None:
        w = torch.softmax(s.masked_fill(~seen[None], -math.inf), dim=-1)
    else:
        w = sigmoid(s + score_bias[:, None, None]) * seen[None]
    return torch.einsum("hij,jhe->ihe", w, v)


def latent_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     shared: Optional[Tuple[torch.Tensor, torch.Tensor]]) -> Tuple[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Returns the mixer's output and (latents [T, R], rotated shared key part [T, P]), which a later layer may use."""
    T, H, D, P, E, R = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    dims, freq, mag = rotation_of(m["rot"])
    q = lin(h, t[p + "q"]).view(T, H, D + P)
    q_plain, q_rot = q[..., :D], _r(rotate_half(q[..., D:], dims, freq, mag))
    if shared is None:
        z = lin(h, t[p + "dkv"])
        c = _r(unit_rms(z[:, :R], eps) * t[p + "dkv.norm"])
        k_rot = _r(rotate_half(z[:, None, R:], dims, freq, mag)[:, 0])
    else:
        c, k_rot = shared
    k_plain = lin(c, t[p + "uk"]).view(T, H, D)
    v = lin(c, t[p + "uv"]).view(T, H, E)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    s = s.masked_fill(~causal(T)[None], -math.inf)
    top = torch.maximum(s.max(dim=-1, keepdim=True).values, t[p + "sink"][:, None, None])
    w = torch.exp(s - top)
    w = w / (w.sum(dim=-1, keepdim=True) + torch.exp(t[p + "sink"][:, None, None] - top))
    y = torch.einsum("hij,jhe->ihe", w, v) * sigmoid(lin(h, t[p + "g"]))[:, :, None]
    return lin(_r(y.reshape(T, H * E)), t[p + "o"]), (c, k_rot)


def sigmoid_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped attention behind a window that keeps the first tokens, whose weights are sigmoid(score + bias of
    the head), not normalised; biases on every projection; queries and keys normed over the whole projection."""
    T, H, G, D, E = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms(lin(h, t[p + "q"], t[p + "q.b"]), eps) * t[p + "q.norm"]
    k = unit_rms(lin(h, t[p + "k"], t[p + "k.b"]), eps) * t[p + "k.norm"]
    v = lin(h, t[p + "v"], t[p + "v.b"]).view(T, G, E)
    dims, freq, mag = rotation_of(m["rot"])
    q = _r(rotate_half(q.view(T, H, D), dims, freq, mag))
    k = _r(rotate_half(k.view(T, G, D), dims, freq, mag)).repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    mask = m.get("mask")
    seen = window_with_first(T, mask["size"], mask.get("keep_first", 0)) if mask else causal(T)
    y = attend(q, k, v, m["scale"], seen, t[p + "pb"])
    return lin(_r(y.reshape(T, H * E)), t[p + "o"], t[p + "o.b"])


def keyed_value_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped causal softmax attention whose values are the keys as projected; queries and keys normed head by
    head with one weight for all heads, then rotated."""
    T, H, G, D = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = lin(h, t[p + "q"]).view(T, H, D)
    k = lin(h, t[p + "k"]).view(T, G, D)
    v = k.repeat_interleave(H // G, dim=1)
    dims, freq, mag = rotation_of(m["rot"])
    q = _r(rotate_half(unit_rms(q, eps) * t[p + "q.norm"], dims, freq, mag))
    k = _r(rotate_half(unit_rms(k, eps) * t[p + "k.norm"], dims, freq, mag)).repeat_interleave(H // G, dim=1)
    y = attend(q, k, v, m["scale"], causal(T))
    return lin(_r(y.reshape(T, H * m["vdim"])), t[p + "o"])


# ---------------------------------------------------------------- the model
def forward(cfg: dict, t: Dict[str, torch.Tensor], ids: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = t["embed"][torch.tensor(ids, dtype=torch.int64)] * cfg["embedding"]["scale"]
    latents: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = unit_rms(x, eps) * (1.0 + t[p + "norm1"])
        hs = token_shift(h, t[p + "shift"])
        if layer["type"] == "latent_attention":
            shared = latents[m["kv_from"]] if m.get("kv_from") is not None else None
            y, made = latent_attention(hs, t, p + "mix.", m, eps, shared)
            if shared is None:
                latents[i] = made
        elif layer["type"] == "attention":
            y = sigmoid_attention(hs, t, p + "mix.", m, eps)
        elif layer["type"] == "attention_2":
            y = keyed_value_attention(hs, t, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + dense_ff(h, t[p + "mlp.up"], t[p + "mlp.down"], t[p + "mlp.act"])
        x = x + mult * y
        if layers_out is not None:
            layers_out.append(x.clone())
    h = unit_rms(x, eps) * (1.0 + t["final.norm"])
    return lin(h, t["head"])


def greedy(cfg: dict, t: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """n_new tokens chosen greedily (the lowest index among equals), the whole sequence computed anew each time."""
    seq, out = list(prompt), []
    for _ in range(n_new):
        tok = int(torch.argmax(forward(cfg, t, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
