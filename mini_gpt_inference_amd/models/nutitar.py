"""Nutitar: a decoder whose layers are listed one by one in config.json, every layer with one norm that both
of its sublayers read, a token shift in front of its mixer, and one of three attention mixers, as data.

What the design fixes, and is therefore set here and handed to the parts as parameters:
- the embedded tokens are multiplied by `embedding.scale`; no position table;
- a layer is x <- x + m (mixer(shifted(h)) + ff(h)) with h = norm1(x) and m = `residual_mult` (the
  `parallel_shift` arrangement); the norms of the layers and of the model are RMS norms with eps `norm.eps`
  whose gain is stored as its distance from one; `mlp: null` leaves the feed-forward out;
- layer type `latent_attention`: keys and values made from a cached latent of `kv_rank` values beside one
  rotated key part of `rot_dim` channels that all heads share; a query head is [dim plain | rot_dim rotated];
  the latent's norm has a plain gain and the model's eps; a sink per head in the softmax's denominator, a sigmoid
  gate per head, causal.  `kv_from: j` reads layer j's cached rows instead of making its own;
- layer type `attention`: grouped heads, biases on all four projections, an RMS norm with plain weights over
  the whole query projection (and the whole key projection) before the rotation, a window of `mask.size`
  positions beside the first `mask.keep_first` ones, and sigmoid weights (score plus a number per head) in
  place of a softmax;
- layer type `attention_2`: grouped heads, no biases, the values are the keys as projected, an RMS norm per
  head with one plain weight vector for all heads before the rotation, causal softmax;
- rotations pair channel i with i + dims/2 over the first `rot.dims` channels of a head; `rot.scaling` with
  `fast` / `slow` ramps the frequencies pair by pair (and scales cosine and sine), with `low` / `high` it
  stretches the long wavelengths;
- feed-forward `dense`: down(xielu(up h)), the activation's two numbers in `mlp.act`;
- the head: the model's norm (`final.norm`), then `head`, untied.

Tensor names: `embed`, `l<i>.norm1`, `l<i>.shift`, `l<i>.mix.{q,o}` and, by type, `l<i>.mix.{dkv,dkv.norm,uk,uv,
sink,g}`, `l<i>.mix.{k,v,q.b,k.b,v.b,o.b,q.norm,k.norm,pb}`, `l<i>.mix.{k,q.norm,k.norm}`; `l<i>.mlp.{up,down,act}`,
`final.norm`, `head`; linear weights are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "Nutitar"
TYPES = ("latent_attention", "attention", "attention_2")


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[Tuple[Tuple[str, float], ...]] = None     # the config's rot.scaling entries, sorted by key

    def part_params(self) -> Dict[str, Any]:
        params: Dict[str, Any] = {"kind": "rotary_half", "dims": self.dims, "base": self.base}
        if self.scaling is not None:
            sc = dict(self.scaling)
            sc["kind"] = "ramp" if "fast" in sc else "stretch"
            params["scaling"] = sc
        return params


@dataclass(frozen=True)
class MixerConfig:
    heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation]            # None (a grouped layer without a rot entry): queries and keys are not rotated
    kv_heads: int = 0                   # attention, attention_2
    window: int = 0                     # attention: mask.size; 0: every earlier key
    keep_first: int = 0                 # attention: mask.keep_first
    kv_rank: int = 0                    # latent_attention
    rot_dim: int = 0                    # latent_attention
    kv_from: Optional[int] = None       # latent_attention: the layer whose cached rows this one reads


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: MixerConfig
    ff: Optional[int]                   # hidden size of the dense feed-forward, None: no feed-forward


@dataclass(frozen=True)
class NutitarConfig:
    architecture: str
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float
    residual_mult: float = 1.0
    embedding_scale: float = 1.0


def _positive(name: str, value: Any) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{name} must be a positive integer, got {value!r}")
    return value


def _rotation(where: str, rot: Any, most: int) -> Rotation:
    if not isinstance(rot, Mapping):
        raise ConfigError(f"{where}: no rot entry")
    dims = _positive(f"{where} rot.dims", rot.get("dims"))
    if dims % 2 or dims > most:
        raise ConfigError(f"{where}: rot.dims must be even and at most {most}, got {dims}")
    if not float(rot.get("base", 0.0)) > 0.0:
        raise ConfigError(f"{where}: rot.base must be positive")
    scaling = rot.get("scaling")
    if scaling is None:
        return Rotation(dims, float(rot["base"]))
    keys = set(scaling)
    if keys not in ({"factor", "original", "fast", "slow"}, {"factor", "original", "low", "high"}):
        raise ConfigError(f"{where}: rot.scaling has factor, original and either fast and slow or low and high, got {sorted(keys)}")
    return Rotation(dims, float(rot["base"]), tuple(sorted((k, float(v)) for k, v in scaling.items())))


def _mixer(where: str, kind: str, m: Mapping[str, Any]) -> MixerConfig:
    heads = _positive(f"{where} heads", m.get("heads"))
    dim = _positive(f"{where} dim", m.get("dim"))
    vdim = _positive(f"{where} vdim", m.get("vdim"))
    scale = float(m["scale"])
    if not scale > 0.0:
        raise ConfigError(f"{where}: scale must be positive")
    if kind == "latent_attention":
        rot_dim = _positive(f"{where} rot_dim", m.get("rot_dim"))
        rot = _rotation(where, m.get("rot"), rot_dim)
        if rot.dims != rot_dim:
            raise ConfigError(f"{where}: the rotation covers the rotated part, rot.dims = rot_dim")
        if m.get("mask") is not None:
            raise ConfigError(f"{where}: a latent-attention layer is causal and takes no mask")
        kv_from = m.get("kv_from")
        if kv_from is not None and (not isinstance(kv_from, int) or isinstance(kv_from, bool) or kv_from < 0):
            raise ConfigError(f"{where}: kv_from names an earlier layer")
        return MixerConfig(heads, dim, vdim, scale, rot, kv_rank=_positive(f"{where} kv_rank", m.get("kv_rank")),
                           rot_dim=rot_dim, kv_from=kv_from)
    kv_heads = _positive(f"{where} kv_heads", m.get("kv_heads"))
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
    rot = _rotation(where, m["rot"], dim) if m.get("rot") is not None else None
    window = keep_first = 0
    mask = m.get("mask")
    if mask is not None:
        if kind != "attention":
            raise ConfigError(f"{where}: only layers of type attention take a mask")
        window = _positive(f"{where} mask.size", mask.get("size"))
        keep_first = mask.get("keep_first", 0)
        if not isinstance(keep_first, int) or isinstance(keep_first, bool) or keep_first < 0:
            raise ConfigError(f"{where}: mask.keep_first must be a non-negative integer")
    if kind == "attention_2" and vdim != dim:
        raise ConfigError(f"{where}: the values are the keys, so vdim = dim")
    return MixerConfig(heads, dim, vdim, scale, rot, kv_heads=kv_heads, window=window, keep_first=keep_first)


def config_from_json(raw: Mapping[str, Any]) -> NutitarConfig:
    if not isinstance(raw.get("layers"), list) or not raw["layers"]:
        raise ConfigError("config.json lists no layers")
    layers: List[LayerConfig] = []
    for i, layer in enumerate(raw["layers"]):
        kind, m = layer.get("type"), layer.get("mixer")
        if kind not in TYPES:
            raise ConfigError(f"layer {i}: unknown mixer type {kind!r}")
        if not isinstance(m, Mapping):
            raise ConfigError(f"layer {i}: no mixer sizes")
        mixer = _mixer(f"layer {i}", kind, m)
        if mixer.kv_from is not None:
            src = layers[mixer.kv_from] if mixer.kv_from < i else None
            if (src is None or src.type != "latent_attention" or src.mixer.kv_from is not None
                    or (src.mixer.kv_rank, src.mixer.rot_dim) != (mixer.kv_rank, mixer.rot_dim)):
                raise ConfigError(f"layer {i}: kv_from names an earlier latent-attention layer that makes its own "
                                  f"latents, with this layer's kv_rank and rot_dim")
        mlp = layer.get("mlp")
        if mlp is not None and mlp.get("kind") != "dense":
            raise ConfigError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append(LayerConfig(kind, mixer, None if mlp is None else _positive(f"layer {i} mlp.ff", mlp.get("ff"))))
    return NutitarConfig(architecture=NAME, vocab=_positive("vocab", raw.get("vocab")),
                         width=_positive("width", raw.get("width")), layers=tuple(layers),
                         norm_eps=float(raw["norm"]["eps"]), residual_mult=float(raw.get("residual_mult", 1.0)),
                         embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)))


def _rotation_json(rot: Rotation) -> Dict[str, Any]:
    out: Dict[str, Any] = {"base": rot.base, "dims": rot.dims}
    if rot.scaling is not None:
        out["scaling"] = {k: (int(v) if k == "original" and float(v).is_integer() else v) for k, v in rot.scaling}
    return out


def config_to_json(cfg: NutitarConfig) -> Dict[str, Any]:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        mixer: Dict[str, Any] = {"dim": m.dim, "heads": m.heads, "scale": m.scale, "vdim": m.vdim}
        if m.rot is not None:
            mixer["rot"] = _rotation_json(m.rot)
        if layer.type == "latent_attention":
            mixer.update(kv_rank=m.kv_rank, rot_dim=m.rot_dim)
            if m.kv_from is not None:
                mixer["kv_from"] = m.kv_from
        else:
            mixer["kv_heads"] = m.kv_heads
            if m.window:
                mixer["mask"] = {"keep_first": m.keep_first, "size": m.window}
        layers.append({"type": layer.type, "mixer": mixer,
                       "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
    return {"architecture": NAME, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
            "norm": {"eps": cfg.norm_eps}, "residual_mult": cfg.residual_mult,
            "embedding": {"scale": cfg.embedding_scale}}


def model_spec(cfg: NutitarConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"width": w, "eps": eps, "one_plus": True}, {"weight": name})

    def mixer_spec(kind: str, m: MixerConfig, p: str) -> PartSpec:
        if kind == "latent_attention":
            names = {"q_weight": p + "q", "gate_weight": p + "g", "uk_weight": p + "uk", "uv_weight": p + "uv",
                     "sink": p + "sink", "out_weight": p + "o"}
            if m.kv_from is None:
                names.update(dkv_weight=p + "dkv", dkv_norm=p + "dkv.norm")
            return PartSpec("latent_attention",
                            {"width": w, "n_head": m.heads, "head_dim": m.dim, "value_dim": m.vdim, "rank": m.kv_rank,
                             "scale": m.scale, "eps": eps, "makes_latent": m.kv_from is None, "rot_dim": m.rot_dim,
                             "rotary": m.rot.part_params(), "gate": "head"}, names)
        names = {"q_weight": p + "q", "k_weight": p + "k", "out_weight": p + "o", "q_norm": p + "q.norm",
                 "k_norm": p + "k.norm"}
        params = {"width": w, "n_head": m.heads, "n_kv_head": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
                  "scale": m.scale, "rotary": m.rot.part_params() if m.rot is not None else None, "qk_norm_eps": eps}
        if kind == "attention":
            names.update(v_weight=p + "v", q_bias=p + "q.b", k_bias=p + "k.b", v_bias=p + "v.b", out_bias=p + "o.b",
                         score_bias=p + "pb")
            params.update(bias=True, out_bias=True, qk_norm_weights="whole", window=m.window, keep_first=m.keep_first,
                          score_bias=True)
        else:
            params.update(qk_norm_weights="head", values_from_keys=True)
        return PartSpec("gated_attention", params, names)

    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts: Dict[str, Tuple[str, PartSpec]] = {"norm1": ("norm", norm(p + "norm1")),
                                                  "mixer": ("mixer", mixer_spec(layer.type, layer.mixer, p + "mix."))}
        if layer.ff is not None:
            parts["feed_forward"] = ("feed_forward", PartSpec(
                "dense_mlp", {"width": w, "hidden": layer.ff, "bias": False, "activation": "xielu"},
                {"fc_weight": p + "mlp.up", "proj_weight": p + "mlp.down", "act": p + "mlp.act"}))
        arrangement = PartSpec("parallel_shift", {"width": w, "residual_mult": cfg.residual_mult,
                                                  "feed_forward": layer.ff is not None, "token_shift": True},
                               {"shift": p + "shift"})
        layers.append(LayerSpec(arrangement, parts=parts))
        order.append(LayerRun(i, reads_cache_of=layer.mixer.kv_from))
    return ModelSpec(
        width=w, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "width": w, "scale": cfg.embedding_scale},
                           {"weight": "embed"}),
        position=PartSpec("none"),
        layers=tuple(layers), order=tuple(order),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": w, "tied": False}, {"weight": "head"}),
        max_positions=None)


def init_plan(cfg: NutitarConfig) -> List[Tuple[str, Tuple[int, ...], str, float]]:
    """Random-weights rule, in drawing order: matrices N(0, 1/sqrt(fan_in)), biases N(0, 0.3), gains stored as their
    distance from one N(0, 0.1), plain gains 1 + N(0, 0.1), shifts around 0.4, sinks and score biases N(0, 1), the
    activation's numbers around 0.5."""
    w = cfg.width
    plan: List[Tuple[str, Tuple[int, ...], str, float]] = [("embed", (cfg.vocab, w), "normal", 1.0)]

    def lin(name: str, out: int, inn: int, bias: bool = False) -> None:
        plan.append((name, (out, inn), "normal", 1.0 / math.sqrt(inn)))
        if bias:
            plan.append((name + ".b", (out,), "normal", 0.3))

    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        plan.append((p + "norm1", (w,), "normal", 0.1))
        x = p + "mix."
        if layer.type == "latent_attention":
            lin(x + "q", m.heads * (m.dim + m.rot_dim), w)
            if m.kv_from is None:
                lin(x + "dkv", m.kv_rank + m.rot_dim, w)
                plan.append((x + "dkv.norm", (m.kv_rank,), "gain", 0.1))
            lin(x + "uk", m.heads * m.dim, m.kv_rank)
            lin(x + "uv", m.heads * m.vdim, m.kv_rank)
            plan.append((x + "sink", (m.heads,), "normal", 1.0))
            lin(x + "g", m.heads, w)
            lin(x + "o", w, m.heads * m.vdim)
        elif layer.type == "attention":
            lin(x + "q", m.heads * m.dim, w, True)
            lin(x + "k", m.kv_heads * m.dim, w, True)
            lin(x + "v", m.kv_heads * m.vdim, w, True)
            plan.append((x + "q.norm", (m.heads * m.dim,), "gain", 0.1))
            plan.append((x + "k.norm", (m.kv_heads * m.dim,), "gain", 0.1))
            plan.append((x + "pb", (m.heads,), "normal", 1.0))
            lin(x + "o", w, m.heads * m.vdim, True)
        else:
            lin(x + "q", m.heads * m.dim, w)
            lin(x + "k", m.kv_heads * m.dim, w)
            plan.append((x + "q.norm", (m.dim,), "gain", 0.1))
            plan.append((x + "k.norm", (m.dim,), "gain", 0.1))
            lin(x + "o", w, m.heads * m.vdim)
        if layer.ff is not None:
            lin(p + "mlp.up", layer.ff, w)
            lin(p + "mlp.down", w, layer.ff)
            plan.append((p + "mlp.act", (2,), "around", 0.5))
        plan.append((p + "shift", (w,), "around", 0.4))
    plan.append(("final.norm", (w,), "normal", 0.1))
    lin("head", cfg.vocab, w)
    return plan


register_architecture(Architecture(NAME, config_from_json, model_spec, init_plan, config_to_json))
