"""Small Rilavik configurations and model folders with random weights for the tests.

The configurations differ from each other in every size and option: the order of the layer types,
widths that are and are not multiples of 16, one head and several, one key/value head, a few and as
many as heads, query/key sizes below, at and above the value size, rotations over part of a head,
over all of it and none, scaled positions or not, windows of one position up to longer than any
request and none, convolutions of two to five taps (different in the two halves) and none, one to
several groups of B and C, one to several parts of the gated norm, one to three experts a token
out of two to nine, layers without a feed-forward, decay projections of different ranks."""

from __future__ import annotations

import dataclasses
import os
from typing import Callable, Dict, Optional

import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.models import rilavik
from mini_gpt_inference_amd.weights.random_init import random_tensors


def _rot(dims, base, factor=None):
    rot = {"dims": dims, "base": base}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return rot


def gla(heads, dim, vdim, tau):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}


def left(heads, kv_heads, dim, vdim, scale, conv=None, window=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    if window:
        m["mask"] = {"size": window}
    if rot is not None:
        m["rot"] = rot
    return m


def right(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def parallel(l, r, left_scale, right_scale):
    return {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


RAW: Dict[str, dict] = {
    # both layer types in turn, two experts a token, a window shorter than a page and one longer than two, grouped
    # key/value heads, rotation over half a head with scaled positions, different taps left and right
    "A": {"architecture": "Rilavik", "vocab": 131, "width": 64, "norm": {"eps": 1e-5},
          "layers": [
              layer("parallel", parallel(left(4, 2, 16, 32, 0.25, conv=3, window=7, rot=_rot(8, 1000.0, 2.0)),
                                         right(4, 16, 8, 2, 4, 1), 0.75, 1.25), moe(5, 2, 48)),
              layer("gla", gla(2, 16, 24, 4.0), moe(3, 1, 80)),
              layer("parallel", parallel(left(2, 1, 24, 16, 0.2, conv=2, window=37, rot=_rot(24, 500.0)),
                                         right(2, 24, 16, 1, 2, 2), 1.0, 0.5), None),
              layer("gla", gla(3, 8, 40, 16.0), moe(4, 3, 32))]},
    # head sizes that the bfloat16 matrix-core attention kernels take (64 both ways), as many key/value heads as
    # heads, a gla layer first, no window, no convolution left, one expert of two, as many groups as heads
    "B": {"architecture": "Rilavik", "vocab": 77, "width": 96, "norm": {"eps": 1e-6},
          "layers": [
              layer("gla", gla(1, 64, 64, 1.0), moe(2, 1, 64)),
              layer("parallel", parallel(left(2, 2, 64, 64, 0.125, rot=_rot(64, 3e5, 6.0)),
                                         right(3, 32, 64, 3, 5, 3), 0.5, 0.5), moe(9, 2, 40)),
              layer("parallel", parallel(left(1, 1, 64, 32, 0.125, conv=4, window=100, rot=_rot(32, 50000.0, 4.0)),
                                         right(1, 128, 128, 1, 4, 4), 1.5, 0.25), None)]},
    # a width and head sizes that only the general kernels take, a window of one position (a token sees itself
    # only), no rotation, every expert chosen, one tap right (no convolution state)
    "C": {"architecture": "Rilavik", "vocab": 59, "width": 40, "norm": {"eps": 1e-4},
          "layers": [
              layer("parallel", parallel(left(3, 1, 20, 12, 0.6, conv=5, window=1),
                                         right(3, 12, 20, 3, 1, 1), 0.3, 1.0), moe(2, 2, 24)),
              layer("parallel", parallel(left(4, 2, 12, 20, 0.5, conv=2, window=16, rot=_rot(6, 200.0, 1.5)),
                                         right(6, 4, 12, 2, 3, 3), 1.0, 1.0), moe(7, 3, 72)),
              layer("gla", gla(2, 36, 20, 2.5), None)]},
    # a parallel layer, then a gla layer
    "D": {"architecture": "Rilavik", "vocab": 33, "width": 32, "norm": {"eps": 1e-5},
          "layers": [
              layer("parallel", parallel(left(2, 1, 16, 16, 0.25, conv=4, window=33, rot=_rot(16, 10000.0)),
                                         right(2, 16, 16, 1, 4, 1), 0.8, 0.6), moe(3, 1, 32)),
              layer("gla", gla(2, 16, 16, 8.0), moe(6, 2, 16))]},
    # gla layers only: no keys and values, no pages with anything in them
    "E": {"architecture": "Rilavik", "vocab": 45, "width": 48, "norm": {"eps": 1e-5},
          "layers": [
              layer("gla", gla(2, 24, 16, 4.0), moe(4, 2, 24)),
              layer("gla", gla(3, 16, 32, 32.0), None)]},
}
SEEDS = {"A": 21, "B": 22, "C": 23, "D": 24, "E": 25}
DECAY_RANKS = {"A": 8, "B": 16, "C": 5, "D": 4, "E": 6}
STD_SCALE = 1.5


def config(name: str):
    return with_decay_rank(rilavik.config_from_json(RAW[name]), DECAY_RANKS[name])


def with_decay_rank(cfg, rank: int):
    """config.json does not say how narrow the middle of the decay's projection is (the stored tensors do):
    random weights are drawn with the rank given here."""
    layers = tuple(dataclasses.replace(l, mixer=dataclasses.replace(l.mixer, decay_rank=rank)) if l.type == "gla" else l
                   for l in cfg.layers)
    return dataclasses.replace(cfg, layers=layers)


def write_raw_model(path: str, raw: dict, seed: int, std_scale: float = STD_SCALE, decay_rank: int = 16,
                    edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    cfg = with_decay_rank(rilavik.config_from_json(raw), decay_rank)
    tensors = random_tensors(cfg, seed, torch.bfloat16, std_scale)
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    return write_raw_model(path, RAW[name], SEEDS[name], decay_rank=DECAY_RANKS[name], edit=edit)


def random_raw(rng) -> dict:
    """A random config.json: two to six layers of random types, widths, head counts and sizes (also no
    multiples of 8), rotations over 2 channels to the whole head or none, scaled or not, windows, taps,
    groups, norm parts, experts, feed-forwards or none."""
    width = int(rng.choice([24, 40, 64, 72, 96, 136, 256]))

    def rot(dim):
        if rng.random() < 0.15:
            return None
        dims = int(rng.choice([d for d in (2, 4, 8, 12, 16, 32, 64, dim - dim % 2) if 0 < d <= dim]))
        return _rot(dims, float(rng.choice([10.0, 1000.0, 50000.0, 1e6])),
                    float(rng.choice([2.0, 8.0])) if rng.random() < 0.5 else None)

    def att():
        dim, vdim = int(rng.choice([8, 12, 16, 24, 32, 48, 64, 128])), int(rng.choice([8, 16, 20, 32, 64, 128]))
        kv = int(rng.integers(1, 4))
        heads = kv * int(rng.integers(1, 4))
        return left(heads, kv, dim, vdim, float(rng.choice([0.1, 0.3, dim ** -0.5])),
                    conv=int(rng.choice([0, 2, 3, 4, 6])), window=int(rng.choice([0, 1, 2, 9, 16, 17, 50, 64, 70, 130])),
                    rot=rot(dim))

    def ssm():
        groups = int(rng.integers(1, 4))
        heads = groups * int(rng.integers(1, 4))
        vdim = int(rng.choice([4, 8, 12, 16, 32, 64]))
        parts = [p for p in (1, 2, 3, 4, heads) if (heads * vdim) % p == 0]
        return right(heads, vdim, int(rng.choice([4, 8, 16, 24, 32, 64, 128])), groups, int(rng.choice([1, 2, 3, 4, 7])),
                     int(rng.choice(parts)))

    def ff():
        if rng.random() < 0.2:
            return None
        experts = int(rng.choice([1, 2, 3, 5, 8, 12, 33]))
        return moe(experts, int(rng.integers(1, min(experts, 4) + 1)), int(rng.choice([16, 24, 40, 100, 128])))

    layers = []
    for _ in range(int(rng.integers(2, 7))):
        if rng.random() < 0.4:
            layers.append(layer("gla", gla(int(rng.integers(1, 5)), int(rng.choice([8, 12, 16, 32, 48, 64, 128])),
                                           int(rng.choice([8, 16, 24, 32, 64, 128])),
                                           float(rng.choice([1.0, 4.0, 16.0, 64.0]))), ff()))
        else:
            layers.append(layer("parallel", parallel(att(), ssm(), float(rng.choice([0.5, 0.8, 1.0])),
                                                     float(rng.choice([0.25, 0.5, 1.0, 1.3]))), ff()))
    return {"architecture": "Rilavik", "vocab": int(rng.choice([50, 131, 300, 577])), "width": width,
            "norm": {"eps": float(rng.choice([1e-6, 1e-5]))}, "layers": layers}
