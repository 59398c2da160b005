"""Small Nutitar configurations and model folders with random weights for the tests.

The configurations differ from each other in every size and option: the order of the layer types, widths that
are and are not multiples of 16, one head and several, grouped and ungrouped key/value heads, value sizes
below, at and above the key size, rotations over part of a head and over all of it, with each kind of frequency
scaling and with none, windows of one position up to longer than any test request, with and without kept first
tokens (fewer and more than the window holds), latents whose cached row is and is not a multiple of 8, layers
that read another layer's latents with other head counts and sizes, layers without a feed-forward, embedding
scales and residual multipliers of one and others."""

from __future__ import annotations

import os
from typing import Callable, Dict, Optional

import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.models import nutitar
from mini_gpt_inference_amd.weights.random_init import random_tensors


def rot(dims, base, ramp=None, stretch=None):
    """ramp = (factor, original, fast, slow); stretch = (factor, original, low, high)."""
    r = {"dims": dims, "base": base}
    if ramp is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), ramp))
    if stretch is not None:
        r["scaling"] = dict(zip(("factor", "original", "low", "high"), stretch))
    return r


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, rotation, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rotation}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def windowed(heads, kv_heads, dim, vdim, scale, rotation, size=None, keep_first=0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rotation}
    if size is not None:
        m["mask"] = {"size": size, "keep_first": keep_first}
    return m


def keyed(heads, kv_heads, dim, scale, rotation):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rotation}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(vocab, width, eps, mult, scale, layers):
    return {"architecture": "Nutitar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "embedding": {"scale": scale}, "layers": layers}


_RAMP_A = rot(8, 1000.0, ramp=(8.0, 64, 16.0, 2.0))
_RAMP_C = rot(6, 200.0, ramp=(3.0, 16, 4.0, 0.5))
RAW: Dict[str, dict] = {
    # every layer type, a layer that reads the first layer's latents with other head counts and sizes, a window
    # shorter than a page beside three kept tokens, a window longer than two pages without kept tokens, a layer
    # without a feed-forward, rotation over half a head, both scalings
    "A": model(131, 64, 1e-5, 0.5, 2.0, [
        layer("latent_attention", latent(4, 16, 8, 24, 40, 0.2, _RAMP_A), 48),
        layer("attention", windowed(4, 2, 16, 32, 0.25, rot(8, 1000.0), size=7, keep_first=3), 80),
        layer("attention_2", keyed(4, 1, 24, 0.2, rot(12, 500.0, stretch=(8.0, 32, 1.0, 4.0))), None),
        layer("latent_attention", latent(2, 8, 8, 16, 40, 0.3, _RAMP_A, kv_from=0), 32),
        layer("attention", windowed(2, 2, 32, 16, 0.15, rot(32, 10000.0), size=37), 40)]),
    # head and row sizes that the bfloat16 matrix-core kernels take (64, and a cached row of 96 + 32 = 128), a window
    # of 100 beside 20 kept tokens, as many key/value heads as heads, multiplier and embedding scale of one
    "B": model(77, 96, 1e-6, 1.0, 1.0, [
        layer("attention_2", keyed(2, 2, 64, 0.125, rot(64, 3e5, stretch=(4.0, 128, 2.0, 8.0))), 64),
        layer("latent_attention", latent(3, 32, 32, 32, 96, 0.125, rot(32, 50000.0, ramp=(4.0, 256, 32.0, 1.0))), 72),
        layer("attention", windowed(2, 1, 64, 64, 0.125, rot(32, 50000.0), size=100, keep_first=20), None),
        layer("latent_attention", latent(1, 64, 32, 64, 96, 0.1, rot(32, 50000.0, ramp=(4.0, 256, 32.0, 1.0)), kv_from=1), 64)]),
    # a width and head sizes that only the general kernels take, a window of one position (a token sees itself and
    # the kept first ones: more kept tokens than the window holds), a cached row that is no multiple of 8, no
    # scaling anywhere but the latent's, one head
    "C": model(59, 40, 1e-4, 0.3, 0.7, [
        layer("attention", windowed(3, 1, 20, 12, 0.4, rot(10, 200.0), size=1, keep_first=5), 24),
        layer("latent_attention", latent(1, 12, 6, 20, 21, 0.3, _RAMP_C), 72),
        layer("attention_2", keyed(3, 3, 12, 0.5, rot(4, 30.0)), None),
        layer("attention", windowed(4, 2, 12, 20, 0.3, rot(12, 1e4), size=16, keep_first=16), 56)]),
    # small, for generation through the engine: one layer of each type, no mask on the windowed type (plain causal)
    "D": model(33, 32, 1e-5, 0.8, 1.5, [
        layer("attention_2", keyed(2, 1, 16, 0.25, rot(16, 10000.0, stretch=(2.0, 16, 1.0, 2.0))), 32),
        layer("attention", windowed(2, 1, 16, 16, 0.25, rot(8, 100.0)), 16),
        layer("latent_attention", latent(2, 16, 4, 16, 16, 0.25, rot(4, 100.0, ramp=(2.0, 8, 2.0, 1.0))), 32)]),
}
SEEDS = {"A": 31, "B": 32, "C": 33, "D": 34}
STD_SCALE = 1.5


def config(name: str):
    return nutitar.config_from_json(RAW[name])


def write_raw_model(path: str, raw: dict, seed: int, std_scale: float = STD_SCALE,
                    edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    cfg = nutitar.config_from_json(raw)
    tensors = random_tensors(cfg, seed, torch.bfloat16, std_scale)
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    return write_raw_model(path, RAW[name], SEEDS[name], edit=edit)


def random_raw(rng) -> dict:
    """A random config.json: two to six layers of random types, widths, head counts and sizes (also no multiples
    of 8), rotations over 2 channels to the whole head, scaled either way or not, windows with and without kept
    tokens or none, latents read by later layers, feed-forwards or none."""
    width = int(rng.choice([24, 36, 40, 50, 64, 72, 96, 100, 136, 256]))

    def rotation(most, exactly=None):
        dims = exactly or int(rng.choice([d for d in (2, 4, 8, 12, 16, 32, 64, most - most % 2) if 0 < d <= most]))
        base = float(rng.choice([10.0, 1000.0, 50000.0, 1e6]))
        pick = rng.random()
        if pick < 0.35:
            return rot(dims, base, ramp=(float(rng.choice([2.0, 4.0, 16.0])), int(rng.choice([8, 64, 512])),
                                         float(rng.choice([8.0, 32.0])), float(rng.choice([0.5, 1.0, 2.0]))))
        if pick < 0.7:
            low = float(rng.choice([0.5, 1.0, 2.0]))
            return rot(dims, base, stretch=(float(rng.choice([2.0, 8.0])), int(rng.choice([16, 128, 1024])), low,
                                            low * float(rng.choice([2.0, 4.0]))))
        return rot(dims, base)

    def ff():
        return None if rng.random() < 0.2 else int(rng.choice([16, 24, 40, 100, 128]))

    layers, makers = [], []
    for i in range(int(rng.integers(2, 7))):
        pick = rng.random()
        dim = int(rng.choice([6, 8, 10, 12, 16, 24, 32, 48, 64, 128]))
        scale = float(rng.choice([0.1, 0.3, dim ** -0.5]))
        if pick < 0.35:
            heads, vdim = int(rng.integers(1, 5)), int(rng.choice([6, 8, 16, 20, 32, 64]))
            if makers and rng.random() < 0.5:
                src = int(rng.choice(makers))
                m = layers[src]["mixer"]
                layers.append(layer("latent_attention", latent(heads, dim, m["rot_dim"], vdim, m["kv_rank"], scale,
                                                               m["rot"], kv_from=src), ff()))
            else:
                rot_dim = int(rng.choice([2, 4, 8, 16, 32]))
                makers.append(i)
                layers.append(layer("latent_attention", latent(heads, dim, rot_dim, vdim, int(rng.choice([16, 21, 32, 40, 96, 112, 160])),
                                                               scale, rotation(rot_dim, exactly=rot_dim)), ff()))
            continue
        kv = int(rng.integers(1, 4))
        heads = kv * int(rng.integers(1, 4))
        if pick < 0.7:
            size = [None, 1, 2, 9, 16, 17, 50, 64, 70, 130][int(rng.integers(0, 10))]
            layers.append(layer("attention", windowed(heads, kv, dim, int(rng.choice([8, 16, 20, 32, 64, 128])), scale,
                                                      rotation(dim), size=size, keep_first=int(rng.choice([0, 1, 4, 16, 33, 70]))), ff()))
        else:
            layers.append(layer("attention_2", keyed(heads, kv, dim, scale, rotation(dim)), ff()))
    return model(int(rng.choice([50, 131, 300, 577])), width, float(rng.choice([1e-6, 1e-5])),
                 float(rng.choice([0.3, 0.5, 1.0])), float(rng.choice([0.5, 1.0, 3.0])), layers)
