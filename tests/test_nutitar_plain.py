"""Nutitar without a GPU: the plain implementation's mechanisms in their limiting cases, the configuration
(round trip, refusals), the cache layout and tensor names that the model asks for, the frequency tables of the
framework's rotation against the plain ones, and that the test models move when any constant changes."""

import copy
import json
import math

import numpy as np
import pytest
import torch

import nutitar_cases as cases
import plain_nutitar as P
from mini_gpt_inference_amd.config.model_config import ConfigError
from mini_gpt_inference_amd.models import nutitar
from mini_gpt_inference_amd.parts.base import POSITIONS, PartSpec
from mini_gpt_inference_amd.parts.model import DecoderModel
from mini_gpt_inference_amd.weights.random_init import random_tensors


def _tensors(name):
    t = random_tensors(cases.config(name), cases.SEEDS[name], torch.bfloat16, cases.STD_SCALE)
    return {k: v.to(P.DTYPE) for k, v in t.items()}


def _ids(n, vocab, seed=0):
    return [int(x) for x in np.random.default_rng(seed).integers(0, vocab, size=n)]


# ---------------------------------------------------------------- mechanisms
def test_token_shift_is_a_blend_with_the_token_before():
    g = torch.Generator().manual_seed(1)
    h = torch.randn(5, 6, generator=g, dtype=P.DTYPE)
    shift = torch.rand(6, generator=g, dtype=P.DTYPE)
    got = P.token_shift(h, shift)
    assert torch.allclose(got[0], h[0] * (1 - shift))                      # zeros before the first token
    assert torch.allclose(got[3], (1 - shift) * h[3] + shift * h[2])
    assert torch.equal(P.token_shift(h, torch.zeros(6, dtype=P.DTYPE)), h)
    assert torch.allclose(P.token_shift(h, torch.ones(6, dtype=P.DTYPE))[1:], h[:-1])


def test_xielu_branches_meet_at_zero_and_follow_their_formulas():
    p, q = torch.tensor(0.3, dtype=P.DTYPE), torch.tensor(-0.7, dtype=P.DTYPE)
    z = torch.tensor([-3.0, -1e-9, 0.0, 1e-9, 2.0], dtype=P.DTYPE)
    y = P.xielu(z, p, q)
    sp = lambda v: math.log1p(math.exp(v))
    assert abs(float(y[4]) - (sp(0.3) * 4.0 + 1.0)) < 1e-12
    assert abs(float(y[0]) - ((0.5 + sp(-0.7)) * (math.exp(-3.0) - 1.0 + 3.0) - 1.5)) < 1e-12
    assert float(y[2]) == 0.0 and abs(float(y[1])) < 1e-8 and abs(float(y[3])) < 1e-8


def test_rotation_depends_on_distance_only_and_keeps_the_rest():
    g = torch.Generator().manual_seed(2)
    q, k = torch.randn(9, 1, 10, generator=g, dtype=P.DTYPE), torch.randn(9, 1, 10, generator=g, dtype=P.DTYPE)
    freq = P.plain_frequencies(6, 100.0)
    rq, rk = P.rotate_half(q, 6, freq), P.rotate_half(k, 6, freq)
    assert torch.equal(rq[..., 6:], q[..., 6:])
    same = q[4:5].repeat(9, 1, 1), k[2:3].repeat(9, 1, 1)          # the same two vectors at every position
    a, b = P.rotate_half(same[0], 6, freq), P.rotate_half(same[1], 6, freq)
    dots = [(a[i + 2, 0] * b[i, 0]).sum() for i in range(7)]
    assert max(abs(float(d - dots[0])) for d in dots) < 1e-12
    # a magnitude multiplies the rotated channels and only those
    m = P.rotate_half(q, 6, freq, 1.5)
    assert torch.allclose(m[..., :6], rq[..., :6] * 1.5) and torch.equal(m[..., 6:], q[..., 6:])


def test_frequency_scalings_at_their_ends():
    dims, base = 16, 10000.0
    plain = P.plain_frequencies(dims, base)
    # stretch: a huge original context leaves every frequency alone, a tiny one divides all by the factor
    assert P.stretched_frequencies(dims, base, 8.0, 1.0, 4.0, 1e9) == plain
    assert np.allclose(P.stretched_frequencies(dims, base, 8.0, 1.0, 4.0, 1e-3), [f / 8.0 for f in plain])
    mid = P.stretched_frequencies(dims, base, 8.0, 1.0, 4.0, 64.0)
    assert mid[0] == plain[0] and abs(mid[-1] - plain[-1] / 8.0) < 1e-18
    assert any(plain[i] / 8.0 < mid[i] < plain[i] for i in range(len(plain)))
    # ramp: fast pairs (few positions a turn) stay, slow ones are divided; cosine and sine grow with the factor
    f, mag = P.ramped_frequencies(dims, base, 4.0, 64.0, 16.0, 1.0)
    assert f[0] == plain[0] and abs(f[-1] - plain[-1] / 4.0) < 1e-18 and abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert all(plain[i] / 4.0 <= f[i] <= plain[i] for i in range(len(plain)))


@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_the_frameworks_frequency_tables_are_the_plain_ones(name):
    for layer in cases.RAW[name]["layers"]:
        dims, freq, mag = P.rotation_of(layer["mixer"]["rot"])
        params = nutitar._rotation("test", layer["mixer"]["rot"], dims).part_params()
        params.pop("kind")
        part = POSITIONS.build(PartSpec("rotary_half", params))
        assert np.allclose(part.frequency_values(), freq, rtol=1e-14, atol=0.0) and abs(part.magnitude - mag) < 1e-15


def test_window_with_kept_first_tokens():
    seen = P.window_with_first(12, 3, 2)
    assert seen[9].tolist() == [True, True] + [False] * 5 + [True] * 3 + [False] * 2
    assert seen[1].tolist() == [True, True] + [False] * 10
    assert torch.equal(P.window_with_first(12, 100, 0), P.causal(12))
    assert P.window_with_first(12, 1, 5)[8].tolist() == [True] * 5 + [False] * 3 + [True] + [False] * 3


def test_sigmoid_attention_as_an_explicit_sum():
    raw = cases.RAW["C"]
    t = _tensors("C")
    m, eps = raw["layers"][0]["mixer"], raw["norm"]["eps"]
    g = torch.Generator().manual_seed(3)
    h = torch.randn(11, raw["width"], generator=g, dtype=P.DTYPE)
    got = P.sigmoid_attention(h, t, "l0.mix.", m, eps)
    T, H, G, D, E = 11, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = P.unit_rms(h @ t["l0.mix.q"].T + t["l0.mix.q.b"], eps) * t["l0.mix.q.norm"]
    k = P.unit_rms(h @ t["l0.mix.k"].T + t["l0.mix.k.b"], eps) * t["l0.mix.k.norm"]
    v = (h @ t["l0.mix.v"].T + t["l0.mix.v.b"]).view(T, G, E)
    dims, freq, mag = P.rotation_of(m["rot"])
    q, k = P.rotate_half(q.view(T, H, D), dims, freq, mag), P.rotate_half(k.view(T, G, D), dims, freq, mag)
    y = torch.zeros(T, H, E, dtype=P.DTYPE)
    for i in range(T):
        for a in range(H):
            for j in range(i + 1):
                if i - j < m["mask"]["size"] or j < m["mask"]["keep_first"]:
                    s = float(q[i, a] @ k[j, a // (H // G)]) * m["scale"] + float(t["l0.mix.pb"][a])
                    y[i, a] += v[j, a // (H // G)] / (1.0 + math.exp(-s))
    want = y.reshape(T, H * E) @ t["l0.mix.o"].T + t["l0.mix.o.b"]
    assert torch.allclose(got, want, rtol=1e-10, atol=1e-10)


def test_latent_attention_as_an_explicit_sum_and_with_shared_latents():
    raw = cases.RAW["A"]
    t = _tensors("A")
    m, eps = raw["layers"][0]["mixer"], raw["norm"]["eps"]
    g = torch.Generator().manual_seed(4)
    h = torch.randn(9, raw["width"], generator=g, dtype=P.DTYPE)
    got, (c, kr) = P.latent_attention(h, t, "l0.mix.", m, eps, None)
    T, H, D, Pn, E, R = 9, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    dims, freq, mag = P.rotation_of(m["rot"])
    q = (h @ t["l0.mix.q"].T).view(T, H, D + Pn)
    z = h @ t["l0.mix.dkv"].T
    assert torch.allclose(c, P.unit_rms(z[:, :R], eps) * t["l0.mix.dkv.norm"])
    assert torch.allclose(kr, P.rotate_half(z[:, None, R:], dims, freq, mag)[:, 0])
    qr = P.rotate_half(q[..., D:], dims, freq, mag)
    gate = P.sigmoid(h @ t["l0.mix.g"].T)
    y = torch.zeros(T, H, E, dtype=P.DTYPE)
    for i in range(T):
        for a in range(H):
            ks = (c[: i + 1] @ t["l0.mix.uk"][a * D:(a + 1) * D].T)
            vs = (c[: i + 1] @ t["l0.mix.uv"][a * E:(a + 1) * E].T)
            s = (ks @ q[i, a, :D] + kr[: i + 1] @ qr[i, a]) * m["scale"]
            w = torch.exp(s)
            y[i, a] = (w[:, None] * vs).sum(0) / (w.sum() + torch.exp(t["l0.mix.sink"][a])) * gate[i, a]
    assert torch.allclose(got, y.reshape(T, H * E) @ t["l0.mix.o"].T, rtol=1e-10, atol=1e-10)
    # a layer that reads them computes with the given latents, whatever its own input would have made
    m3 = raw["layers"][3]["mixer"]
    a, _ = P.latent_attention(h, t, "l3.mix.", m3, eps, (c, kr))
    b, _ = P.latent_attention(h, t, "l3.mix.", m3, eps, (c * 1.5, kr))
    assert not torch.allclose(a, b)
    # a very negative sink is an ordinary softmax, a very large one leaves nothing
    t2 = dict(t)
    t2["l0.mix.sink"] = torch.full_like(t["l0.mix.sink"], 60.0)
    assert P.latent_attention(h, t2, "l0.mix.", m, eps, None)[0].abs().max() < 1e-12


def test_keyed_value_attention_takes_the_keys_as_projected_for_values():
    raw = cases.RAW["A"]
    t = _tensors("A")
    m, eps = raw["layers"][2]["mixer"], raw["norm"]["eps"]
    g = torch.Generator().manual_seed(5)
    h = torch.randn(7, raw["width"], generator=g, dtype=P.DTYPE)
    got = P.keyed_value_attention(h, t, "l2.mix.", m, eps)
    # one token: the softmax has one term, so the output is the head's own projected key through Wo
    one = P.keyed_value_attention(h[:1], t, "l2.mix.", m, eps)
    k = (h[:1] @ t["l2.mix.k"].T).view(1, m["kv_heads"], m["dim"]).repeat_interleave(m["heads"] // m["kv_heads"], dim=1)
    assert torch.allclose(one, k.reshape(1, -1) @ t["l2.mix.o"].T)
    assert torch.allclose(got[:1], one)
    # the norm's weight moves the scores, not the values
    t2 = dict(t)
    t2["l2.mix.k.norm"] = t["l2.mix.k.norm"] * 0.0
    flat = P.keyed_value_attention(h, t2, "l2.mix.", m, eps)      # all scores zero: running means of the keys
    ks = (h @ t["l2.mix.k"].T).view(7, m["kv_heads"], m["dim"]).repeat_interleave(m["heads"] // m["kv_heads"], dim=1)
    means = torch.cumsum(ks, 0) / torch.arange(1, 8, dtype=P.DTYPE)[:, None, None]
    assert torch.allclose(flat, means.reshape(7, -1) @ t["l2.mix.o"].T)


# ---------------------------------------------------------------- configuration, layout
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_config_round_trip_and_layout(name):
    raw = cases.RAW[name]
    cfg = nutitar.config_from_json(raw)
    assert nutitar.config_from_json(json.loads(json.dumps(nutitar.config_to_json(cfg)))) == cfg
    model = DecoderModel(nutitar.model_spec(cfg))
    wanted = model.weight_requests()
    plan = {n: tuple(s) for n, s, _, _ in nutitar.init_plan(cfg)}
    assert {n: tuple(r.shape) for n, r in wanted.items()} == plan
    layout = model.cache_layout
    assert layout.state_numels == [raw["width"]] * len(raw["layers"])      # every layer keeps its last normed row
    for i, (layer, run) in enumerate(zip(raw["layers"], layout.run_bindings)):
        assert run["arrangement"].kind == "state" and run["mixer"].kind == "kv"
        group = layout.groups[run["mixer"].group]
        m = layer["mixer"]
        if layer["type"] == "latent_attention":
            assert group.joint and group.head_dim >= m["kv_rank"] + m["rot_dim"] and group.n_kv_head == 1
            assert run["mixer"].writes == ("kv_from" not in m)
            if "kv_from" in m:
                src = layout.run_bindings[m["kv_from"]]["mixer"]
                assert (src.group, src.index) == (run["mixer"].group, run["mixer"].index)
        elif layer["type"] == "attention":
            mask = m.get("mask")
            assert (group.window, group.keep_first) == ((mask["size"], mask["keep_first"]) if mask else (0, 0))
        else:
            assert group.window == 0 and not group.joint


def test_config_refusals():
    good = cases.RAW["A"]

    def broken(edit):
        raw = copy.deepcopy(good)
        edit(raw)
        with pytest.raises((ConfigError, KeyError)):
            nutitar.config_from_json(raw)

    broken(lambda r: r["layers"][0].update(type="retention"))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=6))               # not the rotated part's size
    broken(lambda r: r["layers"][3]["mixer"].update(kv_from=2))                   # not a latent-attention layer
    broken(lambda r: r["layers"][3]["mixer"].update(kv_from=3))                   # not an earlier layer
    broken(lambda r: r["layers"][3]["mixer"].update(kv_rank=48))                  # another latent size than its source
    broken(lambda r: r["layers"][1]["mixer"].update(kv_heads=3))
    broken(lambda r: r["layers"][2]["mixer"].update(vdim=16))                     # values are keys
    broken(lambda r: r["layers"][2]["mixer"].update(mask={"size": 4}))
    broken(lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7))
    broken(lambda r: r["layers"][2]["mixer"]["rot"]["scaling"].pop("low"))
    broken(lambda r: r["layers"][4].update(mlp={"kind": "moe", "ff": 8}))
    broken(lambda r: r.pop("norm"))


# ---------------------------------------------------------------- every constant matters
def test_the_test_models_move_when_a_constant_changes():
    raw, t = cases.RAW["A"], _tensors("A")
    ids = _ids(48, raw["vocab"], 6)
    base = P.forward(raw, t, ids)

    def moved(edit_raw=None, edit_t=None, frm=0):
        r, tt = copy.deepcopy(raw), dict(t)
        if edit_raw:
            edit_raw(r)
        if edit_t:
            edit_t(tt)
        return float((P.forward(r, tt, ids) - base)[frm:].abs().max())

    assert moved(lambda r: r.update(residual_mult=0.6)) > 1e-3
    assert moved(lambda r: r["embedding"].update(scale=1.9)) > 1e-3
    assert moved(lambda r: r["norm"].update(eps=1e-2)) > 1e-6
    assert moved(lambda r: r["layers"][1]["mixer"]["mask"].update(size=8), frm=10) > 1e-4
    assert moved(lambda r: r["layers"][1]["mixer"]["mask"].update(keep_first=4), frm=12) > 1e-4
    assert moved(lambda r: r["layers"][4]["mixer"]["mask"].update(size=36), frm=37) > 1e-5
    assert moved(lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(factor=4.0)) > 1e-4
    assert moved(lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(slow=0.25)) > 1e-5
    assert moved(lambda r: r["layers"][2]["mixer"]["rot"]["scaling"].update(factor=2.0)) > 1e-5
    assert moved(lambda r: r["layers"][2]["mixer"]["rot"]["scaling"].update(high=2.0)) > 1e-6
    assert moved(lambda r: r["layers"][2]["mixer"]["rot"].update(dims=24)) > 1e-4
    assert moved(lambda r: r["layers"][0]["mixer"].update(scale=0.3)) > 1e-4
    for name in ("l0.shift", "l3.shift", "l0.mix.sink", "l3.mix.sink", "l1.mix.pb", "l0.mix.g", "l0.mlp.act", "l1.mix.o.b",
                 "l1.mix.k.norm", "l2.mix.q.norm", "l0.mix.dkv.norm", "l1.mix.v.b"):
        assert moved(edit_t=lambda tt, n=name: tt.update({n: tt[n] + 0.25})) > 1e-4, name
    # the first tokens: position 0 sees zeros before it, so its logits do not depend on the shift
    r0 = float((P.forward(raw, {**t, "l0.shift": t["l0.shift"] + 0.25, "l3.shift": t["l3.shift"] * 0.0}, ids[:1]) -
                P.forward(raw, t, ids[:1])).abs().max())
    assert r0 > 1e-5        # (1 - shift) still scales what the mixer reads at position 0
