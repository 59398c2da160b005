"""Rilavik on the CPU: limiting cases of the plain implementation's mechanisms (each checked against
a form that is obviously right), config.json in and out, what the architecture refuses, the cache
layout (pages and the convolutions' last inputs for the attention halves, a state for the others),
and the loader's tensor names."""

import copy
import math

import numpy as np
import pytest
import torch

import plain_rilavik as P
import rilavik_cases as cases
from mini_gpt_inference_amd.config.model_config import ConfigError, read_config_json
from mini_gpt_inference_amd.config.registry import architecture_of
from mini_gpt_inference_amd.models import rilavik
from mini_gpt_inference_amd.parts.base import KVNeed, StateNeed
from mini_gpt_inference_amd.parts.model import DecoderModel


def _rnd(g, *shape):
    return torch.randn(*shape, generator=g, dtype=P.DTYPE)


# ---------------------------------------------------------------- the plain mechanisms
def test_short_convolution_is_a_sum_over_the_last_taps_with_zeros_before_the_start():
    g = torch.Generator().manual_seed(0)
    T, C, J = 7, 3, 4
    u, w, b = _rnd(g, T, C), _rnd(g, C, J), _rnd(g, C)
    got = P.short_conv(u, w, b)
    for t in range(T):
        for c in range(C):
            want = float(b[c]) + sum(float(w[c, j]) * float(u[t - J + 1 + j, c]) for j in range(J) if t - J + 1 + j >= 0)
            assert math.isclose(float(got[t, c]), want, abs_tol=1e-12)
    # one tap is a scaling of the current token; a sequence shorter than the taps works
    assert torch.allclose(P.short_conv(u, w[:, -1:]), u * w[:, -1])
    assert torch.allclose(P.short_conv(u[:2], w)[1], w[:, -1] * u[1] + w[:, -2] * u[0])


def test_rotation_depends_on_the_distance_only_and_keeps_lengths():
    g = torch.Generator().manual_seed(1)
    q, k = _rnd(g, 1, 1, 12), _rnd(g, 1, 1, 12)
    scores = []
    for shift in (0, 5, 40):
        seq_q = torch.zeros(shift + 8, 1, 12, dtype=P.DTYPE)
        seq_k = torch.zeros(shift + 8, 1, 12, dtype=P.DTYPE)
        seq_q[shift + 7], seq_k[shift + 3] = q[0], k[0]
        rq, rk = P.rotate_half(seq_q, 8, 100.0, 2.0), P.rotate_half(seq_k, 8, 100.0, 2.0)
        scores.append(float((rq[shift + 7, 0] * rk[shift + 3, 0]).sum()))
        assert math.isclose(float(rq[shift + 7].norm()), float(q.norm()), rel_tol=1e-12)
        assert torch.equal(rq[shift + 7, 0, 8:], q[0, 0, 8:])          # channels beyond `dims` pass
    assert max(scores) - min(scores) < 1e-9
    x = _rnd(g, 9, 2, 8)
    assert torch.allclose(P.rotate_half(x, 8, 50.0)[0], x[0])           # position 0 is not rotated
    same_row = torch.cat([x[8:9]] * 9)
    assert torch.allclose(P.rotate_half(same_row, 8, 50.0, 2.0)[8], P.rotate_half(same_row, 8, 50.0)[4])


def test_gated_linear_attention_is_a_sum_over_the_past_weighted_by_the_decays_in_between():
    g = torch.Generator().manual_seed(2)
    T, H, D, E = 8, 2, 3, 4
    q, k, v = _rnd(g, T, H, D), _rnd(g, T, H, D), _rnd(g, T, H, E)
    alpha = torch.rand(T, H, D, generator=g, dtype=P.DTYPE) * 0.5 + 0.5
    got = P.gla_recurrence(q, k, v, alpha)
    for a in range(H):
        for t in range(T):
            want = torch.zeros(E, dtype=P.DTYPE)
            for s in range(t + 1):
                between = torch.prod(alpha[s + 1:t + 1, a], dim=0)       # the decays of the tokens after s, up to t
                want += float((q[t, a] * between * k[s, a]).sum()) * v[s, a]
            assert torch.allclose(got[t, a], want, atol=1e-12)
    # a decay of one everywhere is plain linear attention
    ones = P.gla_recurrence(q, k, v, torch.ones_like(alpha))
    assert torch.allclose(ones[-1, 0], ((q[-1, 0] @ k[:, 0].T)[:, None] * v[:, 0]).sum(0), atol=1e-12)


def test_window_attention_sees_the_last_positions_only():
    g = torch.Generator().manual_seed(3)
    T, H, G, D, E = 12, 4, 2, 6, 5
    q, k, v = _rnd(g, T, H, D), _rnd(g, T, G, D), _rnd(g, T, G, E)
    assert torch.allclose(P.window_attention(q, k, v, 0.3, 0), P.window_attention(q, k, v, 0.3, T + 5), atol=1e-12)
    grouped = P.window_attention(q, k, v, 0.3, 5)
    full = P.window_attention(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1), 0.3, 5)
    assert torch.allclose(grouped, full, atol=1e-12)
    # a window of one: every token sees itself only
    assert torch.allclose(P.window_attention(q, k, v, 0.3, 1), v.repeat_interleave(2, dim=1))
    # the key just outside the window does not count, the one just inside does
    w = 4
    v2 = v.clone()
    v2[T - 1 - w] += 100.0
    assert torch.equal(P.window_attention(q, k, v2, 0.3, w)[-1], P.window_attention(q, k, v, 0.3, w)[-1])
    v2 = v.clone()
    v2[T - w] += 100.0
    assert float((P.window_attention(q, k, v2, 0.3, w)[-1] - P.window_attention(q, k, v, 0.3, w)[-1]).abs().max()) > 1e-3


def test_state_space_recurrence_is_a_sum_over_the_past():
    g = torch.Generator().manual_seed(4)
    T, H, G, N, E = 7, 4, 2, 3, 5
    x, B, C = _rnd(g, T, H, E), _rnd(g, T, G, N), _rnd(g, T, G, N)
    dt = torch.rand(T, H, generator=g, dtype=P.DTYPE) + 0.1
    A = torch.rand(H, generator=g, dtype=P.DTYPE) + 0.2
    skip = _rnd(g, H)
    got = P.ssd_recurrence(x, B, C, dt, A, skip)
    for a in range(H):
        grp = a // (H // G)
        for t in range(T):
            want = skip[a] * x[t, a]
            for s in range(t + 1):
                decay = math.exp(-float(A[a]) * float(dt[s + 1:t + 1, a].sum()))
                want = want + decay * float(dt[s, a]) * float(C[t, grp] @ B[s, grp]) * x[s, a]
            assert torch.allclose(got[t, a], want, atol=1e-12)


def test_routed_experts_scale_the_input_not_the_output():
    g = torch.Generator().manual_seed(5)
    W, F, n = 6, 5, 4
    h = _rnd(g, 9, W)
    tensors = {"m.router": _rnd(g, n, W)}
    for e in range(n):
        tensors.update({f"m.e{e}.gate": _rnd(g, F, W), f"m.e{e}.up": _rnd(g, F, W), f"m.e{e}.down": _rnd(g, W, F)})
    got = P.routed_experts(h, tensors, "m.", {"router": {"experts": n, "top": 2}, "expert": {"ff": F}})
    scores = P.sigmoid(h @ tensors["m.router"].T)
    for t in range(9):
        order = sorted(range(n), key=lambda e: -float(scores[t, e]))[:2]
        want = torch.zeros(W, dtype=P.DTYPE)
        for e in order:
            u = scores[t, e] * h[t]
            want += tensors[f"m.e{e}.down"] @ (P.silu(tensors[f"m.e{e}.gate"] @ u) * (tensors[f"m.e{e}.up"] @ u))
        assert torch.allclose(got[t], want, atol=1e-12)
    # scaling the input differs from scaling the output (the unit is not linear)
    e = int(scores[0].argmax())
    u = h[0]
    outside = scores[0, e] * (tensors[f"m.e{e}.down"] @ (P.silu(tensors[f"m.e{e}.gate"] @ u) * (tensors[f"m.e{e}.up"] @ u)))
    one = P.routed_experts(h[:1], tensors, "m.", {"router": {"experts": n, "top": 1}, "expert": {"ff": F}})
    assert float((one[0] - outside).abs().max()) > 1e-3


def test_norms_and_activations():
    g = torch.Generator().manual_seed(6)
    x = _rnd(g, 4, 10)
    unit = P.unit_rms(x, 0.0)
    assert torch.allclose((unit * unit).mean(-1), torch.ones(4, dtype=P.DTYPE))
    assert torch.allclose(P.unit_rms(torch.zeros(1, 4, dtype=P.DTYPE), 0.25), torch.zeros(1, 4, dtype=P.DTYPE))
    z = torch.tensor([-800.0, -3.0, 0.0, 2.0, 900.0], dtype=P.DTYPE)
    assert torch.allclose(P.softplus(z)[1:4], torch.log(1.0 + torch.exp(z[1:4])))
    assert float(P.softplus(z)[0]) == 0.0 and float(P.softplus(z)[4]) == 900.0


def test_what_the_test_models_are_sensitive_to(tmp_path):
    """Changing tau, a decay bias, a window by one, the scaling of positions, a tap, a join weight, a
    layer scale, a norm behind a sublayer, the number of norm parts, the experts a token takes or the
    state-space constants moves the logits by far more than the tolerances."""
    folder = cases.write_model(str(tmp_path / "A"), "A")
    cfg, w = P.read_model_folder(folder)
    ids = list(np.random.default_rng(0).integers(0, cfg["vocab"], 60))
    base = P.forward(cfg, w, ids)

    def moved(cfg2=None, w2=None):
        return float((P.forward(cfg2 or cfg, w2 or w, ids) - base).abs().max())

    def with_layer(i, change):
        layers = copy.deepcopy(cfg["layers"])
        change(layers[i])
        return {**cfg, "layers": layers}

    assert moved(with_layer(1, lambda l: l["mixer"].update(tau=1.0))) > 0.05
    assert moved(w2={**w, "l1.mix.a2.b": w["l1.mix.a2.b"] - 2.0}) > 0.05
    assert moved(with_layer(0, lambda l: l["mixer"]["left"]["mask"].update(size=8))) > 0.005
    assert moved(with_layer(0, lambda l: l["mixer"]["left"]["rot"]["scaling"].update(factor=1.0))) > 0.005
    assert moved(w2={**w, "l0.mix.left.k.conv": w["l0.mix.left.k.conv"].flip(1)}) > 0.005
    assert moved(w2={**w, "l0.mix.right.conv": w["l0.mix.right.conv"].flip(1)}) > 0.05
    assert moved(with_layer(0, lambda l: l["mixer"].update(left_scale=1.25, right_scale=0.75))) > 0.05
    assert moved(w2={**w, "l2.ls1": w["l2.ls1"] * 2.0}) > 0.05
    assert moved(w2={**w, "l1.norm2b": w["l1.norm2b"] + 0.5}) > 0.05
    assert moved(with_layer(2, lambda l: l["mixer"]["right"].update(norm_groups=1))) > 0.005
    assert moved(with_layer(3, lambda l: l["mlp"]["router"].update(top=2))) > 0.05
    assert moved(w2={**w, "l0.mix.right.A_log": w["l0.mix.right.A_log"] + 1.0}) > 0.005
    assert moved(w2={**w, "l0.mix.right.dt_bias": w["l0.mix.right.dt_bias"] + 1.0}) > 0.05
    assert moved(w2={**w, "l0.mix.right.D": w["l0.mix.right.D"] + 1.0}) > 0.05
    # (a common factor would be undone by the norm behind the sublayer)
    assert moved(w2={**w, "l1.mix.norm": w["l1.mix.norm"] + torch.linspace(0.0, 2.0, 24, dtype=P.DTYPE)}) > 0.05


def test_residuals_are_reported_layer_by_layer(tmp_path):
    folder = cases.write_model(str(tmp_path / "D"), "D")
    cfg, w = P.read_model_folder(folder)
    res = []
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5], residuals=res)
    assert len(res) == len(cfg["layers"]) and res[0].shape == (5, cfg["width"]) and logits.shape == (5, cfg["vocab"])
    # causal: a later token does not change an earlier position
    assert torch.allclose(P.forward(cfg, w, [1, 2, 3]), logits[:3], atol=1e-9)


# ---------------------------------------------------------------- configuration
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_config_round_trip(name, tmp_path):
    cfg = rilavik.config_from_json(cases.RAW[name])
    assert rilavik.config_from_json(rilavik.config_to_json(cfg)) == cfg
    folder = cases.write_model(str(tmp_path / name), name)
    raw = read_config_json(folder)
    assert architecture_of(raw).name == "Rilavik" and rilavik.config_from_json(raw) == cfg


def test_random_configurations_are_accepted_and_round_trip():
    rng = np.random.default_rng(4)
    for _ in range(30):
        raw = cases.random_raw(rng)
        cfg = rilavik.config_from_json(raw)
        assert rilavik.config_from_json(rilavik.config_to_json(cfg)) == cfg
        DecoderModel(rilavik.model_spec(cfg))


def _edited(name, edit):
    raw = copy.deepcopy(cases.RAW[name])
    edit(raw)
    return raw


@pytest.mark.parametrize("edit", [
    lambda r: r["layers"][0].update(type="retention"),
    lambda r: r["layers"][1]["mixer"].update(tau=0.0),
    lambda r: r["layers"][1]["mixer"].update(heads=0),
    lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3),
    lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=7),
    lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=64),
    lambda r: r["layers"][0]["mixer"]["left"]["mask"].update(size=-1),
    lambda r: r["layers"][0]["mixer"]["right"].update(groups=3),
    lambda r: r["layers"][0]["mixer"]["right"].update(norm_groups=5),
    lambda r: r["layers"][0]["mixer"].pop("right"),
    lambda r: r["layers"][0]["mlp"].update(kind="dense"),
    lambda r: r["layers"][0]["mlp"]["router"].update(top=6),
    lambda r: r.update(layers=[]),
    lambda r: r.update(width=0),
])
def test_refusals(edit):
    with pytest.raises(ConfigError):
        rilavik.config_from_json(_edited("A", edit))


# ---------------------------------------------------------------- model as data
def test_cache_layout_and_tensor_names():
    cfg = cases.config("A")
    model = DecoderModel(rilavik.model_spec(cfg))
    layout = model.cache_layout
    kinds = [{role: b.kind for role, b in run.items()} for run in layout.run_bindings]
    assert kinds == [{"mixer0": "kv", "mixer1": "state"}, {"mixer": "state"}, {"mixer0": "kv", "mixer1": "state"},
                     {"mixer": "state"}]
    # a left half keeps pages of max(dim, vdim) rounded up to 32 channels a head, behind its window
    assert [(g.n_kv_head, g.head_dim, g.n_pools) for g in layout.groups] == [(2, 32, 1), (1, 32, 1)]
    needs = [p.cache_need() for layer in model.layers for r, p in layer.parts.items() if r.startswith("mixer")]
    kv = [n for n in needs if isinstance(n, KVNeed)]
    assert [n.window for n in kv] == [7, 37]
    # ... and beside them the last taps - 1 projected rows of q, k and v in the padded layout
    assert [n.state_numel for n in kv] == [2 * (4 + 2 + 2) * 32, 1 * (2 + 1 + 1) * 32]
    st = [n for n in needs if isinstance(n, StateNeed)]
    # state-space: heads * state * vdim and the last taps - 1 rows of x, B and C; gla: heads * dim * vdim
    assert [n.numel for n in st] == [4 * 8 * 16 + 3 * (64 + 2 * 2 * 8), 2 * 16 * 24, 2 * 16 * 24 + 1 * (48 + 2 * 16), 3 * 8 * 40]
    wanted = model.weight_requests()
    plan_names = {name: tuple(shape) for name, shape, _, _ in rilavik.init_plan(cfg)}
    assert set(wanted) == set(plan_names)
    for name, req in wanted.items():
        assert req.fits(plan_names[name]), name
    assert "l2.norm2" not in wanted and "l2.ls2" not in wanted and "l2.ls1" in wanted
    assert "l0.mix.left.q.conv" in wanted and "l0.mix.right.conv.b" in wanted and "l1.mix.a2.b" in wanted
    assert "l0.mlp.e4.down" in wanted and "l0.mlp.e5.down" not in wanted and "l0.mlp.router" in wanted
    # the decay projection's narrow middle comes from the stored tensors
    assert wanted["l1.mix.a1"].shape[0] == -1 and wanted["l1.mix.a1"].fits((3, 64)) and not wanted["l1.mix.a1"].fits((3, 65))
    assert model.graph_safe and model.plan_safe


def test_no_convolution_no_rotation_no_window_leave_their_tensors_and_state_out():
    cfg = cases.config("B")
    model = DecoderModel(rilavik.model_spec(cfg))
    wanted = model.weight_requests()
    assert "l1.mix.left.q.conv" not in wanted and "l2.mix.left.q.conv" in wanted
    kv = [p.cache_need() for layer in model.layers for r, p in layer.parts.items() if r == "mixer0"]
    assert [(n.window, n.state_numel) for n in kv] == [(0, 0), (100, 3 * 3 * 64)]


def test_a_model_of_state_mixers_only_still_has_a_group_of_pages():
    """No mixer keeps keys and values: the layout holds one group without pools, whose page tables only count
    how far every request has come."""
    model = DecoderModel(rilavik.model_spec(cases.config("E")))
    layout = model.cache_layout
    assert [(g.n_pools, g.window) for g in layout.groups] == [(0, 0)]
    assert [b.kind for run in layout.run_bindings for b in run.values()] == ["state", "state"]
    assert layout.state_numels == [2 * 24 * 16, 3 * 16 * 32]
