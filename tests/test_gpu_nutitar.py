"""Nutitar on the GPU against the plain implementation (tests/plain_nutitar.py): each new kernel alone (the
activation, the norm with the token shift and its kept row per request, the latent's rotated part, norms with
weights in front of the rotation and values taken from the keys, the window that keeps the first tokens and
sigmoid weights in every attention kernel, with a key made to stand out at every edge); whole prompts against
token-by-token decoding, portions down to two tokens and mixed batches with pages, request slots and kept rows
used again, steps that want no logits, in 32-bit and bfloat16; long decoding; configurations drawn at random;
greedy generation through LLMEngine."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import nutitar_cases as cases
import plain_nutitar as P
from mini_gpt_inference_amd import EngineConfig, SamplingParams
from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
from mini_gpt_inference_amd.engine.replay import TraceReplayer
from mini_gpt_inference_amd.ops import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda"
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rnd(g, *shape, dtype="float32", scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(TDT[dtype])


def _d(t):
    return t.to(P.DTYPE)


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


# Steps of a kernel-level schedule: lists of (request, first token of the request, count).  Request r's tokens
# are rows STARTS[r] .. of the test's arrays; its slot is r + 1 (slot 0 and the last stay untouched).
WHOLE = [[(0, 0, 70), (1, 0, 1), (2, 0, 32), (3, 0, 33)]]
PORTIONS = [[(0, 0, 31), (3, 0, 2)], [(0, 31, 2), (1, 0, 1), (3, 2, 30)], [(3, 32, 1), (0, 33, 36), (2, 0, 17)],
            [(0, 69, 1), (2, 17, 15)]]
ONE_BY_ONE = [[(r, t, 1) for r, n in enumerate((70, 1, 32, 33)) if t < n] for t in range(70)]
STARTS, COUNTS = [0, 70, 71, 103], [70, 1, 32, 33]
N_ROWS = 136


def _step_arrays(step):
    rows, cu, pos, req, slots = [], [0], [], [], []
    for i, (r, first, count) in enumerate(step):
        rows += list(range(STARTS[r] + first, STARTS[r] + first + count))
        pos += list(range(first, first + count))
        req += [i] * count
        cu.append(len(rows))
        slots.append(r + 1)
    return rows, _i32(cu), _i32(pos), _i32(req), _i32(slots)


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,hidden", [(1, 24), (9, 130), (70, 256), (300, 1000)])
def test_xielu(dtype, n, hidden):
    g = torch.Generator().manual_seed(n + hidden)
    z = _rnd(g, n, hidden + 3, dtype=dtype, scale=2.0)
    z[0, :4] = torch.tensor([0.0, -0.0, 1e-4, -1e-4]).to(TDT[dtype])
    p, q = torch.tensor(0.4), torch.tensor(-1.1)
    want = P.xielu(_d(z[:, :hidden]), _d(p), _d(q))
    coef = torch.stack([torch.nn.functional.softplus(p), torch.nn.functional.softplus(q) + 0.5]).to(DEV)
    for fast in (False, True):
        out = torch.full((n, hidden + 5), 9.0, dtype=TDT[dtype], device=DEV)
        kernels.xielu(z.to(DEV), out, coef, n, hidden, fast=fast)
        helpers.assert_close(out[:, :hidden], want, dtype, f"xielu fast={fast}")
        assert (out[:, hidden:] == 9.0).all()


@pytest.mark.parametrize("n,k,out,bias", [(300, 256, 1000, True), (8, 2048, 8192, False), (64, 4096, 256, False),
                                          (2048, 512, 2048, True), (33, 64, 72, False)])
def test_xielu_as_the_tiled_products_epilogue(n, k, out, bias):
    """The activation inside the tiled bfloat16 product, also where the inner size is split among workgroups and
    the parts are joined by a second kernel."""
    g = torch.Generator().manual_seed(n + k + out)
    a, w = _rnd(g, n, k, dtype="bfloat16"), _rnd(g, out, k, dtype="bfloat16", scale=k ** -0.5)
    b = _rnd(g, out, scale=0.3) if bias else None
    p, q = torch.tensor(-0.2), torch.tensor(0.6)
    want = P.xielu(_d(a) @ _d(w).T + (_d(b) if bias else 0.0), _d(p), _d(q))
    coef = torch.stack([torch.nn.functional.softplus(p), torch.nn.functional.softplus(q) + 0.5]).to(DEV)
    need = kernels.linear_mfma_partials(n, out, k, kernels.EPI_XIELU)
    partials = torch.empty(need, dtype=torch.float32, device=DEV) if need else None
    got = torch.full((n, out + 8), 9.0, dtype=torch.bfloat16, device=DEV)
    assert kernels.linear_mfma_xielu(a.to(DEV), w.to(DEV), b.to(DEV) if bias else None, got, n, coef, partials=partials)
    helpers.assert_close(got[:, :out], want, "bfloat16", f"xielu epilogue, {'split' if need else 'whole'} inner size")
    assert (got[:, out:] == 9.0).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,pad", [(40, 3), (40, 0), (256, 4), (1030, 2), (2048, 0), (3076, 8)])
def test_norm_and_token_shift_keep_a_row_per_request(dtype, width, pad):
    """Four requests of 70, 1, 32 and 33 tokens: whole, in portions cut anywhere, and one token a step (where one
    kernel norms, shifts and keeps); the kept rows start as NaN, and the slots are used a second time by other
    sequences.  Beside the shift: the pending addition is made, the sums are cleared, h is the norm."""
    g = torch.Generator().manual_seed(width)
    gain, shift = _rnd(g, width, scale=0.2), torch.rand(width, generator=g)
    state = torch.full((6, width + pad), float("nan"), device=DEV)
    for trial in range(2):
        x0, y0 = _rnd(g, N_ROWS, width, scale=3.0), _rnd(g, N_ROWS, width)
        xs = _d(x0) + 0.3 * _d(y0)
        h_want = P.unit_rms(xs, 1e-5) * (1.0 + _d(gain))
        if dtype == "bfloat16":
            h_want = _d(h_want.to(torch.bfloat16))       # the shift reads the rows the other sublayers read
        hs_want = torch.cat([P.token_shift(h_want[s:s + c], _d(shift)) for s, c in zip(STARTS, COUNTS)])
        for plan in (WHOLE, PORTIONS, ONE_BY_ONE):
            got_h, got_hs = torch.zeros(N_ROWS, width, dtype=P.DTYPE), torch.zeros(N_ROWS, width, dtype=P.DTYPE)
            for step in plan:
                rows, cu, pos, req, slots = _step_arrays(step)
                n = len(rows)
                x, y = x0[rows].to(DEV).contiguous(), y0[rows].to(DEV).contiguous()
                h = torch.zeros(n, width, dtype=TDT[dtype], device=DEV)
                hs = torch.zeros(n, width, dtype=TDT[dtype], device=DEV)
                single = all(c == 1 for _, _, c in step)
                kernels.parallel_norm(x, y, 0.3, n, gain=gain.to(DEV), offset=1.0, eps=1e-5, h=h, hs=hs if single else None,
                                      shift=shift.to(DEV), state=state, state_slots=slots, q_req=req, positions=pos)
                if not single:
                    kernels.token_shift(h, hs, shift.to(DEV), state, slots, req, cu, pos, n, len(step))
                assert (y == 0).all()
                helpers.assert_close(x, xs[rows], "float32", "x + mult * y")
                got_h[rows], got_hs[rows] = _d(h.cpu()), _d(hs.cpu())
            helpers.assert_close(got_h, h_want, dtype, "the norm")
            helpers.assert_close(got_hs, hs_want, dtype, f"the shifted rows, trial {trial}")
            last = torch.stack([h_want[s + c - 1] for s, c in zip(STARTS, COUNTS)])
            helpers.assert_close(state[1:5, :width], last, dtype, "the kept rows")
            assert torch.isnan(state[0]).all() and torch.isnan(state[5]).all() and torch.isnan(state[:, width:]).all()
    # the addition alone, as the model makes it before its last norm
    x, y = x0.to(DEV).contiguous(), y0.to(DEV).contiguous()
    kernels.parallel_norm(x, y, 0.3, N_ROWS)
    helpers.assert_close(x, xs, "float32", "the addition alone")
    assert (y == 0).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,R,rank,row", [(4, 16, 8, 40, 48), (1, 12, 6, 21, 32), (3, 32, 32, 96, 128), (2, 0, 4, 16, 24)])
def test_latent_rows_and_rotated_query_parts(dtype, H, D, R, rank, row):
    g = torch.Generator().manual_seed(H + D + rank)
    n, page, pages = 37, 4, 12
    freq, mag = P.ramped_frequencies(R, 1000.0, 4.0, 16.0, 8.0, 1.0)
    q_off, c_off = 0, H * (D + R) + 5
    z = _rnd(g, n, c_off + rank + R + 2, dtype=dtype)
    gain = _rnd(g, rank, scale=0.3) + 1.0
    pos = torch.randint(0, 900, (n,), generator=g)
    slots = torch.randperm(page * pages, generator=g)[:n]
    slots[5] = -1                                    # a token of the padding keeps no row
    pool = torch.full((pages, 1, page, row), float("nan"), dtype=TDT[dtype], device=DEV)
    zd = z.to(DEV).clone()
    kernels.latent_prepare(zd, q_off, H, D, R, _i32(pos.tolist()), torch.tensor(freq, dtype=torch.float64).float().to(DEV), n,
                           mag, c_off=c_off, rank=rank, gain=gain.to(DEV), eps=1e-5, pool=pool, slot_mapping=_i32(slots.tolist()))

    def rotated(x, p):
        full = torch.zeros(int(p.max()) + 1, x.shape[1], x.shape[2], dtype=P.DTYPE)
        out = torch.empty_like(x)
        for i in range(x.shape[0]):
            full[int(p[i])] = x[i]
            out[i] = P.rotate_half(full, R, freq, mag)[int(p[i])]
        return out

    q = _d(z[:, :H * (D + R)]).view(n, H, D + R)
    want_q = torch.cat([q[..., :D], rotated(q[..., D:], pos)], dim=-1).reshape(n, -1)
    helpers.assert_close(zd[:, :H * (D + R)], want_q, dtype, "queries")
    assert torch.equal(zd[:, H * (D + R):].cpu(), z[:, H * (D + R):])
    lat = _d(z[:, c_off:c_off + rank])
    want_c = P.unit_rms(lat, 1e-5) * _d(gain)
    want_kr = rotated(_d(z[:, None, c_off + rank:c_off + rank + R]), pos)[:, 0]
    flat = pool.view(-1, row)
    for i in range(n):
        if int(slots[i]) < 0:
            continue
        helpers.assert_close(flat[int(slots[i]), :rank][None], want_c[i][None], dtype, "latent")
        helpers.assert_close(flat[int(slots[i]), rank:rank + R][None], want_kr[i][None], dtype, "rotated key part")
        assert (flat[int(slots[i]), rank + R:] == 0).all()
    written = set(int(s) for s in slots if int(s) >= 0)
    assert all(torch.isnan(flat[s]).all() for s in range(page * pages) if s not in written)
    # a layer that reads another's rows rotates its queries only
    zd2 = z.to(DEV).clone()
    kernels.latent_prepare(zd2, q_off, H, D, R, _i32(pos.tolist()), torch.tensor(freq, dtype=torch.float64).float().to(DEV), n, mag)
    assert torch.equal(zd2, zd)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("norm,H,G,D,rot,from_keys", [("head", 4, 1, 24, 12, True), ("whole", 3, 1, 20, 10, False),
                                                      ("whole", 6, 3, 96, 24, False), ("head", 2, 2, 64, 64, True),
                                                      ("head", 5, 5, 12, 4, False)])
def test_norms_with_weights_before_the_rotation_and_values_from_keys(dtype, norm, H, G, D, rot, from_keys):
    g = torch.Generator().manual_seed(H * D + rot)
    n, page, pages, E = 29, 4, 10, D
    s = -(-D // 32) * 32
    k_off, v_off = H * s, (H + G) * s
    z = _rnd(g, n, v_off + (0 if from_keys else G * s) + 1, dtype=dtype)
    if not from_keys:       # the stacked projection leaves zeros in the channels a value head does not have
        z[:, v_off:v_off + G * s].view(n, G, s)[..., E:] = 0
    wq = _rnd(g, D if norm == "head" else H * D, scale=0.3) + 1.0
    wk = _rnd(g, D if norm == "head" else G * D, scale=0.3) + 1.0
    pos = torch.randint(0, 700, (n,), generator=g)
    slots = torch.randperm(page * pages, generator=g)[:n]
    freq, mag = P.ramped_frequencies(rot, 500.0, 3.0, 32.0, 8.0, 1.0)
    kp = torch.full((pages, G, page, s), float("nan"), dtype=TDT[dtype], device=DEV)
    vp = torch.full_like(kp, float("nan"))
    zd = z.to(DEV).clone()
    kernels.qk_prepare(zd, 0, k_off, v_off, H, G, D, E, s, n, positions=_i32(pos.tolist()),
                       freq=torch.tensor(freq, dtype=torch.float64).float().to(DEV), norm_eps=1e-5, k_pool=kp, v_pool=vp,
                       slot_mapping=_i32(slots.tolist()), norm=norm, q_norm_weight=wq.to(DEV), k_norm_weight=wk.to(DEV),
                       values_from_keys=from_keys, rot_magnitude=mag)
    q = _d(z[:, :H * s]).view(n, H, s)[..., :D]
    k = _d(z[:, k_off:k_off + G * s]).view(n, G, s)[..., :D]
    if norm == "head":
        qn, kn = P.unit_rms(q, 1e-5) * _d(wq), P.unit_rms(k, 1e-5) * _d(wk)
    else:
        qn = (P.unit_rms(q.reshape(n, H * D), 1e-5) * _d(wq)).view(n, H, D)
        kn = (P.unit_rms(k.reshape(n, G * D), 1e-5) * _d(wk)).view(n, G, D)

    def rotated(x):
        out = torch.empty_like(x)
        for i in range(n):
            full = torch.zeros(int(pos[i]) + 1, x.shape[1], x.shape[2], dtype=P.DTYPE)
            full[int(pos[i])] = x[i]
            out[i] = P.rotate_half(full, rot, freq, mag)[int(pos[i])]
        return out

    helpers.assert_close(zd[:, :H * s].view(n, H, s)[..., :D], rotated(qn), dtype, "queries")
    want_k = rotated(kn)
    want_v = k if from_keys else _d(z[:, v_off:v_off + G * s]).view(n, G, s)[..., :E]
    for i in range(n):
        pg, off = int(slots[i]) // page, int(slots[i]) % page
        helpers.assert_close(kp[pg, :, off, :D], want_k[i], dtype, "cached keys")
        helpers.assert_close(vp[pg, :, off, :E], want_v[i], dtype, "cached values")
        assert (kp[pg, :, off, D:] == 0).all() and (vp[pg, :, off, E:] == 0).all()


def _paged(k, v, page, perm, dtype):
    """[T, G, D] keys and values into pools [pages, G, page, D] with the sequence's pages in the order `perm`."""
    T, G, D = k.shape
    pages = T // page
    kp = torch.full((pages, G, page, D), float("nan"), dtype=TDT[dtype])
    vp = torch.full((pages, G, page, D), float("nan"), dtype=TDT[dtype])
    for i in range(pages):
        kp[perm[i]] = k[i * page:(i + 1) * page].transpose(0, 1)
        vp[perm[i]] = v[i * page:(i + 1) * page].transpose(0, 1)
    return kp.to(DEV), vp.to(DEV)


def _all_attention_kernels(dtype, D, q, k, v, scale, window, keep_first, bias, want, first, tag):
    """The queries from `first` on as a portion on top of cached tokens, and the last one alone, through every
    attention kernel that takes the sizes."""
    T, H, G, page = q.shape[0], q.shape[1], k.shape[1], 16
    g = torch.Generator().manual_seed(T + D)
    pages = T // page
    perm = torch.randperm(pages, generator=g)
    kp, vp = _paged(k, v, page, perm, dtype)
    bt = perm.to(torch.int32).view(1, pages).to(DEV)
    n = T - first
    qd = q[first:].reshape(n, H * D).to(DEV)
    ref = want[first:].reshape(n, H * D)
    kw = {"window": window, "keep_first": keep_first, "score_bias": None if bias is None else bias.to(DEV)}
    out = torch.zeros(n, H * D, dtype=TDT[dtype], device=DEV)
    kernels.paged_attention_generic(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), _i32([0] * n), n, 1, H, scale, **kw)
    helpers.assert_close(out, ref, dtype, f"general kernel, {tag}")
    one = torch.zeros(1, H * D, dtype=TDT[dtype], device=DEV)
    kernels.paged_attention_generic(qd[n - 1:], one, kp, vp, bt, _i32([0, 1]), _i32([T]), _i32([0]), 1, 1, H, scale, **kw)
    helpers.assert_close(one, ref[n - 1:], dtype, f"general kernel, one query, {tag}")
    if dtype != "bfloat16":
        return
    if D in (32, 64, 96, 128):
        out.zero_()
        assert kernels.prefill_attention_bf16(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), 1, n, H, scale, **kw)
        helpers.assert_close(out, ref, dtype, f"tile kernel, {tag}")
    for fast in (True, False) if D <= 256 else ():
        out.zero_()
        assert kernels.paged_attention_split_bf16(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), _i32([0] * n), n, 1, H,
                                                  scale, fast=fast, **kw)
        helpers.assert_close(out, ref, dtype, f"split kernel (fast={fast}), {tag}")
    if D in (32, 64, 128):
        one.zero_()
        assert kernels.paged_attention_decode_bf16(qd[n - 1:], one, kp, vp, bt, _i32([T - 1]), _i32([0]), 1, H, scale,
                                                   identity=True, **kw)
        helpers.assert_close(one, ref[n - 1:], dtype, f"decode kernel, {tag}")


@pytest.mark.parametrize("dtype,D", [("float32", 32), ("bfloat16", 32), ("bfloat16", 64), ("bfloat16", 96), ("bfloat16", 128),
                                     ("float32", 20)])
@pytest.mark.parametrize("window,keep_first", [(1, 5), (2, 1), (16, 16), (17, 3), (70, 64), (40, 20), (100, 130), (30, 0),
                                               (700, 9)])
@pytest.mark.parametrize("sigmoid", [False, True])
def test_a_key_at_every_edge_of_a_window_that_keeps_the_first_tokens(dtype, D, window, keep_first, sigmoid):
    """The last query is made to look like one key, scaled so that this key carries the result if it is seen: the
    oldest key the window still holds, the one before it, the last of the kept first tokens, the one behind it.
    With softmax weights and with sigmoid weights (a negative number per head keeps the other keys' weights small)."""
    H, G, T = 4, 2, 608
    scale = D ** -0.5
    last = T - 1
    edges = {"window_in": last - (window - 1), "window_out": last - window, "first_in": keep_first - 1,
             "first_out": keep_first}
    bias = torch.tensor([-6.0, -5.0, -7.0, -6.5]) if sigmoid else None
    for tag, far in edges.items():
        if not 0 <= far < last:
            continue
        g = torch.Generator().manual_seed(7 + D + window + keep_first)
        q, k, v = _rnd(g, T, H, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype)
        k[far] *= 4.0
        q[-1] = k[far].float().repeat_interleave(H // G, dim=0).to(TDT[dtype])
        kk, vv = _d(k).repeat_interleave(H // G, dim=1), _d(v).repeat_interleave(H // G, dim=1)
        want = P.attend(_d(q), kk, vv, scale, P.window_with_first(T, window, keep_first), None if bias is None else _d(bias))
        if tag.endswith("out") and far >= keep_first and last - far >= window:
            # the key is not seen; were it, the result would be another
            other = P.window_with_first(T, window, keep_first)
            other[last, far] = True
            seen = P.attend(_d(q), kk, vv, scale, other, None if bias is None else _d(bias))
            assert float((want[-1] - seen[-1]).abs().max()) > 0.3
        _all_attention_kernels(dtype, D, q, k, v, scale, window, keep_first, bias, want, 480, f"{tag}, key at {far}")


@pytest.mark.parametrize("dtype,D", [("float32", 24), ("bfloat16", 64), ("bfloat16", 128), ("bfloat16", 144), ("bfloat16", 640),
                                     ("float32", 1000)])
def test_sigmoid_weights_without_a_window_and_a_key_far_back(dtype, D):
    """No window: every earlier key counts with its own sigmoid, one of them hundreds of positions back made large.
    (Heads beyond 256 channels are the general kernel's alone.)"""
    H, G, T = 2, 1, 608
    g = torch.Generator().manual_seed(D)
    q, k, v = _rnd(g, T, H, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype)
    k[3] *= 4.0
    q[-1] = k[3].float().repeat_interleave(H, dim=0).to(TDT[dtype])
    bias = torch.tensor([-5.0, -6.0])
    want = P.attend(_d(q), _d(k).repeat_interleave(H, dim=1), _d(v).repeat_interleave(H, dim=1), D ** -0.5, P.causal(T), _d(bias))
    _all_attention_kernels(dtype, D, q, k, v, D ** -0.5, 0, 0, bias, want, 480, "no window")


# ---------------------------------------------------------------- the model through the step function
LENGTHS = {"A": [5, 70, 23, 41, 2, 64, 37], "B": [1, 9, 33, 17, 130], "C": [40, 3, 64, 21], "D": [75, 12, 30, 6, 49]}
_folders, _plain, _twin = {}, {}, {}


def _folder(tmp_path_factory, name):
    if name not in _folders:
        _folders[name] = cases.write_model(str(tmp_path_factory.mktemp("nutitar") / name), name)
    return _folders[name]


def _requests(folder, name):
    rng = np.random.default_rng(cases.SEEDS[name])
    return {f"r{i}": helpers.random_ids(rng, cases.RAW[name]["vocab"], n) for i, n in enumerate(LENGTHS[name])}


def _plain_logits(folder, name):
    if name not in _plain:
        cfg, w = P.read_model_folder(folder)
        _plain[name] = {rid: P.forward(cfg, w, ids).numpy() for rid, ids in _requests(folder, name).items()}
    return _plain[name]


def _row_errors(got, want):
    """Per position: root mean square over the vocabulary of the difference, its mean taken off."""
    d = np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)
    d = d - d.mean(axis=1, keepdims=True)
    return np.sqrt((d * d).mean(axis=1))


def _rounded_twin(cfg, w, ids):
    """The plain implementation with every matrix product rounded to bfloat16: what rounding alone does."""
    P.ROUNDING = torch.bfloat16
    try:
        return P.forward(cfg, w, ids).numpy()
    finally:
        P.ROUNDING = None


def _assert_within_rounding(folder, key, ids, got, want, what, worst=3.0):
    """bfloat16: a position's error may be `worst` times what rounding alone causes at the request's worst
    position, and the request's mean error three times the mean of that."""
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    if key not in _twin:
        cfg, w = P.read_model_folder(folder)
        _twin[key] = _row_errors(_rounded_twin(cfg, w, ids), want)
    noise, err = _twin[key], _row_errors(got, want)
    assert err.max() <= worst * noise.max(), f"{what}: worst position {err.max():.3e} > {worst} * {noise.max():.3e}"
    assert err.mean() <= 3.0 * noise.mean(), f"{what}: mean {err.mean():.3e} > 3 * {noise.mean():.3e}"


def _check(folder, name, dtype, rid, ids, got, want, what):
    if dtype == "float32":
        assert np.isfinite(got).all(), what
        err = _row_errors(got, want)
        assert err.max() <= 5e-5 * max(1.0, float(np.abs(want).max())), f"{what}: {err.max():.3e}"
    else:
        _assert_within_rounding(folder, (name, rid, len(ids)), ids, got, want, what)


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_every_way_of_cutting_matches_the_plain_implementation(tmp_path_factory, name, dtype, way, page_size):
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(folder, name)
    want = _plain_logits(folder, name)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
    # the pool holds just what the live requests need and starts as NaN, and so do the kept rows; four request slots
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(page_size), page_size=page_size, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cases.RAW[name]["vocab"])
    for rid in reqs:
        _check(folder, name, dtype, rid, reqs[rid], got[rid], want[rid], f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0 and not replayer.live
    assert all(replayer.cache.num_free_pages(g) == replayer.num_pages for g in range(len(replayer.cache.groups)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_that_want_no_logits_leave_the_kept_rows_right(tmp_path_factory, name, dtype):
    """Token-by-token steps of which only every fourth wants its logits, and mixed steps likewise: step shapes come
    back often enough to be replayed from recorded launches and from graphs, and a request's kept rows must have
    seen every token once."""
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(folder, name)
    want = _plain_logits(folder, name)
    for way in ("tail", "mixed"):
        plan = helpers.PLANS[way](reqs, np.random.default_rng(7))
        kept = {}
        for rec in plan.steps:
            rows, keep, at = plan.wanted[rec["step"]], [], 0
            for entry in rec["entries"]:
                n = len(entry["tokens"])
                entry["want"] = [i for i in range(n) if (rec["step"] + i) % 4 == 0]
                keep += [rows[at + i] for i in entry["want"]]
                at += n
            kept[rec["step"]] = keep
        plan.wanted = {s: rows for s, rows in kept.items() if rows}
        replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), page_size=16, max_live=4, poison=True)
        outputs = helpers.run_plan_in_process(replayer, plan)
        vocab = cases.RAW[name]["vocab"]
        for step, rows in plan.wanted.items():
            out = np.asarray(outputs[step], dtype=np.float64).reshape(len(rows), vocab)
            for (rid, pos), row in zip(rows, out):
                ref = want[rid][pos:pos + 1]
                err = float(_row_errors(row[None], ref)[0])
                bound = (5e-5 if dtype == "float32" else 0.03) * max(1.0, float(np.abs(ref).max()))
                assert np.isfinite(row).all() and err <= bound, f"{name} {dtype} {way} {rid} position {pos}: {err:.3e}"


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (tests/nutitar_cases.py: random_raw), five requests of lengths 1 to 200
    each, whole, in portions and mixed, in both dtypes.  bfloat16: a position may be one and a half times over
    three times what rounding alone does, the mean may not."""
    rng = np.random.default_rng(4000 + seed)
    raw = cases.random_raw(rng)
    folder = cases.write_raw_model(str(tmp_path / "m"), raw, seed)
    cfg, w = P.read_model_folder(folder)
    lens = [int(x) for x in rng.choice([1, 2, 5, 17, 33, 64, 70, 97, 130, 200], size=5)]
    reqs = {f"r{i}": helpers.random_ids(rng, raw["vocab"], n) for i, n in enumerate(lens)}
    want = {rid: P.forward(cfg, w, ids).numpy() for rid, ids in reqs.items()}
    noise = {rid: _row_errors(_rounded_twin(cfg, w, ids), want[rid]) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for way in ("whole", "portions", "mixed"):
            plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
            replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), page_size=16, max_live=4, poison=True)
            got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                                raw["vocab"])
            for rid in reqs:
                what = f"seed {seed} {dtype} {way} {rid} ({json.dumps(raw)})"
                assert np.isfinite(got[rid]).all(), what
                err = _row_errors(got[rid], want[rid])
                if dtype == "float32":
                    assert err.max() <= 5e-5 * max(1.0, float(np.abs(want[rid]).max())), f"{err.max():.3e}: {what}"
                else:
                    assert err.max() <= 4.5 * noise[rid].max() and err.mean() <= 3.0 * noise[rid].mean(), \
                        f"{err.max():.3e} / {noise[rid].max():.3e}, mean {err.mean():.3e} / {noise[rid].mean():.3e}: {what}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """Three tokens of prompt, then 300 tokens one by one through pages of four tokens: the kept rows are carried
    over hundreds of steps, both windows of the configuration pass over decoded tokens while the kept first
    tokens stay, the rotations' scalings reach far beyond their original lengths, the decode steps come from graphs."""
    folder = _folder(tmp_path_factory, "A")
    cfg, w = P.read_model_folder(folder)
    ids = helpers.random_ids(np.random.default_rng(9), cases.RAW["A"]["vocab"], 303)
    want = P.forward(cfg, w, ids).numpy()
    plan = helpers.plan_tail({"a": ids}, tail=300)
    replayer = TraceReplayer(folder, dtype, 304, page_size=4, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["A"]["vocab"])
    _check(folder, "A", dtype, "long", ids, got["a"], want, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_at_every_edge_prefill_and_decoding(tmp_path, dtype):
    """Configuration A with the queries and keys of its windowed layers scaled up and their score biases lowered
    (a key's weight is near one or near nothing), and a sharp softmax in the other layers: 90 tokens whole, in
    portions, and with the last 60 one by one, so that both windows (7 and 37 positions) pass over prompt tokens
    and over decoded ones while the three kept first tokens stay."""
    def edit(tensors):
        for layer in (1, 4):
            for n in ("q.norm", "k.norm"):
                tensors[f"l{layer}.mix.{n}"] *= 2.0
            tensors[f"l{layer}.mix.pb"] -= 2.0
        for n in ("l0.mix.q", "l2.mix.q.norm", "l3.mix.q"):
            tensors[n] *= 3.0
    folder = cases.write_model(str(tmp_path / "sharp"), "A", edit=edit)
    cfg, w = P.read_model_folder(folder)
    ids = helpers.random_ids(np.random.default_rng(11), cases.RAW["A"]["vocab"], 90)
    want = P.forward(cfg, w, ids).numpy()
    # the masks matter: one position less, one kept token less, and the logits move
    for key, frm in (("size", 40), ("keep_first", 12)):
        other = json.loads(json.dumps(cfg))
        other["layers"][1]["mixer"]["mask"][key] -= 1
        assert _row_errors(P.forward(other, w, ids).numpy(), want)[frm:].max() > 1e-3
    for way, plan in (("whole", helpers.plan_whole({"a": ids})), ("portions", helpers.plan_portions({"a": ids}, None)),
                      ("tail", helpers.plan_tail({"a": ids}, tail=60))):
        replayer = TraceReplayer(folder, dtype, 128, page_size=16, max_live=4, poison=True)
        got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["A"]["vocab"])
        _check(folder, "sharp", dtype, "a", ids, got["a"], want, f"sharp {dtype} {way}")


def test_pages_behind_the_window_return_but_the_kept_first_ones_stay(tmp_path_factory):
    """Configuration C's first layer sees itself and the first five tokens: while a request decodes, its group's
    pages behind the window go back to the pool, the page of the kept tokens never does."""
    folder = _folder(tmp_path_factory, "C")
    replayer = TraceReplayer(folder, "float32", 128, page_size=4, max_live=4)
    ids = helpers.random_ids(np.random.default_rng(1), cases.RAW["C"]["vocab"], 60)
    replayer.run_step({"step": 0, "entries": [{"id": "a", "tokens": ids, "want": []}], "end": []})
    layout = replayer.model.cache_layout
    g = next(i for i, grp in enumerate(layout.groups) if grp.window == 1)
    slot = replayer.live["a"][0]
    table = replayer.cache.table(slot, g)
    assert table[0] >= 0 and table[1] >= 0 and len(table) == 15 and all(p < 0 for p in table[2:])
    whole = next(i for i, grp in enumerate(layout.groups) if grp.window == 0)
    assert all(p >= 0 for p in replayer.cache.table(slot, whole))


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name):
    folder = _folder(tmp_path_factory, name)
    cfg, w = P.read_model_folder(folder)
    vocab = cases.RAW[name]["vocab"]
    rng = np.random.default_rng(2)
    prompts = [helpers.random_ids(rng, vocab, n) for n in (7, 19, 3, 11, 26)]
    want = [P.greedy(cfg, w, p, 10) for p in prompts]
    # three request slots for five prompts, portions of at most 8 tokens, small pages: requests wait, prompts are
    # cut, slots, pages and kept rows are used again
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=48, max_batch_size=3,
                                                        prefill_chunk=8, dtype="float32"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    assert got == want
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=16, num_blocks=32, max_batch_size=3, dtype="bfloat16"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    for prompt, tokens in zip(prompts, got):
        seq = list(prompt)
        assert len(tokens) == 10
        for tok in tokens:
            logits = P.forward(cfg, w, seq)[-1].numpy()
            margin = 2 * helpers.TOL["bfloat16"] * max(1.0, float(abs(logits).max()))
            assert logits[tok] >= logits.max() - margin
            seq.append(tok)


def test_generation_with_evictions_recomputes_the_kept_rows(tmp_path_factory):
    """A page pool too small for all running requests: the newest is evicted and later recomputed from its prompt
    and outputs, its kept rows starting over; the tokens are those of an engine with room."""
    folder = _folder(tmp_path_factory, "D")
    rng = np.random.default_rng(3)
    prompts = [helpers.random_ids(rng, cases.RAW["D"]["vocab"], n) for n in (9, 14, 5, 12)]
    roomy = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=64, max_batch_size=4, dtype="float32"))
    want = roomy.generate(prompts, SamplingParams(max_tokens=24, temperature=0.0))
    tight = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=22, max_batch_size=4, dtype="float32"))
    got = tight.generate(prompts, SamplingParams(max_tokens=24, temperature=0.0))
    assert got == want
    assert tight.stats()["num_preemptions"] > 0


def test_the_command_line_and_seeded_sampling(tmp_path_factory):
    """`python -m mini_gpt_inference_amd.generate` on a Nutitar folder: the architecture is found by config.json,
    greedy tokens are the plain implementation's; sampling with a seed through the engine gives the same tokens
    whatever the batch a request runs in."""
    folder = _folder(tmp_path_factory, "D")
    cfg, w = P.read_model_folder(folder)
    prompt = [5, 17, 3, 20]
    want = P.greedy(cfg, w, prompt, 6)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-m", "mini_gpt_inference_amd.generate", "--model", folder,
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--temperature", "0",
                           "--dtype", "float32", "--kv-block-size", "4", "--num-kv-blocks", "32"],
                          cwd=root, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Nutitar" in proc.stdout
    line = next(l for l in proc.stdout.splitlines() if l.startswith("sample:"))
    assert [int(t) for t in line.split()[1:]] == want
    rng = np.random.default_rng(4)
    prompts = [helpers.random_ids(rng, cases.RAW["D"]["vocab"], n) for n in (6, 13, 4)]
    params = [SamplingParams(max_tokens=12, temperature=0.9, top_k=10, seed=7 + i) for i in range(3)]
    together = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=64, max_batch_size=4, dtype="float32"))
    got = together.generate(prompts, params)
    for prompt, sp, tokens in zip(prompts, params, got):
        alone = LLMEngine.from_folder(folder, EngineConfig(block_size=16, num_blocks=16, max_batch_size=1, dtype="float32"))
        assert alone.generate([prompt], sp) == [tokens]
