"""Rilavik on the GPU against the plain implementation (tests/plain_rilavik.py): each new kernel
alone (the short convolution with its kept inputs, the state with a decay from the token in both its
forms, token by token and in chunks, the router and the rows scaled by their pair's weight, the
window's edges in every attention kernel); whole prompts against token-by-token decoding, portions
down to two tokens and mixed batches with pages, request slots and states used again, steps that
want no logits, in 32-bit and bfloat16; long decoding; configurations drawn at random; greedy
generation through LLMEngine."""

import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_rilavik as P
import rilavik_cases as cases
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
# are rows starts[r] .. of the test's arrays; its slot is r + 1 (slot 0 and the last stay untouched).
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
    # a request of the padding behind the real ones: no tokens, no slot
    cu.append(len(rows))
    slots.append(-1)
    return rows, _i32(cu), _i32(pos), _i32(req), _i32(slots)


# ---------------------------------------------------------------- the short convolution
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("channels,taps,bias,act", [(24, 4, True, "silu"), (130, 2, False, None), (7, 5, True, None),
                                                   (64, 1, True, "silu"), (300, 3, False, "silu")])
def test_short_convolution_keeps_its_last_inputs_per_request(dtype, channels, taps, bias, act):
    g = torch.Generator().manual_seed(channels + taps)
    u = _rnd(g, N_ROWS, channels + 5, dtype=dtype)
    w, b = _rnd(g, channels, taps), _rnd(g, channels) if bias else None
    want = torch.zeros(N_ROWS, channels, dtype=P.DTYPE)
    for s, c in zip(STARTS, COUNTS):
        y = P.short_conv(_d(u[s:s + c, 3:3 + channels]), _d(w), None if b is None else _d(b))
        want[s:s + c] = P.silu(y) if act else y
    for plan in (WHOLE, PORTIONS, ONE_BY_ONE):
        # the kept inputs start as NaN: a request's first token must not read them
        state = torch.full((6, max((taps - 1) * channels, 1) + 3), float("nan"), device=DEV)
        got = torch.zeros(N_ROWS, channels, dtype=P.DTYPE)
        for step in plan:
            rows, cu, pos, req, slots = _step_arrays(step)
            out = torch.full((len(rows) + 1, channels + 2), 9.0, dtype=TDT[dtype], device=DEV)
            kernels.short_conv(u[rows].to(DEV), 3, w.to(DEV), None if b is None else b.to(DEV), state, slots, cu, req, pos,
                               len(step) + 1, out, 1, len(rows), activation=act)
            got[rows] = out[:len(rows), 1:1 + channels].cpu().to(P.DTYPE)
            assert (out[len(rows)] == 9.0).all() and (out[:, 0] == 9.0).all() and (out[:, -1] == 9.0).all()
        helpers.assert_close(got, want, dtype, f"short convolution, {len(plan)} steps")
        assert torch.isnan(state[0]).all() and torch.isnan(state[5]).all()


# ---------------------------------------------------------------- the state with a decay from the token
def _state_case(mode, H, G, D, E, dtype, seed, tau):
    """Rows as the mixers lay them out, and the plain result for the four requests."""
    g = torch.Generator().manual_seed(seed)
    if mode == "channel_sigmoid":
        z = _rnd(g, N_ROWS, 2 * H * D + H * E + 3, dtype=dtype)
        a = _rnd(g, N_ROWS, H * D + 2, dtype=dtype, scale=2.0)
        a[:, 1] -= 30.0          # one channel forgets at once (a decay of e^-30 a token with tau 1), one keeps nearly all
        a[:, 2] += 12.0
        offs = dict(q_off=0, k_off=H * D, v_off=2 * H * D, a_off=1)
        extra = dict(q_scale=D ** -0.5, tau=tau)
        want = torch.zeros(N_ROWS, H * E, dtype=P.DTYPE)
        for s, c in zip(STARTS, COUNTS):
            rows = _d(z[s:s + c])
            q, k = rows[:, :H * D].view(c, H, D) * D ** -0.5, rows[:, H * D:2 * H * D].view(c, H, D)
            v = rows[:, 2 * H * D:2 * H * D + H * E].view(c, H, E)
            alpha = P.sigmoid(_d(a[s:s + c, 1:1 + H * D])).view(c, H, D) ** (1.0 / tau)
            want[s:s + c] = P.gla_recurrence(q, k, v, alpha).reshape(c, H * E)
        return z, a, offs, extra, want
    z = _rnd(g, N_ROWS, H * E + 2 * G * D + 1, dtype=dtype)
    a = _rnd(g, N_ROWS, H + 4, dtype=dtype, scale=2.0)
    dt_bias, a_log, skip = _rnd(g, H) - 1.0, _rnd(g, H), _rnd(g, H)
    offs = dict(q_off=H * E + G * D, k_off=H * E, v_off=0, a_off=3)
    extra = dict(dt_bias=dt_bias.to(DEV), a_log=a_log.to(DEV), skip=skip.to(DEV))
    want = torch.zeros(N_ROWS, H * E, dtype=P.DTYPE)
    for s, c in zip(STARTS, COUNTS):
        rows = _d(z[s:s + c])
        x = rows[:, :H * E].view(c, H, E)
        B, C = rows[:, H * E:H * E + G * D].view(c, G, D), rows[:, H * E + G * D:H * E + 2 * G * D].view(c, G, D)
        dt = P.softplus(_d(a[s:s + c, 3:3 + H]) + _d(dt_bias))
        want[s:s + c] = P.ssd_recurrence(x, B, C, dt, torch.exp(_d(a_log)), _d(skip)).reshape(c, H * E)
    return z, a, offs, extra, want


def _run_state(plan, chunked, mode, H, G, D, E, z, a, offs, extra, state):
    got = torch.zeros(N_ROWS, H * E, dtype=P.DTYPE)
    for step in plan:
        rows, cu, pos, _, slots = _step_arrays(step)
        n = len(rows)
        zs, as_ = z[rows].to(DEV), a[rows].to(DEV)
        out = torch.full((n + 1, H * E), 9.0, device=DEV)
        if chunked:
            qkg = torch.zeros(n, 3 * H * D, device=DEV)
            assert kernels.gated_state_chunked(zs, offs["q_off"], offs["k_off"], offs["v_off"], H, G, D, E, as_, offs["a_off"],
                                               mode, state, slots, cu, len(step) + 1, n, pos, qkg, out, **extra)
        else:
            kernels.gated_state(zs, offs["q_off"], offs["k_off"], offs["v_off"], H, G, D, E, as_, offs["a_off"], mode, state,
                                slots, cu, len(step) + 1, pos, out, **extra)
        assert (out[n] == 9.0).all()
        got[rows] = out[:n].cpu().to(P.DTYPE)
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode,H,G,D,E,tau", [
    ("channel_sigmoid", 2, 2, 16, 24, 4.0), ("channel_sigmoid", 3, 3, 20, 12, 1.0), ("channel_sigmoid", 1, 1, 64, 64, 16.0),
    ("channel_sigmoid", 2, 2, 128, 128, 2.0), ("channel_sigmoid", 1, 1, 40, 130, 1.0), ("channel_sigmoid", 16, 16, 8, 256, 8.0),
    ("head_softplus", 4, 2, 8, 16, 1.0), ("head_softplus", 3, 3, 20, 12, 1.0), ("head_softplus", 6, 2, 12, 4, 1.0),
    ("head_softplus", 1, 1, 128, 128, 1.0), ("head_softplus", 2, 1, 64, 32, 1.0), ("head_softplus", 16, 4, 16, 256, 1.0)])
def test_state_with_a_decay_from_the_token(dtype, mode, H, G, D, E, tau):
    """Token by token and in chunks: whole requests of 70, 1, 32 and 33 tokens, the same in portions whose cuts fall
    inside, at and one token beside a chunk's border, and one token a step; then the token-by-token kernel
    goes on from the state the chunked one left.  States start as NaN and are compared too."""
    z, a, offs, extra, want = _state_case(mode, H, G, D, E, dtype, H * D + E, tau)
    width = H * D * E
    states = {}
    for chunked in (False, True):
        for name, plan in (("whole", WHOLE), ("portions", PORTIONS), ("one by one", ONE_BY_ONE)):
            pool = torch.full((6, width + 5), float("nan"), device=DEV)      # the state is a view of a wider pool's columns
            state = pool[:, :width]
            got = _run_state(plan, chunked, mode, H, G, D, E, z, a, offs, extra, state)
            helpers.assert_close(got, want, "float32", f"{mode} chunked {chunked} {name}")
            assert torch.isnan(pool[0]).all() and torch.isnan(pool[5]).all() and torch.isnan(pool[:, width:]).all()
            assert torch.isfinite(state[1:5]).all()
            states[(chunked, name)] = state[1:5].cpu()
    ref = states[(False, "whole")]
    for key, st in states.items():
        helpers.assert_close(st, ref, "float32", f"state {key}")
    # chunks first, then single tokens
    pool = torch.full((6, width), float("nan"), device=DEV)
    head = [[(0, 0, 37), (2, 0, 30), (3, 0, 32)]]
    tail = [[(r, t, 1) for r, first, n in ((0, 37, 70), (1, 0, 1), (2, 30, 32), (3, 32, 33)) if first <= t < n] for t in range(70)]
    got = _run_state(head, True, mode, H, G, D, E, z, a, offs, extra, pool)
    got2 = _run_state([s for s in tail if s], False, mode, H, G, D, E, z, a, offs, extra, pool)
    done = torch.zeros(N_ROWS, dtype=torch.bool)
    for r, n in ((0, 37), (2, 30), (3, 32)):
        done[STARTS[r]:STARTS[r] + n] = True
    helpers.assert_close(torch.where(done[:, None], got, got2), want, "float32", "token by token behind chunks")


@pytest.mark.parametrize("chunked", [False, True])
def test_the_state_far_back_matters(chunked):
    """With decays near one the first token's key and value are still in the output after hundreds of tokens (a
    lost or restarted state shows), with fast decays they are gone: the first token's key is scaled up, and the
    last outputs must move with it in the slow head and not in the fast one.  Prompt of 330 tokens in portions,
    then 70 tokens one by one."""
    g = torch.Generator().manual_seed(5)
    T, H, D, E = 400, 2, 16, 16
    z = _rnd(g, T, 2 * H * D + H * E)
    z[0, H * D:2 * H * D] *= 20.0
    a = torch.cat([torch.full((T, D), 9.0), torch.full((T, D), -1.0)], dim=1)     # head 0 keeps, head 1 forgets
    rows = _d(z)
    q, k = rows[:, :H * D].view(T, H, D), rows[:, H * D:2 * H * D].view(T, H, D)
    v = rows[:, 2 * H * D:].view(T, H, E)
    alpha = P.sigmoid(_d(a)).view(T, H, D)
    want = P.gla_recurrence(q, k, v, alpha)
    k2 = k.clone()
    k2[0] /= 20.0
    plain = P.gla_recurrence(q, k2, v, alpha)
    assert float((want[-1, 0] - plain[-1, 0]).abs().max()) > 1.0 and float((want[-1, 1] - plain[-1, 1]).abs().max()) < 1e-9
    state = torch.full((3, H * D * E), float("nan"), device=DEV)
    got = torch.zeros(T, H * E, dtype=P.DTYPE)
    cuts = [0, 100, 102, 197, 330] + list(range(331, T + 1))
    for first, last in zip(cuts[:-1], cuts[1:]):
        n = last - first
        out = torch.zeros(n, H * E, device=DEV)
        args = (z[first:last].to(DEV), 0, H * D, 2 * H * D, H, H, D, E, a[first:last].to(DEV), 0, "channel_sigmoid", state,
                _i32([1]), _i32([0, n]), 1)
        pos = _i32(list(range(first, last)))
        if chunked and n > 1:
            assert kernels.gated_state_chunked(*args, n, pos, torch.zeros(n, 3 * H * D, device=DEV), out)
        else:
            kernels.gated_state(*args, pos, out)
        got[first:last] = out.cpu().to(P.DTYPE)
    helpers.assert_close(got, want.reshape(T, H * E), "float32", "a key 400 tokens back")


# ---------------------------------------------------------------- the router and the scaled rows
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,width,experts,top", [(1, 64, 2, 1), (9, 40, 5, 2), (70, 264, 11, 1), (33, 136, 9, 3),
                                                 (5, 2048, 8, 2), (4, 24, 3, 3), (300, 96, 33, 4), (7, 100, 6, 2), (3, 4100, 9, 2),
                                                 (2, 4096, 17, 3)])
def test_router_picks_the_largest_scores(dtype, n, width, experts, top):
    g = torch.Generator().manual_seed(n + experts)
    h = _rnd(g, n + 1, width + 8, dtype=dtype)
    w = _rnd(g, experts, width, dtype=dtype, scale=width ** -0.5 * 2.0)
    logits = _d(h[:n, :width]) @ _d(w).T
    scores = P.sigmoid(logits)
    order = torch.argsort(scores, dim=1, descending=True)
    chosen = torch.full((n + 1, top), -7, dtype=torch.int32, device=DEV)
    weight = torch.full((n + 1, top), -7.0, device=DEV)
    kernels.router_topk(h.to(DEV), w.to(DEV), n, top, chosen, weight)
    assert (chosen[n] == -7).all() and (weight[n] == -7.0).all()
    chosen, weight = chosen[:n].cpu().long(), weight[:n].cpu().to(P.DTYPE)
    for i in range(n):
        # best first; where two scores are closer than float32 summation can tell, either order will do
        srt = scores[i][order[i]]
        for c in range(top):
            assert abs(float(scores[i][chosen[i, c]] - srt[c])) < 1e-5, f"row {i} choice {c}"
        assert len(set(chosen[i].tolist())) == top
    helpers.assert_close(weight, torch.gather(scores, 1, chosen), "float32", "scores of the chosen")
    # the sum itself as score
    kernels.router_topk(h.to(DEV), w.to(DEV), n, top, ch2 := torch.zeros(n, top, dtype=torch.int32, device=DEV),
                        w2 := torch.zeros(n, top, device=DEV), score="logit")
    helpers.assert_close(w2, torch.gather(logits, 1, ch2.cpu().long()), "float32", "sums of the chosen")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,width,slots", [(5, 40, 16), (70, 256, 300), (3, 1030, 7)])
def test_rows_scaled_by_their_pairs_weight(dtype, n, width, slots):
    g = torch.Generator().manual_seed(width)
    src = _rnd(g, n, width + 8, dtype=dtype)[:, :width]
    pairs = 2 * n
    slot_token = torch.randint(0, n, (slots,), generator=g, dtype=torch.int32)
    slot_pair = torch.randint(0, pairs, (slots,), generator=g, dtype=torch.int32)
    pair_weight = torch.rand(pairs, generator=g)
    out = torch.full((slots + 1, width), 9.0, dtype=TDT[dtype], device=DEV)
    kernels.gather_scale_rows(src.to(DEV), slot_token.to(DEV), slot_pair.to(DEV), pair_weight.to(DEV), out, slots)
    want = _d(pair_weight)[slot_pair.long()][:, None] * _d(src)[slot_token.long()]
    helpers.assert_close(out[:slots], want, dtype, "scaled rows")
    assert (out[slots] == 9.0).all()


# ---------------------------------------------------------------- the window's edges in the attention kernels
def _paged(k, v, page, perm, dtype):
    T, G, D = k.shape
    E = v.shape[2]
    kp = torch.zeros(len(perm), G, page, D, dtype=TDT[dtype])
    vp = torch.zeros(len(perm), G, page, E, dtype=TDT[dtype])
    for j in range(T):
        kp[perm[j // page], :, j % page], vp[perm[j // page], :, j % page] = k[j], v[j]
    return kp.to(DEV), vp.to(DEV)


@pytest.mark.parametrize("dtype,D", [("float32", 32), ("bfloat16", 32), ("bfloat16", 64), ("bfloat16", 128), ("float32", 20)])
@pytest.mark.parametrize("window", [1, 2, 16, 17, 70, 100])
def test_a_key_just_inside_and_just_outside_the_window(dtype, D, window):
    """The last query is made to look like one key, scaled so that this key takes nearly all the weight
    if it is seen: once the key is the oldest the window still holds, once the one before it.  Queries in
    a portion on top of cached tokens, and single queries, through every attention kernel that takes the sizes."""
    H, G, page, T = 4, 2, 16, 208
    scale = D ** -0.5
    for back in (window - 1, window):
        g = torch.Generator().manual_seed(7 + D + window)
        q, k, v = _rnd(g, T, H, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype), _rnd(g, T, G, D, dtype=dtype)
        far = T - 1 - back
        k[far] *= 4.0
        q[-1] = k[far].float().repeat_interleave(H // G, dim=0).to(TDT[dtype])
        want = P.window_attention(_d(q), _d(k), _d(v), scale, window)
        seen = P.window_attention(_d(q), _d(k), _d(v), scale, window + 1)
        if back == window:
            assert float((want[-1] - seen[-1]).abs().max()) > 0.3      # one position more and the key would take over
        pages = T // page
        perm = torch.randperm(pages, generator=g)
        kp, vp = _paged(k, v, page, perm, dtype)
        bt = perm.to(torch.int32).view(1, pages).to(DEV)
        first = 100
        n = T - first
        qd = q[first:].reshape(n, H * D).to(DEV)
        ref = want[first:].reshape(n, H * D)
        out = torch.zeros(n, H * D, dtype=TDT[dtype], device=DEV)
        kernels.paged_attention_generic(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), _i32([0] * n), n, 1, H, scale,
                                        window=window)
        helpers.assert_close(out, ref, dtype, f"general kernel, key {back} back")
        one = torch.zeros(1, H * D, dtype=TDT[dtype], device=DEV)
        kernels.paged_attention_generic(qd[n - 1:], one, kp, vp, bt, _i32([0, 1]), _i32([T]), _i32([0]), 1, 1, H, scale,
                                        window=window)
        helpers.assert_close(one, ref[n - 1:], dtype, f"general kernel, one query, key {back} back")
        if dtype != "bfloat16" or D not in (32, 64, 128):
            continue
        out.zero_()
        assert kernels.prefill_attention_bf16(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), 1, n, H, scale, window=window)
        helpers.assert_close(out, ref, dtype, f"tile kernel, key {back} back")
        for fast in (True, False):
            out.zero_()
            assert kernels.paged_attention_split_bf16(qd, out, kp, vp, bt, _i32([0, n]), _i32([T]), _i32([0] * n), n, 1, H,
                                                      scale, window=window, fast=fast)
            helpers.assert_close(out, ref, dtype, f"split kernel, key {back} back")
        one.zero_()
        assert kernels.paged_attention_decode_bf16(qd[n - 1:], one, kp, vp, bt, _i32([T - 1]), _i32([0]), 1, H, scale,
                                                   window=window, identity=True)
        helpers.assert_close(one, ref[n - 1:], dtype, f"decode kernel, key {back} back")


# ---------------------------------------------------------------- the model through the step function
LENGTHS = {"A": [5, 70, 23, 41, 2, 64, 37], "B": [1, 9, 33, 17, 110], "C": [40, 3, 64, 21], "D": [75, 12, 30, 6, 49],
           "E": [33, 4, 70, 18, 2]}
_folders, _plain, _twin = {}, {}, {}


def _folder(tmp_path_factory, name):
    if name not in _folders:
        _folders[name] = cases.write_model(str(tmp_path_factory.mktemp("rilavik") / name), name)
    return _folders[name]


FIRM_GAP = 0.15     # in a router's logits: a choice decided by less is no test of reduced precision


def _router_gaps(cfg, w, ids):
    """Per position: by how much the least decided router's choice is decided in the plain implementation."""
    P.ROUTER_GAPS = []
    try:
        P.forward(cfg, w, ids)
        gaps = torch.stack(P.ROUTER_GAPS).min(dim=0).values if P.ROUTER_GAPS else torch.full((len(ids),), math.inf)
    finally:
        P.ROUTER_GAPS = None
    return gaps.numpy()


def _firm_ids(cfg, w, rng, vocab, n):
    """n random tokens, each drawn again (up to 50 times) until every router's choice at its position is decided by
    FIRM_GAP: rounding to bfloat16 then chooses the same experts, and the logits can be compared.  (A position's
    routing depends on the tokens up to it only.)"""
    ids = []
    while len(ids) < n:
        for _ in range(50):
            tok = int(rng.integers(0, vocab))
            if _router_gaps(cfg, w, ids + [tok])[-1] >= FIRM_GAP:
                break
        ids.append(tok)
    return ids


def _firm_prefix(cfg, w, ids):
    """The number of positions before the first whose routing is a close call."""
    close = np.nonzero(_router_gaps(cfg, w, ids) < FIRM_GAP)[0]
    return int(close[0]) if len(close) else len(ids)


_requests_made = {}


def _requests(folder, name):
    if name not in _requests_made:
        cfg, w = P.read_model_folder(folder)
        rng = np.random.default_rng(len(name) + ord(name[0]))
        _requests_made[name] = {f"r{i}": _firm_ids(cfg, w, rng, cases.RAW[name]["vocab"], n)
                                for i, n in enumerate(LENGTHS[name])}
    return _requests_made[name]


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


def _assert_within_rounding(folder, key, ids, got, want, what, worst=3.0, upto=None):
    """bfloat16: a position's error may be `worst` times what rounding alone causes at the request's
    worst position, and the request's mean error three times the mean of that (over the first `upto` positions)."""
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    if key not in _twin:
        cfg, w = P.read_model_folder(folder)
        _twin[key] = _row_errors(_rounded_twin(cfg, w, ids), want)
    noise, err = _twin[key][:upto], _row_errors(got, want)[:upto]
    assert err.max() <= worst * noise.max(), f"{what}: worst position {err.max():.3e} > {worst} * {noise.max():.3e}"
    assert err.mean() <= 3.0 * noise.mean(), f"{what}: mean {err.mean():.3e} > 3 * {noise.mean():.3e}"


def _check(folder, name, dtype, rid, ids, got, want, what, upto=None):
    if dtype == "float32":
        assert np.isfinite(got).all(), what
        err = _row_errors(got, want)
        assert err.max() <= 5e-5 * max(1.0, float(np.abs(want).max())), f"{what}: {err.max():.3e}"
    else:
        _assert_within_rounding(folder, (name, rid, len(ids)), ids, got, want, what, upto=upto)


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_every_way_of_cutting_matches_the_plain_implementation(tmp_path_factory, name, dtype, way, page_size):
    folder = _folder(tmp_path_factory, name)
    reqs = _requests(folder, name)
    want = _plain_logits(folder, name)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
    # the pool holds just what the live requests need and starts as NaN, and so do the states; four request slots
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(page_size), page_size=page_size, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cases.RAW[name]["vocab"])
    for rid in reqs:
        _check(folder, name, dtype, rid, reqs[rid], got[rid], want[rid], f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0 and not replayer.live
    assert all(replayer.cache.num_free_pages(g) == replayer.num_pages for g in range(len(replayer.cache.groups)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_that_want_no_logits_leave_the_state_right(tmp_path_factory, name, dtype):
    """Token-by-token steps of which only every fourth wants its logits, and mixed steps likewise:
    step shapes come back often enough to be replayed from recorded launches and from graphs, and a
    request's states and kept convolution inputs must have seen every token once."""
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
                bound = 5e-5 * max(1.0, float(np.abs(ref).max())) if dtype == "float32" else 0.1
                assert np.isfinite(row).all() and err <= bound, f"{name} {dtype} {way} {rid} position {pos}: {err:.3e}"


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (tests/rilavik_cases.py: random_raw), five requests of lengths
    1 to 200 each, whole, in portions and mixed, in both dtypes.  bfloat16: a position may be one and
    a half times over three times what rounding alone does, the mean may not; a request is compared up to
    its first position where a router's choice is a close call."""
    rng = np.random.default_rng(3000 + seed)
    raw = cases.random_raw(rng)
    folder = cases.write_raw_model(str(tmp_path / "m"), raw, seed, decay_rank=int(rng.choice([3, 8, 16])))
    cfg, w = P.read_model_folder(folder)
    lens = [int(x) for x in rng.choice([1, 2, 5, 17, 33, 64, 70, 97, 130, 200], size=5)]
    reqs = {f"r{i}": helpers.random_ids(rng, raw["vocab"], n) for i, n in enumerate(lens)}
    want = {rid: P.forward(cfg, w, ids).numpy() for rid, ids in reqs.items()}
    noise = {rid: _row_errors(_rounded_twin(cfg, w, ids), want[rid]) for rid, ids in reqs.items()}
    firm = {rid: _firm_prefix(cfg, w, ids) for rid, ids in reqs.items()}
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
                    continue
                # bfloat16 may choose other experts where a router's choice is a close call, and what follows in
                # that request differs too: the positions before the first such call are compared
                if not firm[rid]:
                    continue
                e, nz = err[:firm[rid]], noise[rid][:firm[rid]]
                assert e.max() <= 4.5 * nz.max() and e.mean() <= 3.0 * nz.mean(), \
                    f"{e.max():.3e} / {nz.max():.3e}, mean {e.mean():.3e} / {nz.mean():.3e}: {what}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """Three tokens of prompt, then 300 tokens one by one through pages of four tokens: states and kept
    convolution inputs are carried over hundreds of steps, both windows of the configuration pass over
    decoded tokens, the decode steps come from graphs."""
    folder = _folder(tmp_path_factory, "A")
    cfg, w = P.read_model_folder(folder)
    rng = np.random.default_rng(9)
    ids = _firm_ids(cfg, w, rng, cases.RAW["A"]["vocab"], 40) + helpers.random_ids(rng, cases.RAW["A"]["vocab"], 263)
    want = P.forward(cfg, w, ids).numpy()
    plan = helpers.plan_tail({"a": ids}, tail=300)
    replayer = TraceReplayer(folder, dtype, 304, page_size=4, max_live=4, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["A"]["vocab"])
    # (bfloat16: up to the first position where a router's choice is a close call, all of it in 32-bit)
    upto = None if dtype == "float32" else _firm_prefix(cfg, w, ids)
    assert np.isfinite(got["a"]).all() and (upto is None or upto >= 8)
    _check(folder, "A", dtype, "long", ids, got["a"], want, "long decoding", upto=upto)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_at_the_windows_edge_prefill_and_decoding(tmp_path, dtype):
    """Configuration A with the queries and keys of its windowed layers scaled up (a sharp softmax: the
    key that leaves the window carries weight): 90 tokens whole, in portions, and with the last 60 one by
    one, so that both windows (7 and 37 positions) pass over prompt tokens and over decoded ones."""
    def edit(tensors):
        for layer in (0, 2):
            for n in ("q", "k"):
                tensors[f"l{layer}.mix.left.{n}"] *= 3.0
    folder = cases.write_model(str(tmp_path / "sharp"), "A", edit=edit)
    cfg, w = P.read_model_folder(folder)
    ids = _firm_ids(cfg, w, np.random.default_rng(11), cases.RAW["A"]["vocab"], 90)
    want = P.forward(cfg, w, ids).numpy()
    # the window matters: one position less and the logits move
    narrower = json.loads(json.dumps(cfg))
    narrower["layers"][2]["mixer"]["left"]["mask"]["size"] -= 1
    assert _row_errors(P.forward(narrower, w, ids).numpy(), want)[40:].max() > 1e-3
    for way, plan in (("whole", helpers.plan_whole({"a": ids})), ("portions", helpers.plan_portions({"a": ids}, None)),
                      ("tail", helpers.plan_tail({"a": ids}, tail=60))):
        replayer = TraceReplayer(folder, dtype, 128, page_size=16, max_live=4, poison=True)
        got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {"a": len(ids)}, cases.RAW["A"]["vocab"])
        _check(folder, "sharp", dtype, "a", ids, got["a"], want, f"sharp {dtype} {way}")


@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name):
    folder = _folder(tmp_path_factory, name)
    cfg, w = P.read_model_folder(folder)
    vocab = cases.RAW[name]["vocab"]
    rng = np.random.default_rng(2)
    prompts = [_firm_ids(cfg, w, rng, vocab, n) for n in (7, 19, 3, 11, 26)]
    want = [P.greedy(cfg, w, p, 10) for p in prompts]
    # three request slots for five prompts, portions of at most 8 tokens, small pages: requests
    # wait, prompts are cut, slots, pages and states are used again
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=4, num_blocks=48, max_batch_size=3,
                                                        prefill_chunk=8, dtype="float32"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    assert got == want
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=16, num_blocks=32, max_batch_size=3, dtype="bfloat16"))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    checked = 0
    for prompt, tokens in zip(prompts, got):
        seq = list(prompt)
        assert len(tokens) == 10
        for tok in tokens:
            if _firm_prefix(cfg, w, seq) < len(seq):
                break       # a router's close call: from here on bfloat16 may have gone another, as valid, way
            logits = P.forward(cfg, w, seq)[-1].numpy()
            margin = 2 * helpers.TOL["bfloat16"] * max(1.0, float(abs(logits).max()))
            assert logits[tok] >= logits.max() - margin
            seq.append(tok)
            checked += 1
    assert checked >= 10


def test_generation_with_evictions_recomputes_the_state(tmp_path_factory):
    """A page pool too small for all running requests: the newest is evicted and later recomputed
    from its prompt and outputs, its states and kept convolution inputs starting over; the tokens are
    those of an engine with room."""
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
    """`python -m mini_gpt_inference_amd.generate` on a Rilavik folder: the architecture is found by config.json,
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
    assert "Rilavik" in proc.stdout
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


def test_heads_larger_than_the_chunked_form_takes():
    """Head sizes over 128: the chunked form says no and launches nothing, the token-by-token kernel takes them."""
    mode, H, G, D, E = "channel_sigmoid", 1, 1, 160, 24
    z, a, offs, extra, want = _state_case(mode, H, G, D, E, "float32", 3, 2.0)
    state = torch.full((6, H * D * E), float("nan"), device=DEV)
    rows, cu, pos, _, slots = _step_arrays(WHOLE[0])
    out = torch.full((len(rows), H * E), 9.0, device=DEV)
    assert not kernels.gated_state_chunked(z[rows].to(DEV), offs["q_off"], offs["k_off"], offs["v_off"], H, G, D, E,
                                           a[rows].to(DEV), offs["a_off"], mode, state, slots, cu, len(WHOLE[0]) + 1,
                                           len(rows), pos, torch.zeros(len(rows), 3 * H * D, device=DEV), out, **extra)
    assert (out == 9.0).all() and torch.isnan(state).all()
    got = _run_state(PORTIONS, False, mode, H, G, D, E, z, a, offs, extra, state)
    helpers.assert_close(got, want, "float32", "heads of 160")
