"""Typed Python entry points of the HIP kernels.

Each function checks on the host that operand shapes, strides, dtypes and
devices are what the kernel and its grid assume, then launches on the current
HIP stream.  Tensors are torch tensors used as plain device buffers; no torch
operator computes anything here.
"""

from __future__ import annotations

import contextlib
import ctypes
from typing import Dict, Optional

import torch

from . import library

F32, BF16 = 0, 1
EPI_NONE, EPI_GELU, EPI_RESIDUAL = 0, 1, 2
EPI_XIELU = 4      # only through linear_mfma_xielu, which brings the activation's coefficients

_ERRORS = {
    -1: "unsupported dtype combination",
    -2: "unsupported shape",
    -3: "size beyond what the launch grid can hold",
    -4: "null pointer",
    -5: "the shape needs more scratch than the library's own array holds",
}


class KernelError(RuntimeError):
    pass


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 buffers, got {t.dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    """The address for a pointer argument (ctypes takes an int, or None for null, where argtypes say c_void_p)."""
    return None if t is None else t.data_ptr()


_pinned_stream: Optional[ctypes.c_void_p] = None


def _stream() -> ctypes.c_void_p:
    if _pinned_stream is not None:
        return _pinned_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@contextlib.contextmanager
def pinned_stream():
    """Inside the block every launch goes to the stream that is current on entry.  Asking torch for
    the current stream costs about as much as a launch does, and a step is some hundred launches;
    the block must not switch streams."""
    global _pinned_stream
    previous = _pinned_stream
    _pinned_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    try:
        yield
    finally:
        _pinned_stream = previous


launches = 0     # kernels launched so far (a product split over workgroups counts its second kernel too)


def _check(rc: int, what: str, n_kernels: int = 1) -> None:
    global launches
    if rc == 0:
        launches += n_kernels
        return
    if rc < 0:
        raise KernelError(f"{what}: refused, {_ERRORS.get(rc, rc)}")
    raise KernelError(f"{what}: HIP error {rc}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _need_cuda(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _need_i32(name: str, t: torch.Tensor, n: int) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n,
          f"{name} must be a contiguous int32 buffer of at least {n} entries")


def _need_sinks(sinks: Optional[torch.Tensor], n_head: int) -> None:
    _need(sinks is None or (sinks.is_cuda and sinks.dtype == torch.float32 and sinks.is_contiguous()
                            and sinks.numel() == n_head), "sinks must be float32 [n_head] on the GPU")


def embed(ids: torch.Tensor, positions: Optional[torch.Tensor], table: torch.Tensor,
          pos_table: Optional[torch.Tensor], x: torch.Tensor, n_tokens: int) -> None:
    """x[t] = table[ids[t]] (+ pos_table[positions[t]]), into the float32 residual stream."""
    _need_cuda(ids, positions, table, pos_table, x)
    width = table.shape[1]
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be dense [vocab, width]")
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == width and x.shape[0] >= n_tokens,
          "residual stream must be dense float32 [>=n_tokens, width]")
    _need_i32("ids", ids, n_tokens)
    if pos_table is not None:
        _need(pos_table.dtype == table.dtype and pos_table.is_contiguous() and pos_table.shape[1] == width,
              "position table must match the token table's dtype and width")
        _need(positions is not None, "positions are needed with a position table")
        _need_i32("positions", positions, n_tokens)
    rc = library.kernels().mgpt_embed(_ptr(ids), _ptr(positions), _ptr(table), _ptr(pos_table), _ptr(x),
                                      n_tokens, width, _dtype_code(table), _stream())
    _check(rc, "embed")


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
               n_rows: int, eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """out[i] = LayerNorm(x[rows[i]] or x[i]); statistics in float32."""
    _need_cuda(x, weight, bias, out, rows)
    width = x.shape[1]
    _need(x.dtype == torch.float32 and x.is_contiguous(), "LayerNorm input must be dense float32")
    _need(weight.dtype == torch.float32 and weight.numel() == width, "LayerNorm weight must be float32 [width]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == width),
          "LayerNorm bias must be float32 [width]")
    _need(out.is_contiguous() and out.shape[1] == width and out.shape[0] >= n_rows, "LayerNorm output too small")
    if rows is None:
        _need(x.shape[0] >= n_rows, "LayerNorm input has fewer rows than asked for")
    else:
        _need_i32("rows", rows, n_rows)
    rc = library.kernels().mgpt_layernorm(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _ptr(rows), n_rows,
                                          width, float(eps), _dtype_code(out), _stream())
    _check(rc, "layer_norm")


def linear_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                   n_rows: int, epilogue: int = EPI_NONE) -> None:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias), optional GELU, or added into a float32 out."""
    _need_cuda(a, w, bias, out)
    n_out, k_dim = w.shape
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          f"activation must be [>=n_rows, {k_dim}] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == n_out and out.shape[0] >= n_rows,
          f"output must be [>=n_rows, {n_out}] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    rc = library.kernels().mgpt_linear_generic(
        _ptr(a), _dtype_code(a), a.stride(0), _ptr(w), _dtype_code(w), _ptr(bias), _ptr(out), _dtype_code(out),
        out.stride(0), n_rows, n_out, k_dim, epilogue, _stream())
    _check(rc, "linear_generic")


def kv_write(qkv: torch.Tensor, k_off: int, v_off: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
             slot_mapping: torch.Tensor, n_tokens: int) -> None:
    """Stores the new keys and values of n_tokens rows of qkv into their pages.

    Pools are [num_pages, n_kv_head, page_size, head_dim]."""
    _need_cuda(qkv, k_pool, v_pool, slot_mapping)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    _need(qkv.dtype == k_pool.dtype == v_pool.dtype, "pools must have the activations' dtype")
    _need(qkv.stride(1) == 1 and qkv.shape[0] >= n_tokens, "qkv rows must have unit inner stride")
    width = n_kv_head * head_dim
    _need(0 <= k_off and k_off + width <= qkv.shape[1] and 0 <= v_off and v_off + width <= qkv.shape[1],
          "key/value columns lie outside the qkv buffer")
    _need_i32("slot_mapping", slot_mapping, n_tokens)
    rc = library.kernels().mgpt_kv_write(_ptr(qkv), _dtype_code(qkv), qkv.stride(0), k_off, v_off, _ptr(k_pool),
                                         _ptr(v_pool), _ptr(slot_mapping), n_tokens, n_kv_head, head_dim,
                                         page_size, _stream())
    _check(rc, "kv_write")


def _mask_args(keep_first: int, score_bias: Optional[torch.Tensor], n_head: int, sinks, softcap: float):
    """(first positions that a window keeps, pointer of the per-head number added to a score before its sigmoid):
    the two optional arguments behind the gate's.  With score_bias the weights are sigmoids and not a softmax, so
    sinks and a score cap do not go with it."""
    _need(int(keep_first) >= 0, "keep_first must not be negative")
    if score_bias is not None:
        _need(score_bias.is_cuda and score_bias.dtype == torch.float32 and score_bias.is_contiguous()
              and score_bias.numel() == n_head, "score_bias must be float32 [n_head] on the GPU")
        _need(sinks is None and not softcap > 0.0, "sigmoid weights take neither sinks nor a score cap")
    return int(keep_first), _ptr(score_bias)


def _gate_args(gate: Optional[torch.Tensor], q: torch.Tensor, n_tokens: int, n_head: int):
    """(pointer, row stride) of the optional gate [tokens, >= heads] in q's dtype: a head's attention output is
    multiplied by sigmoid(gate[token][head])."""
    if gate is None:
        return None, 0
    _need_cuda(gate)
    _need(gate.dtype == q.dtype and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] >= n_tokens
          and gate.shape[1] >= n_head, "the heads' gate must be rows [tokens, >= heads] in the queries' dtype")
    return _ptr(gate), gate.stride(0)


def _check_attention_args(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head):
    _need_cuda(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    _need(q.dtype == out.dtype == k_pool.dtype == v_pool.dtype, "queries, output and pools must share a dtype")
    _need(q.stride(1) == 1 and out.stride(1) == 1, "query and output rows must have unit inner stride")
    _need(q.shape[0] >= n_tokens and out.shape[0] >= n_tokens, "query/output buffers have too few rows")
    _need(q.shape[1] >= n_head * head_dim and out.shape[1] >= n_head * head_dim,
          "query/output rows are narrower than n_head * head_dim")
    _need(n_head % n_kv_head == 0, "n_head must be a multiple of the number of key/value heads")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_req, "block_tables must be dense int32 [>=requests, max_blocks]")
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("seq_lens", seq_lens, n_req)
    _need_i32("q_req", q_req, n_tokens)
    return n_kv_head, page_size, head_dim


def paged_attention_generic(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor,
                            q_req: torch.Tensor, n_tokens: int, n_req: int, n_head: int, scale: float,
                            window: int = 0, fast_exp: bool = False, sinks: Optional[torch.Tensor] = None,
                            softcap: float = 0.0, gate: Optional[torch.Tensor] = None, keep_first: int = 0,
                            score_bias: Optional[torch.Tensor] = None) -> None:
    """Causal attention of the step's tokens over their requests' pages (any q_len, any dtype).
    sinks: float32 [n_head], one more term exp(sinks[h]) in every softmax denominator of head h.
    softcap > 0: every score becomes softcap * tanh(score / softcap) before the softmax.
    keep_first: behind a window a query also sees the keys at positions below it.  score_bias: float32 [n_head];
    a visible key's weight is sigmoid(score + score_bias[h]), not normalised over the keys."""
    n_kv_head, page_size, head_dim = _check_attention_args(
        q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head)
    _need(head_dim <= 1024, f"head size {head_dim} exceeds the kernel's limit of 1024")
    _need_sinks(sinks, n_head)
    rc = library.kernels().mgpt_paged_attention_generic(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), _ptr(q_req), n_tokens, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), _dtype_code(q), int(fast_exp), _ptr(sinks), float(softcap), *_gate_args(gate, q, n_tokens, n_head),
        *_mask_args(keep_first, score_bias, n_head, sinks, softcap), _stream())
    _check(rc, "paged_attention_generic")


def sample(logits: torch.Tensor, n_rows: int, real_vocab: int, temperature: torch.Tensor,
           top_k: Optional[torch.Tensor], top_p: Optional[torch.Tensor], request_seed: Optional[torch.Tensor],
           out_index: Optional[torch.Tensor], engine_seed: int, out_tokens: torch.Tensor, advance=None,
           tile_best=None) -> None:
    """One token per row of float32 logits: argmax where temperature <= 0, else seeded sampling.

    tile_best = (values, columns), float32 and int32 [>=n_rows, tiles]: what linear_head_best left
    beside these logits with limit = real_vocab; greedy rows then read those instead of the logits.

    advance = (token_ids, positions, seq_lens, q_req, slot_mapping [groups, n_stride], block_tables
    [groups, r_stride, max_blocks], page_sizes [groups], history [rows, stride], history_pos): after
    a decode-only step each row also prepares the next step on the device (token, position, length,
    output index, cache slot) and appends its token to the history."""
    _need_cuda(logits, temperature, top_k, top_p, request_seed, out_index, out_tokens)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1 and logits.shape[0] >= n_rows,
          "logits must be float32 [>=n_rows, vocab] with unit inner stride")
    vocab = logits.shape[1]
    _need(0 < real_vocab <= vocab, "real_vocab must lie in 1..vocab")
    _need(temperature.dtype == torch.float32 and temperature.numel() >= n_rows, "temperature must be float32 [rows]")
    _need(top_k is None or (top_k.dtype == torch.int32 and top_k.numel() >= n_rows), "top_k must be int32 [rows]")
    _need(top_p is None or (top_p.dtype == torch.float32 and top_p.numel() >= n_rows), "top_p must be float32 [rows]")
    _need(request_seed is None or (request_seed.dtype in (torch.int64, torch.uint64) and request_seed.numel() >= n_rows),
          "request_seed must be 64-bit [rows]")
    _need(out_index is None or (out_index.dtype == torch.int32 and out_index.numel() >= n_rows),
          "out_index must be int32 [rows]")
    _need_i32("out_tokens", out_tokens, n_rows)
    tb = ti = None
    n_tiles = 0
    if tile_best is not None:
        tb, ti = tile_best
        _need_cuda(tb, ti)
        _need(tb.dtype == torch.float32 and ti.dtype == torch.int32 and tb.dim() == 2 and tb.is_contiguous()
              and ti.is_contiguous() and tb.shape == ti.shape and tb.shape[0] >= n_rows,
              "tile_best must be dense float32 values and int32 columns [>=n_rows, tiles]")
        n_tiles = tb.shape[1]
    if advance is not None:
        token_ids, positions, seq_lens, q_req, slot_mapping, block_tables, page_sizes, history, history_pos = advance
        _need_cuda(*advance)
        _need(out_index is not None, "advancing needs the output index array")
        _need(slot_mapping.dtype == torch.int32 and slot_mapping.dim() == 2 and slot_mapping.is_contiguous(),
              "slot_mapping must be dense int32 [groups, tokens]")
        n_groups, n_stride = slot_mapping.shape
        _need(block_tables.dtype == torch.int32 and block_tables.dim() == 3 and block_tables.is_contiguous()
              and block_tables.shape[0] == n_groups, "block_tables must be dense int32 [groups, requests, blocks]")
        _, r_stride, max_blocks = block_tables.shape
        _need(n_rows <= n_stride and n_rows <= r_stride, "more rows than the step's arrays hold")
        _need_i32("page_sizes", page_sizes, n_groups)
        _need(history.dtype == torch.int32 and history.dim() == 2 and history.is_contiguous()
              and history.shape[1] >= n_rows, "history must be dense int32 [steps, >=rows]")
        for name, t in (("token_ids", token_ids), ("positions", positions), ("seq_lens", seq_lens),
                        ("q_req", q_req), ("history_pos", history_pos)):
            _need_i32(name, t, n_rows)
        rc = library.kernels().mgpt_sample_advance(
            _ptr(logits), logits.stride(0), n_rows, vocab, real_vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
            _ptr(request_seed), _ptr(out_index), ctypes.c_ulonglong(engine_seed & (2**64 - 1)), _ptr(out_tokens),
            _ptr(token_ids), _ptr(positions), _ptr(seq_lens), _ptr(q_req), _ptr(slot_mapping), _ptr(block_tables),
            _ptr(page_sizes), n_groups, n_stride, r_stride, max_blocks, _ptr(history), _ptr(history_pos),
            history.shape[0], history.stride(0), _ptr(tb), _ptr(ti), n_tiles, _stream())
        _check(rc, "sample_advance")
        return
    rc = library.kernels().mgpt_sample(_ptr(logits), logits.stride(0), n_rows, vocab, real_vocab,
                                       _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(request_seed),
                                       _ptr(out_index), ctypes.c_ulonglong(engine_seed & (2**64 - 1)),
                                       _ptr(out_tokens), _ptr(tb), _ptr(ti), n_tiles, _stream())
    _check(rc, "sample")


SK_EPI_QKV = 3
_SKINNY_MAX_ROWS = 64


def fold_layer_norm(w: torch.Tensor, gain: torch.Tensor, beta: Optional[torch.Tensor],
                    bias: Optional[torch.Tensor]):
    """Folds a LayerNorm's gain and bias into the bfloat16 matrix that reads it.  Returns
    (w', colsum, bias'): LN(x) w^T + bias = rstd * (x w'^T - mean * colsum) + bias'."""
    _need_cuda(w, gain, beta, bias)
    n_out, k_dim = w.shape
    _need(w.dtype == torch.bfloat16 and w.is_contiguous(), "the matrix must be dense bfloat16")
    _need(gain.dtype == torch.float32 and gain.numel() == k_dim, "gain must be float32 [inner]")
    _need(beta is None or (beta.dtype == torch.float32 and beta.numel() == k_dim), "beta must be float32 [inner]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    w_out = torch.empty_like(w)
    colsum = torch.empty(n_out, dtype=torch.float32, device=w.device)
    bias_out = torch.empty(n_out, dtype=torch.float32, device=w.device)
    with library.unrecorded():
        rc = library.kernels().mgpt_fold_layernorm(_ptr(w), _ptr(gain), _ptr(beta), _ptr(bias), _ptr(w_out),
                                                   _ptr(colsum), _ptr(bias_out), n_out, k_dim, _stream())
    _check(rc, "fold_layer_norm")
    return w_out, colsum, bias_out


def linear_skinny(a: Optional[torch.Tensor], w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  n_rows: int, epilogue: int = EPI_NONE, *, ln_x: Optional[torch.Tensor] = None,
                  ln_colsum: Optional[torch.Tensor] = None, ln_eps: float = 0.0,
                  ln_rows: Optional[torch.Tensor] = None, scatter=None, general_only: bool = False,
                  partials: Optional[torch.Tensor] = None, w_packed: Optional[torch.Tensor] = None,
                  rows_mode: int = 0, rows_per_group: int = 0) -> bool:
    """bfloat16 MFMA product for at most 64 rows.  With ln_x (the float32 residual stream; ln_rows an
    optional gather) the rows are read through a LayerNorm that fold_layer_norm folded into w, bias
    and ln_colsum.  scatter = (k_pool, v_pool, slot_mapping, q_width, kv_width) also stores the new
    keys and values into their pages.  Up to 16 rows with an inner size that is a multiple of 32 go
    to the kernel laid out for a decode step's latency unless general_only is set.  partials:
    float32 scratch of linear_skinny_partials(...) elements, with which a long inner size under many
    rows is split over workgroups.  w_packed: pack_weight(w), which the decode kernel reads faster
    than w itself.  rows_mode: how the decode kernel treats 17 to 64 rows (0: it chooses, ROWS_SHARE_W:
    one workgroup per column tile takes all rows, ROWS_GROUPS: one per column tile and 16 rows); rows_per_group:
    16, 8, 4, 2 or 1 rows to a workgroup of one tile (0: the kernel's launcher chooses).  Returns False, having launched nothing, when the kernel does not take the shape."""
    if n_rows > _SKINNY_MAX_ROWS or w.dtype != torch.bfloat16:
        return False
    n_out, k_dim = w.shape
    if k_dim % 16 != 0:
        return False
    _need_cuda(a, w, bias, out, ln_x, ln_colsum, ln_rows)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    if epilogue == EPI_RESIDUAL:
        _need(out.dtype == torch.float32, "the residual stream is float32")
    elif epilogue in (EPI_GELU, SK_EPI_QKV):
        _need(out.dtype == torch.bfloat16, "this epilogue writes bfloat16")
    lda = 0
    if ln_x is not None:
        _need(ln_x.dtype == torch.float32 and ln_x.is_contiguous() and ln_x.shape[1] == k_dim,
              "the residual stream must be dense float32 rows of the inner size")
        _need(ln_colsum is not None and ln_colsum.dtype == torch.float32 and ln_colsum.numel() == n_out,
              "the folded column sums must be float32 [out]")
        if ln_rows is None:
            _need(ln_x.shape[0] >= n_rows, "too few residual rows")
        else:
            _need_i32("ln_rows", ln_rows, n_rows)
    else:
        if a is None or a.dtype != torch.bfloat16:
            return False
        _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
              "activation must be [>=n_rows, inner] with unit inner stride")
        if a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0:
            return False
        lda = a.stride(0)
    if w_packed is not None:
        _need_cuda(w_packed)
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and k_dim % 32 == 0
              and w_packed.numel() == -(-n_out // 16) * 16 * k_dim and w_packed.data_ptr() % 16 == 0,
              "w_packed must be pack_weight(w)")
    if partials is not None:
        _need_cuda(partials)
        _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0,
              "partials must be contiguous, 16-byte aligned float32")
    kp = vp = sm = None
    q_width = kv_width = head_dim = n_kv_head = page_size = 0
    if epilogue == SK_EPI_QKV:
        kp, vp, sm, q_width, kv_width = scatter
        _need(kp.shape == vp.shape and kp.dim() == 4 and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16,
              "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
        _, n_kv_head, page_size, head_dim = kp.shape
        _need_i32("slot_mapping", sm, n_rows)
    rc = library.kernels().mgpt_linear_skinny(
        _ptr(a if ln_x is None else None), lda, _ptr(ln_x), _ptr(ln_rows), _ptr(ln_colsum),
        float(ln_eps), _ptr(w), _ptr(w_packed), _ptr(bias), _ptr(out), _dtype_code(out), out.stride(0), n_rows,
        n_out, k_dim, epilogue, _ptr(kp), _ptr(vp), _ptr(sm), q_width, kv_width, head_dim, n_kv_head, page_size,
        1 if general_only else rows_mode | (rows_per_group << 8), _ptr(partials), 0 if partials is None else partials.numel(), _stream())
    if rc == -2:
        return False
    _check(rc, "linear_skinny", 2 if partials is not None else 1)
    return True


def pack_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """A copy of a bfloat16 matrix [out, in] in the layout the decode step's product loads in 1 KB
    pieces (blocks of 16 rows x 32 columns in MFMA operand order; rows padded to a multiple of 16
    with zeros).  None if the inner size is no multiple of 32."""
    _need_cuda(w)
    _need(w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous(), "the matrix must be dense bfloat16")
    n_out, k_dim = w.shape
    if k_dim % 32 != 0 or w.data_ptr() % 16 != 0:
        return None
    packed = torch.empty(-(-n_out // 16) * 16 * k_dim, dtype=torch.bfloat16, device=w.device)
    with library.unrecorded():
        _check(library.kernels().mgpt_pack_weight(_ptr(w), _ptr(packed), n_out, k_dim, _stream()), "pack_weight")
    return packed


ROWS_SHARE_W, ROWS_GROUPS = 2, 3


def linear_head_best(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, n_rows: int,
                     best_val: torch.Tensor, best_idx: torch.Tensor, limit: int,
                     w_packed: Optional[torch.Tensor] = None) -> bool:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias) in float32 for at most 16 bfloat16 rows, and beside it,
    per row and tile of 16 columns, the largest value among the columns below `limit` and its column
    (the lowest among equals): best_val float32, best_idx int32, both [>=n_rows, out / 16].  What
    sample() takes as tile_best.  False, having launched nothing, if the decode kernel does not take
    the shape."""
    n_out, k_dim = w.shape
    if (n_rows > 16 or w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or out.dtype != torch.float32
            or k_dim % 32 or n_out % 16 or a.stride(0) % 8 or a.data_ptr() % 16 or out.stride(0) % 4
            or out.data_ptr() % 16):
        return False
    _need_cuda(a, w, bias, out, best_val, best_idx, w_packed)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out and bias.data_ptr() % 16 == 0),
          "bias must be aligned float32 [out]")
    tiles = n_out // 16
    _need(best_val.dtype == torch.float32 and best_idx.dtype == torch.int32 and best_val.is_contiguous()
          and best_idx.is_contiguous() and tuple(best_val.shape) == tuple(best_idx.shape)
          and best_val.dim() == 2 and best_val.shape[0] >= n_rows and best_val.shape[1] == tiles,
          "best_val and best_idx must be dense float32 / int32 [>=n_rows, out / 16]")
    _need(0 < limit <= n_out, "limit must lie in 1..out")
    if w_packed is not None:
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and w_packed.numel() == n_out * k_dim
              and w_packed.data_ptr() % 16 == 0, "w_packed must be pack_weight(w)")
    rc = library.kernels().mgpt_linear_head_best(
        _ptr(a), a.stride(0), None, None, None, 0.0, _ptr(w), _ptr(w_packed), _ptr(bias), _ptr(out), out.stride(0),
        n_rows, n_out, k_dim, _ptr(best_val), _ptr(best_idx), int(limit), _stream())
    if rc == -2:
        return False
    _check(rc, "linear_head_best")
    return True


def linear_decode_parts(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], partials: torch.Tensor,
                        n_rows: int, w_packed: Optional[torch.Tensor] = None) -> int:
    """The split product's first half alone: partials[p, :n_rows] (float32 [parts, n_rows, out], dense)
    = a[:n_rows] @ w[:, stretch p of the inner size].T, the first with the bias added; nobody adds them
    up.  Returns the number of parts, or 0, having launched nothing, for a shape that linear_skinny
    would not split (linear_skinny_partials(n_rows, out, inner, False, EPI_RESIDUAL) == 0)."""
    n_out, k_dim = w.shape
    if (w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or a.stride(0) % 8 or a.data_ptr() % 16
            or not linear_skinny_partials(n_rows, n_out, k_dim, False, EPI_RESIDUAL)):
        return 0
    parts = int(library.kernels().mgpt_linear_decode_parts_count())
    _need_cuda(a, w, bias, partials, w_packed)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out and bias.data_ptr() % 16 == 0),
          "bias must be aligned float32 [out]")
    _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0
          and tuple(partials.shape) == (parts, n_rows, n_out), f"partials must be dense float32 [{parts}, n_rows, out]")
    if w_packed is not None:
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and w_packed.numel() == n_out * k_dim
              and w_packed.data_ptr() % 16 == 0, "w_packed must be pack_weight(w)")
    rc = library.kernels().mgpt_linear_decode_parts(_ptr(a), a.stride(0), _ptr(w), _ptr(w_packed), _ptr(bias),
                                                    _ptr(partials), n_rows, n_out, k_dim, _stream())
    if rc == -2:
        return 0
    _check(rc, "linear_decode_parts")
    return parts


def linear_skinny_row_groups(n_rows: int, n_out: int, k_dim: int) -> bool:
    """Whether linear_skinny, left to choose, gives every 16 of these rows workgroups of their own
    (a folded LayerNorm then costs a workgroup what it costs at 16 rows)."""
    return bool(library.kernels().mgpt_linear_skinny_row_groups(n_rows, n_out, k_dim))


def linear_skinny_partials(n_rows: int, n_out: int, k_dim: int, has_ln: bool, epilogue: int) -> int:
    """float32 elements of scratch with which linear_skinny would split this shape's inner size over
    workgroups; 0 if it would not."""
    return int(library.kernels().mgpt_linear_skinny_partials(n_rows, n_out, k_dim, 1 if has_ln else 0, epilogue))


def paged_attention_split_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                               block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor,
                               q_req: torch.Tensor, n_tokens: int, n_req: int, n_head: int, scale: float,
                               window: int = 0, fast: bool = True, sinks: Optional[torch.Tensor] = None,
                               softcap: float = 0.0, gate: Optional[torch.Tensor] = None, keep_first: int = 0,
                               score_bias: Optional[torch.Tensor] = None) -> bool:
    """bfloat16 attention with each (token, head)'s keys split over four waves.  False if refused.
    fast=False keeps to the variant that takes every head size."""
    if q.dtype != torch.bfloat16:
        return False
    n_kv_head, page_size, head_dim = _check_attention_args(
        q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head)
    if head_dim % 8 != 0 or head_dim > 256 or k_pool.data_ptr() % 16 != 0:
        return False
    _need_sinks(sinks, n_head)
    fn = library.kernels().mgpt_paged_attention_split_bf16
    if fast and head_dim in (16, 32, 64, 128) and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0:
        fn = library.kernels().mgpt_paged_attention_split_fast_bf16   # all loads 16 bytes wide
    rc = fn(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), _ptr(q_req), n_tokens, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), _ptr(sinks), float(softcap), *_gate_args(gate, q, n_tokens, n_head),
        *_mask_args(keep_first, score_bias, n_head, sinks, softcap), _stream())
    if rc == -2:
        return False
    _check(rc, "paged_attention_split_bf16")
    return True


def paged_attention_decode_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                                block_tables: torch.Tensor, positions: torch.Tensor, q_req: torch.Tensor,
                                n_tokens: int, n_head: int, scale: float, window: int = 0,
                                identity: bool = False, cu_q: Optional[torch.Tensor] = None,
                                sinks: Optional[torch.Tensor] = None, softcap: float = 0.0,
                                gate: Optional[torch.Tensor] = None, keep_first: int = 0,
                                score_bias: Optional[torch.Tensor] = None) -> bool:
    """bfloat16 attention for single tokens (one query per request and step), keys split over eight
    waves.  positions[n] is token n's absolute position, q_req[n] its block table row or -1 for a
    padded token; identity=True promises q_req[n] in (n, -1).  With cu_q (the requests' token offsets;
    not with identity) tokens of requests that bring more than one token are skipped.  False if
    refused (other head sizes than 16, 32, 64, 128)."""
    if q.dtype != torch.bfloat16:
        return False
    _need_cuda(q, out, k_pool, v_pool, block_tables, positions, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous()
          and k_pool.dtype == torch.bfloat16 and v_pool.dtype == torch.bfloat16,
          "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
    num_pages, n_kv_head, page_size, head_dim = k_pool.shape
    if head_dim not in (16, 32, 64, 128) or q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0 \
            or k_pool.data_ptr() % 16 != 0 or v_pool.data_ptr() % 16 != 0:
        return False
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[0] >= n_tokens and q.shape[1] >= n_head * head_dim,
          "q must be [>=n_tokens, >=heads*head_dim] with unit inner stride")
    _need(out.dtype == torch.bfloat16 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] >= n_tokens
          and out.shape[1] >= n_head * head_dim, "out must be bfloat16 [>=n_tokens, >=heads*head_dim]")
    _need(n_head % n_kv_head == 0, "query heads must be a multiple of key/value heads")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "block_tables must be dense int32 [requests, blocks]")
    _need_i32("positions", positions, n_tokens)
    _need_i32("q_req", q_req, n_tokens)
    _need_sinks(sinks, n_head)
    if identity:
        _need(block_tables.shape[0] >= n_tokens, "a decode-only step needs a block table row per token")
        _need(cu_q is None, "cu_q is for steps that are not decode-only")
    if cu_q is not None:
        _need_cuda(cu_q)
        _need_i32("cu_q", cu_q, block_tables.shape[0] + 1)
    rc = library.kernels().mgpt_paged_attention_decode_bf16(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(positions), _ptr(q_req), _ptr(cu_q), n_tokens, n_head, n_kv_head, head_dim, page_size,
        num_pages, float(scale), int(window), 1 if identity else 0, _ptr(sinks), float(softcap),
        *_gate_args(gate, q, n_tokens, n_head), *_mask_args(keep_first, score_bias, n_head, sinks, softcap), _stream())
    if rc == -2:
        return False
    _check(rc, "paged_attention_decode_bf16")
    return True


_MFMA_PARTIALS: dict = {}   # the library's answer per size: asked at every product of every step


def linear_mfma_partials(n_rows: int, n_out: int, k_dim: int, epilogue: int) -> int:
    """Floats of scratch that linear_mfma would use to split this product along its inner size
    (0: it would not split it)."""
    key = (n_rows, n_out, k_dim, epilogue)
    hit = _MFMA_PARTIALS.get(key)
    if hit is None:
        if len(_MFMA_PARTIALS) > 4096:
            _MFMA_PARTIALS.clear()
        hit = _MFMA_PARTIALS[key] = int(library.kernels().mgpt_linear_mfma_partials(n_rows, n_out, k_dim, epilogue))
    return hit


def linear_mfma_parts(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], partials: torch.Tensor,
                      n_rows: int) -> bool:
    """The tiled product's first half alone where it splits the inner size: partials[p, :n_rows]
    (float32 [parts, n_rows, out], dense, parts = linear_mfma_partials(n_rows, out, inner, EPI_RESIDUAL)
    // (n_rows * out)) = a[:n_rows] @ w[:, stretch p].T, the first with the bias added; nobody adds
    them up.  False, having launched nothing, where the product would not be split."""
    n_out, k_dim = w.shape
    need = linear_mfma_partials(n_rows, n_out, k_dim, EPI_RESIDUAL)
    if (not need or w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or a.stride(0) % 8 or a.data_ptr() % 16
            or w.data_ptr() % 16 or k_dim % 16):
        return False
    parts = need // (n_rows * n_out)
    _need_cuda(a, w, bias, partials)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0
          and tuple(partials.shape) == (parts, n_rows, n_out), f"partials must be dense float32 [{parts}, n_rows, out]")
    rc = library.kernels().mgpt_linear_mfma_parts(_ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(partials),
                                                  partials.numel(), n_rows, n_out, k_dim, _stream())
    if rc == -2:
        return False
    _check(rc, "linear_mfma_parts")
    return True


def linear_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                n_rows: int, epilogue: int, scatter=None, shape: Optional[int] = None,
                partials: Optional[torch.Tensor] = None, k_parts: Optional[int] = None) -> bool:
    """Tiled bfloat16 MFMA product for many rows.  scatter = (k_pool, v_pool, slot_mapping, q_width,
    kv_width) also stores the new keys and values into their pages (bfloat16 output, no other
    epilogue).  `partials`: float32 scratch with which a long inner size over few tiles is split
    among workgroups (linear_mfma_partials says how much it takes).  `shape` (0 = 256 x 256 tiles,
    1 = 128 x 256, 2 = 128 x 64, 3 = 64 x 64, 4 = 32 x 32, 5 and 6 = 64 x 64 and 32 x 32 with four
    steps on their way from memory, 7 = 64 x 64 with two wave groups that share a tile, float32 outputs, 8 to 12 = operand slices straight
    into LDS with tiles of 32 x 32, 64 x 64, 128 x 64, 128 x 192, 32 x 32 with six stages: an inner size that is a
    multiple of 64) and
    `k_parts` fix what the library otherwise chooses by the size.  False when it does not take the shape."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    n_out, k_dim = w.shape
    if k_dim % 16 != 0 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0 or w.data_ptr() % 16 != 0:
        return False
    if scatter is not None and (epilogue != EPI_NONE or out.dtype != torch.bfloat16):
        return False
    if (epilogue, out.dtype) not in ((EPI_NONE, torch.bfloat16), (EPI_NONE, torch.float32),
                                     (EPI_GELU, torch.bfloat16), (EPI_RESIDUAL, torch.float32)):
        return False
    _need_cuda(a, w, bias, out)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    if scatter is not None:
        kp, vp, sm, q_width, kv_width = scatter
        _need_cuda(kp, vp, sm)
        _need(kp.shape == vp.shape and kp.dim() == 4 and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16,
              "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
        _, n_kv_head, page_size, head_dim = kp.shape
        _need_i32("slot_mapping", sm, n_rows)
        rc = library.kernels().mgpt_linear_mfma_qkv(
            _ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(out), out.stride(0), n_rows, n_out, k_dim, _ptr(kp),
            _ptr(vp), _ptr(sm), q_width, kv_width, head_dim, n_kv_head, page_size, -1 if shape is None else int(shape),
            _stream())
    else:
        if partials is not None:
            _need_cuda(partials)
            _need(partials.dtype == torch.float32 and partials.is_contiguous(), "partials must be dense float32")
        args = (_ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(out), _dtype_code(out), out.stride(0), n_rows,
                n_out, k_dim, epilogue, _ptr(partials), 0 if partials is None else partials.numel(), _stream())
        if shape is None and k_parts is None:
            rc = library.kernels().mgpt_linear_mfma(*args)
        else:
            rc = library.kernels().mgpt_linear_mfma_shape(-1 if shape is None else int(shape),
                                                          0 if k_parts is None else int(k_parts), *args)
    if rc == -2:
        return False
    _check(rc, "linear_mfma", 2 if partials is not None else 1)
    return True


def linear_mfma_xielu(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, n_rows: int,
                      coef: torch.Tensor, partials: Optional[torch.Tensor] = None) -> bool:
    """The tiled bfloat16 product with the xIELU activation as its epilogue: out = act(a @ w.T (+ bias)) with
    act(v) = coef[0] v^2 + v / 2 for v > 0 and coef[1] (exp(v) - 1 - v) + v / 2 elsewhere (coef float32 [2]),
    bfloat16 out.  `partials` as for linear_mfma (linear_mfma_partials with EPI_XIELU says how much).  False when
    it does not take the shape."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        return False
    n_out, k_dim = w.shape
    if k_dim % 16 != 0 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0 or w.data_ptr() % 16 != 0:
        return False
    _need_cuda(a, w, bias, out, coef, partials)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    _need(coef.dtype == torch.float32 and coef.is_contiguous() and coef.numel() == 2, "coef must be float32 [2]")
    _need(partials is None or (partials.dtype == torch.float32 and partials.is_contiguous()), "partials must be dense float32")
    rc = library.kernels().mgpt_linear_mfma_xielu(
        _ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(out), out.stride(0), n_rows, n_out, k_dim, _ptr(coef),
        _ptr(partials), 0 if partials is None else partials.numel(), _stream())
    if rc == -2:
        return False
    _check(rc, "linear_mfma_xielu", 2 if partials is not None else 1)
    return True


def prefill_attention_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                           block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor, n_req: int,
                           max_q_len: int, n_head: int, scale: float, window: int = 0,
                           single_below: int = 0, sinks: Optional[torch.Tensor] = None, softcap: float = 0.0,
                           gate: Optional[torch.Tensor] = None, keep_first: int = 0,
                           score_bias: Optional[torch.Tensor] = None) -> bool:
    """MFMA tile attention for steps with prompt portions (every request's tokens are consecutive
    rows of q from cu_q; a request may bring none).  Requests that bring exactly one token, and that
    among the step's first `single_below` tokens, are left to another kernel.  False when it does
    not take the case."""
    if q.dtype != torch.bfloat16:
        return False
    _need_cuda(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    if head_dim not in (32, 64, 96, 128) or q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0 \
            or k_pool.data_ptr() % 16 != 0 or v_pool.data_ptr() % 16 != 0:
        return False
    _need(q.dtype == out.dtype == k_pool.dtype == v_pool.dtype, "queries, output and pools must share a dtype")
    _need(q.stride(1) == 1 and out.stride(1) == 1, "query and output rows must have unit inner stride")
    _need(q.shape[1] >= n_head * head_dim and out.shape[1] >= n_head * head_dim,
          "query/output rows are narrower than n_head * head_dim")
    _need(n_head % n_kv_head == 0, "n_head must be a multiple of the number of key/value heads")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_req, "block_tables must be dense int32 [>=requests, max_blocks]")
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("seq_lens", seq_lens, n_req)
    _need_sinks(sinks, n_head)
    rc = library.kernels().mgpt_prefill_attention_bf16(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), n_req, max_q_len, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), int(single_below), _ptr(sinks), float(softcap),
        *_gate_args(gate, q, q.shape[0], n_head), *_mask_args(keep_first, score_bias, n_head, sinks, softcap), _stream())
    if rc == -2:
        return False
    _check(rc, "prefill_attention_bf16")
    return True


# ---------------------------------------------------------------- decode steps of few rows, fused
FUSED_MAX_WIDTH = 512
FUSED_MLP_SLICE = 64


def fused_parts_limit(width: int) -> int:
    """Most pending sums of a residual of this width that the fused kernels add up on their way in
    (0: they do not take the width)."""
    if width <= 0 or width % 32 or width > FUSED_MAX_WIDTH:
        return 0
    return int(library.kernels().mgpt_fused_parts_limit(width))


def _residual_args(pending, width: int):
    """The argument block of a residual that is still a sum (ops.residual.PendingSums)."""
    base, partials, n_parts = pending.base, pending.partials, pending.n_parts
    tok = pos = ids = positions = None
    if base is None:
        tok, pos, ids, positions = pending.tables
        _need_cuda(tok, pos, ids, positions)
        _need(tok.dtype == torch.bfloat16 and tok.is_contiguous() and tok.shape[1] == width,
              "the token table must be dense bfloat16 [vocab, width]")
        _need(pos is None or (pos.dtype == torch.bfloat16 and pos.is_contiguous() and pos.shape[1] == width),
              "the position table must be dense bfloat16 [positions, width]")
    else:
        _need_cuda(base)
        _need(base.dtype == torch.float32 and base.is_contiguous() and base.shape[1] == width,
              "the residual rows must be dense float32 [rows, width]")
    stride = 0
    if n_parts:
        _need_cuda(partials)
        _need(partials.dtype == torch.float32 and partials.dim() == 3 and partials.is_contiguous()
              and partials.shape[0] >= n_parts and partials.shape[2] == width,
              "pending sums must be dense float32 [parts, rows, width]")
        stride = partials.stride(0)
    return (_ptr(base), _ptr(partials) if n_parts else None, n_parts, stride, _ptr(tok), _ptr(pos), _ptr(ids),
            _ptr(positions))


def _overlap(a: Optional[torch.Tensor], b: Optional[torch.Tensor]) -> bool:
    """Whether two tensors' bytes overlap."""
    if a is None or b is None or not a.numel() or not b.numel():
        return False
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def _residual_rows(pending) -> int:
    """Rows that every array of a pending residual holds."""
    rows = 1 << 30
    if pending.base is not None:
        rows = min(rows, pending.base.shape[0])
    else:
        rows = min(rows, pending.tables[2].numel())
    if pending.n_parts:
        rows = min(rows, pending.partials.shape[1])
    return rows


def fused_attention_tokens(n_rows: int, n_head: int, head_dim: int) -> int:
    """Tokens that a workgroup of fused_attention_decode takes in a step of n_rows rows.  With more
    than one, rows that are no table rows must be handed over normed; 0: the kernel does not take so
    many rows."""
    return int(library.kernels().mgpt_fused_attention_tokens(int(n_rows), int(n_head), int(head_dim)))


def fused_attention_decode(pending, settled: Optional[torch.Tensor], gain: torch.Tensor, beta: Optional[torch.Tensor],
                           eps: float, wqkv_packed: torch.Tensor, bqkv: Optional[torch.Tensor],
                           wproj_packed: torch.Tensor, bproj: Optional[torch.Tensor], out_partials: torch.Tensor,
                           k_pool: torch.Tensor, v_pool: torch.Tensor, slot_mapping: torch.Tensor,
                           block_tables: torch.Tensor, positions: torch.Tensor, q_req: torch.Tensor, n_rows: int,
                           n_head: int, scale: float, normed: Optional[torch.Tensor] = None) -> bool:
    """LayerNorm, one head's q/k/v, cache write, attention and that head's share of the output
    projection, for the single tokens of a decode-only step: out_partials[h, n] is head h's share
    of what token n adds to the residual.  The residual comes as a sum (pending), whose value is
    stored to `settled` on the way.  In a step of so many rows that a workgroup takes several
    tokens (fused_attention_tokens), rows that are no table rows come normed instead (`normed`:
    bfloat16 [rows, width], the LayerNorm of the plain rows `pending.base`; nothing is stored to
    `settled`, which may be None).  False, having launched nothing, if the kernel does not take the
    shape."""
    width = gain.numel()
    _need_cuda(settled, gain, beta, wqkv_packed, bqkv, wproj_packed, bproj, out_partials, k_pool, v_pool,
               slot_mapping, block_tables, positions, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous()
          and k_pool.dtype == torch.bfloat16 and v_pool.dtype == torch.bfloat16,
          "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
    num_pages, n_kv_head, page_size, head_dim = k_pool.shape
    q_width = n_head * head_dim
    if (n_kv_head != n_head or head_dim not in (16, 32, 64, 128) or width % 32 or width > FUSED_MAX_WIDTH
            or q_width % 32 or page_size & (page_size - 1) or pending.n_parts > fused_parts_limit(width)):
        return False
    tokens = fused_attention_tokens(n_rows, n_head, head_dim)
    use_normed = pending.base is not None and tokens > 1
    if tokens == 0 or (use_normed and (normed is None or pending.n_parts)):
        return False
    args = _residual_args(pending, width)
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than the step")
    if use_normed:
        _need_cuda(normed)
        _need(normed.dtype == torch.bfloat16 and normed.is_contiguous() and normed.dim() == 2
              and normed.shape[1] == width and normed.shape[0] >= n_rows, "normed rows must be dense bfloat16 [>=rows, width]")
    else:
        _need(settled is not None and settled.dtype == torch.float32 and settled.is_contiguous()
              and settled.shape[1] == width and settled.shape[0] >= n_rows
              and (pending.base is None or settled.data_ptr() != pending.base.data_ptr()),
              "the settled rows need a dense float32 array of their own")
    for name, t, numel in (("gain", gain, width), ("beta", beta, width), ("qkv bias", bqkv, 3 * q_width),
                           ("projection bias", bproj, width)):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == numel), f"{name} must be float32 [{numel}]")
    _need(wqkv_packed.dtype == torch.bfloat16 and wqkv_packed.numel() == 3 * q_width * width,
          "wqkv_packed must be pack_weight of the [3 * heads * head_dim, width] matrix")
    _need(wproj_packed.dtype == torch.bfloat16 and wproj_packed.numel() == width * q_width,
          "wproj_packed must be pack_weight of the [width, heads * head_dim] matrix")
    _need(out_partials.dtype == torch.float32 and out_partials.dim() == 3 and out_partials.is_contiguous()
          and out_partials.shape[0] >= n_head and out_partials.shape[1] >= n_rows and out_partials.shape[2] == width,
          "out_partials must be dense float32 [>=heads, >=rows, width]")
    # a workgroup adds the pending sums up while others of the launch already store theirs
    _need(not (pending.n_parts and _overlap(out_partials, pending.partials)),
          "out_partials must not be the array that holds the pending sums")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_rows, "block_tables must be dense int32 [>=rows, blocks]")
    _need_i32("slot_mapping", slot_mapping, n_rows)
    _need_i32("positions", positions, n_rows)
    _need_i32("q_req", q_req, n_rows)
    rc = library.kernels().mgpt_fused_attention_decode(
        *args, None if use_normed else _ptr(settled), _ptr(normed) if use_normed else None, _ptr(gain), _ptr(beta),
        float(eps), _ptr(wqkv_packed), _ptr(bqkv), _ptr(wproj_packed),
        _ptr(bproj), _ptr(out_partials), out_partials.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(slot_mapping),
        _ptr(block_tables), block_tables.shape[1], _ptr(positions), _ptr(q_req), n_rows, width, n_head, head_dim,
        page_size, num_pages, float(scale), _stream())
    if rc == -2:
        return False
    _check(rc, "fused_attention_decode")
    return True


def fused_mlp_parts(hidden: int) -> int:
    """Parts that fused_mlp_decode leaves of its output (0: it does not take this hidden size)."""
    return hidden // FUSED_MLP_SLICE if hidden > 0 and hidden % FUSED_MLP_SLICE == 0 else 0


def fused_mlp_decode(pending, settled: torch.Tensor, gain: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
                     wfc_packed: torch.Tensor, bfc: Optional[torch.Tensor], wproj_packed: torch.Tensor,
                     bproj: Optional[torch.Tensor], out_partials: torch.Tensor, n_rows: int, hidden: int) -> bool:
    """LayerNorm, 64 hidden units of the first product with bias and GELU-tanh, and their share of
    the second product, per workgroup: out_partials[j, n] is what hidden units 64 j .. add to row n
    of the residual.  False, having launched nothing, if the kernel does not take the shape."""
    width = gain.numel()
    parts = fused_mlp_parts(hidden)
    if not parts or width % 32 or width > FUSED_MAX_WIDTH or pending.base is None \
            or pending.n_parts > fused_parts_limit(width):
        return False
    _need_cuda(settled, gain, beta, wfc_packed, bfc, wproj_packed, bproj, out_partials)
    args = _residual_args(pending, width)
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than the step")
    _need(settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[1] == width
          and settled.shape[0] >= n_rows and (pending.base is None or settled.data_ptr() != pending.base.data_ptr()),
          "the settled rows need a dense float32 array of their own")
    for name, t, numel in (("gain", gain, width), ("beta", beta, width), ("first bias", bfc, hidden),
                           ("second bias", bproj, width)):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == numel), f"{name} must be float32 [{numel}]")
    _need(wfc_packed.dtype == torch.bfloat16 and wfc_packed.numel() == hidden * width
          and wproj_packed.dtype == torch.bfloat16 and wproj_packed.numel() == hidden * width,
          "the matrices must be pack_weight of [hidden, width] and [width, hidden]")
    _need(out_partials.dtype == torch.float32 and out_partials.dim() == 3 and out_partials.is_contiguous()
          and out_partials.shape[0] >= parts and out_partials.shape[1] >= n_rows and out_partials.shape[2] == width,
          "out_partials must be dense float32 [>=hidden/64, >=rows, width]")
    _need(not (pending.n_parts and _overlap(out_partials, pending.partials)),
          "out_partials must not be the array that holds the pending sums")
    rc = library.kernels().mgpt_fused_mlp_decode(
        *args, _ptr(settled), _ptr(gain), _ptr(beta), float(eps), _ptr(wfc_packed), _ptr(bfc), _ptr(wproj_packed),
        _ptr(bproj), _ptr(out_partials), out_partials.stride(0), n_rows, width, hidden, _stream())
    if rc == -2:
        return False
    _check(rc, "fused_mlp_decode")
    return True


RESIDUAL_MAX_WIDTH = 4096
_RESIDUAL_PARTS_LIMIT: Dict[int, int] = {}


def residual_parts_limit(width: int) -> int:
    """Most parts of a pending residual of this width that residual_layer_norm adds up (0: the width
    is not taken).  Wider than the fused kernels take: a row up to RESIDUAL_MAX_WIDTH."""
    hit = _RESIDUAL_PARTS_LIMIT.get(width)
    if hit is None:
        hit = _RESIDUAL_PARTS_LIMIT[width] = int(library.kernels().mgpt_residual_parts_limit(int(width)))
    return hit


def residual_layer_norm(pending, gain: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
                        rows: Optional[torch.Tensor], out: torch.Tensor, n_rows: int,
                        settled: Optional[torch.Tensor] = None) -> bool:
    """out[i] = LayerNorm of row rows[i] (or i) of a residual that is still a sum.  With `settled`
    (float32 rows; may be the sum's base itself) the rows' sums are stored there too.  False if
    the width is not taken."""
    width = gain.numel()
    if width % 32 or width > RESIDUAL_MAX_WIDTH or pending.base is None or pending.n_parts > residual_parts_limit(width):
        return False
    _need_cuda(gain, beta, rows, out, settled)
    _need(settled is None or (settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[1] == width
                              and settled.shape[0] >= (n_rows if rows is None else 0) and settled.data_ptr() % 16 == 0),
          "the settled rows must be dense float32 of the residual's width")
    _need(settled is None or rows is None, "settling through a row gather is not supported")
    args = _residual_args(pending, width)
    _need(gain.dtype == torch.float32 and (beta is None or (beta.dtype == torch.float32 and beta.numel() == width)),
          "gain and beta must be float32 [width]")
    _need(out.is_contiguous() and out.shape[1] == width and out.shape[0] >= n_rows, "LayerNorm output too small")
    if rows is None:
        _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than asked for")
    else:
        _need_i32("rows", rows, n_rows)
    rc = library.kernels().mgpt_residual_layernorm(*args, _ptr(gain), _ptr(beta), float(eps), _ptr(rows), _ptr(out),
                                                   _dtype_code(out), n_rows, width, _ptr(settled), _stream())
    if rc == -2:
        return False
    _check(rc, "residual_layer_norm")
    return True


def residual_settle(pending, settled: torch.Tensor, n_rows: int) -> bool:
    """settled[:n_rows] = the rows of a residual that is still a sum (settled may be its base).
    False if the width is not taken."""
    width = settled.shape[1]
    if width % 32 or width > RESIDUAL_MAX_WIDTH or pending.base is None:
        return False
    _need_cuda(settled)
    args = _residual_args(pending, width)
    _need(settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[0] >= n_rows,
          "the settled rows must be dense float32")
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than asked for")
    rc = library.kernels().mgpt_residual_settle(*args, _ptr(settled), n_rows, width, _stream())
    if rc == -2:
        return False
    _check(rc, "residual_settle")
    return True


# ---------------------------------------------------------------- several residual streams, soft-capped logits
MAX_STREAMS = 8


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, x: torch.Tensor, n_tokens: int, scale: float,
                 copies: int = 1) -> None:
    """x[t][s] = table[ids[t]] * scale for every s < copies; x is float32 [>=n_tokens, copies * width]."""
    _need_cuda(ids, table, x)
    width = table.shape[1]
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be dense [vocab, width]")
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == copies * width and x.shape[0] >= n_tokens,
          "residual streams must be dense float32 [>=n_tokens, copies * width]")
    _need_i32("ids", ids, n_tokens)
    rc = library.kernels().mgpt_embed_scaled(_ptr(ids), _ptr(table), _ptr(x), n_tokens, width, _dtype_code(table),
                                             float(scale), int(copies), _stream())
    _check(rc, "embed_scaled")


def _need_streams(x: torch.Tensor, n_rows: int, width: int, streams: int) -> None:
    _need(1 <= streams <= MAX_STREAMS, f"the kernels take up to {MAX_STREAMS} residual streams")
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2 and x.shape[1] == streams * width
          and x.shape[0] >= n_rows, "residual streams must be dense float32 [>=n_rows, streams * width]")


def _need_rows_f32(name: str, t: torch.Tensor, n_rows: int, width: int) -> None:
    _need(t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 2 and t.shape[1] == width
          and t.shape[0] >= n_rows, f"{name} must be dense float32 [>=n_rows, {width}]")


def streams_read(x: torch.Tensor, coef: Optional[torch.Tensor], u: torch.Tensor, n_rows: int, streams: int,
                 zero: Optional[torch.Tensor] = None) -> None:
    """u[n] = sum_s coef[s] x[n][s] (coef None: the plain sum); `zero`, shaped like u, is cleared."""
    _need_cuda(x, coef, u, zero)
    width = u.shape[1]
    _need_streams(x, n_rows, width, streams)
    _need_rows_f32("u", u, n_rows, width)
    if zero is not None:
        _need_rows_f32("zero", zero, n_rows, width)
    _need(coef is None or (coef.dtype == torch.float32 and coef.is_contiguous() and coef.numel() == streams),
          "coef must be float32 [streams]")
    rc = library.kernels().mgpt_streams_read(_ptr(x), _ptr(coef), _ptr(u), _ptr(zero), n_rows, width, streams,
                                             _stream())
    _check(rc, "streams_read")


def streams_write(x: torch.Tensor, mix: torch.Tensor, out: torch.Tensor, y: torch.Tensor, n_rows: int,
                  streams: int) -> None:
    """x[n][t] = sum_s mix[s][t] x[n][s] + out[t] y[n], every t from the old streams."""
    _need_cuda(x, mix, out, y)
    width = y.shape[1]
    _need_streams(x, n_rows, width, streams)
    _need_rows_f32("y", y, n_rows, width)
    _need(mix.dtype == torch.float32 and mix.is_contiguous() and tuple(mix.shape) == (streams, streams),
          "mix must be float32 [streams, streams]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.numel() == streams, "out must be float32 [streams]")
    rc = library.kernels().mgpt_streams_write(_ptr(x), _ptr(mix), _ptr(out), _ptr(y), n_rows, width, streams,
                                              _stream())
    _check(rc, "streams_write")


def streams_step(x: torch.Tensor, write, coef: torch.Tensor, u: torch.Tensor, gain: torch.Tensor,
                 beta: Optional[torch.Tensor], eps: float, h: torch.Tensor, n_rows: int, streams: int,
                 zero: Optional[torch.Tensor] = None) -> None:
    """One pass over every token's streams: the write that is still to be made (write = (mix, out, y)
    as for streams_write, or None), `zero` cleared (it may be y), then u = sum_t coef[t] x[t] and
    h = LayerNorm(u) with gain (and beta), in h's dtype."""
    mix, out, y = write if write is not None else (None, None, None)
    _need_cuda(x, mix, out, y, coef, u, gain, beta, h, zero)
    width = u.shape[1]
    _need_streams(x, n_rows, width, streams)
    _need_rows_f32("u", u, n_rows, width)
    for name, t in (("y", y), ("zero", zero)):
        if t is not None:
            _need_rows_f32(name, t, n_rows, width)
    _need(h.dim() == 2 and h.is_contiguous() and h.shape[1] == width and h.shape[0] >= n_rows, "h must be dense [>=n_rows, width]")
    _need(coef.dtype == torch.float32 and coef.is_contiguous() and coef.numel() == streams, "coef must be float32 [streams]")
    if write is not None:
        _need(mix.dtype == torch.float32 and mix.is_contiguous() and tuple(mix.shape) == (streams, streams)
              and out.dtype == torch.float32 and out.is_contiguous() and out.numel() == streams,
              "mix must be float32 [streams, streams] and out float32 [streams]")
    _need(gain.dtype == torch.float32 and gain.numel() == width and (beta is None or (beta.dtype == torch.float32
          and beta.numel() == width)), "gain and beta must be float32 [width]")
    _need(y is None or zero is None or y.data_ptr() == zero.data_ptr(), "the buffer to clear is y itself")
    buf = y if y is not None else zero
    rc = library.kernels().mgpt_streams_step(_ptr(x), _ptr(mix), _ptr(out), _ptr(buf), int(write is not None),
                                             int(zero is not None), _ptr(coef), _ptr(u), _ptr(gain), _ptr(beta),
                                             float(eps), _ptr(h), _dtype_code(h), n_rows, width, streams, _stream())
    _check(rc, "streams_step")


def scale_softcap(logits: torch.Tensor, n_rows: int, scale: float, cap: float, fast: bool) -> None:
    """logits = cap * tanh(logits * scale / cap) in place (cap <= 0: the scale alone)."""
    _need_cuda(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1 and logits.shape[0] >= n_rows,
          "logits must be float32 [>=n_rows, vocab] with unit inner stride")
    rc = library.kernels().mgpt_scale_softcap(_ptr(logits), logits.stride(0), n_rows, logits.shape[1], float(scale),
                                              float(cap), int(fast), _stream())
    _check(rc, "scale_softcap")


# ---------------------------------------------------------------- latent attention
def rms_norm_store(src: torch.Tensor, gain: torch.Tensor, eps: float, pool: torch.Tensor,
                   slot_mapping: torch.Tensor, n_tokens: int) -> None:
    """pool[slot of token n] = src[n] / sqrt(mean(src[n]^2) + eps) * gain; pool [pages, 1, page_size, rank]."""
    _need_cuda(src, gain, pool, slot_mapping)
    _need(pool.dim() == 4 and pool.shape[1] == 1 and pool.is_contiguous(),
          "a latent pool must be dense [pages, 1, page_size, rank]")
    rank = pool.shape[3]
    _need(src.dim() == 2 and src.stride(1) == 1 and src.shape[1] == rank and src.shape[0] >= n_tokens
          and src.dtype == pool.dtype, "latents must be [>=n_tokens, rank] in the pool's dtype")
    _need(gain.dtype == torch.float32 and gain.is_contiguous() and gain.numel() == rank, "gain must be float32 [rank]")
    _need_i32("slot_mapping", slot_mapping, n_tokens)
    rc = library.kernels().mgpt_rms_norm_store(_ptr(src), _dtype_code(src), src.stride(0), _ptr(gain), float(eps),
                                               _ptr(pool), _ptr(slot_mapping), n_tokens, rank, _stream())
    _check(rc, "rms_norm_store")


def latent_prepare(z: torch.Tensor, q_off: int, n_head: int, head_dim: int, rot_dim: int, positions: torch.Tensor,
                   freq: torch.Tensor, n_tokens: int, rot_magnitude: float = 1.0, c_off: int = 0, rank: int = 0,
                   gain: Optional[torch.Tensor] = None, eps: float = 0.0, pool: Optional[torch.Tensor] = None,
                   slot_mapping: Optional[torch.Tensor] = None) -> None:
    """Latent attention with a rotated part: the last rot_dim channels of every query head (heads of head_dim +
    rot_dim channels at q_off of z's rows) are rotated in place by the token's position; with `pool` (latent pages
    whose rows hold at least rank + rot_dim values) the token's row becomes [rms_norm(z[c_off : c_off + rank]) * gain |
    the next rot_dim columns of z, rotated | zeros].  freq: float32 [rot_dim / 2]."""
    _need_cuda(z, positions, freq, gain, pool, slot_mapping)
    _rows_2d("latent_prepare z", z, n_tokens)
    _need(freq.dtype == torch.float32 and freq.is_contiguous() and freq.numel() * 2 == rot_dim, "latent_prepare: float32 frequencies [rot_dim / 2]")
    _need_i32("positions", positions, n_tokens)
    _need(z.shape[1] >= q_off + n_head * (head_dim + rot_dim), "latent_prepare: z is too narrow for the queries")
    row_width = 0
    if pool is not None:
        _need(pool.dtype == z.dtype and pool.is_contiguous() and pool.dim() == 4 and pool.shape[1] == 1
              and pool.shape[3] >= rank + rot_dim, "latent_prepare: the pool must be [pages, 1, page, >= rank + rot_dim] in z's dtype")
        _need(gain is not None and gain.dtype == torch.float32 and gain.is_contiguous() and gain.numel() == rank,
              "latent_prepare: gain must be float32 [rank]")
        _need(z.shape[1] >= c_off + rank + rot_dim, "latent_prepare: z is too narrow for the latent")
        _need_i32("slot_mapping", slot_mapping, n_tokens)
        row_width = pool.shape[3]
    rc = library.kernels().mgpt_latent_prepare(
        _ptr(z), _dtype_code(z), z.stride(0), int(q_off), n_head, head_dim, rot_dim, int(c_off), int(rank), _ptr(gain),
        float(eps), _ptr(positions), _ptr(freq), float(rot_magnitude), _ptr(pool), row_width, _ptr(slot_mapping), n_tokens,
        _stream())
    _check(rc, "latent_prepare")


def parallel_norm(x: torch.Tensor, y: Optional[torch.Tensor], mult: float, n_rows: int, gain: Optional[torch.Tensor] = None,
                  offset: float = 0.0, eps: float = 0.0, h: Optional[torch.Tensor] = None, hs: Optional[torch.Tensor] = None,
                  shift: Optional[torch.Tensor] = None, state: Optional[torch.Tensor] = None,
                  state_slots: Optional[torch.Tensor] = None, q_req: Optional[torch.Tensor] = None,
                  positions: Optional[torch.Tensor] = None) -> None:
    """x += mult * y and y = 0 (y float32 rows like x, or None); with h: h = x / sqrt(mean(x^2) + eps) * (offset + gain);
    with hs (only in a step whose requests bring one token each): hs = h + (kept - h) * shift with `kept` the
    request's row of `state` (zeros at position 0), which then takes h."""
    _need_cuda(x, y, gain, h, hs, shift, state, state_slots, q_req, positions)
    width = x.shape[1]
    for t in (x, y):
        _need(t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.shape[1] == width and t.shape[0] >= n_rows),
              "parallel_norm: x and y must be dense float32 rows of one width")
    dtype = 0
    if h is not None:
        _need(gain is not None and gain.dtype == torch.float32 and gain.is_contiguous() and gain.numel() == width,
              "parallel_norm: gain must be float32 [width]")
        for t in (h, hs):
            _need(t is None or (t.is_contiguous() and t.shape[1] == width and t.shape[0] >= n_rows and t.dtype == h.dtype),
                  "parallel_norm: h and hs must be dense rows as wide as x, of one dtype")
        dtype = _dtype_code(h)
    ld_state = 0
    if hs is not None:
        _need(h is not None, "parallel_norm: the shift reads h")
        ld_state = _need_shift_state(shift, state, state_slots, width)
        _need_i32("q_req", q_req, n_rows)
        _need_i32("positions", positions, n_rows)
    rc = library.kernels().mgpt_parallel_norm(
        _ptr(x), _ptr(y), float(mult), _ptr(gain), float(offset), float(eps), _ptr(h), _ptr(hs), dtype, _ptr(shift),
        _ptr(state), ld_state, _ptr(state_slots), _ptr(q_req), _ptr(positions), n_rows, width, _stream())
    _check(rc, "parallel_norm")


def _need_shift_state(shift, state, state_slots, width: int) -> int:
    _need(shift is not None and shift.dtype == torch.float32 and shift.is_contiguous() and shift.numel() == width,
          "token shift: shift must be float32 [width]")
    _need(state is not None and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= width, "token shift: the state pool must be float32 rows of at least the width")
    _need(state_slots is not None and state_slots.dtype == torch.int32 and state_slots.is_contiguous(),
          "token shift: state_slots must be int32")
    return state.stride(0)


def token_shift(h: torch.Tensor, hs: torch.Tensor, shift: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                q_req: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor, n_rows: int, n_req: int) -> None:
    """hs = h + (h_before - h) * shift for every token of the step, h_before being the row before (same request),
    the request's row of `state` for its first token of the step, zeros at position 0; then every request's row
    of `state` takes the h of its last token."""
    _need_cuda(h, hs, shift, state, state_slots, q_req, cu_q, positions)
    width = h.shape[1]
    _need(h.is_contiguous() and hs.is_contiguous() and hs.shape[1] == width and h.dtype == hs.dtype and h.shape[0] >= n_rows
          and hs.shape[0] >= n_rows, "token_shift: h and hs must be dense rows of one width and dtype")
    ld_state = _need_shift_state(shift, state, state_slots, width)
    _need_i32("q_req", q_req, n_rows)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("positions", positions, n_rows)
    _need(state_slots.numel() >= n_req, "token_shift: a state slot per request")
    lib = library.kernels()
    rc = lib.mgpt_token_shift(_ptr(h), _ptr(hs), _dtype_code(h), _ptr(shift), _ptr(state), ld_state, _ptr(state_slots),
                              _ptr(q_req), _ptr(cu_q), _ptr(positions), n_rows, width, _stream())
    _check(rc, "token_shift")
    rc = lib.mgpt_token_shift_keep(_ptr(h), _dtype_code(h), _ptr(state), ld_state, _ptr(state_slots), _ptr(cu_q), n_req,
                                   width, _stream())
    _check(rc, "token_shift_keep")


def xielu(z: torch.Tensor, out: torch.Tensor, coef: torch.Tensor, n_rows: int, hidden: int, fast: bool = False) -> None:
    """out = coef[0] z^2 + z / 2 where z > 0, coef[1] (exp(z) - 1 - z) + z / 2 elsewhere; coef float32 [2]."""
    _need_cuda(z, out, coef)
    _rows_2d("xielu z", z, n_rows)
    _rows_2d("xielu out", out, n_rows)
    _need(z.dtype == out.dtype and z.shape[1] >= hidden and out.shape[1] >= hidden, "xielu: rows of one dtype, at least `hidden` wide")
    _need(coef.dtype == torch.float32 and coef.is_contiguous() and coef.numel() == 2, "xielu: coef must be float32 [2]")
    rc = library.kernels().mgpt_xielu(_ptr(z), z.stride(0), _ptr(out), out.stride(0), _dtype_code(z), _ptr(coef), n_rows,
                                      hidden, int(fast), _stream())
    _check(rc, "xielu")


def heads_linear(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, n_rows: int,
                 gate: Optional[torch.Tensor] = None, fast: bool = False) -> None:
    """out[n][h] = a[n][h] @ w[h].T for every head h, optionally times sigmoid(gate[n][h]).
    w: [heads, n_out, k_dim]; a: [>=n_rows, >=heads * k_dim]; out, gate: [>=n_rows, >=heads * n_out]."""
    _need_cuda(a, w, out, gate)
    _need(w.dim() == 3 and w.is_contiguous(), "the heads' matrices must be dense [heads, out, in]")
    n_head, n_out, k_dim = w.shape
    _need(a.dtype == w.dtype == out.dtype and (gate is None or gate.dtype == a.dtype), "operands must share a dtype")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] >= n_head * k_dim and a.shape[0] >= n_rows,
          "activations must be [>=n_rows, >=heads * in] with unit inner stride")
    for name, t in (("out", out), ("gate", gate)):
        _need(t is None or (t.dim() == 2 and t.stride(1) == 1 and t.shape[1] >= n_head * n_out and t.shape[0] >= n_rows),
              f"{name} must be [>=n_rows, >=heads * out] with unit inner stride")
    ldg = 0 if gate is None else gate.stride(0)
    if fast and a.dtype == torch.bfloat16:
        # the MFMA kernel; it refuses sizes and alignments that its 16-byte loads do not take
        rc = library.kernels().mgpt_heads_linear_mfma(_ptr(a), a.stride(0), _ptr(w), _ptr(out), out.stride(0),
                                                      _ptr(gate), ldg, n_rows, n_head, n_out, k_dim, _stream())
        if rc != -2:
            _check(rc, "heads_linear_mfma")
            return
    rc = library.kernels().mgpt_heads_linear(_ptr(a), a.stride(0), _ptr(w), _ptr(out), out.stride(0), _ptr(gate),
                                             0 if gate is None else gate.stride(0), n_rows, n_head, n_out, k_dim,
                                             _dtype_code(a), int(fast), _stream())
    _check(rc, "heads_linear")


# ---------------------------------------------------------------- gated feed-forwards and experts
# slots a tile: 16 for the general kernel, 64 for the MFMA kernel of few rows, 256 for the tiled MFMA kernel
EXPERT_TILES = (16, 64, 256)
MAX_EXPERTS = 1024


GATE_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}


def gated_unit(z: torch.Tensor, act: torch.Tensor, n_rows: int, hidden: int, fast: bool = False,
               activation: str = "silu") -> None:
    """act[n][j] = f(z[n][j]) * z[n][hidden + j] with f = silu, relu or the tanh form of gelu."""
    _need(activation in GATE_ACTIVATIONS, f"gated unit: activation {activation!r} is none of {sorted(GATE_ACTIVATIONS)}")
    _need_cuda(z, act)
    _need(z.dtype == act.dtype and z.dim() == 2 and act.dim() == 2 and z.stride(1) == 1 and act.stride(1) == 1
          and z.shape[1] >= 2 * hidden and act.shape[1] >= hidden and z.shape[0] >= n_rows and act.shape[0] >= n_rows,
          "z must be [>=n_rows, >=2 * hidden] and act [>=n_rows, >=hidden], one dtype")
    rc = library.kernels().mgpt_gated_unit(_ptr(z), z.stride(0), _ptr(act), act.stride(0), n_rows, hidden,
                                           _dtype_code(z), int(fast), GATE_ACTIVATIONS[activation], _stream())
    _check(rc, "gated_unit")


def expert_slots(n_rows: int, top: int, n_experts: int, tile: int) -> int:
    """Slots that n_rows tokens with `top` experts each may need once every expert's run of slots is
    padded to whole tiles of `tile` slots."""
    pairs = n_rows * top
    worst = pairs + min(n_experts, pairs) * (tile - 1)
    return -(-worst // tile) * tile


def expert_route(ids: Optional[torch.Tensor], q_req: Optional[torch.Tensor], table: torch.Tensor, n_rows: int, n_experts: int,
                 slot_token: torch.Tensor, slot_pair: torch.Tensor, tile_expert: torch.Tensor, tile: int,
                 pair_slot: Optional[torch.Tensor] = None) -> None:
    """Sorts the (token, choice) pairs by expert into slots; see csrc/hip/experts.hip.  Token n's experts are
    row ids[n] of the table, or row n with ids None (a table made for this step, as a router's).  pair_slot
    ([n_rows * top], optional) receives the slot of every pair."""
    _need_cuda(ids, q_req, table, slot_token, slot_pair, tile_expert, pair_slot)
    _need(table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous(), "the table must be dense int32")
    _need(tile in EXPERT_TILES, f"tiles of {EXPERT_TILES} slots")
    top = table.shape[1]
    n_slots = expert_slots(n_rows, top, n_experts, tile)
    _need(n_experts <= MAX_EXPERTS, f"the route kernel takes up to {MAX_EXPERTS} experts")
    if ids is not None:
        _need_i32("ids", ids, n_rows)
    else:
        _need(table.shape[0] >= n_rows, "a table without ids has a row per token")
    if q_req is not None:
        _need_i32("q_req", q_req, n_rows)
    _need_i32("slot_token", slot_token, n_slots)
    _need_i32("slot_pair", slot_pair, n_slots)
    _need_i32("tile_expert", tile_expert, n_slots // tile)
    if pair_slot is not None:
        _need_i32("pair_slot", pair_slot, n_rows * top)
    rc = library.kernels().mgpt_expert_route(_ptr(ids), _ptr(q_req), _ptr(table), top, n_rows, n_experts,
                                             _ptr(slot_token), _ptr(slot_pair), _ptr(pair_slot), _ptr(tile_expert),
                                             n_slots, n_slots // tile, tile, _stream())
    _check(rc, "expert_route")


def grouped_linear(a: torch.Tensor, a_rows: Optional[torch.Tensor], w: torch.Tensor, tile_expert: torch.Tensor,
                   slot_token: torch.Tensor, out: torch.Tensor, out_rows: Optional[torch.Tensor], n_slots: int,
                   tile: int, fast: bool = False) -> None:
    """out[out_rows[s] or s] = a[a_rows[s] or s] @ w[expert of s's tile].T for every used slot s < n_slots.
    w: [experts, n_out, k_dim]."""
    _need_cuda(a, a_rows, w, tile_expert, slot_token, out, out_rows)
    _need(w.dim() == 3 and w.is_contiguous(), "the experts' matrices must be dense [experts, out, in]")
    _, n_out, k_dim = w.shape
    _need(tile in EXPERT_TILES and n_slots % tile == 0, "slots come in whole tiles")
    _need(a.dtype == w.dtype and a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim,
          "activations must be [rows, in] in the matrices' dtype")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == n_out, "out must be [rows, out]")
    _need(a_rows is not None or a.shape[0] >= n_slots, "activations have fewer rows than slots")
    _need(out_rows is not None or out.shape[0] >= n_slots, "out has fewer rows than slots")
    _need_i32("slot_token", slot_token, n_slots)
    _need_i32("tile_expert", tile_expert, n_slots // tile)
    for t in (a_rows, out_rows):
        if t is not None:
            _need_i32("row index", t, n_slots)
    if fast and tile in (16, 64) and a.dtype == torch.bfloat16:
        # the MFMA kernel; it refuses sizes and alignments that its 16-byte loads do not take
        rc = library.kernels().mgpt_grouped_linear_mfma(_ptr(a), a.stride(0), _ptr(a_rows), _ptr(w), w.stride(0),
                                                        _ptr(tile_expert), _ptr(slot_token), _ptr(out),
                                                        _dtype_code(out), out.stride(0), _ptr(out_rows),
                                                        n_slots // tile, tile, n_out, k_dim, _stream())
        if rc != -2:
            _check(rc, "grouped_linear_mfma")
            return
    rc = library.kernels().mgpt_grouped_linear(_ptr(a), a.stride(0), _ptr(a_rows), _ptr(w), w.stride(0),
                                               _ptr(tile_expert), _ptr(slot_token), _ptr(out), _dtype_code(out),
                                               out.stride(0), _ptr(out_rows), n_slots // tile, tile, n_out, k_dim,
                                               _dtype_code(a), _stream())
    _check(rc, "grouped_linear")


def expert_combine(pair_out: torch.Tensor, y: torch.Tensor, n_rows: int, top: int, weight: float,
                   pair_slot: Optional[torch.Tensor] = None, q_req: Optional[torch.Tensor] = None) -> None:
    """y[n] += weight * sum_k pair_out[pair_slot[n * top + k]] (without pair_slot: row n * top + k); both
    float32.  Tokens whose q_req is negative (padding) are left alone."""
    _need_cuda(pair_out, y, pair_slot, q_req)
    width = y.shape[1]
    _need_rows_f32("y", y, n_rows, width)
    if pair_slot is None:
        _need_rows_f32("pair_out", pair_out, n_rows * top, width)
    else:
        _need_rows_f32("pair_out", pair_out, 0, width)      # its rows are slots: the route kernel's bound holds
        _need_i32("pair_slot", pair_slot, n_rows * top)
    if q_req is not None:
        _need_i32("q_req", q_req, n_rows)
    rc = library.kernels().mgpt_expert_combine(_ptr(pair_out), _ptr(pair_slot), _ptr(q_req), _ptr(y), n_rows, width,
                                               top, float(weight), _stream())
    _check(rc, "expert_combine")


def gather_rows(src: torch.Tensor, slot_token: torch.Tensor, out: torch.Tensor, n_slots: int) -> bool:
    """out[s] = src[slot_token[s]] for every used slot s < n_slots (bfloat16 rows whose width is a
    multiple of 8).  False, with nothing launched, for other rows."""
    _need_cuda(src, slot_token, out)
    width = src.shape[1]
    if src.dtype != torch.bfloat16 or width % 8 or src.stride(0) % 8 or out.stride(0) % 8 \
            or src.data_ptr() % 16 or out.data_ptr() % 16:
        return False
    _need(out.dtype == src.dtype and out.dim() == 2 and out.shape[1] == width and out.shape[0] >= n_slots
          and src.stride(1) == 1 and out.stride(1) == 1, "out must be [>=n_slots, width] like src")
    _need_i32("slot_token", slot_token, n_slots)
    rc = library.kernels().mgpt_gather_rows(_ptr(src), src.stride(0), _ptr(slot_token), _ptr(out), out.stride(0),
                                            n_slots, width, _stream())
    _check(rc, "gather_rows")
    return True


ROUTER_SCORES = {"sigmoid": 0, "logit": 1}


def router_topk(h: torch.Tensor, w: torch.Tensor, n_rows: int, top: int, chosen: torch.Tensor, weight: torch.Tensor,
                q_req: Optional[torch.Tensor] = None, score: str = "sigmoid") -> None:
    """chosen[n] = the `top` experts with the largest w[e] . h[n] (float32 sums), best first; weight[n] = their
    scores (sigmoid of the sum, or the sum itself).  w: dense [experts, width]; chosen int32 and weight float32,
    dense [>= n_rows, top]."""
    _need_cuda(h, w, chosen, weight, q_req)
    _need(score in ROUTER_SCORES, f"router score {score!r} is none of {sorted(ROUTER_SCORES)}")
    _need(w.dim() == 2 and w.is_contiguous() and w.dtype in (torch.float32, torch.bfloat16), "the router's matrix must be dense")
    n_experts, width = w.shape
    _need(0 < top <= n_experts <= MAX_EXPERTS, f"top {top} of {n_experts} experts: need 0 < top <= experts <= {MAX_EXPERTS}")
    _rows_2d("router rows", h, n_rows)
    _need(h.shape[1] >= width, "the router's rows are narrower than its matrix")
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.dim() == 2 and chosen.shape[1] == top
          and chosen.shape[0] >= n_rows, "chosen must be dense int32 [>= n_rows, top]")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.shape == chosen.shape,
          "weight must be float32, shaped like chosen")
    if q_req is not None:
        _need_i32("q_req", q_req, n_rows)
    rc = library.kernels().mgpt_router_topk(_ptr(h), _dtype_code(h), h.stride(0), _ptr(w), _dtype_code(w), _ptr(q_req), n_rows,
                                            width, n_experts, top, ROUTER_SCORES[score], _ptr(chosen), _ptr(weight), _stream())
    _check(rc, "router_topk")


def gather_scale_rows(src: torch.Tensor, slot_token: torch.Tensor, slot_pair: torch.Tensor, pair_weight: torch.Tensor,
                      out: torch.Tensor, n_slots: int) -> None:
    """out[s] = pair_weight[slot_pair[s]] * src[slot_token[s]] for every used slot s < n_slots, the product in float32,
    rounded to the rows' dtype."""
    _need_cuda(src, slot_token, slot_pair, pair_weight, out)
    width = src.shape[1]
    _need(src.dim() == 2 and src.stride(1) == 1 and src.dtype in (torch.float32, torch.bfloat16), "rows must be float32 or bfloat16")
    _need(out.dtype == src.dtype and out.dim() == 2 and out.shape[1] == width and out.shape[0] >= n_slots
          and out.stride(1) == 1, "out must be [>= n_slots, width] like src")
    _need(pair_weight.dtype == torch.float32 and pair_weight.is_contiguous(), "pair weights must be dense float32")
    _need_i32("slot_token", slot_token, n_slots)
    _need_i32("slot_pair", slot_pair, n_slots)
    rc = library.kernels().mgpt_gather_scale_rows(_ptr(src), _dtype_code(src), src.stride(0), _ptr(slot_token), _ptr(slot_pair),
                                                  _ptr(pair_weight), _ptr(out), out.stride(0), n_slots, width, _stream())
    _check(rc, "gather_scale_rows")


def grouped_linear_tiled(a: torch.Tensor, w: torch.Tensor, tile_expert: torch.Tensor, slot_token: torch.Tensor,
                         out: torch.Tensor, n_slots: int) -> bool:
    """out[s] = a[s] @ w[expert of s's tile of 256].T for the slots of every tile in use, through the
    tiled MFMA kernel (bfloat16 operands, bfloat16 or float32 out).  False, with nothing launched,
    if that kernel does not take the sizes."""
    _need_cuda(a, w, tile_expert, slot_token, out)
    _need(w.dim() == 3 and w.is_contiguous(), "the experts' matrices must be dense [experts, out, in]")
    _, n_out, k_dim = w.shape
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or k_dim % 16 or a.stride(0) % 8 or n_slots % 256:
        return False
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_slots,
          "activations must be [>=n_slots, in]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == n_out and out.shape[0] >= n_slots,
          "out must be [>=n_slots, out]")
    _need_i32("slot_token", slot_token, n_slots)
    _need_i32("tile_expert", tile_expert, n_slots // 256)
    rc = library.kernels().mgpt_linear_mfma_grouped(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(tile_expert),
                                                    _ptr(slot_token), 256, _ptr(out), _dtype_code(out), out.stride(0),
                                                    n_slots, n_out, k_dim, _stream())
    if rc == -2:
        return False
    _check(rc, "linear_mfma_grouped")
    return True


# ---------------------------------------------------------------- root-mean-square norms, rotation, decaying state
RMS_GATES = {None: 0, "silu": 1, "sigmoid": 2, "silu_first": 3}


def _rows_2d(name: str, t: torch.Tensor, n_rows: int) -> None:
    _need(t.dim() == 2 and t.stride(1) == 1 and t.shape[0] >= n_rows and t.dtype in (torch.float32, torch.bfloat16),
          f"{name} must be float32 or bfloat16 rows [>= {n_rows}, ...] with unit column stride")


def rms_norm(x: torch.Tensor, gain: Optional[torch.Tensor], out: torch.Tensor, n_rows: int, eps: float, width: int,
             offset: float = 0.0, mult: float = 1.0, rows: Optional[torch.Tensor] = None, groups: int = 1,
             x_group_stride: Optional[int] = None, out_group_stride: Optional[int] = None,
             gate: Optional[torch.Tensor] = None, gate_act: Optional[str] = None, accumulate: bool = False,
             zero: Optional[torch.Tensor] = None) -> None:
    """out[i, g] = (out[i, g] +) mult * x[r, g] / sqrt(mean(x[r, g]^2) + eps) * (offset + gain[g]) (* act(gate[i, g]))
    with r = rows[i] or i; with gate_act "silu_first" the gate acts in front of the norm instead: x * silu(gate)
    takes x's place and nothing follows the gain.  A row holds `groups` segments of `width` values,
    x_group_stride / out_group_stride apart (default: width).  gain: float32 [groups * width] or None.  gate: laid out like out.  zero: float32 rows
    that are cleared on the way (row i for every i)."""
    _need_cuda(x, gain, out, rows, gate, zero)
    xs = width if x_group_stride is None else int(x_group_stride)
    os_ = width if out_group_stride is None else int(out_group_stride)
    _rows_2d("rms_norm out", out, n_rows)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.dtype in (torch.float32, torch.bfloat16), "rms_norm input must be rows")
    _need(groups >= 1 and width >= 1 and xs >= width and os_ >= width, "rms_norm: segments overlap")
    _need(x.shape[1] >= (groups - 1) * xs + width and out.shape[1] >= (groups - 1) * os_ + width,
          "rms_norm: a row is shorter than its segments")
    _need(gain is None or (gain.dtype == torch.float32 and gain.is_contiguous() and gain.numel() == groups * width),
          "rms_norm gain must be float32 [groups * width]")
    if rows is None:
        _need(x.shape[0] >= n_rows, "rms_norm input has fewer rows than asked for")
    else:
        _need_i32("rows", rows, n_rows)
    if gate is not None:
        _rows_2d("rms_norm gate", gate, n_rows)
        _need(gate.shape[1] >= (groups - 1) * os_ + width and gate_act in RMS_GATES, "rms_norm gate: too narrow, or unknown activation")
    zero_width = 0
    if zero is not None:
        _need(zero.dtype == torch.float32 and zero.dim() == 2 and zero.stride(1) == 1 and zero.shape[0] >= n_rows,
              "rms_norm: the buffer to clear must be float32 rows")
        zero_width = zero.shape[1]
    rc = library.kernels().mgpt_rms_norm(
        _ptr(x), _dtype_code(x), x.stride(0), _ptr(rows), _ptr(gain), float(offset), float(eps), float(mult),
        _ptr(gate), _dtype_code(gate) if gate is not None else 0, gate.stride(0) if gate is not None else 0,
        RMS_GATES[gate_act if gate is not None else None], _ptr(out), _dtype_code(out), out.stride(0), int(accumulate),
        _ptr(zero), zero.stride(0) if zero is not None else 0, zero_width, n_rows, groups, xs, os_, width, _stream())
    _check(rc, "rms_norm")


MAX_NORM_BRANCHES = 4


def rms_post_norm(branches, x: torch.Tensor, gain_post: torch.Tensor, n_rows: int, eps: float, offset: float,
                  mult: float, gain_next: Optional[torch.Tensor] = None, h: Optional[torch.Tensor] = None,
                  join_unit: bool = True, scale_post: Optional[torch.Tensor] = None) -> None:
    """branches: [(y float32 [rows, width], gain float32 [width] or None), ...].  With several branches
    y = mean_b unit(y_b) * gain_b (join_unit False: y = sum_b y_b * gain_b, a weighted sum), else y = y_0;
    x += mult * unit(y) * (offset + gain_post) (* scale_post, float32 [width]); with gain_next
    h = unit(x) * (offset + gain_next); every y_b is cleared.  unit(v) = v / sqrt(mean(v^2) + eps)."""
    nb = len(branches)
    _need(1 <= nb <= MAX_NORM_BRANCHES, f"rms_post_norm takes 1 to {MAX_NORM_BRANCHES} branches")
    width = x.shape[1]
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[0] >= n_rows, "rms_post_norm: x must be dense float32 rows")
    ys, gs = [], []
    for y, g in branches:
        _need_cuda(y, g)
        _need(y.dtype == torch.float32 and y.is_contiguous() and y.shape[1] == width and y.shape[0] >= n_rows,
              "rms_post_norm: a branch must be dense float32 rows as wide as x")
        _need(nb == 1 or (g is not None and g.dtype == torch.float32 and g.numel() == width and g.is_contiguous()),
              "rms_post_norm: several branches need a float32 gain each")
        ys.append(_ptr(y))
        gs.append(_ptr(g) if nb > 1 else None)
    ys += [None] * (MAX_NORM_BRANCHES - nb)
    gs += [None] * (MAX_NORM_BRANCHES - nb)
    for g in (gain_post, gain_next, scale_post):
        _need(g is None or (g.dtype == torch.float32 and g.numel() == width and g.is_contiguous()), "rms_post_norm: gains are float32 [width]")
    _need(gain_post is not None, "rms_post_norm needs the gain of the norm behind the sublayer")
    if gain_next is not None:
        _need(h is not None and h.is_contiguous() and h.shape[1] == width and h.shape[0] >= n_rows
              and h.dtype in (torch.float32, torch.bfloat16), "rms_post_norm: h must be dense rows as wide as x")
    _need_cuda(x, gain_post, gain_next, h, scale_post)
    rc = library.kernels().mgpt_rms_post_norm(
        *ys, *gs, nb, 1.0 / nb if join_unit else 1.0, int(join_unit), _ptr(x), _ptr(gain_post), _ptr(scale_post),
        float(offset), float(eps), float(mult), _ptr(gain_next),
        _ptr(h) if gain_next is not None else None, _dtype_code(h) if gain_next is not None else 0, n_rows, width, _stream())
    _check(rc, "rms_post_norm")


QK_NORMS = {None: 0, "head": 1, "whole": 2}


def qk_prepare(z: torch.Tensor, q_off: int, k_off: int, v_off: int, n_head: int, n_kv_head: int, head_dim: int,
               value_dim: int, head_stride: int, n_tokens: int, positions: Optional[torch.Tensor] = None,
               freq: Optional[torch.Tensor] = None, norm_eps: Optional[float] = None,
               mix_lambda: Optional[torch.Tensor] = None, v_other: Optional[torch.Tensor] = None, mix_mode: int = 0,
               k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
               slot_mapping: Optional[torch.Tensor] = None, norm: Optional[str] = None,
               q_norm_weight: Optional[torch.Tensor] = None, k_norm_weight: Optional[torch.Tensor] = None,
               values_from_keys: bool = False, rot_magnitude: float = 1.0) -> None:
    """Projected queries, keys and values of a step's tokens (rows of z; q heads at q_off, k heads at k_off, v heads
    at v_off, head_stride channels apart) made ready for attention: q and k rotated by position with the float32
    frequencies `freq` [rot_dims / 2] (pairs (i, i + rot_dims / 2)), then divided by their root mean square over
    head_dim channels if norm_eps is given; v kept for other layers in v_other (heads value_dim apart; mix_mode 1) or mixed with what
    lies there, (1 - lambda) v + lambda v_other (mix_mode 2); q back in place, k and v into their pages.
    norm "head" / "whole" (with norm_eps and float32 weights [head_dim] / [heads * head_dim] for q and for k): an RMS
    norm with weights *before* the rotation, head by head with the heads sharing a weight vector, or over all of a
    token's query (key) channels at once.  values_from_keys: the values are the keys as projected, z holds none.
    rot_magnitude multiplies every cosine and sine."""
    _need_cuda(z, positions, freq, mix_lambda, v_other, k_pool, v_pool, slot_mapping, q_norm_weight, k_norm_weight)
    _need(norm in QK_NORMS, f"qk_prepare: norm {norm!r} is none of {sorted(QK_NORMS, key=str)}")
    if norm is not None:
        for w, heads in ((q_norm_weight, n_head), (k_norm_weight, n_kv_head)):
            _need(norm_eps is not None and w is not None and w.dtype == torch.float32 and w.is_contiguous()
                  and w.numel() == (head_dim if norm == "head" else heads * head_dim),
                  "qk_prepare: a norm with weights needs eps and float32 weights of the head's (or the projection's) size")
    _need(not values_from_keys or (value_dim == head_dim and mix_mode == 0), "qk_prepare: values that are the keys have their size")
    _rows_2d("qk_prepare z", z, n_tokens)
    rot_dims = 0
    if freq is not None:
        _need(freq.dtype == torch.float32 and freq.is_contiguous() and positions is not None, "rotation needs float32 frequencies and positions")
        _need_i32("positions", positions, n_tokens)
        rot_dims = 2 * freq.numel()
    kv_span = (n_kv_head - 1) * head_stride
    _need(z.shape[1] >= max(q_off + (n_head - 1) * head_stride + head_dim, k_off + kv_span + head_dim,
                            v_off + kv_span + head_stride if k_pool is not None and not values_from_keys else 0),
          "qk_prepare: z is too narrow")
    page_size = 0
    if k_pool is not None:
        _need(v_pool is not None and k_pool.dtype == z.dtype and v_pool.dtype == z.dtype and k_pool.dim() == 4
              and k_pool.shape[1] == n_kv_head and k_pool.shape[3] == head_stride and k_pool.is_contiguous()
              and v_pool.shape == k_pool.shape and v_pool.is_contiguous(),
              "qk_prepare: pools must be [pages, kv heads, page, head stride] in z's dtype")
        _need_i32("slot_mapping", slot_mapping, n_tokens)
        page_size = k_pool.shape[2]
    if mix_mode:
        _need(v_other is not None and v_other.dtype == z.dtype and v_other.dim() == 2 and v_other.stride(1) == 1
              and v_other.shape[0] >= n_tokens and v_other.shape[1] >= n_kv_head * value_dim,
              "qk_prepare: the shared values must be rows of all kv heads in z's dtype")
        _need(mix_mode == 1 or (mix_lambda is not None and mix_lambda.dtype == torch.float32 and mix_lambda.numel() >= 1),
              "qk_prepare: mixing needs a float32 lambda")
    rc = library.kernels().mgpt_qk_prepare(
        _ptr(z), _dtype_code(z), z.stride(0), q_off, k_off, v_off, n_head, n_kv_head, head_dim, value_dim, head_stride,
        _ptr(positions), _ptr(freq), rot_dims, -1.0 if norm_eps is None else float(norm_eps), _ptr(mix_lambda),
        _ptr(v_other), v_other.stride(0) if v_other is not None else 0, int(mix_mode), _ptr(k_pool), _ptr(v_pool),
        _ptr(slot_mapping), page_size, n_tokens, QK_NORMS[norm], _ptr(q_norm_weight) if norm else None,
        _ptr(k_norm_weight) if norm else None, int(values_from_keys), float(rot_magnitude), _stream())
    _check(rc, "qk_prepare")


def decay_state(z: torch.Tensor, q_off: int, k_off: int, v_off: int, g_off: int, n_head: int, head_dim: int,
                value_dim: int, decay: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                n_req: int, positions: torch.Tensor, out: torch.Tensor, silu_inputs: bool = False,
                freq: Optional[torch.Tensor] = None, k_scale: float = 1.0, norm_eps: Optional[float] = None) -> None:
    """Per request and head the state S [head_dim, value_dim] (float32, in the request's slot of `state`, zero
    before position 0) goes over the request's tokens of this step: S = decay_h S + k v^T, o = S^T q.  q, k, v
    (and a gate at g_off, -1 for none) are columns of z's rows; silu_inputs passes them through silu first; freq
    rotates q and k by position; k is multiplied by k_scale.  out[n, h] = o (divided by its root mean square with
    norm_eps given, times silu(gate) with a gate), float32 or z's dtype."""
    _need_cuda(z, decay, state, state_slots, cu_q, positions, out, freq)
    n_tokens = 0
    _rows_2d("decay_state z", z, n_tokens)
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_head * value_dim
          and out.dtype in (torch.float32, torch.bfloat16), "decay_state: out must be rows of all heads' values")
    _need(z.shape[1] >= max(q_off, k_off) + n_head * head_dim and z.shape[1] >= max(v_off, g_off) + n_head * value_dim,
          "decay_state: z is too narrow")
    _need(decay.dtype == torch.float32 and decay.numel() == n_head, "decay_state: one float32 decay per head")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
          and state.shape[1] == n_head * head_dim * value_dim, "decay_state: state must be [slots, heads * dim * vdim] float32")
    _need_i32("state_slots", state_slots, n_req)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need(positions.dtype == torch.int32 and positions.is_contiguous(), "positions must be int32")
    _need(0 < head_dim <= 256 and 0 < value_dim <= 256, "decay_state takes head sizes up to 256")
    rot_dims = 0
    if freq is not None:
        _need(freq.dtype == torch.float32 and freq.is_contiguous() and 2 * freq.numel() <= head_dim, "decay_state: bad frequencies")
        rot_dims = 2 * freq.numel()
    rc = library.kernels().mgpt_decay_state(
        _ptr(z), _dtype_code(z), z.stride(0), q_off, k_off, v_off, g_off, n_head, head_dim, value_dim, int(silu_inputs),
        _ptr(positions), _ptr(freq), rot_dims, float(k_scale), _ptr(decay), _ptr(state), _ptr(state_slots), _ptr(cu_q),
        n_req, -1.0 if norm_eps is None else float(norm_eps), _ptr(out), _dtype_code(out), out.stride(0), _stream())
    _check(rc, "decay_state")


CHUNKED_STATE_MAX_DIM = 128     # largest head size that the chunked form of the decaying state takes


def decay_state_chunked(z: torch.Tensor, q_off: int, k_off: int, v_off: int, n_head: int, head_dim: int, value_dim: int,
                        decay: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                        n_req: int, n_tokens: int, positions: torch.Tensor, qk: torch.Tensor, out: torch.Tensor,
                        silu_inputs: bool = False, freq: Optional[torch.Tensor] = None, k_scale: float = 1.0) -> bool:
    """decay_state for steps with prompt portions: the recurrence 32 tokens at a time as float32 matrix products.
    out: float32 rows, the heads' raw outputs (no norm, no gate); qk: float32 scratch [>= n_tokens, 2 * heads * dim].
    False, with nothing launched, for head sizes beyond CHUNKED_STATE_MAX_DIM."""
    if head_dim > CHUNKED_STATE_MAX_DIM:
        return False
    _need_cuda(z, decay, state, state_slots, cu_q, positions, out, freq, qk)
    _rows_2d("decay_state z", z, n_tokens)
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] >= n_tokens
          and out.shape[1] >= n_head * value_dim, "decay_state_chunked: out must be float32 rows of all heads' values")
    _need(qk.dtype == torch.float32 and qk.is_contiguous() and qk.shape[0] >= n_tokens
          and qk.shape[1] == 2 * n_head * head_dim, "decay_state_chunked: qk must be float32 [tokens, 2 * heads * dim]")
    _need(z.shape[1] >= max(q_off, k_off) + n_head * head_dim and z.shape[1] >= v_off + n_head * value_dim,
          "decay_state_chunked: z is too narrow")
    _need(decay.dtype == torch.float32 and decay.numel() == n_head, "decay_state: one float32 decay per head")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
          and state.shape[1] == n_head * head_dim * value_dim, "decay_state: state must be [slots, heads * dim * vdim] float32")
    _need_i32("state_slots", state_slots, n_req)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("positions", positions, n_tokens)
    _need(0 < value_dim <= 256, "decay_state takes value sizes up to 256")
    rot_dims = 0
    if freq is not None:
        _need(freq.dtype == torch.float32 and freq.is_contiguous() and 2 * freq.numel() <= head_dim, "decay_state: bad frequencies")
        rot_dims = 2 * freq.numel()
    rc = library.kernels().mgpt_decay_state_chunked(
        _ptr(z), _dtype_code(z), z.stride(0), q_off, k_off, v_off, n_head, head_dim, value_dim, int(silu_inputs),
        _ptr(positions), _ptr(freq), rot_dims, float(k_scale), _ptr(decay), _ptr(state), _ptr(state_slots), _ptr(cu_q),
        n_req, n_tokens, _ptr(qk), _ptr(out), out.stride(0), _stream())
    _check(rc, "decay_state_chunked", 2)
    return True


GATED_STATE_MODES = {"channel_sigmoid": 0, "head_softplus": 1}


def gated_state(z: torch.Tensor, q_off: int, k_off: int, v_off: int, n_head: int, n_group: int, head_dim: int,
                value_dim: int, a: torch.Tensor, a_off: int, mode: str, state: torch.Tensor, state_slots: torch.Tensor,
                cu_q: torch.Tensor, n_req: int, positions: torch.Tensor, out: torch.Tensor, q_scale: float = 1.0,
                tau: float = 1.0, dt_bias: Optional[torch.Tensor] = None, a_log: Optional[torch.Tensor] = None,
                skip: Optional[torch.Tensor] = None) -> None:
    """Per request and head the state S [head_dim, value_dim] (float32, in the request's slot of `state`, zero before
    position 0) goes over the request's tokens of this step: S = diag(decay_t) S + k v^T, o = S^T q (+ skip_h v).
    q and k (n_group groups that heads share in turn) and v (per head) are columns of z's rows.  The decay comes
    from columns of a's rows at a_off: mode "channel_sigmoid": sigmoid(a[h][d])^(1/tau) per key channel, and q
    times q_scale; mode "head_softplus": dt = softplus(a[h] + dt_bias[h]), decay exp(-exp(a_log[h]) dt) for the
    whole head, and k times dt.  state: float32 rows (a view of a pool's columns will do) of heads * dim * vdim
    values; out: float32 rows of all heads' values."""
    _need_cuda(z, a, state, state_slots, cu_q, positions, out, dt_bias, a_log, skip)
    _need(mode in GATED_STATE_MODES, f"gated_state: mode {mode!r} is none of {sorted(GATED_STATE_MODES)}")
    _rows_2d("gated_state z", z, 0)
    _rows_2d("gated_state a", a, 0)
    _need(n_head % n_group == 0, "gated_state: heads must be a multiple of groups")
    _need(z.shape[1] >= max(q_off, k_off) + n_group * head_dim and z.shape[1] >= v_off + n_head * value_dim,
          "gated_state: z is too narrow")
    _need(a.shape[1] >= a_off + (n_head * head_dim if mode == "channel_sigmoid" else n_head), "gated_state: a is too narrow")
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_head * value_dim,
          "gated_state: out must be float32 rows of all heads' values")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] == n_head * head_dim * value_dim, "gated_state: state must be float32 rows of heads * dim * vdim")
    for name, t in (("dt_bias", dt_bias), ("a_log", a_log), ("skip", skip)):
        _need(t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n_head),
              f"gated_state: {name} must be float32 [heads]")
    _need(mode != "head_softplus" or (dt_bias is not None and a_log is not None), "gated_state: this mode needs dt_bias and a_log")
    _need(0 < head_dim <= 256 and 0 < value_dim <= 256 and tau > 0.0, "gated_state takes head sizes up to 256")
    _need_i32("state_slots", state_slots, n_req)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need(positions.dtype == torch.int32 and positions.is_contiguous(), "positions must be int32")
    rc = library.kernels().mgpt_gated_state(
        _ptr(z), _dtype_code(z), z.stride(0), q_off, k_off, v_off, n_head, n_group, head_dim, value_dim, _ptr(a),
        _dtype_code(a), a.stride(0), a_off, GATED_STATE_MODES[mode], float(q_scale), 1.0 / float(tau), _ptr(dt_bias),
        _ptr(a_log), _ptr(skip), _ptr(state), state.stride(0), _ptr(state_slots), _ptr(cu_q), n_req, _ptr(positions),
        _ptr(out), out.stride(0), _stream())
    _check(rc, "gated_state")


def gated_state_chunked(z: torch.Tensor, q_off: int, k_off: int, v_off: int, n_head: int, n_group: int, head_dim: int,
                        value_dim: int, a: torch.Tensor, a_off: int, mode: str, state: torch.Tensor,
                        state_slots: torch.Tensor, cu_q: torch.Tensor, n_req: int, n_tokens: int, positions: torch.Tensor,
                        qkg: torch.Tensor, out: torch.Tensor, q_scale: float = 1.0, tau: float = 1.0,
                        dt_bias: Optional[torch.Tensor] = None, a_log: Optional[torch.Tensor] = None,
                        skip: Optional[torch.Tensor] = None) -> bool:
    """gated_state for steps with prompt portions: the recurrence 32 tokens at a time as float32 matrix products,
    the decays between a chunk's tokens from sums of their logarithms.  qkg: float32 scratch [>= n_tokens,
    3 * heads * dim].  False, with nothing launched, for head sizes beyond CHUNKED_STATE_MAX_DIM."""
    if head_dim > CHUNKED_STATE_MAX_DIM:
        return False
    _need_cuda(z, a, state, state_slots, cu_q, positions, out, qkg, dt_bias, a_log, skip)
    _need(mode in GATED_STATE_MODES, f"gated_state: mode {mode!r} is none of {sorted(GATED_STATE_MODES)}")
    _rows_2d("gated_state z", z, n_tokens)
    _rows_2d("gated_state a", a, n_tokens)
    _need(n_head % n_group == 0, "gated_state: heads must be a multiple of groups")
    _need(z.shape[1] >= max(q_off, k_off) + n_group * head_dim and z.shape[1] >= v_off + n_head * value_dim,
          "gated_state: z is too narrow")
    _need(a.shape[1] >= a_off + (n_head * head_dim if mode == "channel_sigmoid" else n_head), "gated_state: a is too narrow")
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] >= n_tokens
          and out.shape[1] >= n_head * value_dim, "gated_state: out must be float32 rows of all heads' values")
    _need(qkg.dtype == torch.float32 and qkg.is_contiguous() and qkg.dim() == 2 and qkg.shape[0] >= n_tokens
          and qkg.shape[1] == 3 * n_head * head_dim, "gated_state_chunked: qkg must be float32 [tokens, 3 * heads * dim]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] == n_head * head_dim * value_dim, "gated_state: state must be float32 rows of heads * dim * vdim")
    for name, t in (("dt_bias", dt_bias), ("a_log", a_log), ("skip", skip)):
        _need(t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n_head),
              f"gated_state: {name} must be float32 [heads]")
    _need(mode != "head_softplus" or (dt_bias is not None and a_log is not None), "gated_state: this mode needs dt_bias and a_log")
    _need(0 < value_dim <= 256 and tau > 0.0, "gated_state takes value sizes up to 256")
    _need_i32("state_slots", state_slots, n_req)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("positions", positions, n_tokens)
    rc = library.kernels().mgpt_gated_state_chunked(
        _ptr(z), _dtype_code(z), z.stride(0), q_off, k_off, v_off, n_head, n_group, head_dim, value_dim, _ptr(a),
        _dtype_code(a), a.stride(0), a_off, GATED_STATE_MODES[mode], float(q_scale), 1.0 / float(tau), _ptr(dt_bias),
        _ptr(a_log), _ptr(skip), _ptr(state), state.stride(0), _ptr(state_slots), _ptr(cu_q), n_req, n_tokens,
        _ptr(positions), _ptr(qkg), _ptr(out), out.stride(0), _stream())
    _check(rc, "gated_state_chunked", 2)
    return True


MAX_CONV_TAPS = 9
CONV_ACTIVATIONS = {None: 0, "silu": 1}


def short_conv(u: torch.Tensor, u_off: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
               state_slots: torch.Tensor, cu_q: torch.Tensor, q_req: torch.Tensor, positions: torch.Tensor, n_req: int,
               out: torch.Tensor, o_off: int, n_tokens: int, activation: Optional[str] = None) -> None:
    """out[t][o_off + c] = act(sum_j weight[c][j] * u_(t - taps + 1 + j)[u_off + c] (+ bias[c])) over time inside each
    request, zeros before position 0; the taps - 1 inputs before the step's first token come from the request's
    slot of `state` (float32 rows holding [taps - 1][channels], a view of a pool's columns will do), which is then
    brought up to date.  weight: float32 [channels, taps]."""
    _need_cuda(u, weight, bias, state, state_slots, cu_q, q_req, positions, out)
    _need(activation in CONV_ACTIVATIONS, f"short_conv: activation {activation!r} is none of {sorted(map(str, CONV_ACTIVATIONS))}")
    _need(weight.dtype == torch.float32 and weight.dim() == 2 and weight.is_contiguous(), "short_conv: weight must be dense float32 [channels, taps]")
    channels, taps = weight.shape
    _need(1 <= taps <= MAX_CONV_TAPS, f"short_conv takes 1 to {MAX_CONV_TAPS} taps")
    _need(bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == channels),
          "short_conv: bias must be float32 [channels]")
    _rows_2d("short_conv input", u, n_tokens)
    _rows_2d("short_conv output", out, n_tokens)
    _need(u.shape[1] >= u_off + channels and out.shape[1] >= o_off + channels, "short_conv: rows are too narrow")
    _need(u.data_ptr() != out.data_ptr(), "short_conv: the output cannot be the input's buffer")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= (taps - 1) * channels, "short_conv: state must be float32 rows of (taps - 1) * channels")
    _need_i32("state_slots", state_slots, n_req)
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("q_req", q_req, n_tokens)
    _need_i32("positions", positions, n_tokens)
    rc = library.kernels().mgpt_short_conv(
        _ptr(u), _dtype_code(u), u.stride(0), u_off, _ptr(weight), _ptr(bias), CONV_ACTIVATIONS[activation], _ptr(state),
        state.stride(0), _ptr(state_slots), _ptr(cu_q), _ptr(q_req), _ptr(positions), n_req, _ptr(out), _dtype_code(out),
        out.stride(0), o_off, n_tokens, channels, taps, _stream())
    _check(rc, "short_conv", 2 if taps > 1 else 1)
