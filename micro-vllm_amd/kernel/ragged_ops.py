"""Ops of layer stacks with an fp32 residual stream over a ragged step (csrc/linear_any.hip,
stream_ops.hip, seq_mix.hip): thin wrappers that check shapes on the host and pass pointers and row
strides.  Two-dimensional operands may be column slices of wider buffers (`buf[:, a:b]`): only the
last stride has to be 1.  `f32` everywhere means "the activation type is fp32" and is read off the
operand that carries it.

No counterpart in the reference, whose only model family is the Llama-shaped one.
"""
from typing import Optional

import torch

from .. import _native as nv
from .linear import StreamedWeight, gemm_prefill, wgemm

SCAN_SEQ_MAX = 16   # rows up to this length are not in a step's chunk table (core/state_cache.py): they take the
                    # token-by-token recurrence and the one-workgroup-per-token attention


def _ld(t: torch.Tensor) -> int:
    assert t.dim() == 2 and t.stride(1) == 1
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], t.stride(0))


def _f32(t):
    assert t.is_cuda and t.dtype == torch.float32, "fp32 device tensor expected"
    return t


def _i32(t):
    assert t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()
    return t


def _is_f32(t) -> int:
    assert t.dtype in (torch.float32, torch.bfloat16)
    return int(t.dtype == torch.float32)


class AnyLinear:
    """y = x W^T with fp32 output for a [N,K] weight of any shape.  bf16 weights whose shape the
    wave-tile projections take (N % 16 == 0, K % 64 == 0) are relaid out for them (mv_wgemm up to 64
    rows, mv_gemm_prefill above); every other shape, and fp32, runs mv_linear_any on the plain
    row-major weight."""

    def __init__(self, w: torch.Tensor, wave_tiles: bool = True):
        assert w.is_cuda and w.dim() == 2 and w.dtype in (torch.bfloat16, torch.float32)
        self.n, self.k = w.shape
        self.f32 = w.dtype == torch.float32
        self.tiles: Optional[StreamedWeight] = None
        self.w = None
        if wave_tiles and not self.f32 and self.n % 16 == 0 and self.k % 64 == 0:
            self.tiles = StreamedWeight.from_linear(w)
        else:
            self.w = w.contiguous()

    @property
    def nbytes(self):
        return self.n * self.k * (4 if self.f32 else 2)

    def __call__(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        m = x.shape[0]
        assert x.is_cuda and x.dim() == 2 and x.shape[1] == self.k and x.stride(1) == 1
        assert x.dtype == (torch.float32 if self.f32 else torch.bfloat16)
        if out is None:
            out = torch.empty(m, self.n, dtype=torch.float32, device=x.device)
        assert out.shape == (m, self.n) and out.dtype == torch.float32 and out.stride(1) == 1
        if m == 0:
            return out
        if self.tiles is not None:
            return wgemm(x, self.tiles, out) if m <= 64 else gemm_prefill(x, self.tiles, out)
        nv.check("mv_linear_any", nv.lib().mv_linear_any(
            x.data_ptr(), _ld(x), self.w.data_ptr(), self.k, out.data_ptr(), _ld(out), m, self.n, self.k,
            int(self.f32), nv.stream_ptr()))
        return out


def embed_scaled(table, ids, scale: float, x, h):
    rows, n = x.shape
    assert table.is_cuda and table.is_contiguous() and table.shape[1] == n and h.shape == x.shape
    assert table.dtype == h.dtype and ids.numel() == rows
    nv.check("mv_embed_scaled", nv.lib().mv_embed_scaled(
        table.data_ptr(), _i32(ids).data_ptr(), _f32(x).data_ptr(), _ld(x), h.data_ptr(), _ld(h), rows, n,
        table.shape[0], float(scale), _is_f32(h), nv.stream_ptr()))


def postnorm_residual(y1, w, eps: float, x, h, y2=None, s1: float = 1.0, s2: float = 0.0):
    """x += unit_rms(s1*y1 + s2*y2) * (1 + w); h = x in the activation type."""
    rows, n = x.shape
    assert y1.shape == (rows, n) and h.shape == (rows, n) and w.numel() == n and w.is_contiguous()
    assert y2 is None or y2.shape == (rows, n)
    nv.check("mv_postnorm_residual", nv.lib().mv_postnorm_residual(
        _f32(y1).data_ptr(), _ld(y1), None if y2 is None else _f32(y2).data_ptr(), 0 if y2 is None else _ld(y2),
        float(s1), float(s2), _f32(w).data_ptr(), float(eps), _f32(x).data_ptr(), _ld(x), h.data_ptr(), _ld(h),
        rows, n, _is_f32(h), nv.stream_ptr()))


def offset_rmsnorm_gather(x, idx, w, eps: float, out):
    rows, n = out.shape
    assert x.shape[1] == n and w.numel() == n and w.is_contiguous()
    assert idx is None or idx.numel() == rows
    nv.check("mv_offset_rmsnorm_gather", nv.lib().mv_offset_rmsnorm_gather(
        _f32(x).data_ptr(), _ld(x), None if idx is None else _i32(idx).data_ptr(), _f32(w).data_ptr(), float(eps),
        out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def relu_squared(v, out):
    rows, n = v.shape
    assert out.shape == (rows, n)
    nv.check("mv_relu_squared", nv.lib().mv_relu_squared(
        _f32(v).data_ptr(), _ld(v), out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def softcap_(v, cap: float):
    assert v.is_contiguous()
    nv.check("mv_softcap", nv.lib().mv_softcap(_f32(v).data_ptr(), v.numel(), float(cap), nv.stream_ptr()))
    return v


def conv_silu(inp, state, w, bias, out, step):
    """inp [T,C] (a column slice), state [slots, taps-1, C] fp32, w [C,taps] fp32."""
    tokens, ch = inp.shape
    taps = w.shape[1]
    assert w.shape == (ch, taps) and w.is_contiguous() and out.shape == (tokens, ch)
    assert state.is_contiguous() and state.shape[1:] == (max(taps - 1, 0), ch)
    assert bias is None or (bias.numel() == ch and bias.is_contiguous())
    assert step.tokens == tokens and int(step.max_slot) < state.shape[0]
    nv.check("mv_conv_silu", nv.lib().mv_conv_silu(
        _f32(inp).data_ptr(), _ld(inp), _f32(state).data_ptr(), _f32(w).data_ptr(),
        None if bias is None else _f32(bias).data_ptr(), _f32(out).data_ptr(), _ld(out),
        step.tok_row.data_ptr(), step.row_start.data_ptr(), step.row_len.data_ptr(), step.row_ctx.data_ptr(),
        step.row_slot.data_ptr(), tokens, step.rows, ch, taps, nv.stream_ptr()))


def softplus_decay(raw, dt_bias, a_log, gain, decay, log_decay=None):
    tokens, heads = raw.shape
    assert gain.shape == (tokens, heads) and decay.shape == (tokens, heads)
    assert gain.is_contiguous() and decay.is_contiguous() and dt_bias.numel() == heads and a_log.numel() == heads
    assert log_decay is None or (log_decay.shape == (tokens, heads) and log_decay.is_contiguous())
    nv.check("mv_softplus_decay", nv.lib().mv_softplus_decay(
        _f32(raw).data_ptr(), _ld(raw), _f32(dt_bias).data_ptr(), _f32(a_log).data_ptr(), _f32(gain).data_ptr(),
        _f32(decay).data_ptr(), None if log_decay is None else _f32(log_decay).data_ptr(), tokens, heads,
        nv.stream_ptr()))


def scan_outer(q, k, v, decay, gain, skip, state, out, step, heads: int, n: int, p: int, q_div: int = 1,
               k_div: int = 1, log_decay=None, chunked: bool = True):
    """state [slots, heads, n, p] fp32; q [T, heads/q_div * n], k [T, heads/k_div * n], v and out
    [T, heads * p]; decay [T, heads] or [heads] (the same for every token); gain [T, heads] or None.
    Rows of up to SCAN_SEQ_MAX tokens run token by token; with `log_decay` (the decay's logarithm, shaped
    like it) longer rows run in chunks of 64 (mv_scan_chunked) unless `chunked` is False or the head
    shape does not fit a workgroup's LDS."""
    tokens = v.shape[0]
    assert q.shape == (tokens, heads // q_div * n) and k.shape == (tokens, heads // k_div * n)
    assert v.shape == (tokens, heads * p) and out.shape == (tokens, heads * p)
    assert state.is_contiguous() and state.shape[1:] == (heads, n, p) and int(step.max_slot) < state.shape[0]
    assert step.tokens == tokens
    if decay.dim() == 1:
        assert decay.numel() == heads and decay.is_contiguous()
        ld_decay = 0
    else:
        assert decay.shape == (tokens, heads)
        ld_decay = _ld(decay)
    assert gain is None or gain.shape == (tokens, heads)
    assert skip is None or (skip.numel() == heads and skip.is_contiguous())
    L = nv.lib()
    use_chunks = (chunked and log_decay is not None and step.n_chunks > 0
                  and L.mv_scan_chunked_lds_bytes(n, p) <= 150 * 1024)
    if use_chunks:
        assert log_decay.shape == decay.shape and log_decay.stride(-1) == 1
        dev = v.device
        ds = torch.empty(step.n_chunks, heads, n, p, dtype=torch.float32, device=dev)
        lsum = torch.empty(tokens, heads, dtype=torch.float32, device=dev)
        atot = torch.empty(step.n_chunks, heads, dtype=torch.float32, device=dev)
        nv.check("mv_scan_chunked", L.mv_scan_chunked(
            _f32(q).data_ptr(), _ld(q), q_div, _f32(k).data_ptr(), _ld(k), k_div, _f32(v).data_ptr(), _ld(v),
            _f32(log_decay).data_ptr(), 0 if log_decay.dim() == 1 else _ld(log_decay),
            None if gain is None else _f32(gain).data_ptr(), 0 if gain is None else _ld(gain),
            None if skip is None else _f32(skip).data_ptr(), _f32(state).data_ptr(), _f32(out).data_ptr(), _ld(out),
            ds.data_ptr(), lsum.data_ptr(), atot.data_ptr(), step.ch_start.data_ptr(), step.ch_len.data_ptr(),
            step.row_ch0.data_ptr(), step.row_nch.data_ptr(), step.row_ctx.data_ptr(), step.row_slot.data_ptr(),
            step.n_chunks, step.rows, heads, n, p, nv.stream_ptr()))
    nv.check("mv_scan_outer", nv.lib().mv_scan_outer(
        _f32(q).data_ptr(), _ld(q), q_div, _f32(k).data_ptr(), _ld(k), k_div, _f32(v).data_ptr(), _ld(v),
        _f32(decay).data_ptr(), ld_decay, None if gain is None else _f32(gain).data_ptr(),
        0 if gain is None else _ld(gain), None if skip is None else _f32(skip).data_ptr(),
        _f32(state).data_ptr(), _f32(out).data_ptr(), _ld(out), step.row_start.data_ptr(),
        step.row_len.data_ptr(), step.row_ctx.data_ptr(), step.row_slot.data_ptr(), step.rows, heads, n, p,
        SCAN_SEQ_MAX if use_chunks else 0, nv.stream_ptr()))


def rotary_pairs_(x, inv_freq, tok_pos, heads: int, dim: int, rot: int, scale: float = 1.0):
    tokens = x.shape[0]
    assert x.shape[1] == heads * dim and tok_pos.numel() == tokens
    assert inv_freq.is_cuda and inv_freq.dtype == torch.float64 and inv_freq.numel() == rot // 2
    nv.check("mv_rotary_pairs", nv.lib().mv_rotary_pairs(
        _f32(x).data_ptr(), _ld(x), inv_freq.data_ptr(), _i32(tok_pos).data_ptr(), tokens, heads, dim, rot,
        float(scale), nv.stream_ptr()))


def gated_group_norm(y, gate, w, out, groups: int, gate_first: bool, eps: float):
    rows, n = y.shape
    assert gate.shape == (rows, n) and out.shape == (rows, n) and n % groups == 0
    assert w is None or (w.numel() == n and w.is_contiguous())
    nv.check("mv_gated_group_norm", nv.lib().mv_gated_group_norm(
        _f32(y).data_ptr(), _ld(y), _f32(gate).data_ptr(), _ld(gate), None if w is None else _f32(w).data_ptr(),
        out.data_ptr(), _ld(out), rows, n, groups, int(gate_first), float(eps), _is_f32(out), nv.stream_ptr()))


def qk_unitnorm_store(qkv, k_cache, v_cache, step, heads: int, kv_heads: int, d: int, dv: int, eps: float):
    tokens = qkv.shape[0]
    assert qkv.shape[1] == (heads + kv_heads) * d + kv_heads * dv and step.tokens == tokens
    page = k_cache.shape[1]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype
    assert k_cache.shape[1:] == (page, kv_heads, d) and v_cache.shape == (k_cache.shape[0], page, kv_heads, dv)
    assert int(step.max_page) < k_cache.shape[0] and page == step.page
    nv.check("mv_qk_unitnorm_store", nv.lib().mv_qk_unitnorm_store(
        _f32(qkv).data_ptr(), _ld(qkv), k_cache.data_ptr(), v_cache.data_ptr(), step.tok_row.data_ptr(),
        step.tok_pos.data_ptr(), step.block_table.data_ptr(), step.block_table.stride(0), page, tokens, heads,
        kv_heads, d, dv, float(eps), _is_f32(k_cache), nv.stream_ptr()))


def qk_rotary_store(qk, q_bias, k_bias, k_cache, v_cache, inv_freq, step, heads: int, kv_heads: int, d: int, rot: int,
                    adjacent: bool = True, act=None):
    """qk [T, (heads + kv_heads) * d] fp32 = queries then keys of one projection.  Biases are added, queries rotated
    in place; a key goes rotated into k_cache and as projected (with its bias) into v_cache: the values of this
    attention are its unrotated keys.  `act` = (a [T, 2n] fp32, out [T, n], kind, limit, slope): the gated activation
    of gated_act in the same launch (a feed-forward whose gate | up columns the same projection produced)."""
    tokens = qk.shape[0]
    a_in = a_out = None
    n_act = kind = 0
    limit = slope = 0.0
    if act is not None:
        a_in, a_out, kind, limit, slope = act
        n_act = a_out.shape[1]
        assert a_in.shape == (tokens, 2 * n_act) and a_out.shape[0] == tokens and a_out.dtype == k_cache.dtype
    assert qk.shape[1] == (heads + kv_heads) * d and step.tokens == tokens
    page = k_cache.shape[1]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype
    assert k_cache.shape[1:] == (page, kv_heads, d) and v_cache.shape == k_cache.shape
    assert int(step.max_page) < k_cache.shape[0] and page == step.page
    assert q_bias is None or (q_bias.numel() == heads * d and q_bias.is_contiguous())
    assert k_bias is None or (k_bias.numel() == kv_heads * d and k_bias.is_contiguous())
    assert rot == 0 or (inv_freq.is_cuda and inv_freq.dtype == torch.float64 and inv_freq.numel() == rot // 2)
    nv.check("mv_qk_rotary_store", nv.lib().mv_qk_rotary_store(
        _f32(qk).data_ptr(), _ld(qk), None if q_bias is None else _f32(q_bias).data_ptr(),
        None if k_bias is None else _f32(k_bias).data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        None if rot == 0 else inv_freq.data_ptr(), step.tok_row.data_ptr(), step.tok_pos.data_ptr(),
        step.block_table.data_ptr(), step.block_table.stride(0), page, tokens, heads, kv_heads, d, rot, int(adjacent),
        None if a_in is None else _f32(a_in).data_ptr(), 0 if a_in is None else _ld(a_in),
        None if a_in is None else a_out.data_ptr(), 0 if a_in is None else _ld(a_out), int(n_act), int(kind), float(limit),
        float(slope), _is_f32(k_cache), nv.stream_ptr()))


def window_attn(q, k_cache, v_cache, out, step, slopes, heads: int, kv_heads: int, d: int, dv: int,
                scale: float, window: int, tiled: bool = True, keep_first: int = 0, sinks=None, part=None, splits: int = 0):
    """`tiled`: rows of more than SCAN_SEQ_MAX tokens go to the matrix-core kernel where it applies (bf16,
    the head shapes it is built for); False keeps every token on the plain kernel.  `keep_first`: positions below it
    stay visible behind the window; `sinks` [heads]: exp(sink) joins each head's denominator.  `part` (fp32, at least
    tokens * heads * splits * (dv + 2) values, `splits` from window_attn_splits): the tokens the matrix-core kernel
    does not take run the kernel that reads every key once for all query heads of its key/value head and cuts the keys
    into `splits` pieces."""
    assert part is None or (splits >= 1 and part.is_contiguous() and part.numel() >= q.shape[0] * heads * splits * (dv + 2))
    assert sinks is None or (sinks.numel() == heads and sinks.is_contiguous())
    tokens = q.shape[0]
    assert q.shape[1] >= heads * d and out.shape == (tokens, heads * dv) and out.dtype == k_cache.dtype
    page = k_cache.shape[1]
    assert k_cache.shape[1:] == (page, kv_heads, d) and v_cache.shape == (k_cache.shape[0], page, kv_heads, dv)
    assert slopes is None or (slopes.numel() == heads and slopes.is_contiguous())
    assert int(step.max_page) < k_cache.shape[0] and page == step.page and step.tokens == tokens
    nv.check("mv_window_attn", nv.lib().mv_window_attn(
        _f32(q).data_ptr(), _ld(q), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ld(out),
        step.tok_row.data_ptr(), step.tok_pos.data_ptr(), step.block_table.data_ptr(), step.block_table.stride(0),
        page, None if slopes is None else _f32(slopes).data_ptr(), tokens, heads, kv_heads, d, dv, float(scale),
        int(window), _is_f32(k_cache), step.row_len.data_ptr(),
        step.ch_start.data_ptr() if step.n_chunks else None, step.ch_len.data_ptr() if step.n_chunks else None,
        step.n_chunks if tiled else 0, SCAN_SEQ_MAX, int(keep_first), None if sinks is None else _f32(sinks).data_ptr(),
        None if part is None else _f32(part).data_ptr(), int(splits) if part is not None else 0,
        int(getattr(step, "short_tokens", -1)) if tiled else -1, nv.stream_ptr()))


def window_attn_splits(tokens: int, heads: int, kv_heads: int, window: int, keep_first: int = 0) -> int:
    """Pieces to cut a token's keys into so that a step of few tokens still fills the chip (1: no cut)."""
    return int(nv.lib().mv_window_attn_splits(int(tokens), heads, kv_heads, int(window), int(keep_first)))


# ---------------------------------------------------------------------------------------------------------
# Dynamic Tanh norms, token shift, gated recurrence without a key, attention over a cached latent, routed
# experts (csrc/stream_ops.hip, seq_mix.hip, latent_attn.hip, moe.hip, linear_any.hip)

def _dyt(norm):
    w, b, alpha = norm
    assert w.is_contiguous() and b.is_contiguous() and w.numel() == b.numel() and alpha.numel() == 1
    return _f32(w).data_ptr(), _f32(b).data_ptr(), _f32(alpha).data_ptr()


def dyt_shift(x, norm, mix, state, h, step):
    """h_t = act(n_t + (n_(t-1) - n_t) * mix) with n = tanh(alpha x) w + b; state [slots, n] keeps each row's
    last n for its next step."""
    tokens, n = x.shape
    assert h.shape == (tokens, n) and norm[0].numel() == n and mix.numel() == n and mix.is_contiguous()
    assert state.is_contiguous() and state.shape[1:] == (n,) and int(step.max_slot) < state.shape[0]
    assert step.tokens == tokens
    w, b, a = _dyt(norm)
    nv.check("mv_dyt_shift", nv.lib().mv_dyt_shift(
        _f32(x).data_ptr(), _ld(x), w, b, a, _f32(mix).data_ptr(), _f32(state).data_ptr(), h.data_ptr(), _ld(h),
        step.tok_row.data_ptr(), step.row_start.data_ptr(), step.row_len.data_ptr(), step.row_ctx.data_ptr(),
        step.row_slot.data_ptr(), tokens, n, _is_f32(h), nv.stream_ptr()))


def dyt_gather(x, idx, norm, out):
    rows, n = out.shape
    assert x.shape[1] == n and norm[0].numel() == n and (idx is None or idx.numel() == rows)
    assert idx is not None or x.shape[0] == rows
    w, b, a = _dyt(norm)
    nv.check("mv_dyt_gather", nv.lib().mv_dyt_gather(
        _f32(x).data_ptr(), _ld(x), None if idx is None else _i32(idx).data_ptr(), w, b, a, out.data_ptr(), _ld(out),
        rows, n, _is_f32(out), nv.stream_ptr()))


def dyt_residual(y, norm, x, h=None, next_norm=None):
    """x += tanh(alpha y) w + b; h (optional) = x in the activation type, or with `next_norm` that norm of the new x
    (what the next sublayer reads)."""
    rows, n = x.shape
    assert y.shape == (rows, n) and norm[0].numel() == n and (h is None or h.shape == (rows, n))
    assert next_norm is None or (h is not None and next_norm[0].numel() == n)
    w, b, a = _dyt(norm)
    w2, b2, a2 = _dyt(next_norm) if next_norm is not None else (None, None, None)
    nv.check("mv_dyt_residual", nv.lib().mv_dyt_residual(
        _f32(y).data_ptr(), _ld(y), w, b, a, _f32(x).data_ptr(), _ld(x), None if h is None else h.data_ptr(),
        0 if h is None else _ld(h), w2, b2, a2, rows, n, 0 if h is None else _is_f32(h), nv.stream_ptr()))


def unitnorm_residual(y, w, eps: float, x, h=None):
    """x += y / sqrt(mean(y^2) + eps) * w; h (optional) = x in the activation type."""
    rows, n = x.shape
    assert y.shape == (rows, n) and w.numel() == n and w.is_contiguous() and (h is None or h.shape == (rows, n))
    nv.check("mv_unitnorm_residual", nv.lib().mv_unitnorm_residual(
        _f32(y).data_ptr(), _ld(y), _f32(w).data_ptr(), float(eps), _f32(x).data_ptr(), _ld(x),
        None if h is None else h.data_ptr(), 0 if h is None else _ld(h), rows, n, 0 if h is None else _is_f32(h),
        nv.stream_ptr()))


def rmsnorm_rows(v, w, eps: float, out, per: int = 1):
    """Each row of v holds `per` groups of w.numel() values: out = act(unit-RMS(group) * w)."""
    rows, n = v.shape[0], w.numel()
    assert v.shape[1] == per * n and out.shape == (rows, per * n) and w.is_contiguous()
    nv.check("mv_rmsnorm_rows", nv.lib().mv_rmsnorm_rows(
        _f32(v).data_ptr(), _ld(v), per, _f32(w).data_ptr(), float(eps), out.data_ptr(), _ld(out), rows, n,
        _is_f32(out), nv.stream_ptr()))


def gelu_gate_rows(a, table, off: int, ids, out):
    rows, n = a.shape
    assert out.shape == (rows, n) and table.is_cuda and table.dim() == 2 and table.stride(1) == 1
    assert table.dtype == out.dtype and off + n <= table.shape[1] and ids.numel() == rows
    nv.check("mv_gelu_gate_rows", nv.lib().mv_gelu_gate_rows(
        _f32(a).data_ptr(), _ld(a), table.data_ptr(), table.stride(0), off, _i32(ids).data_ptr(), table.shape[0],
        out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def silu_mul(a, out):
    rows, n = out.shape
    assert a.shape == (rows, 2 * n)
    nv.check("mv_silu_mul", nv.lib().mv_silu_mul(
        _f32(a).data_ptr(), _ld(a), out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def sigmoid_gate(a, g, out):
    rows, n = a.shape
    assert out.shape == (rows, n) and (g is None or g.shape == (rows, n))
    nv.check("mv_sigmoid_gate", nv.lib().mv_sigmoid_gate(
        _f32(a).data_ptr(), _ld(a), None if g is None else _f32(g).data_ptr(), 0 if g is None else _ld(g),
        out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def linear_heads(x, w, out, heads: int):
    """out[:, h*n : (h+1)*n] = x[:, h*k : (h+1)*k] . w[h]^T for w [heads, n, k] in the activation type; fp32 out.
    `out` may be a strided view [T, heads, n] of a wider buffer (row stride and head stride are passed on)."""
    m = x.shape[0]
    _, n, k = w.shape
    assert w.is_cuda and w.is_contiguous() and w.shape[0] == heads and x.dtype == w.dtype
    assert x.shape == (m, heads * k) and x.stride(1) == 1
    assert out.dim() == 3 and out.shape == (m, heads, n) and out.stride(2) == 1 and out.dtype == torch.float32
    if m == 0:
        return out
    ldy = out.stride(0) if m > 1 else max(out.stride(0), (heads - 1) * out.stride(1) + n)
    nv.check("mv_linear_heads", nv.lib().mv_linear_heads(
        x.data_ptr(), _ld(x), k, w.data_ptr(), k, n * k, out.data_ptr(), ldy, out.stride(1), m, n, k, heads,
        _is_f32(x), nv.stream_ptr()))
    return out


def linear_segments(x, w, out, seg, src, src_div: int, max_rows: int):
    """Rows seg[e] .. seg[e+1] of out = (operand rows src[i] // src_div, or i itself) . w[e]^T; w [E, n, k]."""
    E, n, k = w.shape
    assert w.is_cuda and w.is_contiguous() and x.dtype == w.dtype and x.shape[1] == k and x.stride(1) == 1
    assert out.shape[1] == n and out.dtype == torch.float32 and out.stride(1) == 1 and seg.numel() == E + 1
    assert src is None or src.numel() == out.shape[0]
    assert src is not None or x.shape[0] == out.shape[0]
    if out.shape[0] == 0:
        return out
    nv.check("mv_linear_segments", nv.lib().mv_linear_segments(
        x.data_ptr(), _ld(x), w.data_ptr(), k, n * k, out.data_ptr(), _ld(out), _i32(seg).data_ptr(),
        None if src is None else _i32(src).data_ptr(), src_div, E, min(max_rows, out.shape[0]), out.shape[0], n, k,
        _is_f32(x), nv.stream_ptr()))
    return out


def gate_lower_bound_(q, f, bias, lower):
    tokens, n = q.shape
    assert f.shape == (tokens, n) and lower.numel() == n and lower.is_contiguous()
    assert bias is None or (bias.numel() == n and bias.is_contiguous())
    nv.check("mv_gate_lower_bound", nv.lib().mv_gate_lower_bound(
        _f32(q).data_ptr(), _ld(q), _f32(f).data_ptr(), _ld(f), None if bias is None else _f32(bias).data_ptr(),
        _f32(lower).data_ptr(), tokens, n, nv.stream_ptr()))


def scan_gated(q, f, v, state, out, step, heads: int, n: int, p: int, chunked: bool = True):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t; state [slots, heads, n, p] fp32.  Rows of up to
    SCAN_SEQ_MAX tokens run token by token; longer rows in chunks of 64 side by side unless `chunked` is False."""
    tokens = v.shape[0]
    assert q.shape == (tokens, heads * n) and f.shape == (tokens, heads * n)
    assert v.shape == (tokens, heads * p) and out.shape == (tokens, heads * p)
    assert state.is_contiguous() and state.shape[1:] == (heads, n, p) and int(step.max_slot) < state.shape[0]
    assert step.tokens == tokens
    chunks = step.n_chunks if chunked else 0
    ds = cum = None
    if chunks:
        ds = torch.empty(chunks, heads, n, p, dtype=torch.float32, device=v.device)
        cum = torch.empty(tokens, heads * n, dtype=torch.float32, device=v.device)
    nv.check("mv_scan_gated", nv.lib().mv_scan_gated(
        _f32(q).data_ptr(), _ld(q), _f32(f).data_ptr(), _ld(f), _f32(v).data_ptr(), _ld(v), _f32(state).data_ptr(),
        _f32(out).data_ptr(), _ld(out), step.row_start.data_ptr(), step.row_len.data_ptr(), step.row_ctx.data_ptr(),
        step.row_slot.data_ptr(), step.rows, heads, n, p, None if ds is None else ds.data_ptr(),
        None if cum is None else cum.data_ptr(), step.ch_start.data_ptr() if chunks else None,
        step.ch_len.data_ptr() if chunks else None, step.row_ch0.data_ptr() if chunks else None,
        step.row_nch.data_ptr() if chunks else None, chunks, SCAN_SEQ_MAX, nv.stream_ptr()))


def latent_prep(dkv, w_norm, eps: float, cache, q, q_plain, q_abs, inv_freq, step, heads: int, d: int, r: int,
                rank: int, rot: int, interleaved: bool):
    """cache [pages, page, rank + r] in the activation type; q [T, heads*(d+r)] fp32; q_plain [T, heads*d] in the
    activation type; q_abs [T, heads*(rank+r)] fp32 (its rotated columns are written here)."""
    tokens = q.shape[0]
    assert dkv.shape == (tokens, rank + r) and w_norm.numel() == rank and w_norm.is_contiguous()
    assert cache.is_contiguous() and cache.shape[1:] == (step.page, rank + r) and int(step.max_page) < cache.shape[0]
    assert q.shape == (tokens, heads * (d + r)) and q_plain.shape == (tokens, heads * d)
    assert q_abs.shape == (tokens, heads * (rank + r)) and q_plain.dtype == cache.dtype and step.tokens == tokens
    assert rot == 0 or (inv_freq.is_cuda and inv_freq.dtype == torch.float64 and inv_freq.numel() == rot // 2)
    nv.check("mv_latent_prep", nv.lib().mv_latent_prep(
        _f32(dkv).data_ptr(), _ld(dkv), _f32(w_norm).data_ptr(), float(eps), cache.data_ptr(), _f32(q).data_ptr(),
        _ld(q), q_plain.data_ptr(), _ld(q_plain), _f32(q_abs).data_ptr(), _ld(q_abs),
        None if rot == 0 else inv_freq.data_ptr(), step.tok_row.data_ptr(), step.tok_pos.data_ptr(),
        step.block_table.data_ptr(), step.block_table.stride(0), step.page, tokens, heads, d, r, rank, rot,
        int(interleaved), _is_f32(cache), nv.stream_ptr()))


def latent_attn(q_abs, cache, out, step, sinks, heads: int, rank: int, r: int, scale: float, window: int,
                tiled: bool = True):
    """out [T, heads*rank] in the activation type: weighted sums of the cached latents.  window 0: causal.
    `tiled`: rows of more than SCAN_SEQ_MAX tokens go to the matrix-core kernel where it applies (bf16, the
    shapes it is built for); False keeps every token on the plain kernel."""
    tokens = q_abs.shape[0]
    assert q_abs.shape == (tokens, heads * (rank + r)) and out.shape == (tokens, heads * rank)
    assert cache.is_contiguous() and cache.shape[1:] == (step.page, rank + r) and int(step.max_page) < cache.shape[0]
    assert out.dtype == cache.dtype and step.tokens == tokens
    assert sinks is None or (sinks.numel() == heads and sinks.is_contiguous())
    nv.check("mv_latent_attn", nv.lib().mv_latent_attn(
        _f32(q_abs).data_ptr(), _ld(q_abs), cache.data_ptr(), out.data_ptr(), _ld(out), step.tok_row.data_ptr(),
        step.tok_pos.data_ptr(), step.block_table.data_ptr(), step.block_table.stride(0), step.page,
        None if sinks is None else _f32(sinks).data_ptr(), tokens, heads, rank, r, float(scale), int(window),
        _is_f32(cache), step.row_len.data_ptr(), step.ch_start.data_ptr() if step.n_chunks else None,
        step.ch_len.data_ptr() if step.n_chunks else None, step.n_chunks if tiled else 0, SCAN_SEQ_MAX,
        nv.stream_ptr()))


def moe_route(h, w_router, w_shared_gate, ids, weights, shared_gate):
    tokens, n = h.shape
    E, top = w_router.shape[0], ids.shape[1]
    assert h.stride(1) == 1 and w_router.shape == (E, n) and w_router.is_contiguous()
    assert ids.shape == (tokens, top) and weights.shape == (tokens, top) and ids.is_contiguous()
    assert weights.is_contiguous() and ids.dtype == torch.int32
    assert w_shared_gate is None or (w_shared_gate.numel() == n and w_shared_gate.is_contiguous()
                                     and shared_gate.numel() == tokens and shared_gate.is_contiguous())
    nv.check("mv_moe_route", nv.lib().mv_moe_route(
        h.data_ptr(), _ld(h), _f32(w_router).data_ptr(), None if w_shared_gate is None else _f32(w_shared_gate).data_ptr(),
        ids.data_ptr(), _f32(weights).data_ptr(), None if w_shared_gate is None else _f32(shared_gate).data_ptr(),
        tokens, n, E, top, _is_f32(h), nv.stream_ptr()))


def moe_plan(ids, seg, order, place, experts: int):
    pairs = ids.numel()
    assert seg.numel() == experts + 1 and order.numel() == pairs and place.numel() == pairs
    nv.check("mv_moe_plan", nv.lib().mv_moe_plan(
        _i32(ids).data_ptr(), _i32(seg).data_ptr(), _i32(order).data_ptr(), _i32(place).data_ptr(), pairs, experts,
        nv.stream_ptr()))


def moe_combine(expert_out, place, weights, shared_out, shared_gate, y, norm=None, h=None, ids=None, first_pass: int = 0,
                passed=None):
    """y = the weighted sum of each token's experts (+ shared_gate * shared_out; weights None: ones, shared_gate None:
    one).  With `norm` y is the residual
    stream and receives the sum through that norm, y += tanh(alpha sum) w + b; h (optional) = y in the activation
    type.  With `ids` [tokens, top] a choice >= first_pass is an expert that hands its input through: it adds its
    weight times the token's row of `passed` (activation type)."""
    tokens, n = y.shape
    top = place.numel() // max(tokens, 1) if weights is None else weights.shape[1]
    assert ids is None or (ids.numel() == tokens * top and passed is not None and passed.shape == (tokens, n)
                           and passed.stride(1) == 1)
    assert expert_out.shape == (tokens * top, n) and place.numel() == tokens * top
    assert weights is None or (weights.shape == (tokens, top) and weights.is_contiguous())
    assert shared_out is None or (shared_out.shape == (tokens, n) and (shared_gate is None or shared_gate.numel() == tokens))
    assert h is None or (norm is not None and h.shape == (tokens, n))
    w, b, a = _dyt(norm) if norm is not None else (None, None, None)
    nv.check("mv_moe_combine", nv.lib().mv_moe_combine(
        _f32(expert_out).data_ptr(), _ld(expert_out), _i32(place).data_ptr(),
        None if weights is None else _f32(weights).data_ptr(),
        None if shared_out is None else _f32(shared_out).data_ptr(), 0 if shared_out is None else _ld(shared_out),
        None if shared_out is None or shared_gate is None else _f32(shared_gate).data_ptr(), _f32(y).data_ptr(), _ld(y),
        w, b, a,
        None if h is None else h.data_ptr(), 0 if h is None else _ld(h), tokens, n, top,
        _is_f32(passed) if passed is not None else (0 if h is None else _is_f32(h)),
        None if ids is None else _i32(ids).data_ptr(), int(first_pass), None if ids is None else passed.data_ptr(),
        0 if ids is None else _ld(passed), nv.stream_ptr()))


def moe_route_scored(h, w_router, correction, ids, weights, scale: float, sum_floor: float):
    """Scores = softmax over all router outputs; the `top` largest of score + correction are chosen, their weights are
    the scores divided by their sum (+ sum_floor), times scale."""
    tokens, n = h.shape
    E, top = w_router.shape[0], ids.shape[1]
    assert h.stride(1) == 1 and w_router.shape == (E, n) and w_router.is_contiguous()
    assert ids.shape == (tokens, top) and weights.shape == (tokens, top) and ids.is_contiguous()
    assert weights.is_contiguous() and ids.dtype == torch.int32
    assert correction is None or (correction.numel() == E and correction.is_contiguous())
    nv.check("mv_moe_route_scored", nv.lib().mv_moe_route_scored(
        h.data_ptr(), _ld(h), _f32(w_router).data_ptr(), None if correction is None else _f32(correction).data_ptr(),
        ids.data_ptr(), _f32(weights).data_ptr(), tokens, n, E, top, float(scale), float(sum_floor), _is_f32(h),
        nv.stream_ptr()))


GATE_SILU, GATE_GELU_TANH, GATE_CLAMPED = 0, 1, 2


def gated_act(a, out, kind: int, limit: float = 0.0, slope: float = 1.0):
    """out = act(f(a[:, :n]) * a[:, n:]) with f = SiLU / GELU (tanh form), or the clamped gate
    min(g, limit) * sigmoid(slope * min(g, limit)) * (clamp(u, -limit, limit) + 1)."""
    rows, n = out.shape
    assert a.shape == (rows, 2 * n)
    nv.check("mv_gated_act", nv.lib().mv_gated_act(
        _f32(a).data_ptr(), _ld(a), out.data_ptr(), _ld(out), rows, n, int(kind), float(limit), float(slope),
        _is_f32(out), nv.stream_ptr()))


def embed_pair(table, pairs, ids, prev, x, scale: float, buckets: int, mul_prev: int, mul_cur: int, w=None,
               eps: float = 0.0, h=None):
    """x = table[id] * scale + pairs[(prev * mul_prev + id * mul_cur) mod buckets], row `buckets` where prev < 0.
    With `w`: h = act(x / sqrt(mean(x^2) + eps) * w) out of the same launch."""
    rows, n = x.shape
    assert (w is None) == (h is None) and (w is None or (w.numel() == n and w.is_contiguous() and h.shape == (rows, n)
                                                        and h.dtype == table.dtype))
    assert table.is_cuda and table.is_contiguous() and table.shape[1] == n and table.dtype == pairs.dtype
    assert pairs.is_cuda and pairs.is_contiguous() and pairs.shape == (buckets + 1, n)
    assert ids.numel() == rows and prev.numel() == rows
    nv.check("mv_embed_pair", nv.lib().mv_embed_pair(
        table.data_ptr(), pairs.data_ptr(), _i32(ids).data_ptr(), _i32(prev).data_ptr(), _f32(x).data_ptr(), _ld(x),
        rows, n, table.shape[0], int(buckets), int(mul_prev), int(mul_cur), float(scale),
        None if w is None else _f32(w).data_ptr(), float(eps), None if h is None else h.data_ptr(),
        0 if h is None else _ld(h), _is_f32(table), nv.stream_ptr()))


def add_rmsnorm(x, y1=None, y2=None, w=None, eps: float = 0.0, h=None):
    """x += y1 (+ y2); with `w`: h = act(x / sqrt(mean(x^2) + eps) * w)."""
    rows, n = x.shape
    assert y1 is None or y1.shape == (rows, n)
    assert y2 is None or (y1 is not None and y2.shape == (rows, n))
    assert (w is None) == (h is None) and (w is None or (w.numel() == n and w.is_contiguous() and h.shape == (rows, n)))
    nv.check("mv_add_rmsnorm", nv.lib().mv_add_rmsnorm(
        None if y1 is None else _f32(y1).data_ptr(), 0 if y1 is None else _ld(y1),
        None if y2 is None else _f32(y2).data_ptr(), 0 if y2 is None else _ld(y2), _f32(x).data_ptr(), _ld(x),
        None if w is None else _f32(w).data_ptr(), float(eps), None if h is None else h.data_ptr(),
        0 if h is None else _ld(h), rows, n, 0 if h is None else _is_f32(h), nv.stream_ptr()))


def rmsnorm_gather(x, idx, w, eps: float, out, offset: float = 0.0):
    """out = act(x[idx] / sqrt(mean(x[idx]^2) + eps) * (offset + w))."""
    rows, n = out.shape
    assert x.shape[1] == n and w.numel() == n and w.is_contiguous()
    assert idx is None or idx.numel() == rows
    nv.check("mv_rmsnorm_gather", nv.lib().mv_rmsnorm_gather(
        _f32(x).data_ptr(), _ld(x), None if idx is None else _i32(idx).data_ptr(), _f32(w).data_ptr(), float(eps),
        float(offset), out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


# ---------------------------------------------------------------------------------------------------------
# Gated residual stream, loop input, short convolutions without activation, differential attention, routing by
# sigmoid scores (csrc/stream_ops.hip, seq_mix.hip, diff_attn.hip, moe.hip)

def gated_residual_norm(x, y=None, g=None, b=None, replace: bool = False, w=None, eps: float = 0.0, offset: float = 0.0,
                        n32=None, h=None):
    """The residual step of a pre-norm layer with gated sublayer outputs: x += y * sigmoid(g + b); with `replace`
    x = y + b instead (a pass of a looped span starts from a projection plus a per-pass vector); y None: x as it is.
    With `w`: n = x / sqrt(mean(x^2) + eps) * (offset + w) of the new x, to n32 (fp32) and / or h (activation type)."""
    rows, n = x.shape
    mode = 0 if y is None else (2 if replace else 1)
    assert y is None or y.shape == (rows, n)
    assert (mode == 1) == (g is not None) and (g is None or g.shape == (rows, n))
    assert b is None or (b.numel() == n and b.is_contiguous())
    assert (w is None) == (n32 is None and h is None) and (w is None or (w.numel() == n and w.is_contiguous()))
    assert n32 is None or n32.shape == (rows, n)
    assert h is None or h.shape == (rows, n)
    nv.check("mv_gated_residual_norm", nv.lib().mv_gated_residual_norm(
        None if y is None else _f32(y).data_ptr(), 0 if y is None else _ld(y),
        None if g is None else _f32(g).data_ptr(), 0 if g is None else _ld(g),
        None if b is None else _f32(b).data_ptr(), mode, _f32(x).data_ptr(), _ld(x),
        None if w is None else _f32(w).data_ptr(), float(eps), float(offset),
        None if n32 is None else _f32(n32).data_ptr(), 0 if n32 is None else _ld(n32),
        None if h is None else h.data_ptr(), 0 if h is None else _ld(h), rows, n, 0 if h is None else _is_f32(h),
        nv.stream_ptr()))


def cast_concat(a, b, out):
    """out = act([a | b]) for two fp32 operands of equal shape."""
    rows, n = a.shape
    assert b.shape == (rows, n) and out.shape == (rows, 2 * n)
    nv.check("mv_cast_concat", nv.lib().mv_cast_concat(
        _f32(a).data_ptr(), _ld(a), _f32(b).data_ptr(), _ld(b), out.data_ptr(), _ld(out), rows, n, _is_f32(out),
        nv.stream_ptr()))


def gelu_tanh(v, out):
    rows, n = v.shape
    assert out.shape == (rows, n)
    nv.check("mv_gelu_tanh", nv.lib().mv_gelu_tanh(
        _f32(v).data_ptr(), _ld(v), out.data_ptr(), _ld(out), rows, n, _is_f32(out), nv.stream_ptr()))


def scale_(v, factor: float):
    assert v.is_contiguous()
    nv.check("mv_scale", nv.lib().mv_scale(_f32(v).data_ptr(), v.numel(), float(factor), nv.stream_ptr()))
    return v


def conv_taps(inp, state, w, step, out32=None, out_act=None, add_input: bool = False):
    """y_t = (inp_t +) sum_j w[:, j] inp_(t - taps + 1 + j) per channel, no bias, no activation; inp [T, C] fp32,
    state [slots, taps - 1, C] fp32 (the inputs before the step; updated), w [C, taps] fp32.  y goes to out32 (fp32)
    and / or out_act (activation type)."""
    tokens, ch = inp.shape
    taps = w.shape[1]
    assert w.shape == (ch, taps) and w.is_contiguous() and (out32 is not None or out_act is not None)
    assert out32 is None or out32.shape == (tokens, ch)
    assert out_act is None or out_act.shape == (tokens, ch)
    assert state.is_contiguous() and state.shape[1:] == (max(taps - 1, 0), ch)
    assert step.tokens == tokens and int(step.max_slot) < state.shape[0]
    nv.check("mv_conv_taps", nv.lib().mv_conv_taps(
        _f32(inp).data_ptr(), _ld(inp), _f32(state).data_ptr(), _f32(w).data_ptr(),
        None if out32 is None else _f32(out32).data_ptr(), 0 if out32 is None else _ld(out32),
        None if out_act is None else out_act.data_ptr(), 0 if out_act is None else _ld(out_act), int(add_input),
        step.tok_row.data_ptr(), step.row_start.data_ptr(), step.row_len.data_ptr(), step.row_ctx.data_ptr(),
        step.row_slot.data_ptr(), tokens, step.rows, ch, taps, 0 if out_act is None else _is_f32(out_act),
        nv.stream_ptr()))


def conv_qkv_store(qkv, state, w, q, k_cache, v_cache, step):
    """The q | k | v columns of one projection (qkv [T, cq + ck + cv] fp32) through a causal convolution per channel
    (w [cq + ck + cv, taps] fp32 and state [slots, taps - 1, cq + ck + cv]; w None: no convolution): queries to q
    [T, cq] fp32, keys and values into the token's rows of k_cache [pages, page, ...ck] / v_cache [pages, page, ...cv]."""
    tokens = qkv.shape[0]
    page = k_cache.shape[1]
    cq, ck, cv = q.shape[1], k_cache[0, 0].numel(), v_cache[0, 0].numel()
    taps = 0 if w is None else w.shape[1]
    assert qkv.shape[1] >= cq + ck + cv and q.shape[0] == tokens and step.tokens == tokens
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype
    assert v_cache.shape[:2] == k_cache.shape[:2] and page == step.page and int(step.max_page) < k_cache.shape[0]
    assert w is None or (w.shape == (cq + ck + cv, taps) and w.is_contiguous())
    assert taps <= 1 or (state.is_contiguous() and state.shape[1:] == (taps - 1, cq + ck + cv)
                         and int(step.max_slot) < state.shape[0])
    nv.check("mv_conv_qkv_store", nv.lib().mv_conv_qkv_store(
        _f32(qkv).data_ptr(), _ld(qkv), None if taps <= 1 else _f32(state).data_ptr(),
        None if w is None else _f32(w).data_ptr(), _f32(q).data_ptr(), _ld(q), k_cache.data_ptr(), v_cache.data_ptr(),
        step.tok_row.data_ptr(), step.tok_pos.data_ptr(), step.row_start.data_ptr(), step.row_len.data_ptr(),
        step.row_ctx.data_ptr(), step.row_slot.data_ptr(), step.block_table.data_ptr(), step.block_table.stride(0), page,
        tokens, step.rows, cq, ck, cv, taps, _is_f32(k_cache), nv.stream_ptr()))


def diff_attn(q, k_cache, v_cache, out, gate, step, heads: int, kv_heads: int, d: int, dv: int, scale: float,
              softcap: float, lam: float, out_scale: float, eps: float, tiled: bool = True):
    """Differential attention: q [T, heads * 2 * d] fp32 (per head its two maps' queries), k_cache [pages, page,
    kv_heads, 2 * d], v_cache [pages, page, kv_heads, dv]; causal softmax per map over the same values, o = a1 - lam a2,
    out [T, heads * dv] = act(o / rms(o) * out_scale * sigmoid(gate[t, h])); gate [T, heads] fp32 or None.
    `tiled`: rows of more than SCAN_SEQ_MAX tokens go to the matrix-core kernel where it applies."""
    tokens = q.shape[0]
    page = k_cache.shape[1]
    assert q.shape[1] == heads * 2 * d and out.shape == (tokens, heads * dv) and out.dtype == k_cache.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[1:] == (page, kv_heads, 2 * d) and v_cache.shape == (k_cache.shape[0], page, kv_heads, dv)
    assert gate is None or gate.shape == (tokens, heads)
    assert int(step.max_page) < k_cache.shape[0] and page == step.page and step.tokens == tokens
    chunks = step.n_chunks if tiled else 0
    nv.check("mv_diff_attn", nv.lib().mv_diff_attn(
        _f32(q).data_ptr(), _ld(q), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ld(out),
        None if gate is None else _f32(gate).data_ptr(), 0 if gate is None else _ld(gate), step.tok_row.data_ptr(),
        step.tok_pos.data_ptr(), step.block_table.data_ptr(), step.block_table.stride(0), page, tokens, heads, kv_heads,
        d, dv, float(scale), float(softcap), float(lam), float(out_scale), float(eps), _is_f32(k_cache),
        step.row_len.data_ptr(), step.ch_start.data_ptr() if chunks else None, step.ch_len.data_ptr() if chunks else None,
        chunks, SCAN_SEQ_MAX, int(getattr(step, "short_tokens", -1)) if tiled else -1, nv.stream_ptr()))


def moe_route_sigmoid(h, w_router, ids, weights):
    """The `top` largest router outputs (fp32 logits of the activation-type input; ties to the lower index); the
    weights are the sigmoids of the chosen outputs, not renormalised."""
    tokens, n = h.shape
    E, top = w_router.shape[0], ids.shape[1]
    assert h.stride(1) == 1 and w_router.shape == (E, n) and w_router.is_contiguous()
    assert ids.shape == (tokens, top) and weights.shape == (tokens, top) and ids.is_contiguous()
    assert weights.is_contiguous() and ids.dtype == torch.int32
    nv.check("mv_moe_route_sigmoid", nv.lib().mv_moe_route_sigmoid(
        h.data_ptr(), _ld(h), _f32(w_router).data_ptr(), ids.data_ptr(), _f32(weights).data_ptr(), tokens, n, E, top,
        _is_f32(h), nv.stream_ptr()))


def gated_act_scaled(a, out, kind: int, scale, order=None, limit: float = 0.0, slope: float = 1.0):
    """gated_act with both halves of row i multiplied by scale[order[i]] (order None: scale[i]) first."""
    rows, n = out.shape
    assert a.shape == (rows, 2 * n) and scale.is_contiguous() and (order is None or order.numel() == rows)
    assert scale.numel() >= rows
    nv.check("mv_gated_act_scaled", nv.lib().mv_gated_act_scaled(
        _f32(a).data_ptr(), _ld(a), out.data_ptr(), _ld(out), rows, n, int(kind), float(limit), float(slope),
        _f32(scale).data_ptr(), None if order is None else _i32(order).data_ptr(), _is_f32(out), nv.stream_ptr()))
