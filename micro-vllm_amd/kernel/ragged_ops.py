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


def window_attn(q, k_cache, v_cache, out, step, slopes, heads: int, kv_heads: int, d: int, dv: int,
                scale: float, window: int, tiled: bool = True):
    """`tiled`: rows of more than SCAN_SEQ_MAX tokens go to the matrix-core kernel where it applies (bf16,
    the head shapes it is built for); False keeps every token on the plain kernel."""
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
        step.n_chunks if tiled else 0, SCAN_SEQ_MAX, nv.stream_ptr()))
