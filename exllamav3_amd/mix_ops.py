"""
Python surface of the sequence-mixer library libexl3_mix.so (include/exl3_mix.h): one function per kernel, torch tensors in, raw device
pointers out, on the caller's current HIP stream.  PyTorch is device memory and streams only; there is no eager or CPU fallback -- a
missing library is compiled on first use (seconds) and anything else raises.

Activations and matrix weights are bfloat16 or float32 (`code(dtype)`); the residual stream, norm weights, sinks, decay biases, recurrent
states and router logits are float32 in both modes.  2-D arguments named *_view may be column blocks of a wider matrix (unit column
stride, any row stride).
"""
from __future__ import annotations
import torch
from . import _lib
from ._lib import mix_check as _check

BF16, F32 = 0, 1


def code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float32:
        return F32
    raise RuntimeError(f"mix_ops: activations are bfloat16 or float32, not {dtype}")


def _p(t):
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _req(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _view(t: torch.Tensor, cols: int, name: str) -> int:
    """Row stride of a 2-D column block."""
    _req(t.dim() == 2 and t.shape[1] == cols and (t.stride(1) == 1 or cols == 1), f"{name}: expected [rows, {cols}] with unit column stride, got {tuple(t.shape)} / {t.stride()}")
    return t.stride(0)


def _f32c(t: torch.Tensor, name: str):
    _req(t.dtype == torch.float32 and t.is_contiguous(), f"{name}: contiguous float32 expected")


def _i32c(t: torch.Tensor, name: str):
    _req(t.dtype == torch.int32 and t.is_contiguous(), f"{name}: contiguous int32 expected")


def embed(x: torch.Tensor, h: torch.Tensor | None, table: torch.Tensor, tokens: torch.Tensor, scale: float, norm_w: torch.Tensor | None, eps: float):
    n, width = x.shape
    _f32c(x, "x"); _i32c(tokens, "tokens")
    _req(tokens.numel() == n and table.is_contiguous() and table.shape[1] == width, "embed: shapes")
    if norm_w is not None:
        _f32c(norm_w, "norm_w"); _req(h is not None and h.is_contiguous() and h.shape == x.shape and h.dtype == table.dtype, "embed: h")
    _check(_lib.mixlib().exl3_mix_embed(_p(x), _p(h), _p(table), _p(tokens), scale, _p(norm_w), eps, n, width, table.shape[0], code(table.dtype), _stream(x)))


def rms_norm_rows(h: torch.Tensor, x: torch.Tensor, rows: torch.Tensor | None, w: torch.Tensor, eps: float):
    n, width = h.shape
    _f32c(x, "x"); _f32c(w, "w")
    _req(h.is_contiguous() and x.shape[1] == width and w.numel() == width, "rms_norm_rows: shapes")
    if rows is not None:
        _i32c(rows, "rows"); _req(rows.numel() == n, "rms_norm_rows: rows")
    else:
        _req(x.shape[0] == n, "rms_norm_rows: rows of x")
    _check(_lib.mixlib().exl3_mix_rms_norm_rows(_p(h), _p(x), _p(rows), _p(w), eps, n, width, code(h.dtype), _stream(x)))


def gated_residual(x: torch.Tensor, y_view: torch.Tensor, r_view: torch.Tensor, norm_w: torch.Tensor | None, h: torch.Tensor | None, eps: float):
    n, width = x.shape
    _f32c(x, "x")
    _req(y_view.dtype == r_view.dtype and y_view.shape[0] == n and r_view.shape[0] == n, "gated_residual: y / r")
    if norm_w is not None:
        _f32c(norm_w, "norm_w"); _req(h is not None and h.is_contiguous() and h.shape == x.shape and h.dtype == y_view.dtype, "gated_residual: h")
    _check(_lib.mixlib().exl3_mix_gated_residual(_p(x), _p(y_view), _view(y_view, width, "y"), _p(r_view), _view(r_view, width, "r"), _p(norm_w), _p(h), eps, n, width,
                                                  code(y_view.dtype), _stream(x)))


def polynorm(out: torch.Tensor, z_view: torch.Tensor, coef: torch.Tensor, eps: float):
    n, ff = out.shape
    _f32c(coef, "coef")
    _req(out.is_contiguous() and z_view.dtype == out.dtype and z_view.shape[0] == n and coef.numel() == 4, "polynorm: shapes")
    _check(_lib.mixlib().exl3_mix_polynorm(_p(out), _p(z_view), _view(z_view, ff, "z"), _p(coef), eps, n, ff, code(out.dtype), _stream(out)))


def attn_store(v_norm, ring_k, ring_v, k_view, v_view, tok_seq, tok_pos, slots, len_after, eps: float):
    n, kv_heads, vdim = v_norm.shape
    n_slots, window, g2, dim = ring_k.shape
    _req(g2 == kv_heads and ring_v.shape == (n_slots, window, kv_heads, vdim) and ring_k.is_contiguous() and ring_v.is_contiguous() and v_norm.is_contiguous(),
         "attn_store: cache shapes")
    _req(ring_k.dtype == k_view.dtype == v_view.dtype == v_norm.dtype == ring_v.dtype, "attn_store: element types")
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots"), (len_after, "len_after")):
        _i32c(t, nm)
    _req(tok_seq.numel() == n and tok_pos.numel() == n and k_view.shape[0] == n and v_view.shape[0] == n, "attn_store: rows")
    _check(_lib.mixlib().exl3_mix_attn_store(_p(v_norm), _p(ring_k), _p(ring_v), _p(k_view), _view(k_view, kv_heads * dim, "k"), _p(v_view),
                                              _view(v_view, kv_heads * vdim, "v"), _p(tok_seq), _p(tok_pos), _p(slots), _p(len_after), eps, n, kv_heads, dim, vdim, window,
                                              code(v_norm.dtype), _stream(v_norm)))


# prompt steps from this many rows on (bfloat16, head sizes <= 256) run on the matrix cores
ATTN_MFMA_MIN_ROWS = 32


def attn_prefill(out, q_view, k_view, v_norm, gate_view, sink, cu, tok_seq, tok_pos, heads: int, scale: float, window: int, max_rows: int = 0, mfma: bool | None = None):
    """max_rows: the longest sequence of the step (host number; needed for the matrix-core kernel's grid).  mfma None: chosen by size and type."""
    n, kv_heads, vdim = v_norm.shape
    dim = q_view.shape[1] // heads
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and out.dtype == q_view.dtype == k_view.dtype == v_norm.dtype, "attn_prefill: out / types")
    if sink is not None:
        _f32c(sink, "sink"); _req(sink.numel() == heads, "attn_prefill: sink")
    if mfma is None:
        mfma = out.dtype == torch.bfloat16 and max_rows >= ATTN_MFMA_MIN_ROWS and dim <= 256 and vdim <= 256 and scale > 0
    if mfma:
        _req(out.dtype == torch.bfloat16 and max_rows > 0 and v_norm.is_contiguous(), "attn_prefill: the matrix-core kernel takes bfloat16 and the step's longest sequence")
        _check(_lib.mixlib().exl3_mix_attn_prefill_mfma(_p(out), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_view), _view(k_view, kv_heads * dim, "k"), _p(v_norm),
                                                         _p(gate_view), 0 if gate_view is None else _view(gate_view, heads, "gate"), _p(sink), _p(cu),
                                                         cu.numel() - 1, max_rows, heads, kv_heads, dim, vdim, scale, window, _stream(out)))
        return
    _check(_lib.mixlib().exl3_mix_attn_prefill(_p(out), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_view), _view(k_view, kv_heads * dim, "k"), _p(v_norm),
                                                _p(gate_view), 0 if gate_view is None else _view(gate_view, heads, "gate"), _p(sink), _p(cu), _p(tok_seq), _p(tok_pos),
                                                n, heads, kv_heads, dim, vdim, scale, window, code(out.dtype), _stream(out)))


def attn_decode(out, q_view, ring_k, ring_v, gate_view, sink, slots, len_after, heads: int, scale: float):
    n = out.shape[0]
    n_slots, window, kv_heads, dim = ring_k.shape
    vdim = ring_v.shape[3]
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and out.dtype == q_view.dtype == ring_k.dtype, "attn_decode: out / types")
    _req(slots.numel() == n and len_after.numel() == n, "attn_decode: one row per sequence")
    if sink is not None:
        _f32c(sink, "sink"); _req(sink.numel() == heads, "attn_decode: sink")
    _check(_lib.mixlib().exl3_mix_attn_decode(_p(out), _p(q_view), _view(q_view, heads * dim, "q"), _p(ring_k), _p(ring_v), _p(gate_view),
                                               0 if gate_view is None else _view(gate_view, heads, "gate"), _p(sink), _p(slots), _p(len_after),
                                               n, heads, kv_heads, dim, vdim, scale, window, code(out.dtype), _stream(out)))


def gla_scan(o, state, q_view, k_view, v_view, lr_view, a2, a2_bias, cu, slots, pos0, tau: float, q_scale: float, segments: tuple[int, int] | None = None):
    """segments = (segs, seg_len): the time axis of every sequence cut into parallel segments (long prompts); None: one workgroup chain per sequence."""
    n, heads, vdim = o.shape
    n_slots, h2, dim, v2 = state.shape
    rank = a2.shape[1]
    _f32c(o, "o"); _f32c(state, "state")
    _req(h2 == heads and v2 == vdim and a2.is_contiguous() and a2.shape[0] == heads * dim and a2.dtype == q_view.dtype, "gla_scan: shapes")
    if a2_bias is not None:
        _f32c(a2_bias, "a2_bias")
    batch = slots.numel()
    _req(cu.numel() == batch + 1 and pos0.numel() == batch, "gla_scan: batch tensors")
    args = (_p(o), _p(state), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_view), _view(k_view, heads * dim, "k"), _p(v_view),
            _view(v_view, heads * vdim, "v"), _p(lr_view), _view(lr_view, rank, "lr"), _p(a2), _p(a2_bias), _p(cu), _p(slots), _p(pos0),
            batch, heads, dim, vdim, rank, tau, q_scale)
    if segments is None:
        _check(_lib.mixlib().exl3_mix_gla_scan(*args, code(q_view.dtype), _stream(o)))
        return
    segs, seg_len = segments
    seg_state = torch.empty((batch * segs, heads, dim, vdim), dtype=torch.float32, device=o.device)
    seg_decay = torch.empty((batch * segs, heads, dim), dtype=torch.float32, device=o.device)
    _check(_lib.mixlib().exl3_mix_gla_segmented(*args, segs, seg_len, _p(seg_state), _p(seg_decay), code(q_view.dtype), _stream(o)))


def gla_out(out, o, w, g_view, eps: float):
    n, heads, vdim = o.shape
    _f32c(o, "o"); _f32c(w, "w")
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and w.numel() == vdim and g_view.dtype == out.dtype, "gla_out: shapes")
    _check(_lib.mixlib().exl3_mix_gla_out(_p(out), _p(o), _p(w), _p(g_view), _view(g_view, heads * vdim, "g"), eps, n, heads, vdim, code(out.dtype), _stream(out)))


def topk_softmax(idx, wts, logits):
    n, experts = logits.shape
    top = idx.shape[1]
    _f32c(logits, "logits"); _f32c(wts, "wts"); _i32c(idx, "idx")
    _req(idx.shape == wts.shape == (n, top), "topk_softmax: shapes")
    _check(_lib.mixlib().exl3_mix_topk_softmax(_p(idx), _p(wts), _p(logits), n, experts, top, _stream(logits)))


def moe_gate_up(hid, h, wg, wu, idx):
    n, width = h.shape
    experts, ff, w2 = wg.shape
    top = idx.shape[1]
    _req(h.is_contiguous() and wg.is_contiguous() and wu.is_contiguous() and wu.shape == wg.shape and w2 == width and hid.is_contiguous()
         and hid.shape == (n * top, ff) and hid.dtype == h.dtype == wg.dtype, "moe_gate_up: shapes")
    _i32c(idx, "idx")
    _check(_lib.mixlib().exl3_mix_moe_gate_up(_p(hid), _p(h), _p(wg), _p(wu), _p(idx), n, top, experts, ff, width, code(h.dtype), _stream(h)))


def moe_down(y, hid, wd, idx, wts):
    n, width = y.shape
    experts, w2, ff = wd.shape
    top = idx.shape[1]
    _req(y.is_contiguous() and hid.is_contiguous() and wd.is_contiguous() and w2 == width and hid.shape == (n * top, ff) and y.dtype == hid.dtype == wd.dtype,
         "moe_down: shapes")
    _i32c(idx, "idx"); _f32c(wts, "wts")
    _check(_lib.mixlib().exl3_mix_moe_down(_p(y), _p(hid), _p(wd), _p(idx), _p(wts), n, top, experts, ff, width, code(y.dtype), _stream(y)))


def moe_grouped(y, h, wg, wu, wd, idx, wts, act_kind: int = 0, limit: float = 0.0):
    """Experts of many rows: rows sorted by expert (device), one host read of the per-expert counts, then per expert three vendor matrix products
    with the activation kernel between them, and the weighted un-sort.  Same result as moe_gate_up + moe_down up to rounding."""
    n, width = h.shape
    experts, ff, _ = wg.shape
    top = idx.shape[1]
    flat = idx.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    counts = torch.zeros(experts, dtype=torch.int32, device=h.device).index_add_(0, flat, torch.ones_like(flat, dtype=torch.int32)).tolist()
    where = torch.empty(n * top, dtype=torch.int32, device=h.device)
    where[order] = torch.arange(n * top, dtype=torch.int32, device=h.device)
    xs = h.index_select(0, order // top)
    out = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
    hid = torch.empty((n * top, ff), dtype=h.dtype, device=h.device)
    lib, at = _lib.mixlib(), 0
    for e, c in enumerate(counts):
        if c == 0:
            continue
        seg = xs[at: at + c]
        g, u = torch.nn.functional.linear(seg, wg[e]), torch.nn.functional.linear(seg, wu[e])
        _check(lib.exl3_mix_glu_act(_p(hid[at: at + c]), _p(g), ff, _p(u), ff, c, ff, act_kind, limit, code(h.dtype), _stream(h)))
        torch.mm(hid[at: at + c], wd[e].t(), out=out[at: at + c])
        at += c
    _check(lib.exl3_mix_moe_combine(_p(y), _p(out), _p(where), _p(wts), n, top, width, code(h.dtype), _stream(h)))


_identity: dict = {}


def moe_expert_major(y, h, wg, wu, wd, idx, wts, act_kind: int = 0, limit: float = 0.0):
    """Experts of a handful to a few dozen rows: each chosen expert's weights are streamed once for all its rows (no host read: capturable)."""
    n, width = h.shape
    experts, ff, _ = wg.shape
    top = idx.shape[1]
    _req(h.is_contiguous() and wg.is_contiguous() and wu.is_contiguous() and wd.is_contiguous() and y.is_contiguous() and y.dtype == h.dtype == wg.dtype, "moe_expert_major: layout")
    _i32c(idx, "idx"); _f32c(wts, "wts")
    hid = torch.empty((n * top, ff), dtype=h.dtype, device=h.device)
    per = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
    key = (n * top, h.device)
    if key not in _identity:
        _identity[key] = torch.arange(n * top, dtype=torch.int32, device=h.device)
    lib = _lib.mixlib()
    _check(lib.exl3_mix_moe_expert_major_act(_p(per), _p(hid), _p(h), _p(wg), _p(wu), _p(wd), _p(idx), n, top, experts, ff, width, act_kind, limit, code(h.dtype), _stream(h)))
    _check(lib.exl3_mix_moe_combine(_p(y), _p(per), _p(_identity[key]), _p(wts), n, top, width, code(h.dtype), _stream(h)))


def moe_vector_layout(h, ff: int) -> bool:
    vn = 8 if h.dtype == torch.bfloat16 else 4
    return h.shape[1] % vn == 0 and ff % vn == 0


# ---- pre-norm blocks with a statistics-free norm, gated activations, sigmoid router (csrc/mix_rowops.hip) ------------------------------------------
GLU_SILU, GLU_CLAMPED_SWISH = 0, 1
ACT_RELU2, ACT_GELU_TANH, ACT_SILU = 0, 1, 2
RES_KEEP, RES_ADD, RES_SET = 0, 1, 2
OUT_NONE, OUT_CAST, OUT_DYN_TANH = 0, 1, 2


def embed_copy(x: torch.Tensor, xc_view: torch.Tensor | None, table: torch.Tensor, tokens: torch.Tensor):
    n, width = x.shape
    _f32c(x, "x"); _i32c(tokens, "tokens")
    _req(tokens.numel() == n and table.is_contiguous() and table.shape[1] == width, "embed_copy: shapes")
    if xc_view is not None:
        _req(xc_view.dtype == table.dtype and xc_view.shape[0] == n, "embed_copy: the copy has the table's element type")
    _check(_lib.mixlib().exl3_mix_embed_copy(_p(x), _p(xc_view), 0 if xc_view is None else _view(xc_view, width, "xc"), _p(table), _p(tokens), n, width, table.shape[0],
                                              code(table.dtype), _stream(x)))


def residual_norm(x: torch.Tensor, y_view: torch.Tensor | None, mode: int, rms_w: torch.Tensor | None, eps: float, out: int, alpha: float, w: torch.Tensor | None,
                  b: torch.Tensor | None, h_view: torch.Tensor | None):
    """x (float32 residual, in place) = x | x + y' | y', y' = y or y / rms(y) * rms_w; h = nothing | x in the activation type | tanh(alpha x) w + b."""
    n, width = x.shape
    _f32c(x, "x")
    ref = y_view if y_view is not None else h_view
    _req(ref is not None, "residual_norm: nothing to do")
    if mode != RES_KEEP:
        _req(y_view is not None and y_view.shape[0] == n, "residual_norm: y")
    if rms_w is not None:
        _f32c(rms_w, "rms_w"); _req(rms_w.numel() == width, "residual_norm: rms_w")
    if out != OUT_NONE:
        _req(h_view is not None and h_view.shape[0] == n and h_view.dtype == ref.dtype, "residual_norm: h")
    if out == OUT_DYN_TANH:
        _f32c(w, "w"); _f32c(b, "b"); _req(w.numel() == width and b.numel() == width, "residual_norm: norm weight / bias")
    _check(_lib.mixlib().exl3_mix_residual_norm(_p(x), _p(y_view) if mode != RES_KEEP else None, 0 if (y_view is None or mode == RES_KEEP) else _view(y_view, width, "y"), mode,
                                                 _p(rms_w), eps, out, alpha, _p(w), _p(b), _p(h_view) if out != OUT_NONE else None,
                                                 0 if (h_view is None or out == OUT_NONE) else _view(h_view, width, "h"), n, width, code(ref.dtype), _stream(x)))


def dyn_tanh_rows(h: torch.Tensor, x: torch.Tensor, rows: torch.Tensor | None, alpha: float, w: torch.Tensor, b: torch.Tensor):
    n, width = h.shape
    _f32c(x, "x"); _f32c(w, "w"); _f32c(b, "b")
    _req(h.is_contiguous() and x.shape[1] == width and w.numel() == width and b.numel() == width, "dyn_tanh_rows: shapes")
    if rows is not None:
        _i32c(rows, "rows"); _req(rows.numel() == n, "dyn_tanh_rows: rows")
    else:
        _req(x.shape[0] == n, "dyn_tanh_rows: rows of x")
    _check(_lib.mixlib().exl3_mix_dyn_tanh_rows(_p(h), _p(x), _p(rows), alpha, _p(w), _p(b), n, width, code(h.dtype), _stream(x)))


def act(out: torch.Tensor, z_view: torch.Tensor, kind: int):
    n, ff = out.shape
    _req(out.is_contiguous() and z_view.dtype == out.dtype and z_view.shape[0] == n, "act: shapes")
    _check(_lib.mixlib().exl3_mix_act(_p(out), _p(z_view), _view(z_view, ff, "z"), n, ff, kind, code(out.dtype), _stream(out)))


def glu_act(out: torch.Tensor, g_view: torch.Tensor, u_view: torch.Tensor, kind: int, limit: float = 0.0):
    n, ff = out.shape
    _req(out.is_contiguous() and g_view.dtype == out.dtype == u_view.dtype and g_view.shape[0] == n and u_view.shape[0] == n, "glu_act: shapes")
    _check(_lib.mixlib().exl3_mix_glu_act(_p(out), _p(g_view), _view(g_view, ff, "g"), _p(u_view), _view(u_view, ff, "u"), n, ff, kind, limit, code(out.dtype), _stream(out)))


def token_gate(out: torch.Tensor, gate_view: torch.Tensor, table: torch.Tensor, col0: int, tokens: torch.Tensor):
    n, dim = out.shape
    _i32c(tokens, "tokens")
    _req(out.is_contiguous() and gate_view.dtype == out.dtype == table.dtype and table.is_contiguous() and table.dim() == 2 and tokens.numel() == n
         and 0 <= col0 and col0 + dim <= table.shape[1], "token_gate: shapes")
    _check(_lib.mixlib().exl3_mix_token_gate(_p(out), _p(gate_view), _view(gate_view, dim, "gate"), _p(table), table.shape[1], col0, _p(tokens), n, dim, table.shape[0],
                                              code(out.dtype), _stream(out)))


def heads_gate(out: torch.Tensor, a: torch.Tensor, a_row: int, a_head: int, gate_view: torch.Tensor | None, heads: int, vdim: int):
    """a is addressed as base + n * a_row + h * a_head + v (token-major or head-major); the gate, if any, is [n, heads * vdim] before its sigmoid."""
    n = out.shape[0]
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and a.dtype == out.dtype and a.numel() >= n * heads * vdim, "heads_gate: shapes")
    if gate_view is not None:
        _req(gate_view.dtype == out.dtype and gate_view.shape[0] == n, "heads_gate: gate")
    _check(_lib.mixlib().exl3_mix_heads_gate(_p(out), _p(a), a_row, a_head, _p(gate_view), 0 if gate_view is None else _view(gate_view, heads * vdim, "gate"), n, heads, vdim,
                                              code(out.dtype), _stream(out)))


def topk_sigmoid(idx, wts, logits, correction: torch.Tensor | None, scale: float, normalise: bool = True):
    n, experts = logits.shape
    top = idx.shape[1]
    _f32c(logits, "logits"); _f32c(wts, "wts"); _i32c(idx, "idx")
    _req(idx.shape == wts.shape == (n, top), "topk_sigmoid: shapes")
    if correction is not None:
        _f32c(correction, "correction"); _req(correction.numel() == experts, "topk_sigmoid: correction")
    _check(_lib.mixlib().exl3_mix_topk_sigmoid(_p(idx), _p(wts), _p(logits), _p(correction), scale, 1 if normalise else 0, n, experts, top, _stream(logits)))


# ---- latent attention (csrc/mix_latent.hip) -----------------------------------------------------------------------------------------------------
def latent_prep(ckr, ring, dkv_view, norm_w, q_view, tok_seq, tok_pos, slots, len_after, freq, mag: float, eps: float, heads: int, dim: int, rot_dim: int, rank: int):
    n = ckr.shape[0]
    n_slots, window, row = ring.shape
    _f32c(norm_w, "norm_w"); _f32c(freq, "freq")
    _req(row == rank + rot_dim and ckr.shape == (n, row) and ckr.is_contiguous() and ring.is_contiguous() and norm_w.numel() == rank, "latent_prep: cache shapes")
    _req(ckr.dtype == ring.dtype == dkv_view.dtype == q_view.dtype, "latent_prep: element types")
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots"), (len_after, "len_after")):
        _i32c(t, nm)
    rot_dims = 2 * freq.numel()
    _req(tok_seq.numel() == n and tok_pos.numel() == n and dkv_view.shape[0] == n and q_view.shape[0] == n and rot_dims <= rot_dim, "latent_prep: rows")
    _check(_lib.mixlib().exl3_mix_latent_prep(_p(ckr), _p(ring), _p(dkv_view), _view(dkv_view, row, "dkv"), _p(norm_w), _p(q_view), _view(q_view, heads * (dim + rot_dim), "q"),
                                               _p(tok_seq), _p(tok_pos), _p(slots), _p(len_after), _p(freq), mag, eps, n, heads, dim, rot_dim, rot_dims, rank, window,
                                               code(ckr.dtype), _stream(ckr)))


def latent_fill_k(k: torch.Tensor, ckr: torch.Tensor, heads: int, dim: int, rot_dim: int, rank: int):
    n = k.shape[0]
    _req(k.dtype == ckr.dtype and ckr.is_contiguous() and ckr.shape == (n, rank + rot_dim), "latent_fill_k: shapes")
    _check(_lib.mixlib().exl3_mix_latent_fill_k(_p(k), _view(k, heads * (dim + rot_dim), "k"), _p(ckr), n, heads, dim, rot_dim, rank, code(k.dtype), _stream(k)))


# decode steps on the matrix cores: the cached rows of a sequence are split so that about this many workgroups are in flight (three fit a CU), and no
# split is shorter than two 32-key tiles (every split costs a partial sum as large as 58 cached rows, and a term in the merge)
LATENT_MFMA_TARGET_WAVES = 512


def latent_mfma_ok(dtype, rank: int, rot_dim: int) -> bool:
    return dtype == torch.bfloat16 and rank % 8 == 0 and rot_dim % 8 == 0 and rank <= 512 and rot_dim <= 128


def latent_decode(o_lat: torch.Tensor, q_lat: torch.Tensor, q_view: torch.Tensor, ring: torch.Tensor, sink, slots, len_after, dim: int, rot_dim: int, scale: float,
                  mfma: bool | None = None):
    """o_lat, q_lat: [heads, n, rank] (any strides with a unit last one); q_view [n, heads * (dim + rot_dim)] holds the rotated parts.
    mfma None: the matrix-core kernel where it applies (bfloat16, rank and rot_dim multiples of 8, rank <= 512, rot_dim <= 128)."""
    heads, n, rank = q_lat.shape
    n_slots, window, row = ring.shape
    if mfma is None:
        mfma = latent_mfma_ok(o_lat.dtype, rank, rot_dim)
    if mfma:
        _req(latent_mfma_ok(o_lat.dtype, rank, rot_dim), "latent_decode: the matrix-core kernel takes bfloat16, rank and rot_dim multiples of 8, rank <= 512, rot_dim <= 128")
        _req(o_lat.shape == q_lat.shape and o_lat.stride(2) == 1 and q_lat.stride(2) == 1 and row == rank + rot_dim and ring.is_contiguous(), "latent_decode: shapes")
        _req(o_lat.dtype == q_lat.dtype == q_view.dtype == ring.dtype and slots.numel() == n and len_after.numel() == n and q_view.shape[0] == n, "latent_decode: types / rows")
        if sink is not None:
            _f32c(sink, "sink"); _req(sink.numel() == heads, "latent_decode: sink")
        groups = (heads + 15) // 16
        splits = max(1, min(LATENT_MFMA_TARGET_WAVES // max(1, n * groups), (window + 63) // 64))
        rp = 128 if rank <= 128 else (256 if rank <= 256 else 512)
        scratch = torch.empty(n * splits * heads * (rp + 2), dtype=torch.float32, device=o_lat.device)
        _check(_lib.mixlib().exl3_mix_latent_decode_mfma(_p(o_lat), o_lat.stride(1), o_lat.stride(0), _p(q_lat), q_lat.stride(1), q_lat.stride(0), _p(q_view),
                                                          _view(q_view, heads * (dim + rot_dim), "q"), _p(ring), _p(sink), _p(slots), _p(len_after), _p(scratch), splits,
                                                          n, heads, dim, rot_dim, rank, scale, window, _stream(o_lat)))
        return
    _req(o_lat.shape == q_lat.shape and o_lat.stride(2) == 1 and q_lat.stride(2) == 1 and row == rank + rot_dim and ring.is_contiguous(), "latent_decode: shapes")
    _req(o_lat.dtype == q_lat.dtype == q_view.dtype == ring.dtype, "latent_decode: element types")
    _req(slots.numel() == n and len_after.numel() == n and q_view.shape[0] == n, "latent_decode: one row per sequence")
    if sink is not None:
        _f32c(sink, "sink"); _req(sink.numel() == heads, "latent_decode: sink")
    _check(_lib.mixlib().exl3_mix_latent_decode(_p(o_lat), o_lat.stride(1), o_lat.stride(0), _p(q_lat), q_lat.stride(1), q_lat.stride(0), _p(q_view),
                                                 _view(q_view, heads * (dim + rot_dim), "q"), _p(ring), _p(sink), _p(slots), _p(len_after), n, heads, dim, rot_dim, rank,
                                                 scale, window, code(o_lat.dtype), _stream(o_lat)))


def moe_gate_up_act(hid, h, wg, wu, idx, act_kind: int, limit: float):
    n, width = h.shape
    experts, ff, w2 = wg.shape
    top = idx.shape[1]
    _req(h.is_contiguous() and wg.is_contiguous() and wu.is_contiguous() and wu.shape == wg.shape and w2 == width and hid.is_contiguous()
         and hid.shape == (n * top, ff) and hid.dtype == h.dtype == wg.dtype, "moe_gate_up: shapes")
    _i32c(idx, "idx")
    _check(_lib.mixlib().exl3_mix_moe_gate_up_act(_p(hid), _p(h), _p(wg), _p(wu), _p(idx), n, top, experts, ff, width, act_kind, limit, code(h.dtype), _stream(h)))


# ---- several attention maps per head, chunk masks, soft-capped scores; normed and rotated queries / keys (csrc/mix_attn*.hip, mix_diffattn.hip) ---------
MASK_WINDOW, MASK_CHUNK = 0, 1


def qk_prep(q_view, k_view, v_view, q_norm, k_norm, freq, mag: float, interleaved: bool, eps: float, ring_k, ring_v, tok_seq, tok_pos, slots, len_after, dim: int):
    """In place on the step's queries and keys: RMS norm per (row, head, map) with a shared weight (None: no norm), rotary positions over 2 * len(freq)
    leading entries (None: no rotation); keys and values of the rows a sequence keeps go into the rings."""
    n = q_view.shape[0]
    n_slots, window, k_heads, d2 = ring_k.shape
    v_heads, vdim = ring_v.shape[2], ring_v.shape[3]
    _req(d2 == dim and ring_v.shape[:2] == (n_slots, window) and ring_k.is_contiguous() and ring_v.is_contiguous(), "qk_prep: ring shapes")
    _req(q_view.shape[1] % dim == 0 and k_view.shape == (n, k_heads * dim) and v_view.shape == (n, v_heads * vdim), "qk_prep: step shapes")
    _req(q_view.dtype == k_view.dtype == v_view.dtype == ring_k.dtype == ring_v.dtype, "qk_prep: element types")
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots"), (len_after, "len_after")):
        _i32c(t, nm)
    for t, nm in ((q_norm, "q_norm"), (k_norm, "k_norm")):
        if t is not None:
            _f32c(t, nm); _req(t.numel() == dim, f"qk_prep: {nm}")
    if freq is not None:
        _f32c(freq, "freq")
    q_heads = q_view.shape[1] // dim
    _req(tok_seq.numel() == n and tok_pos.numel() == n, "qk_prep: rows")
    _check(_lib.mixlib().exl3_mix_qk_prep(_p(q_view), _view(q_view, q_heads * dim, "q"), _p(k_view), _view(k_view, k_heads * dim, "k"), _p(v_view),
                                           _view(v_view, v_heads * vdim, "v"), _p(q_norm), _p(k_norm), _p(freq), 0 if freq is None else 2 * freq.numel(), mag,
                                           1 if interleaved else 0, eps, _p(ring_k), _p(ring_v), _p(tok_seq), _p(tok_pos), _p(slots), _p(len_after),
                                           n, q_heads, k_heads, v_heads, dim, vdim, window, code(q_view.dtype), _stream(q_view)))


def attn_prefill_maps(out, q_view, k_view, v_view, gate_view, sink, cu, tok_seq, tok_pos, heads: int, kv_heads: int, maps: int, dim: int, vdim: int, scale: float,
                      softcap: float, window: int, mask: int, max_rows: int = 0, mfma: bool | None = None):
    """Prompt-step attention over the step's own keys with `maps` maps per head, a soft cap and a window or chunk mask.  out [n, heads * maps * vdim] in
    float32 or the activation type.  mfma None: the matrix-core kernel for bfloat16 steps from ATTN_MFMA_MIN_ROWS rows."""
    n = q_view.shape[0]
    _req(out.is_contiguous() and out.shape == (n, heads * maps * vdim) and out.dtype in (torch.float32, q_view.dtype), "attn_prefill_maps: out")
    _req(q_view.dtype == k_view.dtype == v_view.dtype and k_view.shape[0] == n and v_view.shape[0] == n, "attn_prefill_maps: step tensors")
    if sink is not None:
        _f32c(sink, "sink"); _req(sink.numel() == heads and maps == 1, "attn_prefill_maps: sink")
    out_f32 = 1 if (out.dtype == torch.float32 and q_view.dtype != torch.float32) else 0
    gate_ld = 0 if gate_view is None else _view(gate_view, heads, "gate")
    if mfma is None:
        mfma = q_view.dtype == torch.bfloat16 and max_rows >= ATTN_MFMA_MIN_ROWS and dim <= 256 and vdim <= 256 and scale > 0
    if mfma:
        _req(q_view.dtype == torch.bfloat16 and max_rows > 0, "attn_prefill_maps: the matrix-core kernel takes bfloat16 and the step's longest sequence")
        _check(_lib.mixlib().exl3_mix_attn_prefill_mfma_ex(_p(out), out_f32, _p(q_view), _view(q_view, heads * maps * dim, "q"), _p(k_view), _view(k_view, kv_heads * maps * dim, "k"),
                                                            _p(v_view), _view(v_view, kv_heads * vdim, "v"), _p(gate_view), gate_ld, _p(sink), _p(cu), cu.numel() - 1, max_rows,
                                                            heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask, _stream(out)))
        return
    _check(_lib.mixlib().exl3_mix_attn_prefill_ex(_p(out), out_f32, _p(q_view), _view(q_view, heads * maps * dim, "q"), _p(k_view), _view(k_view, kv_heads * maps * dim, "k"),
                                                   _p(v_view), _view(v_view, kv_heads * vdim, "v"), _p(gate_view), gate_ld, _p(sink), _p(cu), _p(tok_seq), _p(tok_pos),
                                                   n, heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask, code(q_view.dtype), _stream(out)))


def diff_mfma_ok(dtype, max_rows: int, dim: int, vdim: int, scale: float) -> bool:
    return dtype == torch.bfloat16 and max_rows >= ATTN_MFMA_MIN_ROWS and dim <= 128 and vdim <= 256 and scale > 0


def attn_prefill_diff(out, q_view, k_view, v_view, gate_view, cu, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, softcap: float, window: int, mask: int,
                      lam: float, diff: float, eps: float, max_rows: int):
    """Prompt-step differential attention on the matrix cores (bfloat16): both maps of every head and their combination in one kernel; out [n, heads * vdim]."""
    n = q_view.shape[0]
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and out.dtype == q_view.dtype == k_view.dtype == v_view.dtype == torch.bfloat16 and max_rows > 0,
         "attn_prefill_diff: bfloat16 tensors and the step's longest sequence")
    _req(k_view.shape[0] == n and v_view.shape[0] == n, "attn_prefill_diff: step tensors")
    if gate_view is not None:
        _req(gate_view.dtype == out.dtype and gate_view.shape[0] == n, "attn_prefill_diff: gate")
    _check(_lib.mixlib().exl3_mix_attn_prefill_mfma_diff(_p(out), _p(q_view), _view(q_view, heads * 2 * dim, "q"), _p(k_view), _view(k_view, kv_heads * 2 * dim, "k"), _p(v_view),
                                                          _view(v_view, kv_heads * vdim, "v"), _p(gate_view), 0 if gate_view is None else _view(gate_view, heads, "gate"), _p(cu),
                                                          cu.numel() - 1, max_rows, heads, kv_heads, dim, vdim, scale, softcap, window, mask, lam, diff, eps, _stream(out)))


def attn_decode_maps(out, q_view, ring_k, ring_v, gate_view, sink, slots, len_after, heads: int, maps: int, scale: float, softcap: float, mask: int):
    """One new row per sequence against the rings (ring_k [slots, window, kv_heads * maps, dim], ring_v [slots, window, kv_heads, vdim])."""
    n = out.shape[0]
    n_slots, window, k_heads, dim = ring_k.shape
    kv_heads, vdim = ring_v.shape[2], ring_v.shape[3]
    _req(k_heads == kv_heads * maps and ring_k.is_contiguous() and ring_v.is_contiguous() and ring_k.dtype == ring_v.dtype == q_view.dtype, "attn_decode_maps: rings")
    _req(out.is_contiguous() and out.shape == (n, heads * maps * vdim) and out.dtype in (torch.float32, q_view.dtype), "attn_decode_maps: out")
    _req(slots.numel() == n and len_after.numel() == n and q_view.shape[0] == n, "attn_decode_maps: one row per sequence")
    if sink is not None:
        _f32c(sink, "sink"); _req(sink.numel() == heads and maps == 1, "attn_decode_maps: sink")
    out_f32 = 1 if (out.dtype == torch.float32 and q_view.dtype != torch.float32) else 0
    _check(_lib.mixlib().exl3_mix_attn_decode_ex(_p(out), out_f32, _p(q_view), _view(q_view, heads * maps * dim, "q"), _p(ring_k), _p(ring_v), _p(gate_view),
                                                  0 if gate_view is None else _view(gate_view, heads, "gate"), _p(sink), _p(slots), _p(len_after),
                                                  n, heads, kv_heads, maps, dim, vdim, scale, softcap, window, mask, code(q_view.dtype), _stream(out)))


def diff_combine(out, a, lam: float, diff: float, eps: float, gate_view, heads: int, vdim: int):
    """a [n, heads * 2 * vdim] float32 (two maps per head) -> out [n, heads * vdim] = rms_unit(a1 - lam a2) (1 - diff) sigmoid(gate)."""
    n = out.shape[0]
    _f32c(a, "a")
    _req(a.shape == (n, heads * 2 * vdim) and out.is_contiguous() and out.shape == (n, heads * vdim), "diff_combine: shapes")
    if gate_view is not None:
        _req(gate_view.dtype == out.dtype and gate_view.shape[0] == n, "diff_combine: gate")
    _check(_lib.mixlib().exl3_mix_diff_combine(_p(out), _p(a), lam, diff, eps, _p(gate_view), 0 if gate_view is None else _view(gate_view, heads, "gate"),
                                                n, heads, vdim, code(out.dtype), _stream(out)))


# ---- residual update + RMS norm + short causal input convolution (csrc/mix_canon.hip) ----------------------------------------------------------------
def residual_rms(x, y_view, mode: int, w, eps: float, h_view, conv_w=None, ring=None, tok_seq=None, tok_pos=None, slots=None):
    """x (float32, in place) = x | x + y | y (RES_*); h = rms_norm(x) * w, and with conv_w [taps, width] (steps of one row per sequence) h + its causal
    convolution over the ring [slots, taps - 1, width] of earlier normed rows, which also receives the new one.  h_view None: the update alone."""
    n, width = x.shape
    _f32c(x, "x")
    ref = y_view if y_view is not None else h_view
    _req(ref is not None, "residual_rms: nothing to do")
    if mode != RES_KEEP:
        _req(y_view is not None and y_view.shape[0] == n, "residual_rms: y")
    if h_view is not None:
        _f32c(w, "w"); _req(w.numel() == width and h_view.shape[0] == n and h_view.dtype == ref.dtype, "residual_rms: h / w")
    taps = 0
    if conv_w is not None:
        _f32c(conv_w, "conv_w"); taps = conv_w.shape[0]
        _req(conv_w.shape[1] == width and ring is not None and ring.is_contiguous() and ring.shape[1:] == (max(taps - 1, 1), width) and ring.dtype == ref.dtype,
             "residual_rms: convolution weights / ring")
        for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots")):
            _i32c(t, nm)
    _check(_lib.mixlib().exl3_mix_residual_rms(_p(x), _p(y_view) if mode != RES_KEEP else None, 0 if (y_view is None or mode == RES_KEEP) else _view(y_view, width, "y"), mode,
                                                _p(w), eps, _p(h_view), 0 if h_view is None else _view(h_view, width, "h"), _p(conv_w), taps, _p(ring), _p(tok_seq), _p(tok_pos),
                                                _p(slots), n, width, code(ref.dtype), _stream(x)))


def canon(out, hn, conv_w, ring, tok_seq, tok_pos, slots, pos0, len_after):
    """out = hn + causal convolution of hn over time per channel (conv_w [taps, width]: tap-major) for a packed step; the ring keeps each sequence's last
    taps - 1 rows."""
    n, width = hn.shape
    taps = conv_w.shape[0]
    _f32c(conv_w, "conv_w")
    _req(out.shape == hn.shape and out.dtype == hn.dtype == ring.dtype and conv_w.shape[1] == width and ring.is_contiguous() and ring.shape[1:] == (max(taps - 1, 1), width),
         "canon: shapes")
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots"), (pos0, "pos0"), (len_after, "len_after")):
        _i32c(t, nm)
    _check(_lib.mixlib().exl3_mix_canon(_p(out), _view(out, width, "out"), _p(hn), _view(hn, width, "hn"), _p(conv_w), taps, _p(ring), _p(tok_seq), _p(tok_pos), _p(slots),
                                         _p(pos0), _p(len_after), n, width, code(hn.dtype), _stream(hn)))


def softcap(x: torch.Tensor, cap: float):
    """x <- cap tanh(x / cap) in place (float32, contiguous)."""
    _f32c(x, "x")
    _check(_lib.mixlib().exl3_mix_softcap(_p(x), x.numel(), cap, _stream(x)))


# ---- grouped routers, experts without weights, ungated experts (csrc/mix_rowops.hip, mix_moe.hip) ------------------------------------------------------
ROUTE_SOFTMAX_ALL, ROUTE_SIGMOID = 0, 1


def topk_grouped(idx, wts, idw, logits, correction, kind: int, real: int, groups: int = 1, keep: int = 1, scale: float = 1.0, normalise: bool = True):
    """logits [n, total]: outputs >= real stand for experts that return their input (written as idx = real, weight 0, their weights summed into idw [n])."""
    n, total = logits.shape
    top = idx.shape[1]
    _f32c(logits, "logits"); _f32c(wts, "wts"); _i32c(idx, "idx")
    _req(idx.shape == wts.shape == (n, top), "topk_grouped: shapes")
    if idw is not None:
        _f32c(idw, "idw"); _req(idw.numel() == n, "topk_grouped: idw")
    if correction is not None:
        _f32c(correction, "correction"); _req(correction.numel() == total, "topk_grouped: correction")
    _check(_lib.mixlib().exl3_mix_topk_grouped(_p(idx), _p(wts), _p(idw), _p(logits), _p(correction), kind, scale, 1 if normalise else 0, groups, keep, n, total, real, top,
                                                _stream(logits)))


def moe_up_act(hid, h, wu, idx, act_kind: int):
    n, width = h.shape
    experts, ff, w2 = wu.shape
    top = idx.shape[1]
    _req(h.is_contiguous() and wu.is_contiguous() and w2 == width and hid.is_contiguous() and hid.shape == (n * top, ff) and hid.dtype == h.dtype == wu.dtype, "moe_up_act: shapes")
    _i32c(idx, "idx")
    _check(_lib.mixlib().exl3_mix_moe_up_act(_p(hid), _p(h), _p(wu), _p(idx), n, top, experts, ff, width, act_kind, code(h.dtype), _stream(h)))


def moe_down_id(y, hid, wd, idx, wts, h_id=None, idw=None):
    n, width = y.shape
    experts, w2, ff = wd.shape
    top = idx.shape[1]
    _req(y.is_contiguous() and hid.is_contiguous() and wd.is_contiguous() and w2 == width and hid.shape == (n * top, ff) and y.dtype == hid.dtype == wd.dtype, "moe_down: shapes")
    _i32c(idx, "idx"); _f32c(wts, "wts")
    if idw is not None:
        _f32c(idw, "idw"); _req(h_id is not None and h_id.is_contiguous() and h_id.shape == y.shape and h_id.dtype == y.dtype, "moe_down: the identity share needs the input rows")
    _check(_lib.mixlib().exl3_mix_moe_down_id(_p(y), _p(hid), _p(wd), _p(idx), _p(wts), _p(h_id) if idw is not None else None, _p(idw), n, top, experts, ff, width,
                                               code(y.dtype), _stream(y)))


def moe_expert_major_plain(y, h, wu, wd, idx, wts, act_kind: int, idw=None):
    """Ungated experts of a handful to a few dozen rows, expert-major; idw: per-row weight of the experts that return their input."""
    n, width = h.shape
    experts, ff, _ = wu.shape
    top = idx.shape[1]
    _req(h.is_contiguous() and wu.is_contiguous() and wd.is_contiguous() and y.is_contiguous() and y.dtype == h.dtype == wu.dtype, "moe_expert_major_plain: layout")
    _i32c(idx, "idx"); _f32c(wts, "wts")
    hid = torch.empty((n * top, ff), dtype=h.dtype, device=h.device)
    per = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
    key = (n * top, h.device)
    if key not in _identity:
        _identity[key] = torch.arange(n * top, dtype=torch.int32, device=h.device)
    lib = _lib.mixlib()
    _check(lib.exl3_mix_moe_expert_major_plain(_p(per), _p(hid), _p(h), _p(wu), _p(wd), _p(idx), n, top, experts, ff, width, act_kind, code(h.dtype), _stream(h)))
    _check(lib.exl3_mix_moe_combine_id(_p(y), _p(per), _p(_identity[key]), _p(wts), _p(idx), experts, _p(h) if idw is not None else None, _p(idw), n, top, width,
                                        code(h.dtype), _stream(h)))


def moe_grouped_plain(y, h, wu, wd, idx, wts, act_kind: int, idw=None):
    """Ungated experts of many rows: rows sorted by expert (device), one host read of the per-expert counts, per expert two vendor matrix products with the
    activation kernel between them, and the weighted un-sort (which leaves out the choices without a stored expert and adds the identity share)."""
    n, width = h.shape
    experts, ff, _ = wu.shape
    top = idx.shape[1]
    flat = idx.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    counts = torch.zeros(experts + 1, dtype=torch.int32, device=h.device).index_add_(0, flat, torch.ones_like(flat, dtype=torch.int32)).tolist()
    where = torch.empty(n * top, dtype=torch.int32, device=h.device)
    where[order] = torch.arange(n * top, dtype=torch.int32, device=h.device)
    stored = sum(counts[:experts])
    xs = h.index_select(0, order[:stored] // top)
    out = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
    hid = torch.empty((max(stored, 1), ff), dtype=h.dtype, device=h.device)
    lib, at = _lib.mixlib(), 0
    for e, c in enumerate(counts[:experts]):
        if c == 0:
            continue
        u = torch.nn.functional.linear(xs[at: at + c], wu[e])
        _check(lib.exl3_mix_act(_p(hid[at: at + c]), _p(u), ff, c, ff, act_kind, code(h.dtype), _stream(h)))
        torch.mm(hid[at: at + c], wd[e].t(), out=out[at: at + c])
        at += c
    _check(lib.exl3_mix_moe_combine_id(_p(y), _p(out), _p(where), _p(wts), _p(idx), experts, _p(h) if idw is not None else None, _p(idw), n, top, width,
                                        code(h.dtype), _stream(h)))


# ---- parallel blocks over a layer norm, attention without softmax over paged keys, recurrent mixers with a scalar decay per head ----

GATE_SILU, GATE_SIGMOID = 0, 1
SIG_MFMA_MIN_ROWS = 32


def embed_sinusoid(x: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor, tok_pos: torch.Tensor, freq: torch.Tensor, scale: float):
    """x (float32) = table[tokens] * scale + the sinusoidal vector of each row's position (freq: float32 [ceil(width / 2)])."""
    n, width = x.shape
    _f32c(x, "x"); _f32c(freq, "freq"); _i32c(tokens, "tokens"); _i32c(tok_pos, "tok_pos")
    _req(tokens.numel() == n and tok_pos.numel() == n and table.is_contiguous() and table.shape[1] == width and freq.numel() >= (width + 1) // 2, "embed_sinusoid: shapes")
    _check(_lib.mixlib().exl3_mix_embed_sinusoid(_p(x), _p(table), _p(tokens), _p(tok_pos), _p(freq), scale, n, width, table.shape[0], code(table.dtype), _stream(x)))


def layer_norm_rows(h: torch.Tensor, x: torch.Tensor, rows: torch.Tensor | None, w: torch.Tensor, b: torch.Tensor | None, eps: float):
    n, width = h.shape
    _f32c(x, "x"); _f32c(w, "w")
    _req(h.is_contiguous() and x.shape[1] == width and w.numel() == width, "layer_norm_rows: shapes")
    if b is not None:
        _f32c(b, "b"); _req(b.numel() == width, "layer_norm_rows: bias")
    if rows is not None:
        _i32c(rows, "rows"); _req(rows.numel() == n, "layer_norm_rows: rows")
    else:
        _req(x.shape[0] == n, "layer_norm_rows: rows of x")
    _check(_lib.mixlib().exl3_mix_layer_norm_rows(_p(h), _p(x), _p(rows), _p(w), _p(b), eps, n, width, code(h.dtype), _stream(x)))


def residual_norm_conv(x, y_view, y2_view, y_scale: float, mode: int, center: bool, w, bias, eps: float, h_view, hn_view=None, conv_w=None, ring=None, tok_seq=None,
                       tok_pos=None, slots=None):
    """x (float32, in place) = x | x + (y + y2) * y_scale | (y + y2) * y_scale; then the norm of x (center: layer norm with weight and optional bias, else RMS norm
    with weight) into hn_view and / or h_view; with conv_w [taps, width] (steps of one row per sequence) h = normed row + its causal convolution over the slot's
    ring, which receives the new normed row."""
    n, width = x.shape
    _f32c(x, "x")
    ref = next((t for t in (y_view, h_view, hn_view) if t is not None), None)
    _req(ref is not None, "residual_norm_conv: nothing to do")
    if mode != RES_KEEP:
        _req(y_view is not None and y_view.shape[0] == n and (y2_view is None or (y2_view.shape[0] == n and y2_view.dtype == y_view.dtype)), "residual_norm_conv: y")
    else:
        y_view = y2_view = None
    if h_view is not None or hn_view is not None:
        _f32c(w, "w"); _req(w.numel() == width, "residual_norm_conv: w")
        if bias is not None:
            _f32c(bias, "bias"); _req(bias.numel() == width and center, "residual_norm_conv: bias")
        for t in (h_view, hn_view):
            _req(t is None or (t.shape[0] == n and t.dtype == ref.dtype), "residual_norm_conv: h")
    taps = 0
    if conv_w is not None:
        _f32c(conv_w, "conv_w"); taps = conv_w.shape[0]
        _req(conv_w.shape[1] == width and ring is not None and ring.is_contiguous() and ring.shape[1:] == (max(taps - 1, 1), width) and ring.dtype == ref.dtype,
             "residual_norm_conv: convolution weights / ring")
        for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots")):
            _i32c(t, nm)
    ld = lambda t, nm: 0 if t is None else _view(t, width, nm)
    _check(_lib.mixlib().exl3_mix_residual_norm_conv(_p(x), _p(y_view), ld(y_view, "y"), _p(y2_view), ld(y2_view, "y2"), y_scale, mode, 1 if center else 0, _p(w), _p(bias), eps,
                                                      _p(h_view), ld(h_view, "h"), _p(hn_view), ld(hn_view, "hn"), _p(conv_w), taps, _p(ring), _p(tok_seq), _p(tok_pos), _p(slots),
                                                      n, width, code(ref.dtype), _stream(x)))


def glu_act_rowgate(out: torch.Tensor, g_view: torch.Tensor, u_view: torch.Tensor, row_gate: torch.Tensor | None, kind: int, limit: float = 0.0):
    """out = glu(g, u) * sigmoid(row_gate[n]) (row_gate: [n, 1] view, one number per row)."""
    n, ff = out.shape
    _req(out.is_contiguous() and g_view.dtype == out.dtype == u_view.dtype and g_view.shape[0] == n and u_view.shape[0] == n, "glu_act_rowgate: shapes")
    if row_gate is not None:
        _req(row_gate.dtype == out.dtype and row_gate.shape == (n, 1), "glu_act_rowgate: the gate is one number per row")
    _check(_lib.mixlib().exl3_mix_glu_act_rowgate(_p(out), _p(g_view), _view(g_view, ff, "g"), _p(u_view), _view(u_view, ff, "u"), _p(row_gate),
                                                   0 if row_gate is None else max(row_gate.stride(0), 1), n, ff, kind, limit, code(out.dtype), _stream(out)))


def topk_grouped_ex(idx, wts, idw, logits, correction, kind: int, real: int, groups: int = 1, keep: int = 1, group_top: int = 1, scale: float = 1.0, normalise: bool = True):
    """topk_grouped with a group's score = the sum of its `group_top` largest choice scores."""
    n, total = logits.shape
    top = idx.shape[1]
    _f32c(logits, "logits"); _f32c(wts, "wts"); _i32c(idx, "idx")
    _req(idx.shape == wts.shape == (n, top), "topk_grouped: shapes")
    if idw is not None:
        _f32c(idw, "idw"); _req(idw.numel() == n, "topk_grouped: idw")
    if correction is not None:
        _f32c(correction, "correction"); _req(correction.numel() == total, "topk_grouped: correction")
    _check(_lib.mixlib().exl3_mix_topk_grouped_ex(_p(idx), _p(wts), _p(idw), _p(logits), _p(correction), kind, scale, 1 if normalise else 0, groups, keep, group_top, n, total, real,
                                                   top, _stream(logits)))


def _paged(k_pages, v_pages, table, name):
    _i32c(table, "page table")
    _req(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dim() == 3 and v_pages.dim() == 3 and k_pages.shape[:2] == v_pages.shape[:2] and table.dim() == 2
         and k_pages.dtype == v_pages.dtype, f"{name}: pools [pages, page, width] and a table [slots, pages per slot]")


def paged_store(k_pages, v_pages, k_view, v_view, table, tok_seq, tok_pos, slots):
    """The step's key / value rows into the pages of their sequences (pools [pages, page, kw] / [pages, page, vw])."""
    _paged(k_pages, v_pages, table, "paged_store")
    n = k_view.shape[0]
    kw, vw = k_pages.shape[2], v_pages.shape[2]
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots")):
        _i32c(t, nm)
    _req(k_view.dtype == k_pages.dtype == v_view.dtype and v_view.shape[0] == n and tok_seq.numel() == n, "paged_store: rows")
    _check(_lib.mixlib().exl3_mix_paged_store(_p(k_pages), _p(v_pages), _p(k_view), _view(k_view, kw, "k"), _p(v_view), _view(v_view, vw, "v"), _p(table), table.stride(0),
                                               k_pages.shape[1], _p(tok_seq), _p(tok_pos), _p(slots), n, kw, vw, code(k_view.dtype), _stream(k_view)))


def sig_mfma_ok(dtype, max_rows: int, dim: int, vdim: int) -> bool:
    return dtype == torch.bfloat16 and max_rows >= SIG_MFMA_MIN_ROWS and dim <= 256 and vdim <= 256


def sigattn_prefill(out, q_view, k_view, v_view, bias, cu, tok_seq, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, max_rows: int):
    """Prompt steps of the attention without softmax: out [n, heads * vdim] = sum over the row's keys of sigmoid(scale q.k + bias[head]) v.  bfloat16 steps of at
    least SIG_MFMA_MIN_ROWS rows run on the matrix cores, everything else in the exact float32-score kernel."""
    n = out.shape[0]
    _i32c(cu, "cu"); _i32c(tok_seq, "tok_seq")
    if bias is not None:
        _f32c(bias, "bias"); _req(bias.numel() == heads, "sigattn_prefill: one bias per head")
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and q_view.dtype == out.dtype == k_view.dtype == v_view.dtype, "sigattn_prefill: shapes")
    args = (_p(out), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_view), _view(k_view, kv_heads * dim, "k"), _p(v_view), _view(v_view, kv_heads * vdim, "v"), _p(bias), _p(cu))
    if sig_mfma_ok(out.dtype, max_rows, dim, vdim):
        _check(_lib.mixlib().exl3_mix_sigattn_prefill_mfma(*args, cu.numel() - 1, max_rows, heads, kv_heads, dim, vdim, scale, _stream(out)))
    else:
        _check(_lib.mixlib().exl3_mix_sigattn_prefill(*args, _p(tok_seq), n, heads, kv_heads, dim, vdim, scale, code(out.dtype), _stream(out)))


def sigattn_decode(out, q_view, k_pages, v_pages, bias, table, slots, len_after, heads: int, kv_heads: int, dim: int, vdim: int, scale: float):
    """Decode steps (one row per sequence): every sequence reads its len_after keys through the page table."""
    _paged(k_pages, v_pages, table, "sigattn_decode")
    n = out.shape[0]
    _i32c(slots, "slots"); _i32c(len_after, "len_after")
    if bias is not None:
        _f32c(bias, "bias"); _req(bias.numel() == heads, "sigattn_decode: one bias per head")
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and q_view.dtype == out.dtype == k_pages.dtype and k_pages.shape[2] == kv_heads * dim
         and v_pages.shape[2] == kv_heads * vdim and slots.numel() == n, "sigattn_decode: shapes")
    _check(_lib.mixlib().exl3_mix_sigattn_decode(_p(out), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_pages), _p(v_pages), _p(bias), _p(table), table.stride(0),
                                                  k_pages.shape[1], _p(slots), _p(len_after), n, heads, kv_heads, dim, vdim, scale, code(out.dtype), _stream(out)))


def mlstm_scan(o, S, nst, mst, q_view, k_view, v_view, zi_view, zf_view, bias_i, bias_f, cu, slots, pos0, q_scale: float, cap: float):
    """o [n, heads, vdim] float32; state per slot S [heads, vdim, dim], n [heads, dim], m [heads] (float32)."""
    n, heads, vdim = o.shape
    dim = S.shape[3]
    for t, nm in ((o, "o"), (S, "S"), (nst, "n"), (mst, "m"), (bias_i, "bias_i"), (bias_f, "bias_f")):
        _f32c(t, nm)
    for t, nm in ((cu, "cu"), (slots, "slots"), (pos0, "pos0")):
        _i32c(t, nm)
    _req(S.shape[1:] == (heads, vdim, dim) and nst.shape[1:] == (heads, dim) and mst.shape[1:] == (heads,) and bias_i.numel() == heads and bias_f.numel() == heads
         and q_view.dtype == k_view.dtype == v_view.dtype == zi_view.dtype == zf_view.dtype, "mlstm_scan: shapes")
    _check(_lib.mixlib().exl3_mix_mlstm_scan(_p(o), _p(S), _p(nst), _p(mst), _p(q_view), _view(q_view, heads * dim, "q"), _p(k_view), _view(k_view, heads * dim, "k"),
                                              _p(v_view), _view(v_view, heads * vdim, "v"), _p(zi_view), _view(zi_view, heads, "zi"), _p(zf_view), _view(zf_view, heads, "zf"),
                                              _p(bias_i), _p(bias_f), _p(cu), _p(slots), _p(pos0), cu.numel() - 1, heads, dim, vdim, q_scale, cap, code(q_view.dtype), _stream(o)))


def delta_prep(qo, ko, vo, beta, decay, x_view, conv_w, ring, zb_view, za_view, A_log, dt_bias, tok_seq, tok_pos, slots, pos0, len_after, heads: int, kv_heads: int, dim: int,
               vdim: int, q_scale: float):
    """The delta rule's input stage over x = q | k | v [n, C]: short convolutions (conv_w [taps, C], ring [slots, taps - 1, C]) with silu, unit query / key vectors,
    beta and decay; float32 results."""
    n = x_view.shape[0]
    C = 2 * kv_heads * dim + heads * vdim
    taps = conv_w.shape[0]
    for t, nm in ((qo, "qo"), (ko, "ko"), (vo, "vo"), (beta, "beta"), (decay, "decay"), (conv_w, "conv_w"), (A_log, "A_log"), (dt_bias, "dt_bias")):
        _f32c(t, nm)
    for t, nm in ((tok_seq, "tok_seq"), (tok_pos, "tok_pos"), (slots, "slots"), (pos0, "pos0"), (len_after, "len_after")):
        _i32c(t, nm)
    _req(qo.shape == ko.shape == (n, kv_heads * dim) and vo.shape == (n, heads * vdim) and beta.shape == decay.shape == (n, heads) and conv_w.shape[1] == C
         and ring.is_contiguous() and ring.shape[1:] == (max(taps - 1, 1), C) and ring.dtype == x_view.dtype == zb_view.dtype == za_view.dtype
         and A_log.numel() == heads and dt_bias.numel() == heads, "delta_prep: shapes")
    _check(_lib.mixlib().exl3_mix_delta_prep(_p(qo), _p(ko), _p(vo), _p(beta), _p(decay), _p(x_view), _view(x_view, C, "x"), _p(conv_w), taps, _p(ring),
                                              _p(zb_view), _view(zb_view, heads, "zb"), _p(za_view), _view(za_view, heads, "za"), _p(A_log), _p(dt_bias),
                                              _p(tok_seq), _p(tok_pos), _p(slots), _p(pos0), _p(len_after), n, heads, kv_heads, dim, vdim, q_scale, code(x_view.dtype), _stream(qo)))


def delta_scan(o, S, q, k, v, beta, decay, cu, slots, pos0, kv_heads: int):
    """o [n, heads, vdim] float32; state per slot S [heads, vdim, dim] float32; q / k [n, kv_heads * dim], v [n, heads * vdim], beta / decay [n, heads] float32."""
    n, heads, vdim = o.shape
    dim = S.shape[3]
    for t, nm in ((o, "o"), (S, "S"), (q, "q"), (k, "k"), (v, "v"), (beta, "beta"), (decay, "decay")):
        _f32c(t, nm)
    for t, nm in ((cu, "cu"), (slots, "slots"), (pos0, "pos0")):
        _i32c(t, nm)
    _req(S.shape[1:] == (heads, vdim, dim) and q.shape == k.shape == (n, kv_heads * dim) and v.shape == (n, heads * vdim) and beta.shape == decay.shape == (n, heads),
         "delta_scan: shapes")
    _check(_lib.mixlib().exl3_mix_delta_scan(_p(o), _p(S), _p(q), _p(k), _p(v), _p(beta), _p(decay), _p(cu), _p(slots), _p(pos0), cu.numel() - 1, heads, kv_heads, dim, vdim,
                                              _stream(o)))


def head_norm_gate(out, o, w, g_view, gate: int, eps: float):
    """out [n, heads * vdim] = o / rms(o per head) * w * gate(g); w has vdim entries (shared by the heads) or heads * vdim; gate GATE_SILU / GATE_SIGMOID."""
    n, heads, vdim = o.shape
    _f32c(o, "o"); _f32c(w, "w")
    _req(out.is_contiguous() and out.shape == (n, heads * vdim) and w.numel() in (vdim, heads * vdim) and g_view.dtype == out.dtype, "head_norm_gate: shapes")
    per_head = 1 if (w.numel() == heads * vdim and heads > 1) else 0
    _check(_lib.mixlib().exl3_mix_head_norm_gate(_p(out), _p(o), _p(w), per_head, _p(g_view), _view(g_view, heads * vdim, "g"), gate, eps, n, heads, vdim, code(out.dtype),
                                                  _stream(out)))


def rms_pair(out, a_view, wa, b_view, wb, scale: float, eps: float):
    """out = scale * (a / rms(a) * wa + b / rms(b) * wb) row by row."""
    n, width = out.shape
    _f32c(wa, "wa"); _f32c(wb, "wb")
    _req(out.is_contiguous() and a_view.dtype == out.dtype == b_view.dtype and a_view.shape[0] == n and b_view.shape[0] == n and wa.numel() == width and wb.numel() == width,
         "rms_pair: shapes")
    _check(_lib.mixlib().exl3_mix_rms_pair(_p(out), _p(a_view), _view(a_view, width, "a"), _p(wa), _p(b_view), _view(b_view, width, "b"), _p(wb), scale, eps, n, width,
                                            code(out.dtype), _stream(out)))
