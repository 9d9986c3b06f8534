"""
Building blocks of the unquantized mixer models: each mechanism is one class with its constants as constructor arguments, its tensors
read through the framework's SafetensorsCollection, its per-slot state declared as StateSpec, and a forward over a packed StepBatch that
runs the kernels of libexl3_mix.so (mix_ops) around vendor matrix products (torch.nn.functional.linear: hipBLASLt / rocBLAS with
float32 accumulation; true float32 when the model runs in float32).

    FusedInput              several linears over one input as one matrix product, outputs as column views
    SlidingSinkAttention    grouped-query attention over a sliding window, optional learned sink in the softmax denominator, optional unit-RMS
                            values, optional head-wise sigmoid output gate, no rotation; ring cache of `window` entries per slot
    GatedLinearAttention    linear attention with a low-rank per-channel decay sigmoid(z)^(1/tau), float32 state per head, per-head RMS norm,
                            silu output gate
    PolyNormMLP             W_down act(W_up h), act = a N(z) + b N(z^2) + c N(z^3) + e
    SparseExperts           top-k of n experts (router in float32, softmax over the chosen logits), experts W_down (silu(W_gate h) * W_up h)
    GatedResidualBlock      x += sublayer(norm(x)) * sigmoid(W norm(x) + b) for a mixer and an optional feed-forward, residual in float32
    DynTanh                 the norm tanh(alpha x) w + b (no statistics), fused into the residual update that precedes it
    LatentAttention         attention whose keys and values are up-projections of one cached low-rank latent per token plus one rotated key part
                            shared by the heads; rotary positions (optionally YaRN-scaled), sliding window, optional sink, optional element-wise
                            sigmoid output gate; ring cache of [latent | rotated key] per slot; decode in the absorbed form
    ActMLP                  W_down act(W_up h) with a plain activation (relu^2, gelu, silu)
    GatedMLP                W_down glu(W_gate h, W_up h) with a gated activation (silu, or the clamped swish with its limit)
    TokenSide               per-layer token input: a gate on the residual times a slice of a second embedding, projected back and RMS-normed
    PreNormBlock            x += mixer(norm1(x)); x += ff(norm2(x)); x += side(x), each update fused with what the next consumer reads
  SparseExperts also routes by sigmoid scores with a selection-only correction, takes either gated activation and an always-on shared expert;
  with a softmax over all experts, groups of experts of which only the best are eligible, ungated experts (W_down act(W_up h)) and trailing router
  outputs that stand for experts which return their input.
    CanonNorm               RMS norm with a one-plus weight followed by the short causal per-channel input convolution h + conv(h), fused into the
                            residual update that precedes it; the last taps - 1 normed rows of a sequence live in its slot
    DifferentialAttention   grouped-query attention with two maps per head over shared values, o = a1 - lambda a2, per-head unit RMS, head-wise
                            sigmoid gate; RMS-normed queries / keys, rotary positions (rotate-half layout, partial, YaRN), soft-capped scores, chunk
                            (or window) mask; rings of one chunk per slot
    CanonBlock              x += mixer(canon1(x)); x += ff(canon2(x)) over CanonNorm inputs

    LayerNormConv           layer norm (weight and bias) followed by the same input convolution; hands out both the normed rows and the convolved rows
    SigmoidAttention        grouped-query causal attention without softmax (weights sigmoid(scale q.k + bias_head), not normalised), no window: keys and
                            values in the cache's pages
    MatrixLSTM              matrix memory with exponential gating (mLSTM): capped log gates, running maximum, float32 state [heads, vdim, dim] + normaliser
    GatedDeltaRule          delta-rule memory with a scalar decay per head and token, short convolutions with silu on q / k / v, unit query / key vectors
    ParallelMixer           two mixers side by side over ONE fused input product, their outputs RMS-normed and averaged
    ParallelBlock           x += m (mixer(conv(n(x))) + ff(n(x))): one norm, both sublayers read it, the residual factor m

Every sum that the model's exactness rests on (norms, scores, softmax, decays, states, the residual) is float32 inside the kernels in
both modes; the element type only decides how matrix products and their outputs are held.
"""
from __future__ import annotations
from dataclasses import dataclass
import torch
import torch.nn.functional as F
from . import mix_ops
from .state_cache import StateSpec, StepBatch


def _w(stc, key: str, dtype, device) -> torch.Tensor:
    return stc.get_tensor(key, device="cpu").to(dtype).to(device).contiguous()


def _f32(stc, key: str, device) -> torch.Tensor:
    return stc.get_tensor(key, device="cpu").to(torch.float32).to(device).contiguous()


class FusedInput:
    """Linears that read the same input, stacked into one weight: one matrix product instead of several, and every consumer kernel takes its
    column block in place (row stride = total width).  Parts without a bias get zeros in the fused bias (adding zero is exact)."""

    def __init__(self, parts: list[tuple[str, torch.Tensor, torch.Tensor | None]]):
        self.names = [p[0] for p in parts]
        self.sizes = [p[1].shape[0] for p in parts]
        self.weight = torch.cat([p[1] for p in parts], dim=0).contiguous()
        if any(p[2] is not None for p in parts):
            self.bias = torch.cat([p[2].to(self.weight.dtype) if p[2] is not None else torch.zeros(p[1].shape[0], dtype=self.weight.dtype, device=self.weight.device)
                                   for p in parts]).contiguous()
        else:
            self.bias = None
        self.offsets, at = {}, 0
        for n, s in zip(self.names, self.sizes):
            self.offsets[n] = (at, s); at += s

    def __call__(self, h: torch.Tensor) -> dict[str, torch.Tensor]:
        out = F.linear(h, self.weight, self.bias)
        p = {n: out[:, a: a + s] for n, (a, s) in self.offsets.items()}
        p[self.ALL] = out                     # the whole product, for a consumer that reads several neighbouring parts as one block
        return p

    ALL = "*"

    def block(self, p: dict, first: str, last: str) -> torch.Tensor:
        """The column block from part `first` to part `last` (neighbours in the order they were given)."""
        a, b = self.offsets[first][0], self.offsets[last][0] + self.offsets[last][1]
        return p[self.ALL][:, a:b]


class SlidingSinkAttention:
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, eps: float, sink: bool = True,
                 value_norm: bool = True, gate: bool = True, bias: bool = True):
        if heads % kv_heads:
            raise RuntimeError(f"attention: {heads} query heads over {kv_heads} key/value heads")
        if not value_norm:
            raise RuntimeError("attention: the cache store kernel normalises values; an un-normalised variant is not built")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.scale, self.window, self.eps = float(scale), int(window), float(eps)
        self.has_sink, self.has_gate, self.has_bias = sink, gate, bias

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = []
        for nm in ("q", "k", "v"):
            parts.append((nm, _w(stc, prefix + nm, dtype, device), _w(stc, prefix + nm + ".b", dtype, device) if self.has_bias else None))
        if self.has_gate:
            parts.append(("g", _w(stc, prefix + "g", dtype, device), None))
        self.inp = FusedInput(parts + list(extra_parts))
        self.sink = _f32(stc, prefix + "sink", device) if self.has_sink else None
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.inp.offsets["q"][1] == self.heads * self.dim and self.inp.offsets["v"][1] == self.kv_heads * self.vdim
        assert self.w_o.shape == (self.width, self.heads * self.vdim)
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("ring_k", (self.window, self.kv_heads, self.dim), self.dtype), StateSpec("ring_v", (self.window, self.kv_heads, self.vdim), self.dtype)]

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        v_norm = torch.empty((sb.n, self.kv_heads, self.vdim), dtype=self.dtype, device=h.device)
        mix_ops.attn_store(v_norm, state["ring_k"], state["ring_v"], p["k"], p["v"], sb.tok_seq, sb.tok_pos, sb.slots, sb.len_after, self.eps)
        out = torch.empty((sb.n, self.heads * self.vdim), dtype=self.dtype, device=h.device)
        if sb.decode:
            mix_ops.attn_decode(out, p["q"], state["ring_k"], state["ring_v"], p.get("g"), self.sink, sb.slots, sb.len_after, self.heads, self.scale)
        else:
            mix_ops.attn_prefill(out, p["q"], p["k"], v_norm, p.get("g"), self.sink, sb.cu, sb.tok_seq, sb.tok_pos, self.heads, self.scale, self.window,
                                 max_rows=sb.max_rows)
        return F.linear(out, self.w_o), p


class GatedLinearAttention:
    # prompt steps whose longest sequence has at least this many rows are cut into parallel time segments (mix_ops.gla_scan)
    SEGMENT_MIN_ROWS = 256
    SEGMENT_TARGET_WORKGROUPS = 1024

    def __init__(self, width: int, heads: int, dim: int, vdim: int, tau: float, eps: float):
        self.width, self.heads, self.dim, self.vdim, self.tau, self.eps = width, heads, dim, vdim, float(tau), float(eps)
        self.q_scale = float(dim) ** -0.5

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = [(nm, _w(stc, prefix + nm, dtype, device), None) for nm in ("q", "k", "v", "g", "a1")]
        self.inp = FusedInput(parts + list(extra_parts))
        self.a2 = _w(stc, prefix + "a2", dtype, device)
        self.a2_bias = _f32(stc, prefix + "a2.b", device)
        self.norm_w = _f32(stc, prefix + "norm", device)
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.inp.offsets["q"][1] == self.heads * self.dim and self.inp.offsets["v"][1] == self.heads * self.vdim
        assert self.a2.shape[0] == self.heads * self.dim and self.a2.shape[1] == self.inp.offsets["a1"][1]
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("S", (self.heads, self.dim, self.vdim), torch.float32)]

    def segments(self, sb: StepBatch) -> tuple[int, int] | None:
        """(segments per sequence, rows per segment) for a long prompt step: enough workgroups to fill the device, segments of at least 64 rows."""
        if sb.max_rows < self.SEGMENT_MIN_ROWS:
            return None
        chains = sb.batch * self.heads * ((self.vdim + 63) // 64)
        segs = min(max(1, -(-self.SEGMENT_TARGET_WORKGROUPS // chains)), sb.max_rows // 64)
        if segs < 2:
            return None
        seg_len = -(-sb.max_rows // segs)
        seg_len = -(-seg_len // 16) * 16
        return -(-sb.max_rows // seg_len), seg_len

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        o = torch.empty((sb.n, self.heads, self.vdim), dtype=torch.float32, device=h.device)
        mix_ops.gla_scan(o, state["S"], p["q"], p["k"], p["v"], p["a1"], self.a2, self.a2_bias, sb.cu, sb.slots, sb.pos0, self.tau, self.q_scale,
                         segments=self.segments(sb))
        out = torch.empty((sb.n, self.heads * self.vdim), dtype=self.dtype, device=h.device)
        mix_ops.gla_out(out, o, self.norm_w, p["g"], self.eps)
        return F.linear(out, self.w_o), p


class PolyNormMLP:
    def __init__(self, width: int, ff: int, eps: float):
        self.width, self.ff, self.eps = width, ff, float(eps)

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        self.inp = FusedInput([("up", _w(stc, prefix + "up", dtype, device), None)] + list(extra_parts))
        self.coef = _f32(stc, prefix + "act", device)
        self.w_down = _w(stc, prefix + "down", dtype, device)
        assert self.inp.offsets["up"][1] == self.ff and self.w_down.shape == (self.width, self.ff)
        self.dtype = dtype

    def forward(self, h: torch.Tensor, sb: StepBatch) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        a = torch.empty((sb.n, self.ff), dtype=self.dtype, device=h.device)
        mix_ops.polynorm(a, p["up"], self.coef, self.eps)
        return F.linear(a, self.w_down), p


def rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> tuple[torch.Tensor, float]:
    """Per-pair frequencies base^(-2i/dims), i < dims/2, and the magnitude that multiplies cos and sin.  `scaling` (YaRN: factor, original, fast, slow)
    blends every frequency with its `factor`-times slower version along a linear ramp between the pair indices at which the original context
    holds `fast` and `slow` turns, and sets the magnitude to 0.1 ln(factor) + 1.  Computed in float64, returned as float32."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling is not None:
        factor, original = float(scaling["factor"]), float(scaling["original"])
        at = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
        lo = max(math.floor(at(float(scaling["fast"]))), 0)
        hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32), float(mag)


class DynTanh:
    """tanh(alpha x) * w + b: a norm without mean or variance.  It is never a kernel of its own: the residual update before it writes it."""

    def __init__(self, width: int):
        self.width = width

    def load(self, stc, name: str, device):
        self.w, self.b = _f32(stc, name, device), _f32(stc, name + ".b", device)
        self.alpha = float(stc.get_tensor(name + ".alpha", device="cpu").to(torch.float32).reshape(-1)[0])
        assert self.w.numel() == self.width and self.b.numel() == self.width
        return self


@dataclass
class NextInput:
    """What the kernel that updates the residual also writes: the input of the next consumer.  norm None: the stream itself in the activation type."""
    norm: DynTanh | None
    out: torch.Tensor            # [n, width] view (any row stride)


def update_residual(x: torch.Tensor, y: torch.Tensor | None, nxt: NextInput | None, mode: int = mix_ops.RES_ADD, rms_w: torch.Tensor | None = None, eps: float = 0.0):
    if nxt is None:
        if y is not None and mode != mix_ops.RES_KEEP:
            mix_ops.residual_norm(x, y, mode, rms_w, eps, mix_ops.OUT_NONE, 0.0, None, None, None)
    elif nxt.norm is None:
        mix_ops.residual_norm(x, y, mode, rms_w, eps, mix_ops.OUT_CAST, 0.0, None, None, nxt.out)
    else:
        mix_ops.residual_norm(x, y, mode, rms_w, eps, mix_ops.OUT_DYN_TANH, nxt.norm.alpha, nxt.norm.w, nxt.norm.b, nxt.out)


class LatentAttention:
    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, rank: int, scale: float, window: int, eps: float, rot_dims: int, rot_base: float,
                 rot_scaling: dict | None = None, sink: bool = False, gate: bool = False):
        if rot_dims > rot_dim or rot_dims % 2:
            raise RuntimeError(f"latent attention: {rot_dims} rotated dimensions of {rot_dim}")
        if rank > 1024:
            raise RuntimeError("latent attention: the decode kernel holds a latent of at most 1024 entries")
        self.width, self.heads, self.dim, self.rot_dim, self.vdim, self.rank = width, heads, dim, rot_dim, vdim, rank
        self.scale, self.window, self.eps = float(scale), int(window), float(eps)
        self.rot_dims, self.rot_base, self.rot_scaling = rot_dims, float(rot_base), rot_scaling
        self.has_sink, self.has_gate = sink, gate
        self.qk = dim + rot_dim

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = [("q", _w(stc, prefix + "q", dtype, device), None), ("dkv", _w(stc, prefix + "dkv", dtype, device), None)]
        if self.has_gate:
            parts.append(("g", _w(stc, prefix + "g", dtype, device), None))
        self.inp = FusedInput(parts + list(extra_parts))
        self.c_norm = _f32(stc, prefix + "dkv.norm", device)
        w_uk, self.w_uv = _w(stc, prefix + "uk", dtype, device), _w(stc, prefix + "uv", dtype, device)
        H, d, r, dv, rank = self.heads, self.dim, self.rot_dim, self.vdim, self.rank
        assert self.inp.offsets["q"][1] == H * self.qk and self.inp.offsets["dkv"][1] == rank + r
        assert w_uk.shape == (H * d, rank) and self.w_uv.shape == (H * dv, rank)
        # prompt steps: keys of all heads as ONE product whose result already has room for the rotated part behind every head (zero weight rows there)
        padded = torch.zeros((H, self.qk, rank), dtype=dtype, device=device)
        padded[:, :d] = w_uk.view(H, d, rank)
        self.w_uk_padded = padded.view(H * self.qk, rank)
        # decode steps, absorbed form: per head q_lat = q_unrotated W_uk[h] and o = o_lat W_uv[h]^T
        self.w_uk_heads = w_uk.view(H, d, rank)
        self.w_uv_heads_t = self.w_uv.view(H, dv, rank).transpose(1, 2)
        self.sink = _f32(stc, prefix + "sink", device) if self.has_sink else None
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.w_o.shape == (self.width, H * dv)
        f, self.rot_mag = rotary_frequencies(self.rot_dims, self.rot_base, self.rot_scaling)
        self.freq = f.to(device).contiguous()
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("ring", (self.window, self.rank + self.rot_dim), self.dtype)]

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        H, d, r, dv, rank = self.heads, self.dim, self.rot_dim, self.vdim, self.rank
        p = self.inp(h)
        q = p["q"]
        ckr = torch.empty((sb.n, rank + r), dtype=self.dtype, device=h.device)
        mix_ops.latent_prep(ckr, state["ring"], p["dkv"], self.c_norm, q, sb.tok_seq, sb.tok_pos, sb.slots, sb.len_after, self.freq, self.rot_mag, self.eps, H, d, r, rank)
        if sb.decode:
            q_heads = q.as_strided((H, sb.n, d), (self.qk, q.stride(0), 1), q.storage_offset())
            q_lat = torch.bmm(q_heads, self.w_uk_heads)                          # [H, n, rank]
            o_lat = torch.empty_like(q_lat)
            mix_ops.latent_decode(o_lat, q_lat, q, state["ring"], self.sink, sb.slots, sb.len_after, d, r, self.scale)
            o = torch.bmm(o_lat, self.w_uv_heads_t)                              # [H, n, vdim]
            if sb.n == 1 and not self.has_gate:
                out = o.view(1, H * dv)                                          # one row: head-major is token-major
            else:
                out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=h.device)
                mix_ops.heads_gate(out, o, dv, sb.n * dv, p.get("g"), H, dv)
        else:
            out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=h.device)
            c = ckr[:, :rank]
            k = F.linear(c, self.w_uk_padded)                                    # [n, H * (d + r)], the rotated slots still zero
            v = F.linear(c, self.w_uv).view(sb.n, H, dv)
            mix_ops.latent_fill_k(k, ckr, H, d, r, rank)
            if self.has_gate:
                o = torch.empty((sb.n, H * dv), dtype=self.dtype, device=h.device)
                mix_ops.attn_prefill(o, q, k, v, None, self.sink, sb.cu, sb.tok_seq, sb.tok_pos, H, self.scale, self.window, max_rows=sb.max_rows)
                mix_ops.heads_gate(out, o, H * dv, dv, p["g"], H, dv)
            else:
                mix_ops.attn_prefill(out, q, k, v, None, self.sink, sb.cu, sb.tok_seq, sb.tok_pos, H, self.scale, self.window, max_rows=sb.max_rows)
        return F.linear(out, self.w_o), p


class ActMLP:
    KINDS = {"relu2": mix_ops.ACT_RELU2, "gelu_tanh": mix_ops.ACT_GELU_TANH, "silu": mix_ops.ACT_SILU}

    def __init__(self, width: int, ff: int, act: str = "relu2"):
        self.width, self.ff, self.kind = width, ff, self.KINDS[act]

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        self.inp = FusedInput([("up", _w(stc, prefix + "up", dtype, device), None)] + list(extra_parts))
        self.w_down = _w(stc, prefix + "down", dtype, device)
        assert self.inp.offsets["up"][1] == self.ff and self.w_down.shape == (self.width, self.ff)
        self.dtype = dtype

    def forward(self, h: torch.Tensor, sb: StepBatch) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        a = torch.empty((sb.n, self.ff), dtype=self.dtype, device=h.device)
        mix_ops.act(a, p["up"], self.kind)
        return F.linear(a, self.w_down), p


class GatedMLP:
    KINDS = {"silu": mix_ops.GLU_SILU, "clamped_swish": mix_ops.GLU_CLAMPED_SWISH}

    def __init__(self, width: int, ff: int, act: str = "silu", limit: float = 0.0, row_gate: str | None = None):
        """row_gate: name of a [1, width] weight; the sublayer's output is multiplied by sigmoid(W_row_gate h), one number per row (applied to the hidden
        activation, ahead of the linear down projection, so that the product's epilogue can still add it to another sum)."""
        self.width, self.ff, self.kind, self.limit, self.row_gate = width, ff, self.KINDS[act], float(limit), row_gate

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        extra_parts = list(extra_parts) + ([("row_gate", _w(stc, prefix + self.row_gate, dtype, device).view(1, self.width), None)] if self.row_gate else [])
        self.inp = FusedInput([("gate", _w(stc, prefix + "gate", dtype, device), None), ("up", _w(stc, prefix + "up", dtype, device), None)] + list(extra_parts))
        self.w_down = _w(stc, prefix + "down", dtype, device)
        assert self.inp.offsets["up"][1] == self.ff and self.w_down.shape == (self.width, self.ff)
        self.dtype = dtype

    def hidden(self, h: torch.Tensor) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        a = torch.empty((h.shape[0], self.ff), dtype=self.dtype, device=h.device)
        if self.row_gate:
            mix_ops.glu_act_rowgate(a, p["gate"], p["up"], p["row_gate"], self.kind, self.limit)
        else:
            mix_ops.glu_act(a, p["gate"], p["up"], self.kind, self.limit)
        return a, p

    def forward(self, h: torch.Tensor, sb: StepBatch, add_to: torch.Tensor | None = None) -> tuple[torch.Tensor, dict]:
        """add_to: a [n, width] tensor that the down projection is added to (the product's epilogue), e.g. the routed experts' sum."""
        a, p = self.hidden(h)
        if add_to is not None:
            return torch.addmm(add_to, a, self.w_down.t()), p
        return F.linear(a, self.w_down), p


class TokenSide:
    """x += rms_norm(W_proj (gelu(W_gate x) * e)) * w, e = the layer's slice of a second embedding row of the token.  The gate reads the residual
    stream itself (in the activation type), not a normed copy."""

    def __init__(self, width: int, dim: int, index: int, eps: float):
        self.width, self.dim, self.index, self.eps = width, dim, index, float(eps)

    def load(self, stc, prefix: str, table: torch.Tensor, dtype, device):
        self.table = table                                       # [vocab, layers * dim], shared by the layers
        self.w_gate, self.w_proj = _w(stc, prefix + "gate", dtype, device), _w(stc, prefix + "proj", dtype, device)
        self.norm_w = _f32(stc, prefix + "norm", device)
        assert self.w_gate.shape == (self.dim, self.width) and self.w_proj.shape == (self.width, self.dim) and (self.index + 1) * self.dim <= table.shape[1]
        self.dtype = dtype

    def forward(self, xc: torch.Tensor, sb: StepBatch) -> torch.Tensor:
        gate = F.linear(xc, self.w_gate)
        g = torch.empty((sb.n, self.dim), dtype=self.dtype, device=xc.device)
        mix_ops.token_gate(g, gate, self.table, self.index * self.dim, sb.tokens)
        return F.linear(g, self.w_proj)


class PreNormBlock:
    """x += mixer(norm1(x)); x += ff(norm2(x)) (if a feed-forward); x += side(x) (if a token side input).  Every update of the float32 residual is one
    kernel that also writes what comes next: the next norm's output, or the stream in the activation type."""

    def __init__(self, width: int, eps: float, mixer, mlp, side: TokenSide | None):
        self.width, self.eps, self.mixer, self.mlp, self.side = width, float(eps), mixer, mlp, side
        self.norm1, self.norm2 = DynTanh(width), (DynTanh(width) if mlp is not None else None)

    def load(self, stc, prefix: str, dtype, device, side_table: torch.Tensor | None = None):
        self.norm1.load(stc, prefix + "norm1", device)
        self.mixer.load(stc, prefix + "mix.", dtype, device)
        if self.mlp is not None:
            self.norm2.load(stc, prefix + "norm2", device)
            self.mlp.load(stc, prefix + "mlp.", dtype, device)
        if self.side is not None:
            self.side.load(stc, prefix + "side.", side_table, dtype, device)
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return self.mixer.state_specs()

    def forward(self, x: torch.Tensor, h: torch.Tensor, sb: StepBatch, state: dict, nxt: NextInput | None):
        """x: float32 residual (updated in place); h = norm1(x).  nxt: what the block's last update writes for whoever reads the stream next."""
        new = lambda: torch.empty((sb.n, self.width), dtype=self.dtype, device=x.device)
        y, _ = self.mixer.forward(h, sb, state)
        if self.mlp is not None:
            h2 = new()
            update_residual(x, y, NextInput(self.norm2, h2))
            y, _ = self.mlp.forward(h2, sb)
        if self.side is None:
            update_residual(x, y, nxt)
            return
        xc = new()
        update_residual(x, y, NextInput(None, xc))
        update_residual(x, self.side.forward(xc, sb), nxt, rms_w=self.side.norm_w, eps=self.eps)


class SparseExperts:
    # rows from which the expert-sorted matrix products take over from the weight-streaming kernels, and rows from which the streaming kernels
    # walk each chosen expert once for all its rows instead of once per (row, choice)
    GROUPED_MIN_ROWS = 64
    EXPERT_MAJOR_MIN_ROWS = 4

    def __init__(self, width: int, ff: int, experts: int, top: int, router: str = "softmax", router_bias: bool = True, correction: bool = False,
                 route_scale: float = 1.0, act: str = "silu", limit: float = 0.0, shared: GatedMLP | None = None, gated: bool = True, identity: int = 0,
                 groups: int = 1, keep_groups: int = 1, group_top: int = 1):
        """router "softmax": the top logits, weights = softmax over them.  "sigmoid": scores sigmoid(z), chosen by score (+ a stored correction that the
        weights do not see), weights = chosen scores / their sum * route_scale.  "softmax_all": scores = softmax over all router outputs, chosen by score +
        correction inside the `keep_groups` best of `groups` groups of neighbouring outputs, weights = chosen scores / their sum * route_scale (the grouped
        form also serves "sigmoid" when groups > 1).  identity: the router has this many outputs beyond the stored experts; they stand for experts that return
        their input.  group_top: a group's score is the sum of its group_top largest choice scores (1: its largest).  gated False: experts are W_down act(W_up h) with a plain activation (ActMLP.KINDS).  shared: an expert that every row runs, added to
        the routed sum."""
        if not 0 < top <= experts + identity:
            raise RuntimeError(f"router: top {top} of {experts + identity} experts")
        if router not in ("softmax", "sigmoid", "softmax_all"):
            raise RuntimeError(f"router: unknown kind {router!r}")
        if (identity or groups > 1) and router == "softmax":
            raise RuntimeError("router: groups and identity experts go with the softmax_all and sigmoid routers")
        if groups < 1 or (experts + identity) % groups or not 1 <= keep_groups <= groups or top > keep_groups * ((experts + identity) // groups):
            raise RuntimeError(f"router: {groups} groups (keep {keep_groups}) over {experts + identity} outputs cannot give {top} choices")
        self.width, self.ff, self.experts, self.top = width, ff, experts, top
        self.router, self.has_router_bias, self.has_correction, self.route_scale = router, router_bias, correction, float(route_scale)
        self.gated, self.identity, self.groups, self.keep_groups, self.group_top = gated, int(identity), int(groups), int(keep_groups), int(group_top)
        self.act_kind = GatedMLP.KINDS[act] if gated else ActMLP.KINDS[act]
        self.limit, self.shared = float(limit), shared

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        stack = lambda nm: torch.stack([_w(stc, f"{prefix}e{e}.{nm}", dtype, device) for e in range(self.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = (stack("gate") if self.gated else None), stack("up"), stack("down")
        self.w_router = _f32(stc, prefix + "router", device)
        self.b_router = _f32(stc, prefix + "router.b", device) if self.has_router_bias else None
        self.correction = _f32(stc, prefix + "correction", device) if self.has_correction else None
        if self.shared is not None:
            self.shared.load(stc, prefix + "shared.", dtype, device)
        self.inp = FusedInput(list(extra_parts)) if extra_parts else None
        assert self.w_up.shape == (self.experts, self.ff, self.width) and self.w_down.shape == (self.experts, self.width, self.ff)
        assert self.w_router.shape == (self.experts + self.identity, self.width)
        self.dtype = dtype

    def forward(self, h: torch.Tensor, sb: StepBatch) -> tuple[torch.Tensor, dict]:
        p = self.inp(h) if self.inp is not None else {}
        hf = h.float()                                                              # float32 product of the (rounded) input
        logits = torch.addmm(self.b_router, hf, self.w_router.t()) if self.b_router is not None else torch.mm(hf, self.w_router.t())
        idx = torch.empty((sb.n, self.top), dtype=torch.int32, device=h.device)
        wts = torch.empty((sb.n, self.top), dtype=torch.float32, device=h.device)
        idw = None                                                                  # per row: the weights of the chosen experts that return their input
        if self.router == "softmax":
            mix_ops.topk_softmax(idx, wts, logits)
        elif self.router == "sigmoid" and self.groups == 1 and not self.identity:
            mix_ops.topk_sigmoid(idx, wts, logits, self.correction, self.route_scale)
        else:
            idw = torch.empty((sb.n,), dtype=torch.float32, device=h.device) if self.identity else None
            mix_ops.topk_grouped_ex(idx, wts, idw, logits, self.correction, mix_ops.ROUTE_SOFTMAX_ALL if self.router == "softmax_all" else mix_ops.ROUTE_SIGMOID,
                                    self.experts, self.groups, self.keep_groups, self.group_top, self.route_scale)
        y = torch.empty((sb.n, self.width), dtype=self.dtype, device=h.device)
        if not self.gated:
            if sb.n >= self.GROUPED_MIN_ROWS:
                mix_ops.moe_grouped_plain(y, h, self.w_up, self.w_down, idx, wts, self.act_kind, idw)
            elif sb.n >= self.EXPERT_MAJOR_MIN_ROWS and mix_ops.moe_vector_layout(h, self.ff):
                mix_ops.moe_expert_major_plain(y, h, self.w_up, self.w_down, idx, wts, self.act_kind, idw)
            else:
                hid = torch.empty((sb.n * self.top, self.ff), dtype=self.dtype, device=h.device)
                mix_ops.moe_up_act(hid, h, self.w_up, idx, self.act_kind)
                mix_ops.moe_down_id(y, hid, self.w_down, idx, wts, h, idw)
        elif idw is not None:
            raise RuntimeError("experts: the gated experts' kernels carry no identity share")
        elif sb.n >= self.GROUPED_MIN_ROWS:
            mix_ops.moe_grouped(y, h, self.w_gate, self.w_up, self.w_down, idx, wts, self.act_kind, self.limit)
        elif sb.n >= self.EXPERT_MAJOR_MIN_ROWS and mix_ops.moe_vector_layout(h, self.ff):
            mix_ops.moe_expert_major(y, h, self.w_gate, self.w_up, self.w_down, idx, wts, self.act_kind, self.limit)
        else:
            hid = torch.empty((sb.n * self.top, self.ff), dtype=self.dtype, device=h.device)
            mix_ops.moe_gate_up_act(hid, h, self.w_gate, self.w_up, idx, self.act_kind, self.limit)
            mix_ops.moe_down(y, hid, self.w_down, idx, wts)
        if self.shared is not None:
            y, _ = self.shared.forward(h, sb, add_to=y)
        return y, p


class GatedResidualBlock:
    """One layer: x <- x + mixer(n1(x)) * sigmoid(W1 n1(x) + b1); x <- x + ff(n2(x)) * sigmoid(W2 n2(x) + b2) (the second half only with a
    feed-forward).  The gate's linear rides in the sublayer's fused input product; the residual add, the gate and the NEXT norm are one kernel."""

    def __init__(self, width: int, eps: float, mixer, mlp):
        self.width, self.eps, self.mixer, self.mlp = width, float(eps), mixer, mlp

    def load(self, stc, prefix: str, dtype, device):
        self.norm1 = _f32(stc, prefix + "norm1", device)
        self.mixer.load(stc, prefix + "mix.", dtype, device, extra_parts=[("rg", _w(stc, prefix + "rg1", dtype, device), _w(stc, prefix + "rg1.b", dtype, device))])
        if self.mlp is not None:
            self.norm2 = _f32(stc, prefix + "norm2", device)
            self.mlp.load(stc, prefix + "mlp.", dtype, device, extra_parts=[("rg", _w(stc, prefix + "rg2", dtype, device), _w(stc, prefix + "rg2.b", dtype, device))])

    def state_specs(self) -> list[StateSpec]:
        return self.mixer.state_specs()

    def forward(self, x: torch.Tensor, h: torch.Tensor, sb: StepBatch, state: dict, next_norm: torch.Tensor | None) -> torch.Tensor | None:
        """x: float32 residual (updated in place); h = norm1(x) in the activation type.  Returns the next layer's h (None when next_norm is None)."""
        y, p = self.mixer.forward(h, sb, state)
        after = self.norm2 if self.mlp is not None else next_norm
        h2 = torch.empty_like(h) if after is not None else None
        mix_ops.gated_residual(x, y, p["rg"], after, h2, self.eps)
        if self.mlp is None:
            return h2
        y, p = self.mlp.forward(h2, sb)
        h3 = torch.empty_like(h) if next_norm is not None else None
        mix_ops.gated_residual(x, y, p["rg"], next_norm, h3, self.eps)
        return h3


class CanonNorm:
    """What a sublayer reads in blocks with an input convolution: hn = x / sqrt(mean(x^2) + eps) * (1 + w), then h_t = hn_t + sum_j c[:, j] hn_(t - taps + 1 + j)
    per channel, rows before the sequence's start being zero.  It is never a kernel chain of its own: the residual update before it writes it.  A step
    of one row per sequence is ONE launch (update, norm, convolution against the slot's ring of the last taps - 1 normed rows, ring store); a prompt step is
    two (update + norm of every row, then the convolution over the step's own rows)."""

    def __init__(self, width: int, taps: int, eps: float):
        if taps < 1 or taps > 16:
            raise RuntimeError(f"input convolution: {taps} taps")
        self.width, self.taps, self.eps = width, int(taps), float(eps)
        self.dtype = torch.bfloat16                                  # until load() says otherwise

    def load(self, stc, norm_key: str, conv_key: str, dtype, device):
        self.w = (1.0 + _f32(stc, norm_key, device)).contiguous()              # the checkpoint holds w, the norm multiplies by 1 + w
        self.conv = _f32(stc, conv_key, device).t().contiguous()               # stored [width, taps]; the kernels read one tap of neighbouring channels at once
        assert self.w.numel() == self.width and self.conv.shape == (self.taps, self.width)
        self.dtype = dtype
        return self

    def state_spec(self, name: str) -> StateSpec:
        return StateSpec(name, (max(self.taps - 1, 1), self.width), self.dtype)

    def apply(self, x: torch.Tensor, y: torch.Tensor | None, mode: int, sb: StepBatch, ring: torch.Tensor) -> torch.Tensor:
        """x <- x | x + y | y, returns the sublayer's input [n, width] in the activation type."""
        h = torch.empty((sb.n, self.width), dtype=self.dtype, device=x.device)
        if sb.decode:
            mix_ops.residual_rms(x, y, mode, self.w, self.eps, h, self.conv, ring, sb.tok_seq, sb.tok_pos, sb.slots)
            return h
        hn = torch.empty_like(h)
        mix_ops.residual_rms(x, y, mode, self.w, self.eps, hn)
        mix_ops.canon(h, hn, self.conv, ring, sb.tok_seq, sb.tok_pos, sb.slots, sb.pos0, sb.len_after)
        return h


class DifferentialAttention:
    """H query heads over G key/value heads, every head with `maps` = 2 attention maps over the same values: q [H][2][dim], k [G][2][dim], v [G][vdim].
    Queries and keys: bias, RMS norm per (head, map) with one weight for all, rotary positions on the first rot_dims entries (rotate-half pairs, optional
    YaRN blend and magnitude).  score = scale q.k, soft-capped; mask = the row's own chunk of `span` positions ("chunk") or the last `span` positions
    ("window"); plain softmax.  o = a1 - lambda a2 with lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff, divided by its RMS over vdim, times (1 - diff), times
    sigmoid(W_g h) per head; then W_o with bias.  Per slot: rings of `span` keys and values (entry = position mod span: with the chunk mask a row's chunk
    is the entries 0 .. position mod span)."""
    MAPS = 2

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, softcap: float, span: int, mask: str, diff: float, eps: float,
                 rot_dims: int = 0, rot_base: float = 10000.0, rot_scaling: dict | None = None, gate: bool = True):
        if heads % kv_heads:
            raise RuntimeError(f"attention: {heads} query heads over {kv_heads} key/value heads")
        if rot_dims % 2 or rot_dims > dim:
            raise RuntimeError(f"attention: {rot_dims} rotated dimensions of {dim}")
        if mask not in ("chunk", "window") or span < 1:
            raise RuntimeError(f"attention: mask {mask!r} over {span} positions")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.scale, self.softcap, self.span, self.diff, self.eps = float(scale), float(softcap or 0.0), int(span), float(diff), float(eps)
        self.mask = mix_ops.MASK_CHUNK if mask == "chunk" else mix_ops.MASK_WINDOW
        self.rot_dims, self.rot_base, self.rot_scaling, self.has_gate = int(rot_dims), float(rot_base), rot_scaling, gate
        self.dtype = torch.bfloat16                                  # until load() says otherwise

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = [(nm, _w(stc, prefix + nm, dtype, device), _w(stc, prefix + nm + ".b", dtype, device)) for nm in ("q", "k", "v")]
        if self.has_gate:
            parts.append(("g", _w(stc, prefix + "g", dtype, device), None))
        self.inp = FusedInput(parts + list(extra_parts))
        H, G, d, dv, M = self.heads, self.kv_heads, self.dim, self.vdim, self.MAPS
        assert self.inp.offsets["q"][1] == H * M * d and self.inp.offsets["k"][1] == G * M * d and self.inp.offsets["v"][1] == G * dv
        self.q_norm, self.k_norm = _f32(stc, prefix + "q.norm", device), _f32(stc, prefix + "k.norm", device)
        l = {nm: stc.get_tensor(prefix + nm, device="cpu").to(torch.float64) for nm in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = float(torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum()) + self.diff)
        self.w_o, self.b_o = _w(stc, prefix + "o", dtype, device), _w(stc, prefix + "o.b", dtype, device)
        assert self.w_o.shape == (self.width, H * dv)
        if self.rot_dims:
            f, self.rot_mag = rotary_frequencies(self.rot_dims, self.rot_base, self.rot_scaling)
            self.freq = f.to(device).contiguous()
        else:
            self.freq, self.rot_mag = None, 1.0
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("ring_k", (self.span, self.kv_heads * self.MAPS, self.dim), self.dtype), StateSpec("ring_v", (self.span, self.kv_heads, self.vdim), self.dtype)]

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        H, G, d, dv, M = self.heads, self.kv_heads, self.dim, self.vdim, self.MAPS
        p = self.inp(h)
        mix_ops.qk_prep(p["q"], p["k"], p["v"], self.q_norm, self.k_norm, self.freq, self.rot_mag, False, self.eps, state["ring_k"], state["ring_v"],
                        sb.tok_seq, sb.tok_pos, sb.slots, sb.len_after, d)
        out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=h.device)
        if not sb.decode and mix_ops.diff_mfma_ok(self.dtype, sb.max_rows, d, dv, self.scale):
            # matrix cores: both maps of a head in one workgroup, combined in the epilogue
            mix_ops.attn_prefill_diff(out, p["q"], p["k"], p["v"], p.get("g"), sb.cu, H, G, d, dv, self.scale, self.softcap, self.span, self.mask, self.lam, self.diff,
                                      self.eps, sb.max_rows)
            return F.linear(out, self.w_o, self.b_o), p
        a = torch.empty((sb.n, H * M * dv), dtype=torch.float32, device=h.device)      # the maps' weighted sums stay float32 until they are combined
        if sb.decode:
            mix_ops.attn_decode_maps(a, p["q"], state["ring_k"], state["ring_v"], None, None, sb.slots, sb.len_after, H, M, self.scale, self.softcap, self.mask)
        else:
            mix_ops.attn_prefill_maps(a, p["q"], p["k"], p["v"], None, None, sb.cu, sb.tok_seq, sb.tok_pos, H, G, M, d, dv, self.scale, self.softcap, self.span,
                                      self.mask, max_rows=sb.max_rows)
        mix_ops.diff_combine(out, a, self.lam, self.diff, self.eps, p.get("g"), H, dv)
        return F.linear(out, self.w_o, self.b_o), p


class CanonBlock:
    """x += mixer(in1(x)); x += ff(in2(x)) (if a feed-forward), in1 / in2 being CanonNorm inputs.  The block is entered with its first input already
    computed and leaves by computing the next block's (the residual update and the norm behind it are one kernel), or by the bare update."""

    def __init__(self, width: int, eps: float, taps: int, mixer, mlp):
        self.width, self.eps, self.mixer, self.mlp = width, float(eps), mixer, mlp
        self.in1, self.in2 = CanonNorm(width, taps, eps), (CanonNorm(width, taps, eps) if mlp is not None else None)

    def load(self, stc, prefix: str, dtype, device):
        self.in1.load(stc, prefix + "norm1", prefix + "canon1", dtype, device)
        self.mixer.load(stc, prefix + "mix.", dtype, device)
        if self.mlp is not None:
            self.in2.load(stc, prefix + "norm2", prefix + "canon2", dtype, device)
            self.mlp.load(stc, prefix + "mlp.", dtype, device)
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return self.mixer.state_specs() + [self.in1.state_spec("canon1")] + ([self.in2.state_spec("canon2")] if self.in2 is not None else [])

    def forward(self, x: torch.Tensor, h: torch.Tensor, sb: StepBatch, state: dict, nxt: tuple | None) -> torch.Tensor | None:
        """x: float32 residual (updated in place); h = in1(x).  nxt = (the next block's in1, its ring): returns the next block's input; None: returns None."""
        y, _ = self.mixer.forward(h, sb, state)
        if self.mlp is not None:
            h2 = self.in2.apply(x, y, mix_ops.RES_ADD, sb, state["canon2"])
            y, _ = self.mlp.forward(h2, sb)
        if nxt is None:
            mix_ops.residual_rms(x, y, mix_ops.RES_ADD, None, self.eps, None)
            return None
        return nxt[0].apply(x, y, mix_ops.RES_ADD, sb, nxt[1])


class LayerNormConv:
    """What the sublayers of a parallel block read: hn = (x - mean) / sqrt(var + eps) * w + b (var = mean of the squared deviations), and h = hn + conv(hn),
    conv(hn)_t = sum_j c[:, j] hn_(t - taps + 1 + j) per channel with zeros before the sequence's start.  Like CanonNorm it is never a kernel chain of its own:
    the residual update before it writes it (one launch for steps of one row per sequence, two for prompt steps), and it hands out BOTH rows -- the
    feed-forward reads hn, the mixer reads h.  The last taps - 1 normed rows of a sequence live in its slot."""

    def __init__(self, width: int, taps: int, eps: float):
        if taps < 1 or taps > 16:
            raise RuntimeError(f"input convolution: {taps} taps")
        self.width, self.taps, self.eps = width, int(taps), float(eps)
        self.dtype = torch.bfloat16

    def load(self, stc, norm_key: str, conv_key: str, dtype, device):
        self.w, self.b = _f32(stc, norm_key, device), _f32(stc, norm_key + ".b", device)
        self.conv = _f32(stc, conv_key, device).t().contiguous()               # stored [width, taps]; the kernels read one tap of neighbouring channels at once
        assert self.w.numel() == self.width and self.b.numel() == self.width and self.conv.shape == (self.taps, self.width)
        self.dtype = dtype
        return self

    def state_spec(self, name: str) -> StateSpec:
        return StateSpec(name, (max(self.taps - 1, 1), self.width), self.dtype)

    def apply(self, x: torch.Tensor, y: torch.Tensor | None, y2: torch.Tensor | None, scale: float, mode: int, sb: StepBatch, ring: torch.Tensor):
        """x <- x | x + (y + y2) scale | (y + y2) scale; returns (hn, h) [n, width] in the activation type."""
        hn = torch.empty((sb.n, self.width), dtype=self.dtype, device=x.device)
        h = torch.empty_like(hn)
        if sb.decode:
            mix_ops.residual_norm_conv(x, y, y2, scale, mode, True, self.w, self.b, self.eps, h, hn, self.conv, ring, sb.tok_seq, sb.tok_pos, sb.slots)
        else:
            mix_ops.residual_norm_conv(x, y, y2, scale, mode, True, self.w, self.b, self.eps, None, hn)
            mix_ops.canon(h, hn, self.conv, ring, sb.tok_seq, sb.tok_pos, sb.slots, sb.pos0, sb.len_after)
        return hn, h


class _SideMixer:
    """Shared plumbing of the mixers below: a mixer either owns its fused input product (load / forward) or lends its parts to a ParallelMixer, which runs
    one product for both of its mixers and calls `run` with the parts' views.  `tag` prefixes the mixer's part names and its state names."""
    tag = ""

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        self.inp = FusedInput(self.input_parts(stc, prefix, dtype, device) + list(extra_parts))
        self.load_rest(stc, prefix, dtype, device)

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        return self.run(p, self.inp, sb, state), p


class SigmoidAttention(_SideMixer):
    """H query heads over G key/value heads, no biases, no rotation (positions do not enter the scores), causal without a window.  The weight of a visible key
    is sigmoid(scale q.k + bias_head); weights are NOT normalised over keys.  Keys and values of every token stay: they live in the cache's pages."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float):
        if heads % kv_heads:
            raise RuntimeError(f"attention: {heads} query heads over {kv_heads} key/value heads")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim, self.scale = width, heads, kv_heads, dim, vdim, float(scale)
        self.dtype = torch.bfloat16

    def input_parts(self, stc, prefix, dtype, device):
        return [(self.tag + nm, _w(stc, prefix + nm, dtype, device), None) for nm in ("q", "k", "v")]

    def load_rest(self, stc, prefix, dtype, device):
        self.bias = _f32(stc, prefix + "pb", device)
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.bias.numel() == self.heads and self.w_o.shape == (self.width, self.heads * self.vdim)
        self.dtype = dtype

    def state_specs(self) -> list:
        from .state_cache import PagedSpec
        return [PagedSpec(self.tag + "k", (self.kv_heads * self.dim,), self.dtype), PagedSpec(self.tag + "v", (self.kv_heads * self.vdim,), self.dtype)]

    def run(self, p: dict, inp: FusedInput, sb: StepBatch, state: dict) -> torch.Tensor:
        H, G, d, dv, t = self.heads, self.kv_heads, self.dim, self.vdim, self.tag
        q, k, v = p[t + "q"], p[t + "k"], p[t + "v"]
        assert q.shape[1] == H * d and k.shape[1] == G * d and v.shape[1] == G * dv
        kp, vp, table = state[t + "k"], state[t + "v"], state["page_table"]
        mix_ops.paged_store(kp, vp, k, v, table, sb.tok_seq, sb.tok_pos, sb.slots)
        out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=q.device)
        if sb.decode:
            mix_ops.sigattn_decode(out, q, kp, vp, self.bias, table, sb.slots, sb.len_after, H, G, d, dv, self.scale)
        else:
            mix_ops.sigattn_prefill(out, q, k, v, self.bias, sb.cu, sb.tok_seq, H, G, d, dv, self.scale, sb.max_rows)
        return F.linear(out, self.w_o)


class MatrixLSTM(_SideMixer):
    """mLSTM: q = W_q h dim^(-1/2), k, v per head; log gates i = cap tanh((W_i h + b_i) / cap), f = logsigmoid(cap tanh((W_f h + b_f) / cap)); running maximum
    m' = max(f + m, i) (m = 0 at the start); S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k; o = S^T q / (max(|n.q|, e^(-m')) + 1e-6); per-head unit
    RMS, a weight over all heads' values, sigmoid(W_g h), W_o.  State per slot: S [heads, vdim, dim], n [heads, dim], m [heads], float32."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float):
        self.width, self.heads, self.dim, self.vdim, self.cap, self.eps = width, heads, dim, vdim, float(gate_cap), float(eps)
        self.q_scale = float(dim) ** -0.5
        self.dtype = torch.bfloat16

    def input_parts(self, stc, prefix, dtype, device):
        return [(self.tag + nm, _w(stc, prefix + nm, dtype, device), None) for nm in ("q", "k", "v", "g", "i", "f")]

    def load_rest(self, stc, prefix, dtype, device):
        self.bias_i, self.bias_f = _f32(stc, prefix + "i.b", device), _f32(stc, prefix + "f.b", device)
        self.norm_w = _f32(stc, prefix + "norm", device)
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.norm_w.numel() == self.heads * self.vdim and self.w_o.shape == (self.width, self.heads * self.vdim) and self.bias_i.numel() == self.heads
        self.dtype = dtype

    def state_specs(self) -> list:
        t = self.tag
        return [StateSpec(t + "S", (self.heads, self.vdim, self.dim), torch.float32), StateSpec(t + "n", (self.heads, self.dim), torch.float32),
                StateSpec(t + "m", (self.heads,), torch.float32)]

    def run(self, p: dict, inp: FusedInput, sb: StepBatch, state: dict) -> torch.Tensor:
        H, d, dv, t = self.heads, self.dim, self.vdim, self.tag
        assert p[t + "q"].shape[1] == H * d and p[t + "v"].shape[1] == H * dv and p[t + "i"].shape[1] == H
        o = torch.empty((sb.n, H, dv), dtype=torch.float32, device=self.w_o.device)
        mix_ops.mlstm_scan(o, state[t + "S"], state[t + "n"], state[t + "m"], p[t + "q"], p[t + "k"], p[t + "v"], p[t + "i"], p[t + "f"], self.bias_i, self.bias_f,
                           sb.cu, sb.slots, sb.pos0, self.q_scale, self.cap)
        out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=o.device)
        mix_ops.head_norm_gate(out, o, self.norm_w, p[t + "g"], mix_ops.GATE_SIGMOID, self.eps)
        return F.linear(out, self.w_o)


class GatedDeltaRule(_SideMixer):
    """Gated delta rule: q, k (kv_heads x dim) and v (heads x vdim) pass a short causal convolution per channel and silu; q, k become unit vectors per head
    (x / sqrt(sum x^2 + 1e-6)), q times dim^(-1/2); beta = sigmoid(W_b h); decay g = exp(-exp(A_log) softplus(W_a h + dt_bias)) per head; per head S <- g S,
    u = beta (v - S^T k), S <- S + k u^T, o = S^T q; per-head unit RMS, a weight over vdim shared by the heads, silu(W_g h), W_o.  State per slot: S
    [heads, vdim, dim] float32 and the last taps - 1 rows of the projections q | k | v."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, eps: float):
        if heads % kv_heads:
            raise RuntimeError(f"delta rule: {heads} value heads over {kv_heads} query/key heads")
        if taps < 1 or taps > 16:
            raise RuntimeError(f"delta rule: {taps} taps")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.eps = width, heads, kv_heads, dim, vdim, int(taps), float(eps)
        self.channels = 2 * kv_heads * dim + heads * vdim
        self.q_scale = float(dim) ** -0.5
        self.dtype = torch.bfloat16

    def input_parts(self, stc, prefix, dtype, device):
        return [(self.tag + nm, _w(stc, prefix + nm, dtype, device), None) for nm in ("q", "k", "v", "b", "a", "g")]       # q, k, v side by side: one block

    def load_rest(self, stc, prefix, dtype, device):
        conv = torch.cat([_f32(stc, prefix + nm + ".conv", device) for nm in ("q", "k", "v")], dim=0)      # [channels, taps]
        self.conv = conv.t().contiguous()
        self.A_log, self.dt_bias = _f32(stc, prefix + "A_log", device), _f32(stc, prefix + "dt_bias", device)
        self.norm_w = _f32(stc, prefix + "norm", device)
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.conv.shape == (self.taps, self.channels) and self.A_log.numel() == self.heads and self.norm_w.numel() == self.vdim
        assert self.w_o.shape == (self.width, self.heads * self.vdim)
        self.dtype = dtype

    def state_specs(self) -> list:
        t = self.tag
        return [StateSpec(t + "S", (self.heads, self.vdim, self.dim), torch.float32), StateSpec(t + "conv", (max(self.taps - 1, 1), self.channels), self.dtype)]

    def run(self, p: dict, inp: FusedInput, sb: StepBatch, state: dict) -> torch.Tensor:
        H, G, d, dv, t = self.heads, self.kv_heads, self.dim, self.vdim, self.tag
        x = inp.block(p, t + "q", t + "v")
        assert x.shape[1] == self.channels and p[t + "b"].shape[1] == H and p[t + "g"].shape[1] == H * dv
        dev, f32 = self.w_o.device, torch.float32
        q, k = torch.empty((sb.n, G * d), dtype=f32, device=dev), torch.empty((sb.n, G * d), dtype=f32, device=dev)
        v = torch.empty((sb.n, H * dv), dtype=f32, device=dev)
        beta, decay = torch.empty((sb.n, H), dtype=f32, device=dev), torch.empty((sb.n, H), dtype=f32, device=dev)
        mix_ops.delta_prep(q, k, v, beta, decay, x, self.conv, state[t + "conv"], p[t + "b"], p[t + "a"], self.A_log, self.dt_bias, sb.tok_seq, sb.tok_pos, sb.slots,
                           sb.pos0, sb.len_after, H, G, d, dv, self.q_scale)
        o = torch.empty((sb.n, H, dv), dtype=f32, device=dev)
        mix_ops.delta_scan(o, state[t + "S"], q, k, v, beta, decay, sb.cu, sb.slots, sb.pos0, G)
        out = torch.empty((sb.n, H * dv), dtype=self.dtype, device=dev)
        mix_ops.head_norm_gate(out, o, self.norm_w, p[t + "g"], mix_ops.GATE_SILU, self.eps)
        return F.linear(out, self.w_o)


class ParallelMixer(_SideMixer):
    """Two mixers side by side that read the same input: ONE fused input product for both, then
    result = mean of the two outputs, each RMS-normed over the model width with its own plain weight."""

    def __init__(self, width: int, left, right, eps: float):
        self.width, self.left, self.right, self.eps = width, left, right, float(eps)
        left.tag, right.tag = "left.", "right."

    def input_parts(self, stc, prefix, dtype, device):
        return self.left.input_parts(stc, prefix + "left.", dtype, device) + self.right.input_parts(stc, prefix + "right.", dtype, device)

    def load_rest(self, stc, prefix, dtype, device):
        self.left.load_rest(stc, prefix + "left.", dtype, device)
        self.right.load_rest(stc, prefix + "right.", dtype, device)
        self.w_left, self.w_right = _f32(stc, prefix + "left.out", device), _f32(stc, prefix + "right.out", device)
        assert self.w_left.numel() == self.width and self.w_right.numel() == self.width
        self.dtype = dtype

    def state_specs(self) -> list:
        return self.left.state_specs() + self.right.state_specs()

    def run(self, p: dict, inp: FusedInput, sb: StepBatch, state: dict) -> torch.Tensor:
        a = self.left.run(p, inp, sb, state)
        b = self.right.run(p, inp, sb, state)
        out = torch.empty((sb.n, self.width), dtype=self.dtype, device=a.device)
        mix_ops.rms_pair(out, a, self.w_left, b, self.w_right, 0.5, self.eps)
        return out


class ParallelBlock:
    """x <- x + m (mixer(h) + ff(hn)) with hn = norm(x) and h = hn + conv(hn): ONE norm per layer, the feed-forward reads the normed rows, the mixer their short
    causal convolution; m is the residual factor.  The block is entered with (hn, h) already computed and leaves by computing the next block's pair: the
    residual update (both sublayers' outputs, the factor, float32) and the next layer norm are one kernel."""

    def __init__(self, width: int, eps: float, taps: int, mixer, mlp, residual_mult: float = 1.0):
        self.width, self.eps, self.mixer, self.mlp, self.mult = width, float(eps), mixer, mlp, float(residual_mult)
        self.in1 = LayerNormConv(width, taps, eps)

    def load(self, stc, prefix: str, dtype, device):
        self.in1.load(stc, prefix + "norm1", prefix + "canon1", dtype, device)
        self.mixer.load(stc, prefix + "mix.", dtype, device)
        if self.mlp is not None:
            self.mlp.load(stc, prefix + "mlp.", dtype, device)
        self.dtype = dtype

    def state_specs(self) -> list:
        return self.mixer.state_specs() + [self.in1.state_spec("canon1")]

    def forward(self, x: torch.Tensor, hn: torch.Tensor, h: torch.Tensor, sb: StepBatch, state: dict, nxt: tuple | None):
        """x: float32 residual (updated in place).  nxt = (the next block's LayerNormConv, its ring): returns the next block's (hn, h); None: the bare update."""
        y, _ = self.mixer.forward(h, sb, state)
        y2 = self.mlp.forward(hn, sb)[0] if self.mlp is not None else None
        if nxt is None:
            mix_ops.residual_norm_conv(x, y, y2, self.mult, mix_ops.RES_ADD, False, None, None, self.eps, None)
            return None
        return nxt[0].apply(x, y, y2, self.mult, mix_ops.RES_ADD, sb, nxt[1])
