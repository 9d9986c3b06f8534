"""
Dikopel: a decoder-only model of PARALLEL blocks over a float32 stream -- one layer norm per layer whose output feeds both sublayers, the feed-forward
directly and the mixer through a short causal convolution, x <- x + m (mixer + ff) with a residual factor m.  The embedding is scaled and gets a
sinusoidal position vector.  A layer's mixer is either a matrix memory with exponential gating (mLSTM), or two mixers side by side whose outputs are
RMS-normed and averaged: causal attention without softmax (sigmoid weights with a bias per head, no rotation, no window) and a gated delta rule with
short convolutions.  The feed-forward is a gated silu layer, a mixture of such experts (sigmoid scores, a selection-only correction, groups of experts
scored by the sum of their two best choice scores, a shared expert behind a sigmoid gate per token), or none.  A layer may use another layer's weights
with a state of its own.  The order of layers and every size and constant come from config.json:

    architecture "Dikopel"; vocab; width; norm.eps; canon.taps; embedding.scale; residual_mult
    layers[i]: type "mlstm":    mixer {heads, dim, vdim, gate_cap}
               type "parallel": mixer {left {heads, kv_heads, dim, vdim, scale}, right {heads, kv_heads, dim, vdim, conv}}
               mlp: null | {"kind": "dense", ff} | {"kind": "moe", expert {ff}, router {experts, top, scale, groups {count, keep}}, shared {ff}}
               weights_of: j (optional): the layer runs with layer j's tensors

Tensor names: embed, head, final.norm(.b), l<i>.norm1(.b), l<i>.canon1; mLSTM l<i>.mix.{q,k,v,g,o,norm,i,i.b,f,f.b}; parallel l<i>.mix.left.{q,k,v,pb,o,out},
l<i>.mix.right.{q,k,v}(.conv), right.{b,a,A_log,dt_bias,g,norm,o,out}; l<i>.mlp.{gate,up,down} or l<i>.mlp.e<j>.{gate,up,down}, mlp.router, mlp.correction,
mlp.shared.{gate,up,down,sg}.

The model is a list of ParallelBlock over the mechanisms of modules.py; its state is a SlotStateCache with one entry per layer (a layer that borrows
weights has its own); `step` is the one function the generator, the command line and the trace runner call.
"""
from __future__ import annotations
import json
import os
import torch
import torch.nn.functional as F
from . import mix_ops
from .loader import SafetensorsCollection
from .modules import GatedDeltaRule, GatedMLP, MatrixLSTM, ParallelBlock, ParallelMixer, SigmoidAttention, SparseExperts, _f32, _w
from .state_cache import SlotStateCache, StepBatch

# a group of experts is scored by the sum of this many of its largest choice scores; the position vector's base
GROUP_TOP = 2
POSITION_BASE = 10000.0


class DikopelConfig:
    def __init__(self, d: dict):
        self.vocab = int(d["vocab"])
        self.width = int(d["width"])
        self.eps = float(d["norm"]["eps"])
        self.taps = int((d.get("canon") or {}).get("taps", 1))
        self.embed_scale = float((d.get("embedding") or {}).get("scale", 1.0))
        self.mult = float(d.get("residual_mult", 1.0))
        self.layers = d["layers"]
        if not self.layers:
            raise RuntimeError("Dikopel: config has no layers")
        self.source = []                         # layer -> the layer whose tensors it uses
        for i, L in enumerate(self.layers):
            j = L.get("weights_of")
            j = i if j is None else int(j)
            if not 0 <= j < len(self.layers) or self.layers[j].get("weights_of") is not None and j != i:
                raise RuntimeError(f"Dikopel: layer {i} borrows the weights of layer {j}, which has none of its own")
            self.source.append(j)

    def _mixer(self, i: int, L: dict):
        m, w = L["mixer"], self.width
        if L["type"] == "mlstm":
            return MatrixLSTM(w, int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), float(m["gate_cap"]), self.eps)
        if L["type"] == "parallel":
            a, b = m["left"], m["right"]
            left = SigmoidAttention(w, int(a["heads"]), int(a.get("kv_heads", a["heads"])), int(a["dim"]), int(a.get("vdim", a["dim"])), float(a["scale"]))
            right = GatedDeltaRule(w, int(b["heads"]), int(b.get("kv_heads", b["heads"])), int(b["dim"]), int(b.get("vdim", b["dim"])), int(b.get("conv", 1)), self.eps)
            return ParallelMixer(w, left, right, self.eps)
        raise RuntimeError(f"Dikopel: layer {i} has an unknown mixer type {L['type']!r}")

    def _mlp(self, i: int, L: dict):
        f, w = L.get("mlp"), self.width
        if f is None:
            return None
        if f["kind"] == "dense":
            return GatedMLP(w, int(f["ff"]), "silu")
        if f["kind"] == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            count = int(g.get("count", 1))
            sh = f.get("shared")
            shared = GatedMLP(w, int(sh["ff"]), "silu", row_gate="sg") if sh else None
            return SparseExperts(w, int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), router="sigmoid", router_bias=False, correction=True,
                                 route_scale=float(r.get("scale", 1.0)), act="silu", shared=shared, groups=count, keep_groups=int(g.get("keep", count)),
                                 group_top=GROUP_TOP)
        raise RuntimeError(f"Dikopel: layer {i} has an unknown feed-forward kind {f['kind']!r}")

    def build_blocks(self) -> dict:
        """One block per layer that has tensors of its own."""
        return {i: ParallelBlock(self.width, self.eps, self.taps, self._mixer(i, L), self._mlp(i, L), self.mult)
                for i, L in enumerate(self.layers) if self.source[i] == i}


class DikopelModel:
    architecture = "Dikopel"
    native_libraries = ("mix",)          # what a fresh checkout has to compile before this model runs
    PAGE_SIZE = 64

    def __init__(self, config: dict, stc, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("Dikopel runs in bfloat16 or float32")
        self.cfg = DikopelConfig(config)
        self.device, self.dtype = torch.device(device), dtype
        self.vocab = self.cfg.vocab
        own = self.cfg.build_blocks()
        for i, blk in own.items():
            blk.load(stc, f"l{i}.", dtype, self.device)
        self.blocks = [own[j] for j in self.cfg.source]          # in execution order; a borrowing layer is the lender's block over its own state
        self.embed = _w(stc, "embed", dtype, self.device)
        self.head = _w(stc, "head", dtype, self.device)
        self.final_w, self.final_b = _f32(stc, "final.norm", self.device), _f32(stc, "final.norm.b", self.device)
        w = self.cfg.width
        assert self.embed.shape == (self.vocab, w) and self.head.shape == (self.vocab, w) and self.final_w.numel() == w
        i = torch.arange((w + 1) // 2, dtype=torch.float64)
        self.pos_freq = (POSITION_BASE ** (-2.0 * i / w)).to(torch.float32).to(self.device).contiguous()       # computed in float64, rounded once
        self.layer_taps = None               # diagnostics: a list that receives a copy of the residual after every layer

    @classmethod
    def from_directory(cls, directory: str, device="cuda:0", dtype=torch.bfloat16) -> "DikopelModel":
        with open(os.path.join(directory, "config.json")) as f:
            config = json.load(f)
        return cls(config, SafetensorsCollection(directory), device=device, dtype=dtype)

    def new_cache(self, slots: int = 4, tokens: int = 0) -> SlotStateCache:
        """One state entry per layer; tokens: the most tokens alive at once, if known (sizes the pages of the attention layers)."""
        return SlotStateCache([blk.state_specs() for blk in self.blocks], self.device, slots=slots, page_size=self.PAGE_SIZE, tokens=tokens)

    @torch.no_grad()
    def step(self, sb: StepBatch, cache: SlotStateCache) -> torch.Tensor | None:
        """Run the step's rows through every layer over the slots of `cache`; returns float32 logits [wanted rows, vocab] (None if none are wanted)."""
        w, n = self.cfg.width, sb.n
        x = torch.empty((n, w), dtype=torch.float32, device=self.device)
        mix_ops.embed_sinusoid(x, self.embed, sb.tokens, sb.tok_pos, self.pos_freq, self.cfg.embed_scale)
        hn, h = self.blocks[0].in1.apply(x, None, None, 1.0, mix_ops.RES_KEEP, sb, cache.layers[0]["canon1"])
        for r, blk in enumerate(self.blocks):
            nxt = (self.blocks[r + 1].in1, cache.layers[r + 1]["canon1"]) if r + 1 < len(self.blocks) else None
            pair = blk.forward(x, hn, h, sb, cache.layers[r], nxt)
            if pair is not None:
                hn, h = pair
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        if sb.want_rows is None or sb.want_rows.numel() == 0:
            return None
        hw = torch.empty((sb.want_rows.numel(), w), dtype=self.dtype, device=self.device)
        mix_ops.layer_norm_rows(hw, x, sb.want_rows, self.final_w, self.final_b, self.cfg.eps)
        return F.linear(hw, self.head).float()
