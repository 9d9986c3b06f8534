"""
Fimunex: a decoder-only model of pre-norm blocks over a float32 stream whose sublayers read a short causal convolution of the normed stream.  The mixer is
differential attention (two attention maps per head over shared values, RMS-normed and rotated queries / keys, soft-capped scores, a chunk mask, a
head-wise sigmoid gate); the feed-forward is a mixture of ungated relu^2 experts chosen by a softmax router with a selection-only correction, groups of
experts of which only the best are eligible, and trailing router outputs that stand for experts which return their input -- or none.  A block of
consecutive layers may run several times in a row with the same weights, state being kept per pass.  The order of layers and every size and constant
come from config.json:

    architecture "Fimunex"; vocab; width; norm.eps; canon.taps; logit_softcap (optional); loop {start, stop, times} (optional)
    layers[i]: type "attention", mixer {heads, kv_heads, dim, vdim, scale, softcap, diff, mask.size, rot {base, dims, scaling {factor, original, fast, slow} (optional)}},
               mlp ({"kind": "moe", "expert": {ff}, "router": {experts, top, identity, groups {count, keep}}} | null)

Tensor names: embed, head, final.norm, l<i>.norm1 / norm2 / canon1 / canon2, l<i>.mix.{q,k,v,o}(.b), mix.q.norm, mix.k.norm, mix.lq1 / lk1 / lq2 / lk2, mix.g,
l<i>.mlp.e<j>.up / down, mlp.router, mlp.correction.

The model is a list of CanonBlock over the mechanisms of modules.py; its state is a SlotStateCache with one entry per layer RUN (a looped layer has its
rings once per pass); `step` is the one function the generator, the command line and the trace runner call.
"""
from __future__ import annotations
import json
import os
import torch
import torch.nn.functional as F
from . import mix_ops
from .loader import SafetensorsCollection
from .modules import CanonBlock, DifferentialAttention, SparseExperts, _f32, _w
from .state_cache import SlotStateCache, StepBatch


class FimunexConfig:
    def __init__(self, d: dict):
        self.vocab = int(d["vocab"])
        self.width = int(d["width"])
        self.eps = float(d["norm"]["eps"])
        self.taps = int((d.get("canon") or {}).get("taps", 1))
        self.logit_softcap = float(d.get("logit_softcap") or 0.0)
        self.layers = d["layers"]
        if not self.layers:
            raise RuntimeError("Fimunex: config has no layers")
        loop, n = d.get("loop"), len(self.layers)
        if loop:
            self.loop = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
            a, b, t = self.loop
            if not (0 <= a < b <= n and t >= 1):
                raise RuntimeError(f"Fimunex: loop {self.loop} does not fit {n} layers")
        else:
            self.loop = None

    def runs(self) -> list[int]:
        """Layer indices in execution order, the loop unrolled."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        a, b, t = self.loop
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    def build_layers(self) -> list[CanonBlock]:
        out = []
        for i, L in enumerate(self.layers):
            if L["type"] != "attention":
                raise RuntimeError(f"Fimunex: layer {i} has an unknown mixer type {L['type']!r}")
            m = L["mixer"]
            rot, mask = m.get("rot"), m.get("mask")
            if not mask:
                raise RuntimeError(f"Fimunex: layer {i} has no mask: its cache would not be bounded")
            dim = int(m["dim"])
            mixer = DifferentialAttention(self.width, int(m["heads"]), int(m.get("kv_heads", m["heads"])), dim, int(m.get("vdim", dim)), float(m["scale"]),
                                          float(m.get("softcap") or 0.0), int(mask["size"]), "chunk", float(m["diff"]), self.eps,
                                          rot_dims=int(rot.get("dims", dim)) if rot else 0, rot_base=float(rot["base"]) if rot else 1.0,
                                          rot_scaling=rot.get("scaling") if rot else None)
            f = L.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                mlp = SparseExperts(self.width, int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), router="softmax_all", router_bias=False, correction=True,
                                    act="relu2", gated=False, identity=int(r.get("identity", 0)), groups=int(g.get("count", 1)), keep_groups=int(g.get("keep", 1)))
            else:
                raise RuntimeError(f"Fimunex: layer {i} has an unknown feed-forward kind {f['kind']!r}")
            out.append(CanonBlock(self.width, self.eps, self.taps, mixer, mlp))
        return out


class FimunexModel:
    architecture = "Fimunex"
    native_libraries = ("mix",)          # what a fresh checkout has to compile before this model runs

    def __init__(self, config: dict, stc, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("Fimunex runs in bfloat16 or float32")
        self.cfg = FimunexConfig(config)
        self.device, self.dtype = torch.device(device), dtype
        self.vocab = self.cfg.vocab
        self.blocks = self.cfg.build_layers()
        for i, blk in enumerate(self.blocks):
            blk.load(stc, f"l{i}.", dtype, self.device)
        self.runs = self.cfg.runs()
        self.embed = _w(stc, "embed", dtype, self.device)
        self.head = _w(stc, "head", dtype, self.device)
        self.final_norm = (1.0 + _f32(stc, "final.norm", self.device)).contiguous()
        w = self.cfg.width
        assert self.embed.shape == (self.vocab, w) and self.head.shape == (self.vocab, w) and self.final_norm.numel() == w
        self.layer_taps = None               # diagnostics: a list that receives a copy of the residual after every layer run

    @classmethod
    def from_directory(cls, directory: str, device="cuda:0", dtype=torch.bfloat16) -> "FimunexModel":
        with open(os.path.join(directory, "config.json")) as f:
            config = json.load(f)
        return cls(config, SafetensorsCollection(directory), device=device, dtype=dtype)

    def new_cache(self, slots: int = 4) -> SlotStateCache:
        """One state entry per layer run: a layer inside the loop holds its rings once per pass."""
        return SlotStateCache([self.blocks[i].state_specs() for i in self.runs], self.device, slots=slots)

    @torch.no_grad()
    def step(self, sb: StepBatch, cache: SlotStateCache) -> torch.Tensor | None:
        """Run the step's rows through every layer run over the slots of `cache`; returns float32 logits [wanted rows, vocab] (None if none are wanted)."""
        w, n = self.cfg.width, sb.n
        x = torch.empty((n, w), dtype=torch.float32, device=self.device)
        mix_ops.embed_copy(x, None, self.embed, sb.tokens)
        h = self.blocks[self.runs[0]].in1.apply(x, None, mix_ops.RES_KEEP, sb, cache.layers[0]["canon1"])
        for r, i in enumerate(self.runs):
            nxt = (self.blocks[self.runs[r + 1]].in1, cache.layers[r + 1]["canon1"]) if r + 1 < len(self.runs) else None
            h = self.blocks[i].forward(x, h, sb, cache.layers[r], nxt)
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        if sb.want_rows is None or sb.want_rows.numel() == 0:
            return None
        hw = torch.empty((sb.want_rows.numel(), w), dtype=self.dtype, device=self.device)
        mix_ops.rms_norm_rows(hw, x, sb.want_rows, self.final_norm, self.cfg.eps)
        logits = F.linear(hw, self.head).float()
        if self.cfg.logit_softcap:
            mix_ops.softcap(logits, self.cfg.logit_softcap)
        return logits
