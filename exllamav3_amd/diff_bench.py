"""
`bench.py --diff-family`: prefill and decode throughput of Fimunex layers (differential chunked attention behind input convolutions, with ungated relu^2
experts under a grouped softmax router with identity experts, or without a feed-forward; random weights) at sizes that resemble real models' layers, beside
the closest existing model -- Vofanex layers (sliding-window sink attention with softmax-routed gated experts, or without a feed-forward counterpart: its
PolyNorm layer) of the same width / head / expert shape, timed in the same process -- and each kernel of the design alone against its roofline, next to the
like kernel of the closest model.  Prints one JSON line; the default workload of bench.py and the JSON line it prints are untouched.
"""
from __future__ import annotations
import json
import math
import time
import torch
from .mixer_bench import PEAK_BF16, PEAK_HBM, SIZES, TensorDict, _time, kernel_legs, model_legs

# differential attention at the sizes of mixer_bench.SIZES: half the heads, each with two maps of the head dim and values twice as wide, so that the
# projections and the attention core do the work of the plain attention layer of the same name; chunk = that layer's window
TAPS = 4
YARN = {"factor": 8.0, "original": 8192, "fast": 24.0, "slow": 2.0}
SOFTCAP, DIFF, ROT_BASE = 30.0, 0.5, 1.0e6
KINDS = [("attention", "none"), ("attention", "moe")]


def shape(size: dict) -> dict:
    return dict(heads=size["heads"] // 2, kv_heads=size["kv_heads"] // 2, dim=size["dim"], vdim=2 * size["dim"], chunk=size["window"], identity=2, groups=(2, 1))


def synth(size: dict, kinds, vocab=32000, seed=0, device="cuda:0", loop=None):
    """Random Fimunex weights and their config: size = width / heads / window / moe (experts, top, expert ff); loop = (start, stop, times)."""
    g = torch.Generator(device=device).manual_seed(seed)
    w, t, layers, sh = size["width"], {}, [], shape(size)

    def lin(name, o, i, s=1.0):
        t[name] = (torch.randn(o, i, generator=g, device=device) * (s / math.sqrt(i))).to(torch.bfloat16)

    def vec(name, n, mean=0.0, s=0.1):
        t[name] = (mean + s * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)
    lin("embed", vocab, w, math.sqrt(w)); lin("head", vocab, w); vec("final.norm", w)
    H, G, d, dv = sh["heads"], sh["kv_heads"], sh["dim"], sh["vdim"]
    for i, (mix, ff) in enumerate(kinds):
        p = f"l{i}."
        vec(p + "norm1", w); t[p + "canon1"] = (0.3 * torch.randn(w, TAPS, generator=g, device=device)).to(torch.bfloat16)
        lin(p + "mix.q", H * 2 * d, w); lin(p + "mix.k", G * 2 * d, w); lin(p + "mix.v", G * dv, w); lin(p + "mix.g", H, w); lin(p + "mix.o", w, H * dv)
        for b, n in (("q", H * 2 * d), ("k", G * 2 * d), ("v", G * dv), ("o", w)):
            vec(p + f"mix.{b}.b", n)
        vec(p + "mix.q.norm", d, 1.0); vec(p + "mix.k.norm", d, 1.0)
        for nm in ("lq1", "lk1", "lq2", "lk2"):
            vec(p + "mix." + nm, d)
        mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5, "softcap": SOFTCAP, "diff": DIFF, "mask": {"size": sh["chunk"]},
                 "rot": {"base": ROT_BASE, "dims": d, "scaling": YARN}}
        if ff == "none":
            mlp = None
        else:
            E, top, eff = size["moe"]
            vec(p + "norm2", w); t[p + "canon2"] = (0.3 * torch.randn(w, TAPS, generator=g, device=device)).to(torch.bfloat16)
            for e in range(E):
                lin(f"{p}mlp.e{e}.up", eff, w); lin(f"{p}mlp.e{e}.down", w, eff)
            lin(p + "mlp.router", E + sh["identity"], w); vec(p + "mlp.correction", E + sh["identity"])
            mlp = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top, "identity": sh["identity"], "groups": {"count": sh["groups"][0], "keep": sh["groups"][1]}}}
        layers.append({"type": mix, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Fimunex", "vocab": vocab, "width": w, "norm": {"eps": 1e-5}, "canon": {"taps": TAPS}, "logit_softcap": 20.0, "layers": layers}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg, TensorDict(t)


def _make(size, kind, reps, dev):
    from .fimunex import FimunexModel
    cfg, td = synth(size, [kind] * reps, device=dev)
    return FimunexModel(cfg, td, device=dev, dtype=torch.bfloat16)


def diff_kernel_legs(size_name: str, prompt: int, ctx: int, dev):
    """Each kernel of the design alone at the size's shapes: time and the fraction of the roofline that bounds it."""
    from . import mix_ops
    from .modules import rotary_frequencies
    s = SIZES[size_name]
    sh = shape(s)
    out, bf = {}, torch.bfloat16
    rnd = lambda *a: torch.randn(*a, device=dev).to(bf)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    H, G, d, dv, C, w = sh["heads"], sh["kv_heads"], sh["dim"], sh["vdim"], sh["chunk"], s["width"]
    n = prompt
    cu, seq, pos = i32([0, n]), torch.zeros(n, dtype=torch.int32, device=dev), torch.arange(n, dtype=torch.int32, device=dev)
    sl, la, p0 = i32([0]), i32([n]), i32([0])
    hbm = lambda by, t: {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    freq, mag = rotary_frequencies(d, ROT_BASE, YARN)
    freq = freq.to(dev)
    q, k, v = rnd(n, H * 2 * d), rnd(n, G * 2 * d), rnd(n, G * dv)
    rk, rv = torch.zeros((16, C, G * 2, d), dtype=bf, device=dev), torch.zeros((16, C, G, dv), dtype=bf, device=dev)
    qn = torch.ones(d, device=dev)
    t = _time(lambda: mix_ops.qk_prep(q, k, v, qn, qn, freq, mag, False, 1e-5, rk, rv, seq, pos, sl, la, d), 20)
    out["qk_prep_prefill"] = hbm(n * (H + G) * 2 * d * 2 * 2 + C * (G * 2 * d + G * dv) * 2 * 2, t)
    a = torch.empty((n, H * 2 * dv), dtype=torch.float32, device=dev)
    pairs = sum(i % C + 1 for i in range(n))
    fl = 2.0 * (d + dv) * pairs * H * 2
    for cap in (SOFTCAP, 0.0):
        t = _time(lambda: mix_ops.attn_prefill_maps(a, q, k, v, None, None, cu, seq, pos, H, G, 2, d, dv, d ** -0.5, cap, C, mix_ops.MASK_CHUNK, max_rows=n, mfma=True), 10)
        out["attn_prefill_mfma_two_maps_chunk" + ("_softcap" if cap else "_no_softcap")] = {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_bf16_peak": fl / t / PEAK_BF16}
    o, gt = torch.empty((n, H * dv), dtype=bf, device=dev), rnd(n, H)
    for cap in (SOFTCAP, 0.0):
        t = _time(lambda: mix_ops.attn_prefill_diff(o, q, k, v, gt, cu, H, G, d, dv, d ** -0.5, cap, C, mix_ops.MASK_CHUNK, 0.7, DIFF, 1e-5, n), 10)
        out["attn_prefill_mfma_diff_fused" + ("_softcap" if cap else "_no_softcap")] = {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_bf16_peak": fl / t / PEAK_BF16}
    t = _time(lambda: mix_ops.diff_combine(o, a, 0.7, DIFF, 1e-5, gt, H, dv), 20)
    out["diff_combine_prefill"] = hbm(n * H * dv * (2 * 4 + 2), t)
    for bs in (1, 16):
        qd, ad = rnd(bs, H * 2 * d), torch.empty((bs, H * 2 * dv), dtype=torch.float32, device=dev)
        sld, lad = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        t = _time(lambda: mix_ops.attn_decode_maps(ad, qd, rk, rv, None, None, sld, lad, H, 2, d ** -0.5, SOFTCAP, mix_ops.MASK_CHUNK), 50)
        keys = (ctx - 1) % C + 1
        out[f"attn_decode_two_maps_bs{bs}"] = hbm(bs * keys * (G * 2 * d + G * dv) * 2, t)
        kd, vd, sq, pd = rnd(bs, G * 2 * d), rnd(bs, G * dv), torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx - 1] * bs)
        t = _time(lambda: mix_ops.qk_prep(qd, kd, vd, qn, qn, freq, mag, False, 1e-5, rk, rv, sq, pd, sld, lad, d), 50)
        out[f"qk_prep_bs{bs}"] = {"us": t * 1e6}
        od, gd = torch.empty((bs, H * dv), dtype=bf, device=dev), rnd(bs, H)
        t = _time(lambda: mix_ops.diff_combine(od, ad, 0.7, DIFF, 1e-5, gd, H, dv), 50)
        out[f"diff_combine_bs{bs}"] = {"us": t * 1e6}
    x, y, nw, cw = torch.randn(n, w, device=dev), rnd(n, w), torch.ones(w, device=dev), 0.3 * torch.randn(TAPS, w, device=dev)
    hn, h, ring = torch.empty((n, w), dtype=bf, device=dev), torch.empty((n, w), dtype=bf, device=dev), torch.zeros((16, TAPS - 1, w), dtype=bf, device=dev)
    t1 = _time(lambda: mix_ops.residual_rms(x, y, mix_ops.RES_ADD, nw, 1e-5, hn), 20)
    t2 = _time(lambda: mix_ops.canon(h, hn, cw, ring, seq, pos, sl, p0, la), 20)
    out["residual_rms_prefill"] = hbm(n * w * (4 + 4 + 2 + 2), t1)
    out["canon_prefill"] = hbm(n * w * (2 + 2), t2)
    out["residual_rms_plus_canon_prefill"] = hbm(n * w * (4 + 4 + 2 + 2), t1 + t2)          # what one fused pass would have to move
    for bs in (1, 16):
        xd, yd, hd = torch.randn(bs, w, device=dev), rnd(bs, w), torch.empty((bs, w), dtype=bf, device=dev)
        sq, pd, sld = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx - 1] * bs), torch.arange(bs, dtype=torch.int32, device=dev)
        t = _time(lambda: mix_ops.residual_rms(xd, yd, mix_ops.RES_ADD, nw, 1e-5, hd, cw, ring, sq, pd, sld), 50)
        out[f"residual_rms_canon_fused_bs{bs}"] = {"us": t * 1e6}
    E, top, eff = s["moe"]
    tot = E + sh["identity"]
    lg, idx, wt, idw, corr = torch.randn(n, tot, device=dev), torch.empty((n, top), dtype=torch.int32, device=dev), torch.empty((n, top), device=dev), torch.empty(n, device=dev), torch.zeros(tot, device=dev)
    t = _time(lambda: mix_ops.topk_grouped(idx, wt, idw, lg, corr, mix_ops.ROUTE_SOFTMAX_ALL, E, sh["groups"][0], sh["groups"][1]), 20)
    out["topk_grouped_prefill"] = {"us": t * 1e6}
    wu, wd = rnd(E, eff, w), rnd(E, w, eff)
    for bs in (1, 16):
        hh, ix = rnd(bs, w), torch.stack([torch.randperm(E, device=dev)[:top] for _ in range(bs)]).int().contiguous()
        wts, hid, yy, iw = torch.full((bs, top), 1.0 / top, device=dev), torch.empty((bs * top, eff), dtype=bf, device=dev), torch.empty((bs, w), dtype=bf, device=dev), torch.zeros(bs, device=dev)
        if bs == 1:
            def moe():
                mix_ops.moe_up_act(hid, hh, wu, ix, mix_ops.ACT_RELU2); mix_ops.moe_down_id(yy, hid, wd, ix, wts, hh, iw)
        else:
            def moe():
                mix_ops.moe_expert_major_plain(yy, hh, wu, wd, ix, wts, mix_ops.ACT_RELU2, iw)
        t = _time(moe, 50)
        by = min(bs * top, E) * 2 * eff * w * 2
        out[f"moe_ungated_decode_bs{bs}"] = {"us": t * 1e6, "GBps_distinct_weights": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    return out


def run(args) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from . import _lib
    _lib.mixlib()
    prompt, ctx = args.prefill_tokens, 1000
    res = {"metric": "diff_family_layer_times", "unit": "ms per layer", "dtype": "bf16", "data": "synthetic", "prompt": prompt, "ctx": ctx, "sizes": {}}
    for name in (args.mixer_sizes.split(",") if args.mixer_sizes else list(SIZES)):
        t0 = time.time()
        entry = {"shape": shape(SIZES[name]), "fimunex_layers": model_legs(name, prompt, ctx, args.steps, dev, kinds=KINDS, make=_make),
                 "kernels": diff_kernel_legs(name, prompt, ctx, dev)}
        try:
            entry["closest_model_vofanex_layers"] = model_legs(name, prompt, ctx, args.steps, dev, kinds=[("attention", "dense"), ("attention", "moe")])
            entry["closest_model_kernels"] = kernel_legs(name, prompt, ctx, dev)
        except Exception as e:                       # the comparison leg must not hide the new design's numbers
            entry["closest_model_error"] = f"{type(e).__name__}: {e}"
        entry["seconds"] = round(time.time() - t0, 1)
        res["sizes"][name] = entry
    print(json.dumps(res))
    return 0
