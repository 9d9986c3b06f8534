"""
`bench.py --parallel-family`: prefill and decode throughput of Dikopel layers (parallel blocks over one layer norm: sigmoid attention over paged keys beside a
gated delta rule, or an mLSTM, with a gated silu feed-forward, sigmoid-routed experts with a gated shared expert, or none; random weights) at sizes that
resemble real models' layers, beside the closest existing model -- Vofanex layers (gated linear attention or window attention with a PolyNorm feed-forward or
softmax-routed experts: the same library, unquantized bfloat16, float32 residual, a recurrent layer and an attention layer) of the same width / head /
expert shape, timed in the same process -- and each kernel of the design alone against its roofline, next to the like kernel of the closest model.
Prints one JSON line; the default workload of bench.py and the JSON line it prints are untouched.
"""
from __future__ import annotations
import json
import math
import time
import torch
from .mixer_bench import PEAK_BF16, PEAK_F32, PEAK_HBM, SIZES, TensorDict, _time, kernel_legs, model_legs

TAPS, CONV, GATE_CAP = 4, 4, 15.0
KINDS = [("parallel", "dense"), ("parallel", "moe"), ("mlstm", "moe"), ("mlstm", "none")]


def shape(size: dict) -> dict:
    """Attention with the heads of the plain layer of the same name; recurrent heads as that size's linear-attention layer (heads x (dim, vdim)), the delta
    rule's query / key heads shared by two value heads."""
    rh, rd, rv = size["gla"]
    return dict(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["dim"], vdim=size["dim"], r_heads=rh, r_kv=rh // 2, r_dim=rd, r_vdim=rv, groups=(4, 2),
                shared_ff=size["moe"][2])


def synth(size: dict, kinds, vocab=32000, seed=0, device="cuda:0"):
    """Random Dikopel weights and their config."""
    g = torch.Generator(device=device).manual_seed(seed)
    w, t, layers, sh = size["width"], {}, [], shape(size)

    def lin(name, o, i, s=1.0):
        t[name] = (torch.randn(o, i, generator=g, device=device) * (s / math.sqrt(i))).to(torch.bfloat16)

    def vec(name, n, mean=0.0, s=0.1):
        t[name] = (mean + s * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)

    def ff(p, n):
        lin(p + "gate", n, w); lin(p + "up", n, w); lin(p + "down", w, n)
    lin("embed", vocab, w, math.sqrt(w)); lin("head", vocab, w); vec("final.norm", w, 1.0); vec("final.norm.b", w)
    H, G, d, dv = sh["heads"], sh["kv_heads"], sh["dim"], sh["vdim"]
    RH, RG, rd, rv = sh["r_heads"], sh["r_kv"], sh["r_dim"], sh["r_vdim"]
    for i, (mix, f) in enumerate(kinds):
        p = f"l{i}."
        vec(p + "norm1", w, 1.0); vec(p + "norm1.b", w); t[p + "canon1"] = (0.3 * torch.randn(w, TAPS, generator=g, device=device)).to(torch.bfloat16)
        if mix == "mlstm":
            for nm, n in (("q", RH * rd), ("k", RH * rd), ("v", RH * rv), ("g", RH * rv), ("i", RH), ("f", RH)):
                lin(p + "mix." + nm, n, w)
            vec(p + "mix.i.b", RH); vec(p + "mix.f.b", RH, 3.0); vec(p + "mix.norm", RH * rv, 1.0); lin(p + "mix.o", w, RH * rv)
            mixer = {"heads": RH, "dim": rd, "vdim": rv, "gate_cap": GATE_CAP}
        else:
            lin(p + "mix.left.q", H * d, w); lin(p + "mix.left.k", G * d, w); lin(p + "mix.left.v", G * dv, w); vec(p + "mix.left.pb", H, -4.0, 1.0)
            lin(p + "mix.left.o", w, H * dv); vec(p + "mix.left.out", w, 1.0)
            for nm, n in (("q", RG * rd), ("k", RG * rd), ("v", RH * rv)):
                lin(p + "mix.right." + nm, n, w); t[p + f"mix.right.{nm}.conv"] = (0.5 * torch.randn(n, CONV, generator=g, device=device)).to(torch.bfloat16)
            for nm, n in (("b", RH), ("a", RH), ("g", RH * rv)):
                lin(p + "mix.right." + nm, n, w)
            vec(p + "mix.right.A_log", RH, 0.0, 0.5); vec(p + "mix.right.dt_bias", RH, 0.0, 1.0); vec(p + "mix.right.norm", rv, 1.0)
            lin(p + "mix.right.o", w, RH * rv); vec(p + "mix.right.out", w, 1.0)
            mixer = {"left": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5}, "right": {"heads": RH, "kv_heads": RG, "dim": rd, "vdim": rv, "conv": CONV}}
        if f == "none":
            mlp = None
        elif f == "dense":
            ff(p + "mlp.", size["ff"])
            mlp = {"kind": "dense", "ff": size["ff"]}
        else:
            E, top, eff = size["moe"]
            for e in range(E):
                ff(f"{p}mlp.e{e}.", eff)
            ff(p + "mlp.shared.", sh["shared_ff"]); lin(p + "mlp.shared.sg", 1, w)
            lin(p + "mlp.router", E, w); vec(p + "mlp.correction", E)
            mlp = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top, "scale": 1.5, "groups": {"count": sh["groups"][0], "keep": sh["groups"][1]}},
                   "shared": {"ff": sh["shared_ff"]}}
        layers.append({"type": mix, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Dikopel", "vocab": vocab, "width": w, "norm": {"eps": 1e-5}, "canon": {"taps": TAPS}, "embedding": {"scale": math.sqrt(w)}, "residual_mult": 0.5,
           "layers": layers}
    return cfg, TensorDict(t)


def _make(size, kind, reps, dev):
    from .dikopel import DikopelModel
    cfg, td = synth(size, [kind] * reps, device=dev)
    return DikopelModel(cfg, td, device=dev, dtype=torch.bfloat16)


def parallel_kernel_legs(size_name: str, prompt: int, ctx: int, dev):
    """Each kernel of the design alone at the size's shapes: time and the fraction of the roofline that bounds it."""
    from . import mix_ops
    s = SIZES[size_name]
    sh = shape(s)
    out, bf, f32 = {}, torch.bfloat16, torch.float32
    rnd = lambda *a: torch.randn(*a, device=dev).to(bf)
    rf = lambda *a: torch.randn(*a, device=dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    H, G, d, dv, w = sh["heads"], sh["kv_heads"], sh["dim"], sh["vdim"], s["width"]
    RH, RG, rd, rv = sh["r_heads"], sh["r_kv"], sh["r_dim"], sh["r_vdim"]
    n, page = prompt, 64
    cu, seq, pos = i32([0, n]), torch.zeros(n, dtype=torch.int32, device=dev), torch.arange(n, dtype=torch.int32, device=dev)
    sl, la, p0 = i32([0]), i32([n]), i32([0])
    hbm = lambda by, t: {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    # attention without softmax: prompt step on the matrix cores, page store, decode through the page table
    q, k, v, pb = rnd(n, H * d), rnd(n, G * d), rnd(n, G * dv), rf(H) - 4.0
    o = torch.empty((n, H * dv), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.sigattn_prefill(o, q, k, v, pb, cu, seq, H, G, d, dv, d ** -0.5, n), 10)
    fl = 2.0 * (d + dv) * (n * (n + 1) / 2) * H
    out["sigattn_prefill_mfma"] = {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_bf16_peak": fl / t / PEAK_BF16}
    per = -(-max(n, ctx) // page)
    table = torch.arange(16 * per, dtype=torch.int32, device=dev).reshape(16, per).contiguous()
    kp, vp = torch.zeros((16 * per, page, G * d), dtype=bf, device=dev), torch.zeros((16 * per, page, G * dv), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.paged_store(kp, vp, k, v, table, seq, pos, sl), 20)
    out["paged_store_prefill"] = hbm(n * (G * d + G * dv) * 2 * 2, t)
    for bs in (1, 16):
        qd, od = rnd(bs, H * d), torch.empty((bs, H * dv), dtype=bf, device=dev)
        sld, lad = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        t = _time(lambda: mix_ops.sigattn_decode(od, qd, kp, vp, pb, table, sld, lad, H, G, d, dv, d ** -0.5), 50)
        out[f"sigattn_decode_bs{bs}"] = hbm(bs * ctx * (G * d + G * dv) * 2, t)
    # mLSTM: scan over a prompt, one token from the slots; output norm and gate
    wide = rnd(n, RH * (2 * rd + 2 * rv) + 2 * RH)
    c0, c1, c2, c3 = RH * rd, 2 * RH * rd, 2 * RH * rd + RH * rv, 2 * RH * rd + 2 * RH * rv
    S, ns, ms = torch.zeros((16, RH, rv, rd), device=dev), torch.zeros((16, RH, rd), device=dev), torch.zeros((16, RH), device=dev)
    bi, bfg = rf(RH), rf(RH) + 3.0
    om = torch.empty((n, RH, rv), dtype=f32, device=dev)
    t = _time(lambda: mix_ops.mlstm_scan(om, S, ns, ms, wide[:, :c0], wide[:, c0:c1], wide[:, c1:c2], wide[:, c3: c3 + RH], wide[:, c3 + RH:], bi, bfg, cu, sl, p0, rd ** -0.5, GATE_CAP), 5)
    fl = n * RH * rv * rd * 6.0
    out["mlstm_scan_prefill"] = {"ms": t * 1e3, "tflops_useful": fl / t / 1e12, "of_f32_vector_peak": fl / t / PEAK_F32, "workgroups": RH * ((rv + 15) // 16)}
    og = torch.empty((n, RH * rv), dtype=bf, device=dev)
    nw = torch.ones(RH * rv, device=dev)
    t = _time(lambda: mix_ops.head_norm_gate(og, om, nw, wide[:, c2:c3], mix_ops.GATE_SIGMOID, 1e-5), 20)
    out["head_norm_gate_prefill"] = hbm(n * RH * rv * (4 + 2 + 2), t)
    for bs in (1, 16):
        wd_ = rnd(bs, wide.shape[1])
        cud, sld, pd = torch.arange(bs + 1, dtype=torch.int32, device=dev), torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        od = torch.empty((bs, RH, rv), dtype=f32, device=dev)
        t = _time(lambda: mix_ops.mlstm_scan(od, S, ns, ms, wd_[:, :c0], wd_[:, c0:c1], wd_[:, c1:c2], wd_[:, c3: c3 + RH], wd_[:, c3 + RH:], bi, bfg, cud, sld, pd, rd ** -0.5, GATE_CAP), 50)
        out[f"mlstm_decode_bs{bs}"] = hbm(bs * RH * rv * rd * 4 * 2, t)
    # gated delta rule: input stage and scan
    C = 2 * RG * rd + RH * rv
    xw = rnd(n, C + 2 * RH)
    conv, ring = 0.5 * rf(CONV, C), torch.zeros((16, CONV - 1, C), dtype=bf, device=dev)
    A_log, dtb = 0.5 * rf(RH), rf(RH)
    qo, ko, vo = torch.empty((n, RG * rd), device=dev), torch.empty((n, RG * rd), device=dev), torch.empty((n, RH * rv), device=dev)
    be, de = torch.empty((n, RH), device=dev), torch.empty((n, RH), device=dev)
    t = _time(lambda: mix_ops.delta_prep(qo, ko, vo, be, de, xw[:, :C], conv, ring, xw[:, C: C + RH], xw[:, C + RH:], A_log, dtb, seq, pos, sl, p0, la, RH, RG, rd, rv, rd ** -0.5), 20)
    out["delta_prep_prefill"] = hbm(n * C * (2 + 4), t)
    S2 = torch.zeros((16, RH, rv, rd), device=dev)
    t = _time(lambda: mix_ops.delta_scan(om, S2, qo, ko, vo, be, de, cu, sl, p0, RG), 5)
    fl = n * RH * rv * rd * 8.0
    out["delta_scan_prefill"] = {"ms": t * 1e3, "tflops_useful": fl / t / 1e12, "of_f32_vector_peak": fl / t / PEAK_F32, "workgroups": RH * ((rv + 15) // 16)}
    for bs in (1, 16):
        xd = rnd(bs, C + 2 * RH)
        cud, sq, sld, pd, lad = torch.arange(bs + 1, dtype=torch.int32, device=dev), torch.arange(bs, dtype=torch.int32, device=dev), torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs), i32([ctx + 1] * bs)
        qd, kd, vd = torch.empty((bs, RG * rd), device=dev), torch.empty((bs, RG * rd), device=dev), torch.empty((bs, RH * rv), device=dev)
        bd, dd, od = torch.empty((bs, RH), device=dev), torch.empty((bs, RH), device=dev), torch.empty((bs, RH, rv), device=dev)
        t = _time(lambda: mix_ops.delta_prep(qd, kd, vd, bd, dd, xd[:, :C], conv, ring, xd[:, C: C + RH], xd[:, C + RH:], A_log, dtb, sq, pd, sld, pd, lad, RH, RG, rd, rv, rd ** -0.5), 50)
        out[f"delta_prep_bs{bs}"] = {"us": t * 1e6}
        t = _time(lambda: mix_ops.delta_scan(od, S2, qd, kd, vd, bd, dd, cud, sld, pd, RG), 50)
        out[f"delta_decode_bs{bs}"] = hbm(bs * RH * rv * rd * 4 * 2, t)
    # the two branches' norms, the residual update with the layer norm, the convolution
    a, b_, ow = rnd(n, w), rnd(n, w), torch.ones(w, device=dev)
    pr = torch.empty((n, w), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.rms_pair(pr, a, ow, b_, ow, 0.5, 1e-5), 20)
    out["rms_pair_prefill"] = hbm(n * w * 2 * 3, t)
    x, cw = rf(n, w), 0.3 * rf(TAPS, w)
    hn, h, rg = torch.empty((n, w), dtype=bf, device=dev), torch.empty((n, w), dtype=bf, device=dev), torch.zeros((16, TAPS - 1, w), dtype=bf, device=dev)
    t1 = _time(lambda: mix_ops.residual_norm_conv(x, a, b_, 0.5, mix_ops.RES_ADD, True, ow, ow, 1e-5, None, hn), 20)
    t2 = _time(lambda: mix_ops.canon(h, hn, cw, rg, seq, pos, sl, p0, la), 20)
    out["residual_layer_norm_prefill"] = hbm(n * w * (4 + 4 + 2 + 2 + 2), t1)
    out["canon_prefill"] = hbm(n * w * (2 + 2), t2)
    out["residual_layer_norm_plus_canon_prefill"] = hbm(n * w * (4 + 4 + 2 + 2 + 2 + 2), t1 + t2)
    for bs in (1, 16):
        xd, ad, bd2 = rf(bs, w), rnd(bs, w), rnd(bs, w)
        hd, hnd = torch.empty((bs, w), dtype=bf, device=dev), torch.empty((bs, w), dtype=bf, device=dev)
        sq, pd, sld = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs), torch.arange(bs, dtype=torch.int32, device=dev)
        t = _time(lambda: mix_ops.residual_norm_conv(xd, ad, bd2, 0.5, mix_ops.RES_ADD, True, ow, ow, 1e-5, hd, hnd, cw, rg, sq, pd, sld), 50)
        out[f"residual_layer_norm_canon_fused_bs{bs}"] = {"us": t * 1e6}
    E, top, eff = s["moe"]
    lg, idx, wt, corr = rf(n, E), torch.empty((n, top), dtype=torch.int32, device=dev), torch.empty((n, top), device=dev), torch.zeros(E, device=dev)
    t = _time(lambda: mix_ops.topk_grouped_ex(idx, wt, None, lg, corr, mix_ops.ROUTE_SIGMOID, E, sh["groups"][0], sh["groups"][1], 2, 1.5), 20)
    out["topk_grouped_sum2_prefill"] = {"us": t * 1e6}
    gu, sg, act = rnd(n, 2 * eff), rnd(n, 1), torch.empty((n, eff), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.glu_act_rowgate(act, gu[:, :eff], gu[:, eff:], sg, mix_ops.GLU_SILU), 20)
    out["glu_act_rowgate_prefill"] = hbm(n * eff * 2 * 3, t)
    return out


def run(args) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from . import _lib
    _lib.mixlib()
    prompt, ctx = args.prefill_tokens, 1000
    res = {"metric": "parallel_family_layer_times", "unit": "ms per layer", "dtype": "bf16", "data": "synthetic", "prompt": prompt, "ctx": ctx, "sizes": {}}
    for name in (args.mixer_sizes.split(",") if args.mixer_sizes else list(SIZES)):
        t0 = time.time()
        entry = {"shape": shape(SIZES[name]), "dikopel_layers": model_legs(name, prompt, ctx, args.steps, dev, kinds=KINDS, make=_make),
                 "kernels": parallel_kernel_legs(name, prompt, ctx, dev)}
        try:
            entry["closest_model_vofanex_layers"] = model_legs(name, prompt, ctx, args.steps, dev, kinds=[("gla", "dense"), ("gla", "moe"), ("attention", "moe")])
            entry["closest_model_kernels"] = kernel_legs(name, prompt, ctx, dev)
        except Exception as e:                       # the comparison leg must not hide the new design's numbers
            entry["closest_model_error"] = f"{type(e).__name__}: {e}"
        entry["seconds"] = round(time.time() - t0, 1)
        res["sizes"][name] = entry
    print(json.dumps(res))
    return 0
