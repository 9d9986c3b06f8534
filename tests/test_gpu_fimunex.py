"""GPU tests of the Fimunex design (csrc/mix_canon.hip, mix_diffattn.hip, the map / chunk / softcap forms of mix_attn*.hip, the grouped router and the
ungated experts, modules.py, fimunex.py) against the float64 oracle of tests/fimunex_oracle.py: every mechanism alone, whole models of several small
shapes (written to a checkpoint folder and loaded through the registry), prefill against token-by-token decoding, unequal batches against each request
alone, slots that are freed and used again, keys just inside and just outside a chunk in prompts and in decoding, the first tokens, long decoding over a
ring that is refilled many times, trace replay and greedy generation through the scheduler.  float32 runs are held to float32 rounding; bfloat16 runs to
a loose bar (the oracle does not round)."""
import io
import json
import math
import os
import numpy as np
import pytest
import torch
import fimunex_oracle as fo

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {torch.float32: 3e-5, torch.bfloat16: 4e-2}


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from exllamav3_amd import _lib
    _lib.mixlib()
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    return torch.device("cuda:0")


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / (b.abs().max() + 1e-30))


def mk(gpu, v):
    return torch.tensor(v, dtype=torch.int32, device=gpu)


def batch_tensors(gpu, lens, pos0=None, slots=None):
    pos0 = pos0 or [0] * len(lens)
    slots = slots or list(range(len(lens)))
    cu = [0]
    for l in lens: cu.append(cu[-1] + l)
    seq = [i for i, l in enumerate(lens) for _ in range(l)]
    pos = [pos0[i] + j for i, l in enumerate(lens) for j in range(l)]
    return mk(gpu, cu), mk(gpu, seq), mk(gpu, pos), mk(gpu, slots), mk(gpu, pos0), mk(gpu, [p + l for p, l in zip(pos0, lens)])


# ---- small random models ------------------------------------------------------------------------------------------------------------------------

YARN = {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 1.5}


def attn_layer(heads, kv_heads, dim, vdim, chunk, rot_dims, base=10000.0, scaling=None, softcap=20.0, diff=0.35, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 1.3 / math.sqrt(dim), "diff": diff, "mask": {"size": chunk}, "rot": rot}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def moe(ff, experts, top, identity=0, groups=None):
    r = {"experts": experts, "top": top, "identity": identity}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def config(layers, width=64, vocab=80, taps=3, loop=None, logit_softcap=12.0, eps=1e-5):
    c = {"architecture": "Fimunex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps}, "layers": layers}
    if logit_softcap:
        c["logit_softcap"] = logit_softcap
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


def weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W, w, taps = {}, cfg["width"], cfg["canon"]["taps"]
    lin = lambda o, i, gain=1.0: (torch.randn(o, i, generator=g) * gain / math.sqrt(i))
    vec = lambda n, s: s * torch.randn(n, generator=g)
    W["embed"] = torch.randn(cfg["vocab"], w, generator=g)
    W["head"] = lin(cfg["vocab"], w, 3.0)
    W["final.norm"] = vec(w, 0.2)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = vec(w, 0.2); W[p + "canon1"] = 0.4 * torch.randn(w, taps, generator=g)
        W[p + "mix.q"] = lin(H * 2 * d, w, 2.0); W[p + "mix.k"] = lin(G * 2 * d, w, 2.0); W[p + "mix.v"] = lin(G * dv, w)
        W[p + "mix.q.b"] = vec(H * 2 * d, 0.3); W[p + "mix.k.b"] = vec(G * 2 * d, 0.3); W[p + "mix.v.b"] = vec(G * dv, 0.3)
        W[p + "mix.q.norm"] = 1.0 + vec(d, 0.3); W[p + "mix.k.norm"] = 1.0 + vec(d, 0.3)
        for nm in ("lq1", "lk1", "lq2", "lk2"):
            W[p + "mix." + nm] = vec(d, 0.25)
        W[p + "mix.g"] = lin(H, w, 2.0); W[p + "mix.o"] = lin(w, H * dv); W[p + "mix.o.b"] = vec(w, 0.1)
        f = L.get("mlp")
        if f:
            W[p + "norm2"] = vec(w, 0.2); W[p + "canon2"] = 0.4 * torch.randn(w, taps, generator=g)
            r = f["router"]
            for e in range(r["experts"]):
                W[f"{p}mlp.e{e}.up"] = lin(f["expert"]["ff"], w, 2.0); W[f"{p}mlp.e{e}.down"] = lin(w, f["expert"]["ff"])
            total = r["experts"] + r.get("identity", 0)
            W[p + "mlp.router"] = lin(total, w, 3.0); W[p + "mlp.correction"] = vec(total, 0.3) - 0.2          # choice scores go below zero
    return {k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}


def save_and_load(tmp, cfg, W, gpu, dtype):
    from safetensors.torch import save_file
    from exllamav3_amd import registry
    os.makedirs(tmp, exist_ok=True)
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(W, os.path.join(tmp, "model.safetensors"))
    return registry.load_model(str(tmp), gpu, dtype)


# shapes chosen so that nothing the design allows happens to be equal or 1 by accident, and some things are: one head, kv_heads = heads, one key/value
# head, top 1, every expert chosen, no identity expert, more identity experts than stored ones, groups that restrict nothing, a chunk of one token, a chunk
# longer than any prompt, no feed-forward, fewer rotated dimensions than dim, no scaling, no soft cap, one tap, a loop that starts after the first layer, a
# loop of one pass, no loop, sizes that are no multiple of 8
MODELS = {
    "loop_front": lambda: config([attn_layer(4, 2, 16, 24, 9, 8, scaling=YARN, mlp=moe(24, 6, 2, identity=2, groups=(4, 2))),
                                  attn_layer(2, 2, 8, 8, 5, 8, mlp=None),
                                  attn_layer(3, 1, 12, 10, 300, 6, base=500.0, softcap=None, mlp=moe(16, 5, 5))], loop=(0, 2, 3)),
    "loop_middle": lambda: config([attn_layer(1, 1, 24, 24, 7, 24, scaling=YARN, mlp=None),
                                   attn_layer(4, 4, 8, 8, 1, 4, mlp=moe(8, 1, 1, identity=3, groups=(2, 1))),
                                   attn_layer(2, 1, 12, 20, 11, 12, mlp=moe(8, 9, 3, identity=3, groups=(3, 3))),
                                   attn_layer(2, 2, 8, 8, 4, 2, mlp=moe(40, 4, 1))], width=48, taps=4, loop=(1, 3, 2), logit_softcap=None),
    "one_tap": lambda: config([attn_layer(2, 1, 16, 16, 6, 16, mlp=moe(16, 5, 2, identity=1, groups=(3, 2))),
                               attn_layer(2, 2, 16, 8, 13, 10, base=300.0, mlp=moe(24, 8, 3, groups=(4, 2)))], taps=1, logit_softcap=5.0),
    "one_pass": lambda: config([attn_layer(2, 1, 8, 8, 8, 8, scaling=YARN, mlp=moe(48, 3, 2, identity=1))], width=40, taps=2, loop=(0, 1, 1)),
}


@pytest.fixture(scope="module")
def zoo(gpu, tmp_path_factory):
    """name -> (config, weights, {dtype: loaded model}); models are loaded once."""
    out = {}
    for k, (name, mkcfg) in enumerate(MODELS.items()):
        cfg = mkcfg()
        W = weights(cfg, 300 + k)
        d = tmp_path_factory.mktemp(name)
        out[name] = (cfg, W, {dt: save_and_load(str(d), cfg, W, gpu, dt) for dt in (torch.float32, torch.bfloat16)})
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


_truth = {}


def truth(name, cfg, W, toks):
    key = (name, tuple(toks))
    if key not in _truth:
        taps = []
        _truth[key] = (fo.forward(cfg, W, toks, taps), taps)
    return _truth[key]


def logit_err(got, want):
    """Per position: RMS over the vocabulary of the difference (mean taken off), over the spread of the expected logits."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.std()).reshape(-1)


def check_logits(got, want, dtype):
    e = logit_err(got, want)
    if dtype == torch.float32:
        assert float(e.max()) < 3e-5, float(e.max())
    else:
        # bfloat16: judged at the median and the ninth decile -- a router whose two best choice scores lie within bfloat16 rounding of its input may pick
        # the other expert at one position (with top 1: another output altogether); the float32 run has no such freedom
        assert torch.isfinite(e).all() and float(e.median()) < 6e-2 and float(e.quantile(0.9)) < 0.3, (float(e.median()), float(e.quantile(0.9)), float(e.max()))


def run_whole(model, cache, toks, want=None):
    s = cache.alloc()
    lg = model.step(cache.begin_step([(s, toks)], [want if want is not None else list(range(len(toks)))]), cache)
    cache.release(s)
    return lg.cpu()


def poison(cache):
    for layer in cache.layers:
        for t in layer.values():
            t.fill_(float("nan"))


# ---- mechanisms alone -----------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_norm_and_input_convolution_prompt_then_decode(gpu, dtype, taps):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(taps)
    w, lens, extra = 72, [1, 9, 2, 5], 7
    total = [l + extra for l in lens]
    nw, cw = 0.2 * torch.randn(w, generator=g), 0.5 * torch.randn(w, taps, generator=g)
    xs = [torch.randn(t, w, generator=g) for t in total]
    ys = [torch.randn(t, w, generator=g).to(dtype) for t in total]
    want = [fo.causal_taps(fo.norm_one_plus(x.to(F64) + y.to(F64), nw.to(F64), 1e-5), cw.to(F64)) for x, y in zip(xs, ys)]
    ring = torch.full((6, max(taps - 1, 1), w), float("nan"), dtype=dtype, device=gpu)
    slots = [4, 0, 5, 2]
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=slots)
    x = torch.cat([a[:l] for a, l in zip(xs, lens)]).to(gpu); y = torch.cat([a[:l] for a, l in zip(ys, lens)]).to(gpu)
    hn = torch.empty((sum(lens), w), dtype=dtype, device=gpu); h = torch.empty_like(hn)
    one_plus = (1.0 + nw).to(gpu)
    mix_ops.residual_rms(x, y, mix_ops.RES_ADD, one_plus, 1e-5, hn)
    mix_ops.canon(h, hn, cw.t().contiguous().to(gpu), ring, seq, pos, sl, p0, la)
    assert rel(x, torch.cat([(a.to(F64) + b.to(F64))[:l] for a, b, l in zip(xs, ys, lens)])) < 1e-6
    assert rel(h, torch.cat([a[:l] for a, l in zip(want, lens)])) < TOL[dtype] / 4
    for t in range(extra):                                      # one row per sequence against the ring, the fused kernel
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, [1] * 4, pos0=[l + t for l in lens], slots=slots)
        x = torch.stack([a[l + t] for a, l in zip(xs, lens)]).to(gpu); y = torch.stack([a[l + t] for a, l in zip(ys, lens)]).to(gpu)
        h = torch.empty((4, w), dtype=dtype, device=gpu)
        mix_ops.residual_rms(x, y, mix_ops.RES_ADD, one_plus, 1e-5, h, cw.t().contiguous().to(gpu), ring, seq, pos, sl)
        assert rel(h, torch.stack([a[l + t] for a, l in zip(want, lens)])) < TOL[dtype] / 4, t
    assert torch.isnan(ring[1]).all() and torch.isnan(ring[3]).all()          # slots of other sequences are untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,dims,pad", [(3, 1, 12, 10, 6, 5), (3, 1, 16, 24, 8, 8), (4, 2, 64, 128, 64, 0)])      # the last two: rows that allow 16-byte accesses
def test_query_key_norm_rotation_and_ring_store(gpu, dtype, H, G, d, dv, dims, pad):
    from exllamav3_amd import mix_ops
    from exllamav3_amd.modules import rotary_frequencies
    g = torch.Generator().manual_seed(5)
    span = 5
    lens = [7, 3]
    n = sum(lens)
    wide = torch.randn(n, H * 2 * d + G * 2 * d + G * dv + pad, generator=g).to(dtype)
    qn, kn = 1.0 + 0.3 * torch.randn(d, generator=g), 1.0 + 0.3 * torch.randn(d, generator=g)
    dev = wide.to(gpu)
    q, k, v = dev[:, :H * 2 * d], dev[:, H * 2 * d: (H + G) * 2 * d], dev[:, (H + G) * 2 * d: (H + G) * 2 * d + G * dv]
    ring_k = torch.full((3, span, G * 2, d), float("nan"), dtype=dtype, device=gpu); ring_v = torch.full((3, span, G, dv), float("nan"), dtype=dtype, device=gpu)
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=[2, 0])
    freq, mag = rotary_frequencies(dims, 500.0, YARN)
    mix_ops.qk_prep(q, k, v, qn.to(gpu), kn.to(gpu), freq.to(gpu), mag, False, 1e-5, ring_k, ring_v, seq, pos, sl, la, d)
    at = 0
    for b, (l, slot) in enumerate(zip(lens, [2, 0])):
        cos, sin = fo.rotary_half_tables(l, dims, 500.0, YARN)
        rows = wide[at: at + l].to(F64)
        wq = fo.rotate_half(fo.rms_unit(rows[:, :H * 2 * d].reshape(l, H * 2, d), 1e-5) * qn.to(F64), cos, sin, dims)
        wk = fo.rotate_half(fo.rms_unit(rows[:, H * 2 * d: (H + G) * 2 * d].reshape(l, G * 2, d), 1e-5) * kn.to(F64), cos, sin, dims)
        assert rel(q[at: at + l].reshape(l, H * 2, d), wq) < TOL[dtype] / 4
        assert rel(k[at: at + l].reshape(l, G * 2, d), wk) < TOL[dtype] / 4
        for p in range(max(0, l - span), l):                    # the rows a sequence keeps sit at position mod span
            assert rel(ring_k[slot, p % span], wk[p]) < TOL[dtype] / 4
            assert torch.equal(ring_v[slot, p % span].reshape(-1).cpu(), wide[at + p, (H + G) * 2 * d: (H + G) * 2 * d + G * dv])
        at += l
    assert torch.isnan(ring_k[1]).all() and torch.isnan(ring_k[0, 3:]).all()


def _attention_case(gpu, dtype, H, G, d, dv, span, softcap, lens, seed, spike=None):
    """Random normed queries / keys; spike = (sequence, query position, key position): that key is made to dominate that query's first map."""
    g = torch.Generator().manual_seed(seed)
    n = sum(lens)
    q = torch.randn(n, H * 2 * d, generator=g); k = torch.randn(n, G * 2 * d, generator=g); v = torch.randn(n, G * dv, generator=g)
    if spike:
        b, qi, kj = spike
        base = sum(lens[:b])
        q0 = q[base + qi, :d]                                   # head 0, map 0; its key/value head is 0
        k[base + kj, :d] = 6.0 * q0 / q0.norm() * math.sqrt(d)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    want, at = [], 0
    for l in lens:
        qq, kk, vv = q[at: at + l].to(F64).reshape(l, H, 2, d), k[at: at + l].to(F64).reshape(l, G, 2, d), v[at: at + l].to(F64).reshape(l, G, dv)
        o = torch.zeros(l, H, 2, dv, dtype=F64)
        for hh in range(H):
            for m in range(2):
                o[:, hh, m] = fo.chunk_softmax_attention(qq[:, hh, m], kk[:, hh // (H // G), m], vv[:, hh // (H // G)], 0.4, softcap, span)
        want.append(o.reshape(l, -1)); at += l
    return q, k, v, want


@pytest.mark.parametrize("dtype,mfma", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("H,G,d,dv,span,softcap", [(4, 2, 16, 24, 9, 7.0), (2, 2, 8, 8, 1, 0.0), (3, 1, 12, 10, 64, 3.0), (2, 1, 40, 72, 130, 0.0)])
def test_chunked_two_map_attention_prompt(gpu, dtype, mfma, H, G, d, dv, span, softcap):
    from exllamav3_amd import mix_ops
    lens = [150, 1, 37, 2]
    q, k, v, want = _attention_case(gpu, dtype, H, G, d, dv, span, softcap, lens, 11)
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens)
    for out_dtype in (torch.float32, dtype):
        out = torch.empty((sum(lens), H * 2 * dv), dtype=out_dtype, device=gpu)
        mix_ops.attn_prefill_maps(out, q.to(gpu), k.to(gpu), v.to(gpu), None, None, cu, seq, pos, H, G, 2, d, dv, 0.4, softcap, span, mix_ops.MASK_CHUNK, max_rows=max(lens), mfma=mfma)
        assert rel(out, torch.cat(want)) < TOL[dtype]


@pytest.mark.parametrize("H,G,d,dv,span,softcap", [(4, 2, 16, 24, 9, 7.0), (2, 2, 8, 8, 1, 0.0), (3, 1, 12, 10, 64, 3.0), (2, 1, 40, 72, 130, 0.0), (2, 1, 128, 256, 100, 30.0),
                                                   (2, 2, 64, 128, 200, 0.0)])
def test_two_maps_and_their_combination_in_one_kernel(gpu, H, G, d, dv, span, softcap):
    """The matrix-core kernel that keeps both maps of a head in one workgroup and combines them in its epilogue, against the oracle's maps combined in
    float64 -- among them a dominant key just inside and just outside a chunk's start."""
    from exllamav3_amd import mix_ops
    lens = [150, 1, 37, 2, 300]
    for spike in (None, (4, 2 * span + 3, 2 * span) if 2 * span + 3 < 300 else None, (4, 2 * span + 3, 2 * span - 1) if 2 * span + 3 < 300 else None):
        q, k, v, want = _attention_case(gpu, torch.bfloat16, H, G, d, dv, span, softcap, lens, 17, spike=spike)
        g = torch.Generator().manual_seed(3)
        gate = torch.randn(sum(lens), H, generator=g).to(torch.bfloat16)
        lam, diff = 0.77, 0.3
        a = torch.cat(want).reshape(-1, H, 2, dv)
        truth_out = (fo.rms_unit(a[:, :, 0] - lam * a[:, :, 1], 1e-5) * (1.0 - diff) * torch.sigmoid(gate.to(F64))[:, :, None]).reshape(-1, H * dv)
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens)
        out = torch.empty((sum(lens), H * dv), dtype=torch.bfloat16, device=gpu)
        mix_ops.attn_prefill_diff(out, q.to(gpu), k.to(gpu), v.to(gpu), gate.to(gpu), cu, H, G, d, dv, 0.4, softcap, span, mix_ops.MASK_CHUNK, lam, diff, 1e-5, max(lens))
        assert rel(out, truth_out) < TOL[torch.bfloat16], spike


@pytest.mark.parametrize("dtype,mfma", [(torch.float32, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("edge", ["inside", "outside"])
def test_a_dominant_key_at_the_chunk_edge_in_a_prompt(gpu, dtype, mfma, edge):
    """The query at position 70 of a chunk that starts at 64: the key at 64 is the first it sees, the key at 63 the last it does not.  A mask that is one
    position off changes the result completely (the dominant key carries nearly all of the weight when it is visible)."""
    from exllamav3_amd import mix_ops
    H, G, d, dv, span, lens = 2, 1, 16, 16, 64, [40, 100]
    kj = 64 if edge == "inside" else 63
    q, k, v, want = _attention_case(gpu, dtype, H, G, d, dv, span, 0.0, lens, 21, spike=(1, 70, kj))
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens)
    out = torch.empty((sum(lens), H * 2 * dv), dtype=torch.float32, device=gpu)
    mix_ops.attn_prefill_maps(out, q.to(gpu), k.to(gpu), v.to(gpu), None, None, cu, seq, pos, H, G, 2, d, dv, 0.4, 0.0, span, mix_ops.MASK_CHUNK, max_rows=max(lens), mfma=mfma)
    assert rel(out, torch.cat(want)) < TOL[dtype]
    row = out[40 + 70].reshape(H, 2, dv)[0, 0].double().cpu()
    dominant = v[40 + kj].to(F64)[:dv]
    close = float((row - dominant).abs().max())
    assert (close < 0.05) == (edge == "inside"), close


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,span,softcap", [(4, 2, 16, 24, 9, 7.0), (2, 2, 8, 8, 1, 0.0), (3, 1, 12, 10, 300, 3.0), (1, 1, 40, 136, 33, 0.0)])
def test_chunked_two_map_attention_decode_over_refilled_rings(gpu, dtype, H, G, d, dv, span, softcap):
    """Token by token through qk_prep-free rings written by hand: the ring is refilled chunk after chunk, and the rows of earlier chunks that still lie in
    it (entries above position mod span) must not be read."""
    from exllamav3_amd import mix_ops
    lens = [3 * span + 2 if span < 50 else 70, 5]
    q, k, v, want = _attention_case(gpu, dtype, H, G, d, dv, span, softcap, lens, 31)
    ring_k = torch.full((3, span, G * 2, d), float("nan"), dtype=dtype, device=gpu); ring_v = torch.full((3, span, G, dv), float("nan"), dtype=dtype, device=gpu)
    slots, base = [2, 0], [0, lens[0]]
    for t in range(max(lens)):
        live = [b for b in range(2) if t < lens[b]]
        for b in live:
            ring_k[slots[b], t % span] = k[base[b] + t].reshape(G * 2, d).to(gpu); ring_v[slots[b], t % span] = v[base[b] + t].reshape(G, dv).to(gpu)
        out = torch.empty((len(live), H * 2 * dv), dtype=torch.float32, device=gpu)
        qs = torch.stack([q[base[b] + t] for b in live]).to(gpu)
        mix_ops.attn_decode_maps(out, qs, ring_k, ring_v, None, None, mk(gpu, [slots[b] for b in live]), mk(gpu, [t + 1] * len(live)), H, 2, 0.4, softcap, mix_ops.MASK_CHUNK)
        assert rel(out, torch.stack([want[b][t] for b in live])) < TOL[dtype], t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_difference_of_maps_unit_rms_and_head_gate(gpu, dtype):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(8)
    n, H, dv, lam, diff = 6, 3, 20, 0.83, 0.35
    a = torch.randn(n, H * 2 * dv, generator=g)
    wide = torch.randn(n, H + 3, generator=g).to(dtype)
    out = torch.empty((n, H * dv), dtype=dtype, device=gpu)
    mix_ops.diff_combine(out, a.to(gpu), lam, diff, 1e-5, wide.to(gpu)[:, 2: 2 + H], H, dv)
    aa = a.to(F64).reshape(n, H, 2, dv)
    want = fo.rms_unit(aa[:, :, 0] - lam * aa[:, :, 1], 1e-5) * (1.0 - diff) * torch.sigmoid(wide[:, 2: 2 + H].to(F64))[:, :, None]
    assert rel(out, want.reshape(n, -1)) < TOL[dtype] / 4


@pytest.mark.parametrize("total,real,top,groups,keep", [(8, 6, 2, 4, 2), (4, 1, 1, 2, 1), (12, 9, 3, 3, 3), (5, 5, 5, 1, 1), (70, 64, 6, 7, 3), (16, 12, 3, 2, 1)])
def test_grouped_router_with_correction_and_identity(gpu, total, real, top, groups, keep):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(total)
    n = 50
    z = 2.0 * torch.randn(n, total, generator=g)
    corr = 0.3 * torch.randn(total, generator=g) - 0.4          # most choice scores are negative: a group that is left out must count as -inf, not 0
    idx = torch.empty((n, top), dtype=torch.int32, device=gpu); wts = torch.empty((n, top), dtype=torch.float32, device=gpu)
    idw = torch.empty((n,), dtype=torch.float32, device=gpu)
    mix_ops.topk_grouped(idx, wts, idw if real < total else None, z.to(gpu), corr.to(gpu), mix_ops.ROUTE_SOFTMAX_ALL, real, groups, keep)
    wi, ww = fo.grouped_router(z.to(F64), corr.to(F64), top, groups, keep)
    for t in range(n):
        want = {int(e): float(w) for e, w in zip(wi[t], ww[t])}
        got = {int(e): float(w) for e, w in zip(idx[t].cpu(), wts[t].cpu()) if int(e) < real}
        assert set(got) == {e for e in want if e < real}, t
        for e, w in got.items():
            assert abs(w - want[e]) < 1e-6
        if real < total:
            assert abs(float(idw[t]) - sum(w for e, w in want.items() if e >= real)) < 1e-6
            assert int((idx[t] == real).sum()) == sum(1 for e in want if e >= real)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 3, 17, 90])
def test_ungated_experts_with_identity_experts_every_path(gpu, dtype, n):
    """Rows 1-3: per (row, choice) kernels; 4-63: expert-major; from 64: expert-sorted vendor products.  All against the oracle's mixture."""
    from exllamav3_amd.modules import SparseExperts
    from exllamav3_amd.state_cache import StepBatch
    g = torch.Generator().manual_seed(n)
    w, ff, E, I, top = 48, 24, 5, 3, 3
    W = {f"e{e}.up": (torch.randn(ff, w, generator=g) * 2 / math.sqrt(w)).to(torch.bfloat16) for e in range(E)}
    W.update({f"e{e}.down": (torch.randn(w, ff, generator=g) / math.sqrt(ff)).to(torch.bfloat16) for e in range(E)})
    W["router"] = (torch.randn(E + I, w, generator=g) * 3 / math.sqrt(w)).to(torch.bfloat16); W["correction"] = (0.3 * torch.randn(E + I, generator=g) - 0.2).to(torch.bfloat16)

    class Stc:
        def get_tensor(self, key, device="cpu"):
            return W[key]
    mlp = SparseExperts(w, ff, E, top, router="softmax_all", router_bias=False, correction=True, act="relu2", gated=False, identity=I, groups=4, keep_groups=2)
    mlp.load(Stc(), "", dtype, gpu)
    h = torch.randn(n, w, generator=g).to(dtype)
    sb = StepBatch(n=n, batch=1, decode=False, max_rows=n, tokens=None, cu=None, tok_seq=None, tok_pos=None, slots=None, pos0=None, len_after=None)
    y, _ = mlp.forward(h.to(gpu), sb)
    f = {"expert": {"ff": ff}, "router": {"experts": E, "identity": I, "top": top, "groups": {"count": 4, "keep": 2}}}
    want = fo.expert_mixture(h.to(F64), {k: v.to(F64) for k, v in W.items()}, "", f)
    assert rel(y, want) < TOL[dtype]


# ---- whole models -----------------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(MODELS))
def test_whole_prompt_logits_and_stream_after_every_layer_run(zoo, name, dtype):
    cfg, W, models = zoo[name]
    model = models[dtype]
    toks = tokens(cfg, 41, 1)
    want, taps = truth(name, cfg, W, toks)
    cache = model.new_cache()
    poison(cache)
    model.layer_taps = []
    try:
        got = run_whole(model, cache, toks)
        assert len(model.layer_taps) == len(taps) == len(fo.layer_runs(cfg))
        for r, (a, b) in enumerate(zip(model.layer_taps, taps)):
            if dtype == torch.float32:
                assert rel(a, b) < 2e-5, r
            else:
                # a router whose best choice scores lie within bfloat16 rounding of its input may pick another expert at one position (with top 1 that is
                # another output altogether), so rows are judged at the median; the float32 run has no such freedom
                per_row = (a.double().cpu() - b).abs().amax(1) / b.abs().max()
                assert torch.isfinite(per_row).all() and float(per_row.median()) < 4e-2, r
    finally:
        model.layer_taps = None
    check_logits(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("prompt", [1, 2, 30])
def test_prompt_then_token_by_token_equals_whole(zoo, name, dtype, prompt):
    """The first tokens of a sequence (a prompt of one or two), then decoding through chunk borders: chunks of 1, 4, 5, 7, 8, 9 ... positions are crossed
    many times in 41 tokens, and every decoded position is compared."""
    cfg, W, models = zoo[name]
    model = models[dtype]
    toks = tokens(cfg, 41, 2)
    want, _ = truth(name, cfg, W, toks)
    cache = model.new_cache()
    poison(cache)
    s = cache.alloc()
    outs = [model.step(cache.begin_step([(s, toks[:prompt])], [list(range(prompt))]), cache)]
    for p in range(prompt, len(toks)):
        outs.append(model.step(cache.begin_step([(s, [toks[p]])]), cache))
    check_logits(torch.cat(outs), want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["loop_front", "loop_middle"])
def test_unequal_batch_equals_each_alone_and_slots_are_reused(zoo, name, dtype):
    """Four requests of unequal length start together and decode together; the shorter ones end earlier and their slots go to a second wave of requests
    that starts while the first still runs its own steps.  Every logit row is compared with the request's own whole-sequence truth."""
    cfg, W, models = zoo[name]
    model = models[dtype]
    cache = model.new_cache(slots=2)                           # grows while in use
    poison(cache)
    reqs = {i: tokens(cfg, n, 40 + i) for i, n in enumerate([1, 23, 9, 14])}
    cut = {0: 1, 1: 17, 2: 2, 3: 9}
    slot = {i: cache.alloc() for i in reqs}
    got = {i: [] for i in reqs}
    lg = model.step(cache.begin_step([(slot[i], reqs[i][:cut[i]]) for i in reqs], [list(range(cut[i])) for i in reqs]), cache)
    at = 0
    for i in reqs:
        got[i].append(lg[at: at + cut[i]]); at += cut[i]
    done = {i: cut[i] for i in reqs}
    live = [i for i in reqs if done[i] < len(reqs[i])]
    for i in reqs:
        if i not in live:
            cache.release(slot[i])
    while live:
        lg = model.step(cache.begin_step([(slot[i], [reqs[i][done[i]]]) for i in live]), cache)
        for j, i in enumerate(live):
            got[i].append(lg[j: j + 1]); done[i] += 1
        for i in [i for i in live if done[i] == len(reqs[i])]:
            cache.release(slot[i]); live.remove(i)
    for i in reqs:
        check_logits(torch.cat(got[i]), truth(name, cfg, W, reqs[i])[0], dtype)
    # second wave over the freed slots (they hold the first wave's rows)
    again = {i: tokens(cfg, n, 60 + i) for i, n in enumerate([12, 3])}
    slot = {i: cache.alloc() for i in again}
    lg = model.step(cache.begin_step([(slot[i], again[i][:-1]) for i in again], [list(range(len(again[i]) - 1)) for i in again]), cache)
    last = model.step(cache.begin_step([(slot[i], [again[i][-1]]) for i in again]), cache)
    at = 0
    for j, i in enumerate(again):
        n = len(again[i]) - 1
        check_logits(torch.cat([lg[at: at + n], last[j: j + 1]]), truth(name, cfg, W, again[i])[0], dtype)
        at += n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_decoding_refills_the_rings_many_times(zoo, dtype):
    cfg, W, models = zoo["loop_front"]
    model = models[dtype]
    toks = tokens(cfg, 120, 9)
    want, _ = truth("loop_front", cfg, W, toks)
    cache = model.new_cache()
    s = cache.alloc()
    outs = [model.step(cache.begin_step([(s, toks[:3])], [[0, 1, 2]]), cache)]
    for p in range(3, len(toks)):
        outs.append(model.step(cache.begin_step([(s, [toks[p]])]), cache))
    check_logits(torch.cat(outs), want, dtype)


def test_a_far_key_inside_the_chunk_decides_the_logits(zoo, gpu):
    """In a chunk longer than the prompt the first token stays visible to the last one: changing it must change the last position's logits, in prompts and in
    decoding alike, and by the amount the oracle says."""
    cfg, W, models = zoo["loop_front"]                          # its last layer has a chunk of 300 positions
    model = models[torch.float32]
    a = tokens(cfg, 90, 12)
    b = [(a[0] + 1) % cfg["vocab"]] + a[1:]
    cache = model.new_cache()
    for toks in (a, b):
        want, _ = truth("loop_front", cfg, W, toks)
        s = cache.alloc()
        model.step(cache.begin_step([(s, toks[:60])], [[]]), cache)
        outs = [model.step(cache.begin_step([(s, [toks[p]])]), cache) for p in range(60, 90)]
        cache.release(s)
        check_logits(torch.cat(outs), want[60:], torch.float32)
    wa, wb = truth("loop_front", cfg, W, a)[0], truth("loop_front", cfg, W, b)[0]
    assert float(logit_err(wa[-1:], wb[-1:])) > 1e-3             # the far token matters at all


# ---- the framework's entry points ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["loop_front", "one_tap"])
def test_greedy_generation_through_the_scheduler(zoo, name):
    from exllamav3_amd.generator import Generator
    cfg, W, models = zoo[name]
    model = models[torch.float32]
    prompts = [tokens(cfg, n, 70 + n) for n in (5, 1, 12)]
    want = [fo.greedy(cfg, W, p, 10) for p in prompts]
    for graphs in (False, True):
        gen = Generator(model, max_batch=2, graphs=graphs)         # the third prompt waits for a slot of the first two
        assert gen.generate(prompts, 10) == want
        if graphs:
            assert gen.graph_replays > 0


def test_trace_replay_writes_the_wanted_rows(zoo, tmp_path):
    from exllamav3_amd.trace import TraceSession
    cfg, W, models = zoo["loop_middle"]
    model = models[torch.float32]
    a, b = tokens(cfg, 11, 80), tokens(cfg, 4, 81)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [a[9]], "want": [0]}, {"id": "b", "tokens": [b[3]], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": [a[10]], "want": []}], "end": ["a"]}]
    out = io.StringIO()
    sess = TraceSession(model, str(tmp_path))
    sess.run([json.dumps(s) for s in steps], out)
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2"] and sess.cache.in_use() == 0
    ta, tb = truth("loop_middle", cfg, W, a)[0], truth("loop_middle", cfg, W, b)[0]
    r0 = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    r1 = torch.from_numpy(np.fromfile(tmp_path / "1.f32", dtype="<f4").reshape(2, -1))
    check_logits(r0, ta[[0, 8]], torch.float32)
    check_logits(r1, torch.stack([ta[9], tb[3]]), torch.float32)
    assert not (tmp_path / "2.f32").exists()
