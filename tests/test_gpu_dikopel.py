"""GPU tests of the Dikopel design (csrc/mix_recur.hip, mix_sigattn*.hip, the layer-norm form of mix_canon.hip, the router's group scores, the paged part
of state_cache.py, modules.py, dikopel.py) against the float64 oracle of tests/dikopel_oracle.py: every mechanism alone, whole models of several small
shapes (written to a checkpoint folder and loaded through the registry), prefill against token-by-token decoding, unequal batches against each request
alone, slots and pages that are freed and used again, a dominant key far back and at page borders in prompts and in decoding, the first tokens, long
decoding, trace replay and greedy generation through the scheduler.  float32 runs are held to float32 rounding; bfloat16 runs to a loose bar (the oracle
does not round)."""
import io
import json
import math
import os
import numpy as np
import pytest
import torch
import dikopel_oracle as do

pytestmark = pytest.mark.gpu
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


def npy(t):
    return t.detach().double().cpu().numpy()


def rel(a, b):
    a = npy(a) if isinstance(a, torch.Tensor) else np.asarray(a, dtype=np.float64)
    b = npy(b) if isinstance(b, torch.Tensor) else np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / (np.abs(b).max() + 1e-30))


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


def rnd(g, *shape, s=1.0):
    return s * torch.randn(*shape, generator=g)


# ---- small random models ------------------------------------------------------------------------------------------------------------------------

def par(lh, lg, ld, lv, rh, rg, rd, rv, conv, scale=None, mlp=None, **kw):
    L = {"type": "parallel", "mixer": {"left": {"heads": lh, "kv_heads": lg, "dim": ld, "vdim": lv, "scale": scale or 1.0 / math.sqrt(ld)},
                                       "right": {"heads": rh, "kv_heads": rg, "dim": rd, "vdim": rv, "conv": conv}}, "mlp": mlp}
    L.update(kw)
    return L


def xl(heads, dim, vdim, cap=10.0, mlp=None, **kw):
    L = {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}
    L.update(kw)
    return L


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=None, scale=1.0, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    f = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers, width=64, vocab=96, taps=3, mult=0.5, embed_scale=4.0, eps=1e-5):
    for i, L in enumerate(layers):                              # a borrowing layer's entry equals the lender's
        if L.get("weights_of") is not None:
            layers[i] = dict(layers[L["weights_of"]], weights_of=L["weights_of"])
    return {"architecture": "Dikopel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps}, "embedding": {"scale": embed_scale},
            "residual_mult": mult, "layers": layers}


def weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W, w, taps = {}, cfg["width"], cfg["canon"]["taps"]
    lin = lambda o, i, gain=1.0: torch.randn(o, i, generator=g) * gain / math.sqrt(i)
    vec = lambda n, s: s * torch.randn(n, generator=g)
    W["embed"] = torch.randn(cfg["vocab"], w, generator=g)
    W["head"] = lin(cfg["vocab"], w, 3.0)
    W["final.norm"] = 1.0 + vec(w, 0.2); W["final.norm.b"] = vec(w, 0.2)

    def ff(p, n):
        W[p + "gate"] = lin(n, w, 2.0); W[p + "up"] = lin(n, w, 2.0); W[p + "down"] = lin(w, n)

    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        W[p + "norm1"] = 1.0 + vec(w, 0.2); W[p + "norm1.b"] = vec(w, 0.2); W[p + "canon1"] = 0.4 * torch.randn(w, taps, generator=g)
        if L["type"] == "mlstm":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            for nm, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                W[p + "mix." + nm] = lin(n, w, 2.0)
            W[p + "mix.i"] = lin(H, w, 4.0); W[p + "mix.f"] = lin(H, w, 4.0)
            W[p + "mix.i.b"] = vec(H, 1.0); W[p + "mix.f.b"] = 2.0 + vec(H, 1.0)
            W[p + "mix.norm"] = 1.0 + vec(H * dv, 0.2); W[p + "mix.o"] = lin(w, H * dv)
        else:
            a, b = m["left"], m["right"]
            W[p + "mix.left.q"] = lin(a["heads"] * a["dim"], w, 2.0); W[p + "mix.left.k"] = lin(a["kv_heads"] * a["dim"], w, 2.0)
            W[p + "mix.left.v"] = lin(a["kv_heads"] * a["vdim"], w); W[p + "mix.left.pb"] = vec(a["heads"], 1.0) - 1.0
            W[p + "mix.left.o"] = lin(w, a["heads"] * a["vdim"]); W[p + "mix.left.out"] = 1.0 + vec(w, 0.2)
            H, G, d, dv, c = b["heads"], b["kv_heads"], b["dim"], b["vdim"], b["conv"]
            for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                W[p + "mix.right." + nm] = lin(n, w, 2.0); W[p + f"mix.right.{nm}.conv"] = 0.6 * torch.randn(n, c, generator=g)
            W[p + "mix.right.b"] = lin(H, w, 3.0); W[p + "mix.right.a"] = lin(H, w, 3.0)
            W[p + "mix.right.A_log"] = vec(H, 0.7); W[p + "mix.right.dt_bias"] = vec(H, 1.0)
            W[p + "mix.right.norm"] = 1.0 + vec(dv, 0.2); W[p + "mix.right.g"] = lin(H * dv, w, 2.0)
            W[p + "mix.right.o"] = lin(w, H * dv); W[p + "mix.right.out"] = 1.0 + vec(w, 0.2)
        f = L.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            ff(p + "mlp.", f["ff"])
        else:
            r = f["router"]
            for e in range(r["experts"]):
                ff(f"{p}mlp.e{e}.", f["expert"]["ff"])
            W[p + "mlp.router"] = lin(r["experts"], w, 3.0); W[p + "mlp.correction"] = vec(r["experts"], 0.5) - 0.6      # choice scores go below zero
            if f.get("shared"):
                ff(p + "mlp.shared.", f["shared"]["ff"]); W[p + "mlp.shared.sg"] = lin(1, w, 3.0)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}


def save_and_load(tmp, cfg, W, gpu, dtype):
    from safetensors.torch import save_file
    from exllamav3_amd import registry
    os.makedirs(tmp, exist_ok=True)
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(W, os.path.join(tmp, "model.safetensors"))
    return registry.load_model(str(tmp), gpu, dtype)


# shapes chosen so that nothing the design allows happens to be equal or 1 by accident, and some things are: one head, kv_heads = heads, one key/value head, value
# heads of another size than key heads, top 1, every expert chosen, groups that restrict nothing, no groups, no shared expert, no feed-forward, one tap (no
# convolution state), a borrowing layer of either kind, an mLSTM layer first, factor 1, widths that are no multiple of 8, head sizes that are no multiple of 16
MODELS = {
    "mixed": lambda: config([par(4, 2, 16, 24, 4, 2, 16, 8, 4, mlp=dense(48)),
                             xl(2, 24, 40, mlp=moe(16, 8, 2, groups=(4, 2), scale=2.0, shared=24)),
                             {"weights_of": 0},
                             xl(3, 8, 8, cap=4.0, mlp=None),
                             {"weights_of": 1}]),
    "odd": lambda: config([xl(1, 8, 12, mlp=dense(20)),
                           par(2, 2, 8, 8, 2, 2, 8, 12, 1, scale=0.5, mlp=moe(12, 3, 1)),
                           par(3, 1, 12, 10, 6, 1, 20, 6, 2, mlp=None)], width=36, vocab=50, taps=1, mult=1.0, embed_scale=1.0),
    "wide": lambda: config([par(2, 1, 64, 128, 2, 1, 128, 64, 4, mlp=moe(24, 4, 4, groups=(2, 2), scale=0.7, shared=40)),
                            xl(2, 96, 64, cap=15.0, mlp=moe(16, 6, 2, groups=(3, 1)))], width=128, vocab=64, taps=4, mult=0.25),
}


@pytest.fixture(scope="module")
def zoo(gpu, tmp_path_factory):
    """name -> (config, float64 weights, {dtype: loaded model}); models are loaded once."""
    out = {}
    for k, (name, mkcfg) in enumerate(MODELS.items()):
        cfg = mkcfg()
        W = weights(cfg, 500 + k)
        d = tmp_path_factory.mktemp(name)
        out[name] = (cfg, {n: npy(t) for n, t in W.items()}, {dt: save_and_load(str(d), cfg, W, gpu, dt) for dt in (torch.float32, torch.bfloat16)})
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


_truth = {}


def truth(name, cfg, W, toks):
    key = (name, tuple(toks))
    if key not in _truth:
        taps = []
        _truth[key] = (do.forward(cfg, W, toks, taps), taps)
    return _truth[key]


def logit_err(got, want):
    """Per position: RMS over the vocabulary of the difference (mean taken off), over the spread of the expected logits."""
    got, want = npy(got) if isinstance(got, torch.Tensor) else got, np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return (np.sqrt((d * d).mean(-1)) / want.std()).reshape(-1)


def check_logits(got, want, dtype):
    e = logit_err(got, want)
    if dtype == torch.float32:
        assert float(e.max()) < 3e-5, float(e.max())
    else:
        # bfloat16: judged at the median and the ninth decile -- a router whose best choice scores lie within bfloat16 rounding of its input may pick another
        # expert at one position, which the recurrent states then carry; the float32 run has no such freedom
        assert np.isfinite(e).all() and float(np.median(e)) < 6e-2 and float(np.quantile(e, 0.9)) < 0.3, (float(np.median(e)), float(np.quantile(e, 0.9)), float(e.max()))


def run_whole(model, cache, toks, want=None):
    s = cache.alloc()
    lg = model.step(cache.begin_step([(s, toks)], [want if want is not None else list(range(len(toks)))]), cache)
    cache.release(s)
    return lg.cpu()


def run_decoded(model, cache, toks, prompt):
    """The first `prompt` tokens in one step, the rest one by one; logits of every position."""
    s = cache.alloc()
    rows = [model.step(cache.begin_step([(s, toks[:prompt])], [list(range(prompt))]), cache).cpu()]
    for t in toks[prompt:]:
        rows.append(model.step(cache.begin_step([(s, [t])], [[0]]), cache).cpu())
    cache.release(s)
    return torch.cat(rows)


def poison(cache):
    for layer in cache.layers:
        for name, t in layer.items():
            if t.dtype != torch.int32:
                t.fill_(float("nan"))


# ---- mechanisms alone -----------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [36, 64, 130])
def test_scaled_embedding_with_position_vector(gpu, dtype, width):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(width)
    table = rnd(g, 40, width).to(dtype)
    toks, pos = [3, 39, 0, 7, 7], [0, 1, 977, 5, 4096]
    freq = (10000.0 ** (-2.0 * torch.arange((width + 1) // 2, dtype=torch.float64) / width)).float().to(gpu)
    x = torch.empty((5, width), dtype=torch.float32, device=gpu)
    mix_ops.embed_sinusoid(x, table.to(gpu), mk(gpu, toks), mk(gpu, pos), freq, 3.5)
    want = npy(table)[toks] * 3.5 + do.position_vectors(4097, width)[pos]
    assert np.abs(npy(x) - want).max() < 3e-4                  # float32 angles: position 4096 times a frequency near 1 carries 2^-12 of absolute error


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,w", [(1, 72), (2, 36), (4, 72)])
def test_layer_norm_and_input_convolution_prompt_then_decode(gpu, dtype, taps, w):
    """x += (y + y2) m, layer norm, convolution: the two kernels of a prompt step, then the fused kernel of decode steps against the slot's ring."""
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(taps)
    lens, extra, m = [1, 9, 2, 5], 7, 0.5
    total = [l + extra for l in lens]
    nw, nb, cw = 1.0 + rnd(g, w, s=0.2), rnd(g, w, s=0.3), rnd(g, w, taps, s=0.5)
    xs = [rnd(g, t, w) + 3.0 for t in total]                   # a mean far from zero: a norm that forgets to centre shows
    ys = [rnd(g, t, w).to(dtype) for t in total]
    y2 = [rnd(g, t, w).to(dtype) for t in total]
    xn = [npy(x) + (npy(a) + npy(b)) * m for x, a, b in zip(xs, ys, y2)]
    hn_want = [do.layer_norm(x, npy(nw), npy(nb), 1e-5) for x in xn]
    h_want = [do.causal_conv(h, npy(cw), identity=True) for h in hn_want]
    ring = torch.full((6, max(taps - 1, 1), w), float("nan"), dtype=dtype, device=gpu)
    slots = [4, 0, 5, 2]
    conv = cw.t().contiguous().to(gpu)
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=slots)
    cat = lambda parts: torch.cat([a[:l] for a, l in zip(parts, lens)]).to(gpu)
    x = cat(xs)
    hn = torch.empty((sum(lens), w), dtype=dtype, device=gpu); h = torch.empty_like(hn)
    mix_ops.residual_norm_conv(x, cat(ys), cat(y2), m, mix_ops.RES_ADD, True, nw.to(gpu), nb.to(gpu), 1e-5, None, hn)
    mix_ops.canon(h, hn, conv, ring, seq, pos, sl, p0, la)
    assert rel(x, np.concatenate([a[:l] for a, l in zip(xn, lens)])) < 1e-6
    assert rel(hn, np.concatenate([a[:l] for a, l in zip(hn_want, lens)])) < TOL[dtype] / 4
    assert rel(h, np.concatenate([a[:l] for a, l in zip(h_want, lens)])) < TOL[dtype] / 4
    for t in range(extra):
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, [1] * 4, pos0=[l + t for l in lens], slots=slots)
        pick = lambda parts: torch.stack([a[l + t] for a, l in zip(parts, lens)]).to(gpu)
        x = pick(xs)
        hn = torch.empty((4, w), dtype=dtype, device=gpu); h = torch.empty_like(hn)
        mix_ops.residual_norm_conv(x, pick(ys), pick(y2), m, mix_ops.RES_ADD, True, nw.to(gpu), nb.to(gpu), 1e-5, h, hn, conv, ring, seq, pos, sl)
        assert rel(hn, np.stack([a[l + t] for a, l in zip(hn_want, lens)])) < TOL[dtype] / 4, t
        assert rel(h, np.stack([a[l + t] for a, l in zip(h_want, lens)])) < TOL[dtype] / 4, t
    assert torch.isnan(ring[1]).all() and torch.isnan(ring[3]).all()          # slots of other sequences are untouched


def _sig_case(dtype, H, G, d, dv, lens, seed, scale, spike=None):
    """Random queries / keys / values and biases low enough that a common key weighs little; spike = (sequence, query position, key position): that key is made
    to dominate head 0 of that query, and its value is made large."""
    g = torch.Generator().manual_seed(seed)
    n = sum(lens)
    q, k, v = rnd(g, n, H * d), rnd(g, n, G * d), rnd(g, n, G * dv)
    bias = rnd(g, H) - 6.0
    if spike:
        b, qi, kj = spike
        base = sum(lens[:b])
        q0 = q[base + qi, :d]
        k[base + kj, :d] = (12.0 / scale) * q0 / q0.norm() ** 2
        v[base + kj, :dv] = 50.0
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    want, at = [], 0
    for l in lens:
        qq, kk, vv = npy(q[at: at + l]).reshape(l, H, d), npy(k[at: at + l]).reshape(l, G, d), npy(v[at: at + l]).reshape(l, G, dv)
        o = np.zeros((l, H, dv))
        vis = np.tril(np.ones((l, l)))
        for a in range(H):
            gg = a // (H // G)
            o[:, a] = (do.sigmoid(qq[:, a] @ kk[:, gg].T * scale + npy(bias)[a]) * vis) @ vv[:, gg]
        want.append(o.reshape(l, -1)); at += l
    return q, k, v, bias, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 16, 24), (2, 2, 8, 8), (3, 1, 12, 10), (2, 1, 64, 128), (6, 1, 40, 72)])
def test_sigmoid_attention_prompt(gpu, dtype, H, G, d, dv):
    """Both prompt kernels (a step whose longest sequence is short takes the exact one; bfloat16 steps from 32 rows run on the matrix cores)."""
    from exllamav3_amd import mix_ops
    for lens in ([150, 1, 37, 2, 300], [9, 1, 20]):
        q, k, v, bias, want = _sig_case(dtype, H, G, d, dv, lens, 11, 0.3)
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens)
        out = torch.empty((sum(lens), H * dv), dtype=dtype, device=gpu)
        mix_ops.sigattn_prefill(out, q.to(gpu), k.to(gpu), v.to(gpu), bias.to(gpu), cu, seq, H, G, d, dv, 0.3, max(lens))
        assert rel(out, np.concatenate(want)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kj", [0, 1, 63, 64, 65, 127, 128, 500, 899, 900])
def test_a_dominant_key_anywhere_behind_a_prompt_row(gpu, dtype, kj):
    """Query 900 of a 1000-token sequence; one key -- the first token, a key at a tile's or a page's edge, a far one, the one before the query, the query's own --
    carries nearly all of the weight and a large value.  A key that is lost, or one position off, changes the row completely."""
    from exllamav3_amd import mix_ops
    H, G, d, dv, lens = 2, 1, 16, 16, [40, 1000]
    q, k, v, bias, want = _sig_case(dtype, H, G, d, dv, lens, 21, 0.25, spike=(1, 900, kj))
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens)
    out = torch.empty((sum(lens), H * dv), dtype=dtype, device=gpu)
    mix_ops.sigattn_prefill(out, q.to(gpu), k.to(gpu), v.to(gpu), bias.to(gpu), cu, seq, H, G, d, dv, 0.25, max(lens))
    assert rel(out, np.concatenate(want)) < TOL[dtype]
    row = npy(out[40 + 900]).reshape(H, dv)[0]
    assert row.min() > 40.0                                     # the dominant key's value (50) is there
    before = npy(out[40 + kj - 1]).reshape(H, dv)[0] if kj > 0 else None
    assert before is None or np.abs(before).max() < 30.0        # and it is not seen by a row before it


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("page", [1, 8, 64])
def test_sigmoid_attention_decode_over_scattered_pages(gpu, dtype, page):
    """Keys stored through a page table whose pages lie in no order, read back by the decode kernel: every length around page borders, and the rows of a prompt
    step against the same rows decoded."""
    from exllamav3_amd import mix_ops
    H, G, d, dv, scale = 4, 2, 16, 24, 0.3
    lens = [3 * 64 + 2, 1, 64, 65, 130]
    q, k, v, bias, want = _sig_case(dtype, H, G, d, dv, lens, 31, scale)
    pages_per = [-(-l // page) for l in lens]
    order = torch.randperm(sum(pages_per) + 5, generator=torch.Generator().manual_seed(2)).tolist()
    table = torch.zeros((7, max(pages_per)), dtype=torch.int32)
    slots, at = [5, 0, 3, 6, 1], 0
    for s, n in zip(slots, pages_per):
        table[s, :n] = torch.tensor(order[at: at + n], dtype=torch.int32); at += n
    table = table.to(gpu)
    kp = torch.full((len(order), page, G * d), float("nan"), dtype=dtype, device=gpu); vp = torch.full((len(order), page, G * dv), float("nan"), dtype=dtype, device=gpu)
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=slots)
    mix_ops.paged_store(kp, vp, k.to(gpu), v.to(gpu), table, seq, pos, sl)
    base = [sum(lens[:i]) for i in range(len(lens))]
    for back in (0, 1, 2, 63, 64, 65, 129):                     # decode the row at length - back of every sequence that is long enough
        who = [i for i, l in enumerate(lens) if l > back]
        rows = [base[i] + lens[i] - 1 - back for i in who]
        out = torch.empty((len(who), H * dv), dtype=dtype, device=gpu)
        mix_ops.sigattn_decode(out, q[rows].to(gpu), kp, vp, bias.to(gpu), table, mk(gpu, [slots[i] for i in who]), mk(gpu, [lens[i] - back for i in who]), H, G, d, dv, scale)
        assert rel(out, np.concatenate(want)[rows]) < TOL[dtype], back


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kj", [0, 63, 64, 700, 898, 899])
def test_a_dominant_key_anywhere_behind_a_decoded_row(gpu, dtype, kj):
    from exllamav3_amd import mix_ops
    H, G, d, dv, page, n = 2, 1, 16, 16, 64, 900
    q, k, v, bias, want = _sig_case(dtype, H, G, d, dv, [n], 41, 0.25, spike=(0, n - 1, kj))
    table = torch.arange(16, dtype=torch.int32).flip(0).reshape(1, 16).contiguous().to(gpu)
    kp = torch.zeros((16, page, G * d), dtype=dtype, device=gpu); vp = torch.zeros((16, page, G * dv), dtype=dtype, device=gpu)
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, [n])
    mix_ops.paged_store(kp, vp, k.to(gpu), v.to(gpu), table, seq, pos, sl)
    out = torch.empty((1, H * dv), dtype=dtype, device=gpu)
    mix_ops.sigattn_decode(out, q[n - 1:].to(gpu), kp, vp, bias.to(gpu), table, mk(gpu, [0]), mk(gpu, [n]), H, G, d, dv, 0.25)
    assert rel(out, want[0][n - 1:]) < TOL[dtype] and npy(out).reshape(H, dv)[0].min() > 40.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,dv,cap", [(2, 24, 40, 10.0), (1, 8, 8, 3.0), (3, 16, 16, 15.0), (2, 96, 64, 15.0), (1, 130, 20, 8.0)])
def test_mlstm_scan_prompt_then_decode(gpu, dtype, H, d, dv, cap):
    """The matrix memory against the oracle's token loop; gates strong enough that the running maximum moves, the normaliser's floor exp(-m) and |n.q| both
    decide the denominator at some tokens; a second sequence that starts later in another slot; then token-by-token decoding from the slots."""
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(int(cap) + d)
    w, lens, extra = 32, [37, 5], 6
    total = [l + extra for l in lens]
    Wt = {nm: rnd(g, n, w, s=2.0 / math.sqrt(w)).to(dtype) for nm, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("o", H * dv))}
    Wt["i"], Wt["f"] = rnd(g, H, w, s=1.5).to(dtype), rnd(g, H, w, s=1.5).to(dtype)
    Wt["i.b"], Wt["f.b"] = rnd(g, H), rnd(g, H) + 1.0
    Wt["norm"] = 1.0 + rnd(g, H * dv, s=0.2)
    Wt["o"] = torch.eye(H * dv)                                 # the oracle's output projection as the identity: the mixer's result before W_o
    hs = [rnd(g, t, w).to(dtype) for t in total]
    # the oracle reads the SAME projections as the kernel: rounded to the activation type, as the model's fused product leaves them (its own weights pick them
    # out of the wide row)
    order = ("q", "k", "v", "g", "i", "f")
    wcat = torch.cat([Wt[nm] for nm in order])
    wides = [(h.float() @ wcat.float().t()).to(dtype) for h in hs]
    Wn, at = {"m.i.b": npy(Wt["i.b"]), "m.f.b": npy(Wt["f.b"]), "m.norm": npy(Wt["norm"]), "m.o": np.eye(H * dv)}, 0
    for nm in order:
        sel = np.zeros((Wt[nm].shape[0], wcat.shape[0])); sel[:, at: at + Wt[nm].shape[0]] = np.eye(Wt[nm].shape[0])
        Wn["m." + nm] = sel; at += Wt[nm].shape[0]
    want = [do.mlstm(npy(x), Wn, "m.", {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}, 1e-5) for x in wides]
    dev = {nm: t.to(gpu) for nm, t in Wt.items()}
    cols = {nm: (sum(Wt[o].shape[0] for o in order[:i]), Wt[nm].shape[0]) for i, nm in enumerate(order)}
    S = torch.full((4, H, dv, d), float("nan"), device=gpu); nst = torch.full((4, H, d), float("nan"), device=gpu); mst = torch.full((4, H), float("nan"), device=gpu)
    slots = [2, 0]

    def run(rows, lens_now, pos0):
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens_now, pos0=pos0, slots=slots)
        h = rows.to(gpu)
        lin = lambda nm: h[:, cols[nm][0]: cols[nm][0] + cols[nm][1]]           # column blocks of the wide row, in place
        o = torch.empty((h.shape[0], H, dv), dtype=torch.float32, device=gpu)
        mix_ops.mlstm_scan(o, S, nst, mst, lin("q"), lin("k"), lin("v"), lin("i"), lin("f"), dev["i.b"], dev["f.b"], cu, sl, p0, d ** -0.5, cap)
        out = torch.empty((h.shape[0], H * dv), dtype=dtype, device=gpu)
        mix_ops.head_norm_gate(out, o, dev["norm"], lin("g"), mix_ops.GATE_SIGMOID, 1e-5)
        return out

    out = run(torch.cat([h[:l] for h, l in zip(wides, lens)]), lens, None)
    assert rel(out, np.concatenate([a[:l] for a, l in zip(want, lens)])) < TOL[dtype] / 2
    for t in range(extra):
        out = run(torch.stack([h[l + t] for h, l in zip(wides, lens)]), [1, 1], [l + t for l in lens])
        assert rel(out, np.stack([a[l + t] for a, l in zip(want, lens)])) < TOL[dtype] / 2, t
    assert torch.isnan(S[1]).all() and torch.isnan(S[3]).all() and torch.isnan(mst[1]).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 16, 8, 4), (2, 2, 8, 12, 1), (6, 1, 20, 6, 2), (2, 1, 128, 64, 3), (1, 1, 40, 100, 3), (2, 1, 200, 24, 2)])
def test_gated_delta_rule_prompt_then_decode(gpu, dtype, H, G, d, dv, taps):
    """Input stage (short convolutions with silu, unit vectors, step size, decay) and scan against the oracle's token loop, then decoding from the slots: the
    convolution's predecessors then come from the slot's ring, the state from the slot."""
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(taps + d)
    w, lens, extra = 32, [29, 1, 6], 5
    total = [l + extra for l in lens]
    C = 2 * G * d + H * dv
    Wt = {nm: rnd(g, n, w, s=2.0 / math.sqrt(w)).to(dtype) for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv), ("g", H * dv))}
    Wt["b"], Wt["a"] = rnd(g, H, w, s=0.7).to(dtype), rnd(g, H, w, s=0.7).to(dtype)
    for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
        Wt[nm + ".conv"] = rnd(g, n, taps, s=0.6)
    Wt["A_log"], Wt["dt_bias"], Wt["norm"] = rnd(g, H, s=0.7), rnd(g, H), 1.0 + rnd(g, dv, s=0.2)
    Wt["o"] = torch.eye(H * dv)
    hs = [rnd(g, t, w).to(dtype) for t in total]
    # one product, as the model runs it; the oracle reads the same rounded projections (its own weights pick them out of the wide row)
    order = ("q", "k", "v", "b", "a", "g")
    wcat = torch.cat([Wt[nm] for nm in order])
    wides = [(h.float() @ wcat.float().t()).to(dtype) for h in hs]
    Wn, at = {"m." + nm: npy(t) for nm, t in Wt.items() if nm not in order}, 0
    for nm in order:
        sel = np.zeros((Wt[nm].shape[0], wcat.shape[0])); sel[:, at: at + Wt[nm].shape[0]] = np.eye(Wt[nm].shape[0])
        Wn["m." + nm] = sel; at += Wt[nm].shape[0]
    Wn["m.o"] = np.eye(H * dv)
    want = [do.gated_delta(npy(x), Wn, "m.", {"heads": H, "kv_heads": G, "dim": d, "vdim": dv}, 1e-5) for x in wides]
    dev = {nm: t.to(gpu) for nm, t in Wt.items()}
    conv = torch.cat([Wt[nm + ".conv"] for nm in ("q", "k", "v")]).t().contiguous().to(gpu)
    S = torch.full((5, H, dv, d), float("nan"), device=gpu)
    ring = torch.full((5, max(taps - 1, 1), C), float("nan"), dtype=dtype, device=gpu)
    slots = [3, 0, 4]

    def run(rows, lens_now, pos0):
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens_now, pos0=pos0, slots=slots)
        wide = rows.to(gpu)
        n = wide.shape[0]
        f32 = dict(dtype=torch.float32, device=gpu)
        q, k, v = torch.empty((n, G * d), **f32), torch.empty((n, G * d), **f32), torch.empty((n, H * dv), **f32)
        beta, decay = torch.empty((n, H), **f32), torch.empty((n, H), **f32)
        mix_ops.delta_prep(q, k, v, beta, decay, wide[:, :C], conv, ring, wide[:, C: C + H], wide[:, C + H: C + 2 * H], dev["A_log"], dev["dt_bias"], seq, pos, sl, p0, la,
                           H, G, d, dv, d ** -0.5)
        o = torch.empty((n, H, dv), **f32)
        mix_ops.delta_scan(o, S, q, k, v, beta, decay, cu, sl, p0, G)
        out = torch.empty((n, H * dv), dtype=dtype, device=gpu)
        mix_ops.head_norm_gate(out, o, dev["norm"], wide[:, C + 2 * H:], mix_ops.GATE_SILU, 1e-5)
        return out

    out = run(torch.cat([h[:l] for h, l in zip(wides, lens)]), lens, None)
    assert rel(out, np.concatenate([a[:l] for a, l in zip(want, lens)])) < TOL[dtype] / 2
    for t in range(extra):
        out = run(torch.stack([h[l + t] for h, l in zip(wides, lens)]), [1] * 3, [l + t for l in lens])
        assert rel(out, np.stack([a[l + t] for a, l in zip(want, lens)])) < TOL[dtype] / 2, t
    assert torch.isnan(S[1]).all() and torch.isnan(S[2]).all() and torch.isnan(ring[1]).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_normed_branches_averaged(gpu, dtype):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    n, w = 7, 36
    wide = rnd(g, n, 2 * w + 5, s=3.0).to(dtype)
    wa, wb = 1.0 + rnd(g, w, s=0.3), 1.0 + rnd(g, w, s=0.3)
    dev = wide.to(gpu)
    out = torch.empty((n, w), dtype=dtype, device=gpu)
    mix_ops.rms_pair(out, dev[:, :w], wa.to(gpu), dev[:, w + 5:], wb.to(gpu), 0.5, 1e-5)
    a, b = npy(wide[:, :w]), npy(wide[:, w + 5:])
    assert rel(out, 0.5 * (do.rms_unit(a, 1e-5) * npy(wa) + do.rms_unit(b, 1e-5) * npy(wb))) < TOL[dtype] / 2


@pytest.mark.parametrize("experts,top,groups,keep", [(8, 2, 4, 2), (12, 3, 3, 2), (6, 2, 3, 1), (4, 4, 2, 2), (9, 1, 1, 1), (10, 2, 5, 2), (130, 5, 13, 3)])
def test_router_group_scores_are_sums_of_two(gpu, experts, top, groups, keep):
    """Sigmoid scores, a correction that pushes choice scores below zero (a left-out group must count as minus infinity, not 0), groups scored by the sum of
    their two best choice scores: the best single expert may sit in a group that loses."""
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(experts)
    n = 64
    z = rnd(g, n, experts, s=2.0)
    corr = rnd(g, experts, s=0.5) - 1.2
    r = {"experts": experts, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}}
    idx = torch.empty((n, top), dtype=torch.int32, device=gpu); wts = torch.empty((n, top), dtype=torch.float32, device=gpu)
    mix_ops.topk_grouped_ex(idx, wts, None, z.to(gpu), corr.to(gpu), mix_ops.ROUTE_SIGMOID, experts, groups, keep, 2, 1.7)
    differs_from_max_rule = 0
    for t in range(n):
        chosen, w = do.route(npy(z[t]), npy(corr), r)
        assert idx[t].tolist() == chosen, t
        assert np.abs(npy(wts[t]) - w).max() < 1e-5
        c = do.sigmoid(npy(z[t])) + npy(corr)
        per = experts // groups
        by_max = sorted(range(groups), key=lambda gi: (-c[gi * per:(gi + 1) * per].max(), gi))[:keep]
        differs_from_max_rule += any((e // per) not in by_max for e in chosen)
    if groups > keep and experts // groups > 1:
        assert differs_from_max_rule > 0                        # the inputs do tell the two rules apart


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 3, 17, 100])
def test_experts_with_gated_shared_expert(gpu, dtype, rows):
    """Every path of the experts by row count (per (row, choice), expert-major, expert-sorted products) with the shared expert behind its sigmoid gate."""
    from exllamav3_amd.modules import GatedMLP, SparseExperts
    from exllamav3_amd.state_cache import StepBatch
    g = torch.Generator().manual_seed(rows)
    w, ff, E, top = 64, 24, 8, 3
    f = moe(ff, E, top, groups=(4, 2), scale=1.5, shared=40)
    W = {}
    lin = lambda o, i, gain=1.0: (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(torch.bfloat16)
    for e in range(E):
        W[f"x.e{e}.gate"], W[f"x.e{e}.up"], W[f"x.e{e}.down"] = lin(ff, w, 2.0), lin(ff, w, 2.0), lin(w, ff)
    W["x.router"], W["x.correction"] = lin(E, w, 3.0), (rnd(g, E, s=0.5) - 0.6).to(torch.bfloat16)
    W["x.shared.gate"], W["x.shared.up"], W["x.shared.down"], W["x.shared.sg"] = lin(40, w, 2.0), lin(40, w, 2.0), lin(w, 40), lin(1, w, 3.0)

    class Stc:
        def get_tensor(self, key, device="cpu"):
            return W[key]
    m = SparseExperts(w, ff, E, top, router="sigmoid", router_bias=False, correction=True, route_scale=1.5, act="silu", shared=GatedMLP(w, 40, "silu", row_gate="sg"),
                      groups=4, keep_groups=2, group_top=2)
    m.load(Stc(), "x.", dtype, gpu)
    h = rnd(g, rows, w).to(dtype)
    sb = StepBatch(n=rows, batch=1, decode=False, max_rows=rows, tokens=None, cu=None, tok_seq=None, tok_pos=None, slots=None, pos0=None, len_after=None)
    y, _ = m.forward(h.to(gpu), sb)
    want = do.moe(npy(h), {k: npy(v) for k, v in W.items()}, "x.", f)
    e = np.abs(npy(y) - want).max(-1) / np.abs(want).max()
    if dtype == torch.float32:
        assert e.max() < 3e-5
    else:
        assert np.median(e) < 2e-2 and np.quantile(e, 0.9) < 0.2


# ---- whole models -----------------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(MODELS))
def test_whole_prompt_and_the_stream_after_every_layer(gpu, zoo, name, dtype):
    cfg, W, models = zoo[name]
    model = models[dtype]
    toks = tokens(cfg, 90, 1)
    want, taps = truth(name, cfg, W, toks)
    cache = model.new_cache()
    poison(cache)
    model.layer_taps = []
    got = run_whole(model, cache, toks)
    got_taps, model.layer_taps = model.layer_taps, None
    check_logits(got, want, dtype)
    assert len(got_taps) == len(cfg["layers"])
    if dtype == torch.float32:
        for r, (a, b) in enumerate(zip(got_taps, taps)):
            assert rel(a, b) < 3e-5, r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("prompt", [1, 2, 30, 64])
def test_prompt_then_token_by_token(gpu, zoo, name, dtype, prompt):
    """The first tokens of a sequence (a prompt of one or two tokens: convolutions and recurrences start from nothing), a prompt that ends at a page's border,
    then decoding across page borders."""
    cfg, W, models = zoo[name]
    model = models[dtype]
    toks = tokens(cfg, 140, 2)
    want, _ = truth(name, cfg, W, toks)
    cache = model.new_cache()
    poison(cache)
    check_logits(run_decoded(model, cache, toks, prompt), want, dtype)


@pytest.mark.parametrize("name", list(MODELS))
def test_decoded_equals_whole_in_float32(gpu, zoo, name):
    cfg, W, models = zoo[name]
    model = models[torch.float32]
    toks = tokens(cfg, 100, 3)
    cache = model.new_cache()
    a, b = run_whole(model, cache, toks), run_decoded(model, cache, toks, 17)
    assert float(logit_err(a, npy(b)).max()) < 3e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(MODELS))
def test_unequal_batch_against_each_alone_with_reused_slots_and_pages(gpu, zoo, name, dtype):
    """Requests of 1, 2, 70 and 129 tokens start in ONE packed step and decode together; the shorter ones end earlier and give their slot and pages back, a new
    request takes them over (whatever they held).  Every request's logits equal the oracle's for that request alone."""
    cfg, W, models = zoo[name]
    model = models[dtype]
    lens_total = [12, 40, 100, 150]
    prompts = [1, 2, 70, 129]
    reqs = [tokens(cfg, n, 10 + i) for i, n in enumerate(lens_total)]
    cache = model.new_cache(slots=2)                            # the pool of slots grows while the batch is admitted
    poison(cache)
    slots = [cache.alloc() for _ in reqs]
    got = [[] for _ in reqs]
    lg = model.step(cache.begin_step([(s, r[:p]) for s, r, p in zip(slots, reqs, prompts)], [list(range(p)) for p in prompts]), cache).cpu()
    at = 0
    for i, p in enumerate(prompts):
        got[i].append(lg[at: at + p]); at += p
    alive, step = list(range(len(reqs))), 0
    late = None
    while alive:
        ent = [(slots[i], [reqs[i][prompts[i] + step]]) for i in alive]
        lg = model.step(cache.begin_step(ent, [[0]] * len(ent)), cache).cpu()
        for j, i in enumerate(alive):
            got[i].append(lg[j: j + 1])
        step += 1
        for i in list(alive):
            if prompts[i] + step == lens_total[i]:
                cache.release(slots[i]); alive.remove(i)
                if late is None:                                # the first slot that comes back goes to a new request at once
                    late = tokens(cfg, 70, 99)
                    s2 = cache.alloc()
                    assert s2 == slots[i]
                    check_logits(model.step(cache.begin_step([(s2, late)], [list(range(70))]), cache).cpu(), truth(name, cfg, W, late)[0], dtype)
                    cache.release(s2)
    for i, r in enumerate(reqs):
        check_logits(torch.cat(got[i]), truth(name, cfg, W, r)[0], dtype)
    assert cache.in_use() == 0 and cache.pages_in_use() == 0


def test_pages_are_returned_and_reused(gpu, zoo):
    cfg, W, models = zoo["mixed"]
    model = models[torch.float32]
    cache = model.new_cache(slots=1, tokens=200)
    before = cache.num_pages
    toks = tokens(cfg, 130, 5)
    want = truth("mixed", cfg, W, toks)[0]
    for _ in range(3):                                          # the same pages, in another order each time (a stack), filled with something else in between
        check_logits(run_whole(model, cache, toks), want, torch.float32)
        poison(cache)
    assert cache.num_pages == before and cache.pages_in_use() == 0
    a, b = cache.alloc(), cache.alloc()                         # two sequences that need more pages than the pool holds: it grows, what is there stays
    model.step(cache.begin_step([(a, toks[:100])], [[]]), cache)
    model.step(cache.begin_step([(b, tokens(cfg, 500, 6))], [[]]), cache)
    assert cache.num_pages > before
    rows = [model.step(cache.begin_step([(a, [t])], [[0]]), cache).cpu() for t in toks[100:]]
    check_logits(torch.cat(rows), want[100:], torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_decoding(gpu, zoo, dtype):
    """300 tokens decoded one by one after a two-token prompt: five pages per attention layer, recurrent states carried 300 times."""
    cfg, W, models = zoo["odd"]
    model = models[dtype]
    toks = tokens(cfg, 302, 7)
    cache = model.new_cache()
    poison(cache)
    check_logits(run_decoded(model, cache, toks, 2), truth("odd", cfg, W, toks)[0], dtype)


def test_a_step_that_continues_by_several_tokens_is_refused(gpu, zoo):
    cfg, W, models = zoo["odd"]
    cache = models[torch.float32].new_cache()
    s = cache.alloc()
    cache.begin_step([(s, [1, 2, 3])])
    with pytest.raises(RuntimeError):
        cache.begin_step([(s, [4, 5])])


def test_trace_replay(gpu, zoo, tmp_path):
    from exllamav3_amd.trace import TraceSession
    cfg, W, models = zoo["mixed"]
    model = models[torch.float32]
    a, b = tokens(cfg, 70, 20), tokens(cfg, 9, 21)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}, {"id": "b", "tokens": b[:7], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [a[66]], "want": [0]}, {"id": "b", "tokens": [b[7]], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [a[67]], "want": []}, {"id": "b", "tokens": [b[8]], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": [a[68]], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "c", "tokens": b, "want": [8]}, ], "end": ["c"]},
             {"step": 5, "entries": [{"id": "a", "tokens": [a[69]], "want": [0]}], "end": ["a"]}]
    out = io.StringIO()
    sess = TraceSession(model, str(tmp_path), max_tokens=100)
    sess.run([json.dumps(s) for s in steps], out=out)
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2", "done", "3", "done", "4", "done", "5"]
    ta, tb = truth("mixed", cfg, W, a)[0], truth("mixed", cfg, W, b)[0]
    rd = lambda n: np.fromfile(os.path.join(str(tmp_path), f"{n}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])
    check_logits(rd(0), ta[[0, 65]], torch.float32)
    check_logits(rd(1), np.stack([ta[66], tb[7]]), torch.float32)
    check_logits(rd(2), tb[8:9], torch.float32)
    check_logits(rd(3), ta[68:69], torch.float32)
    check_logits(rd(4), tb[8:9], torch.float32)
    check_logits(rd(5), ta[69:70], torch.float32)
    assert sess.cache.in_use() == 0 and sess.cache.pages_in_use() == 0


@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_greedy_generation_through_the_scheduler(gpu, zoo, name):
    """Generator (continuous batching, decode steps replayed as graphs) against the oracle's own greedy loop, token for token, in float32."""
    from exllamav3_amd.generator import Generator
    cfg, W, models = zoo[name]
    model = models[torch.float32]
    prompts = [tokens(cfg, n, 30 + n) for n in (3, 61, 1, 20)]
    new = 9
    gen = Generator(model, model.new_cache(slots=2), max_batch=3)           # the fourth prompt waits for a slot that another request gives back
    outs = gen.generate(prompts, max_new_tokens=new)
    assert gen.graph_replays > 0
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(new):
            seq.append(int(np.argmax(do.forward(cfg, W, seq)[-1])))
        assert o == seq[len(p):]
    assert gen.cache.in_use() == 0 and gen.cache.pages_in_use() == 0
