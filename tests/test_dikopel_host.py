"""CPU tests around the Dikopel design: closed forms that pin the float64 oracle (tests/dikopel_oracle.py) independently of any kernel, the configuration reader,
loading a written checkpoint without a GPU, the paged part of the slot state manager, the registry and the C ABI's declarations."""
import json
import math
import numpy as np
import pytest
import torch
import dikopel_oracle as do


def test_oracle_position_vector_and_layer_norm():
    p = do.position_vectors(5, 6)
    assert np.allclose(p[0], [0, 1, 0, 1, 0, 1])
    f1 = 10000.0 ** (-2.0 / 6)
    assert np.allclose(p[3, 2:4], [math.sin(3 * f1), math.cos(3 * f1)]) and np.allclose(p[4, :2], [math.sin(4.0), math.cos(4.0)])
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    y = do.layer_norm(x, np.full(4, 2.0), np.full(4, 0.5), 0.0)
    assert np.allclose(y, (x - 3.0) / math.sqrt(3.5) * 2.0 + 0.5)         # deviations -2, -1, 0, 3: their squares average 3.5
    assert abs(do.rms_unit(np.array([3.0, 4.0]), 0.0)[0] - 3.0 / math.sqrt(12.5)) < 1e-12


def test_oracle_convolutions():
    h = np.arange(1.0, 9.0).reshape(4, 2)
    w = np.array([[0.5, 2.0, -1.0], [0.0, 1.0, 3.0]])
    c = do.causal_conv(h, w, identity=False)
    assert np.allclose(c[0], [-1.0 * 1.0, 3.0 * 2.0])                       # the last column is the current token's; nothing before the start
    assert np.allclose(c[2], [0.5 * 1 + 2.0 * 3 - 1.0 * 5, 0.0 * 2 + 1.0 * 4 + 3.0 * 6])
    assert np.allclose(do.causal_conv(h, w, identity=True), h + c)
    assert np.allclose(do.causal_conv(h, w[:, 2:], identity=False), h * w[:, 2])


def test_oracle_sigmoid_attention_is_an_unnormalised_causal_sum():
    W = {"a.q": np.eye(2), "a.k": np.eye(2), "a.v": np.eye(2), "a.o": np.eye(2), "a.pb": np.array([0.5])}
    h = np.array([[1.0, 0.0], [0.0, 2.0], [1.0, 1.0]])
    o = do.sigmoid_attention(h, W, "a.", {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 2.0})
    s = lambda z: 1.0 / (1.0 + math.exp(-z))
    assert np.allclose(o[0], s(2.0 + 0.5) * h[0])
    assert np.allclose(o[2], s(2.0 + 0.5) * h[0] + s(4.0 + 0.5) * h[1] + s(4.0 + 0.5) * h[2])      # three keys, weights that do not sum to one


def test_oracle_delta_rule_stores_and_overwrites():
    """With beta = 1, no decay and orthogonal unit keys the memory returns exactly what was written, and writing a key again replaces its value."""
    H = G = 1; d = 2; dv = 3
    big = 60.0                                                              # sigmoid(big) = 1, softplus(-big) = 0
    W = {"r.q": np.zeros((2, 4)), "r.k": np.zeros((2, 4)), "r.v": np.zeros((3, 4)), "r.b": np.array([[0, 0, 0, big]]), "r.a": np.array([[0, 0, 0, -big]]),
         "r.A_log": np.zeros(1), "r.dt_bias": np.zeros(1), "r.norm": np.ones(3), "r.g": np.zeros((3, 4)), "r.o": np.eye(3)}
    for nm, n in (("q", 2), ("k", 2), ("v", 3)):
        W[f"r.{nm}.conv"] = np.ones((n, 1))
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv}
    S = np.zeros((d, dv))
    k1, k2 = np.array([1.0, 0.0]), np.array([0.0, 1.0])
    for k, v in ((k1, [1.0, 2.0, 3.0]), (k2, [4.0, 5.0, 6.0]), (k1, [7.0, 8.0, 9.0])):
        u = np.asarray(v) - S.T @ k
        S = S + np.outer(k, u)
    assert np.allclose(S.T @ k1, [7.0, 8.0, 9.0]) and np.allclose(S.T @ k2, [4.0, 5.0, 6.0])
    # the same through the oracle's function: inputs chosen so that silu(conv(.)) gives those keys, queries equal to the keys
    h = np.zeros((3, 4)); h[:, 3] = 1.0
    inv_silu = lambda y: float(np.interp(y, [z / (1 + math.exp(-z)) for z in np.linspace(0, 20, 20001)], np.linspace(0, 20, 20001)))
    W["r.k"][0, 0] = W["r.q"][0, 0] = 1.0; W["r.k"][1, 1] = W["r.q"][1, 1] = 1.0
    for t, k in enumerate((k1, k2, k1)):
        h[t, :2] = [inv_silu(5.0) if x else 0.0 for x in k]
    W["r.v"][:, 2] = 1.0
    h[:, 2] = [inv_silu(1.0), inv_silu(2.0), inv_silu(3.0)]
    o = do.gated_delta(h, W, "r.", m, 0.0)                                   # gate silu(0) = 0 would wipe the result: give it a gate of its own
    assert np.allclose(o, 0.0)
    W["r.g"][:, 3] = 50.0
    o = do.gated_delta(h, W, "r.", m, 0.0)
    unit = lambda x: x / math.sqrt(np.mean(x * x))
    assert np.allclose(o[2], unit(np.full(3, 3.0)) * 50.0, rtol=1e-4) and np.allclose(o[1], unit(np.full(3, 2.0)) * 50.0, rtol=1e-4)


def test_oracle_mlstm_against_the_unstabilised_sums():
    """With small gates the running maximum is only a rescaling: the result equals sums of exp(i_s + f_(s+1) + ... + f_t) k_s v_s over the past, divided by
    max(|n.q|, 1) + 1e-6 in those unscaled units."""
    rng = np.random.default_rng(0)
    T, w, H, d, dv, cap = 6, 5, 2, 3, 4, 50.0
    W = {"m." + nm: rng.normal(size=(n, w)) * 0.4 for nm, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("i", H), ("f", H))}
    W["m.i.b"], W["m.f.b"], W["m.norm"], W["m.o"] = rng.normal(size=H) * 0.1, rng.normal(size=H) * 0.1, np.ones(H * dv), np.eye(H * dv)
    h = rng.normal(size=(T, w))
    got = do.mlstm(h, W, "m.", {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}, 1e-5)
    q = (h @ W["m.q"].T).reshape(T, H, d) / math.sqrt(d); k = (h @ W["m.k"].T).reshape(T, H, d); v = (h @ W["m.v"].T).reshape(T, H, dv)
    ig = cap * np.tanh((h @ W["m.i"].T + W["m.i.b"]) / cap); fg = do.logsigmoid(cap * np.tanh((h @ W["m.f"].T + W["m.f.b"]) / cap))
    raw = np.zeros((T, H, dv))
    for a in range(H):
        for t in range(T):
            wts = [math.exp(ig[s, a] + fg[s + 1: t + 1, a].sum()) for s in range(t + 1)]
            num = sum(ws * (k[s, a] @ q[t, a]) * v[s, a] for s, ws in enumerate(wts))
            den = sum(ws * (k[s, a] @ q[t, a]) for s, ws in enumerate(wts))
            m = max([0.0 + fg[1 - 1: t + 1, a].sum()] + [ig[s, a] + fg[s + 1: t + 1, a].sum() for s in range(t + 1)])      # the maximum's closed form (it starts at 0)
            raw[t, a] = num / (max(abs(den), 1.0) + 1e-6 * math.exp(m))
    want = (do.rms_unit(raw, 1e-5).reshape(T, -1) * do.sigmoid(h @ W["m.g"].T))
    assert np.allclose(got, want, rtol=1e-9, atol=1e-12)


def test_oracle_router_groups_by_the_sum_of_two():
    r = {"experts": 6, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 1}}
    z = np.array([4.0, -9.0, 1.0, 1.2, 0.0, 0.0])                            # the best single expert (0) sits beside a very bad one
    chosen, w = do.route(z, np.zeros(6), r)
    assert chosen == [3, 2]                                                 # group 1 wins: 0.73 + 0.77 > 0.98 + 0.0001
    s = do.sigmoid(z)
    assert np.allclose(w, s[[3, 2]] / (s[3] + s[2]) * 3.0)
    # a correction decides the choice and stays out of the weights; choice scores below zero still beat a left-out group
    chosen, w = do.route(z, np.array([0.0, -3.0, -5.0, -5.0, -2.0, -2.1]), dict(r, groups={"count": 3, "keep": 2}))
    assert chosen == [0, 4] and np.allclose(w, s[[0, 4]] / (s[0] + s[4]) * 3.0)
    assert do.route(z, np.zeros(6), {"experts": 6, "top": 3})[0] == [0, 3, 2]


LEFT = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.3}
RIGHT = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 10, "conv": 3}
MOE = {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 4, "top": 2, "scale": 1.5, "groups": {"count": 2, "keep": 1}}, "shared": {"ff": 12}}
LAYERS = [{"type": "parallel", "mixer": {"left": LEFT, "right": RIGHT}, "mlp": {"kind": "dense", "ff": 20}},
          {"type": "mlstm", "mixer": {"heads": 2, "dim": 4, "vdim": 6, "gate_cap": 9.0}, "mlp": MOE},
          {"type": "parallel", "mixer": {"left": LEFT, "right": RIGHT}, "mlp": {"kind": "dense", "ff": 20}, "weights_of": 0},
          {"type": "mlstm", "mixer": {"heads": 2, "dim": 4, "vdim": 6, "gate_cap": 9.0}, "mlp": None}]
BASE = {"architecture": "Dikopel", "vocab": 10, "width": 16, "norm": {"eps": 1e-6}, "canon": {"taps": 3}, "embedding": {"scale": 2.0}, "residual_mult": 0.5}


def test_config_reader_and_refusals():
    from exllamav3_amd.dikopel import DikopelConfig
    from exllamav3_amd.state_cache import PagedSpec, StateSpec
    cfg = DikopelConfig(dict(BASE, layers=LAYERS))
    assert cfg.source == [0, 1, 0, 3] and cfg.mult == 0.5 and cfg.embed_scale == 2.0 and cfg.taps == 3
    blocks = cfg.build_blocks()
    assert sorted(blocks) == [0, 1, 3]                                      # the borrowing layer has no block of its own
    b0, b1, b3 = blocks[0], blocks[1], blocks[3]
    assert b0.mixer.left.scale == 0.3 and b0.mixer.right.taps == 3 and b0.mixer.right.channels == 2 * 8 + 2 * 10 and b0.mlp.ff == 20
    assert b1.mixer.cap == 9.0 and b1.mlp.group_top == 2 and b1.mlp.groups == 2 and b1.mlp.keep_groups == 1 and b1.mlp.route_scale == 1.5
    assert b1.mlp.shared.row_gate == "sg" and b1.mlp.shared.ff == 12 and b3.mlp is None
    specs = {s.name: s for s in b0.state_specs()}
    assert isinstance(specs["left.k"], PagedSpec) and specs["left.k"].shape == (16,) and specs["left.v"].shape == (12,)
    assert isinstance(specs["right.S"], StateSpec) and specs["right.S"].shape == (2, 10, 8) and specs["right.conv"].shape == (2, 36) and specs["canon1"].shape == (2, 16)
    assert {s.name: s.shape for s in b1.state_specs()} == {"S": (2, 6, 4), "n": (2, 4), "m": (2,), "canon1": (2, 16)}
    # defaults: no residual factor, no embedding scale, one tap, a router without groups or scale, no shared expert
    bare = DikopelConfig({"vocab": 4, "width": 8, "norm": {"eps": 1e-5}, "layers": [dict(LAYERS[1], mlp={"kind": "moe", "expert": {"ff": 4}, "router": {"experts": 3, "top": 1}})]})
    blk = bare.build_blocks()[0]
    assert bare.mult == 1.0 and bare.embed_scale == 1.0 and bare.taps == 1 and blk.mlp.groups == 1 and blk.mlp.shared is None and blk.mlp.route_scale == 1.0
    with pytest.raises(RuntimeError):
        DikopelConfig(dict(BASE, layers=[dict(LAYERS[0], type="attention")])).build_blocks()
    with pytest.raises(RuntimeError):
        DikopelConfig(dict(BASE, layers=[dict(LAYERS[0], mlp={"kind": "polynorm"})])).build_blocks()
    with pytest.raises(RuntimeError):
        DikopelConfig(dict(BASE, layers=[LAYERS[0], LAYERS[1], LAYERS[2], dict(LAYERS[0], weights_of=2)]))        # layer 2 has no tensors of its own
    with pytest.raises(RuntimeError):
        DikopelConfig(dict(BASE, layers=[]))


def _weights(cfg, g):
    w = cfg["width"]
    W = {"embed": torch.randn(cfg["vocab"], w, generator=g), "head": torch.randn(cfg["vocab"], w, generator=g), "final.norm": torch.full((w,), 0.75),
         "final.norm.b": torch.full((w,), -0.25)}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        W[p + "norm1"] = torch.ones(w); W[p + "norm1.b"] = torch.zeros(w); W[p + "canon1"] = torch.randn(w, cfg["canon"]["taps"], generator=g)
        if L["type"] == "mlstm":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            for nm, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv), ("i", H), ("f", H)):
                W[p + "mix." + nm] = torch.randn(n, w, generator=g)
            W[p + "mix.i.b"] = torch.zeros(H); W[p + "mix.f.b"] = torch.ones(H); W[p + "mix.norm"] = torch.ones(H * dv); W[p + "mix.o"] = torch.randn(w, H * dv, generator=g)
        else:
            a, b = m["left"], m["right"]
            for nm, n in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]), ("v", a["kv_heads"] * a["vdim"])):
                W[p + "mix.left." + nm] = torch.randn(n, w, generator=g)
            W[p + "mix.left.pb"] = torch.zeros(a["heads"]); W[p + "mix.left.o"] = torch.randn(w, a["heads"] * a["vdim"], generator=g); W[p + "mix.left.out"] = torch.ones(w)
            H, G, d, dv = b["heads"], b["kv_heads"], b["dim"], b["vdim"]
            for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                W[p + "mix.right." + nm] = torch.randn(n, w, generator=g); W[p + f"mix.right.{nm}.conv"] = torch.randn(n, b["conv"], generator=g)
            for nm, n in (("b", H), ("a", H), ("g", H * dv)):
                W[p + "mix.right." + nm] = torch.randn(n, w, generator=g)
            W[p + "mix.right.A_log"] = torch.zeros(H); W[p + "mix.right.dt_bias"] = torch.zeros(H); W[p + "mix.right.norm"] = torch.ones(dv)
            W[p + "mix.right.o"] = torch.randn(w, H * dv, generator=g); W[p + "mix.right.out"] = torch.ones(w)
        f = L.get("mlp")
        if f and f["kind"] == "dense":
            W[p + "mlp.gate"] = torch.randn(f["ff"], w, generator=g); W[p + "mlp.up"] = torch.randn(f["ff"], w, generator=g); W[p + "mlp.down"] = torch.randn(w, f["ff"], generator=g)
        elif f:
            for e in list(range(f["router"]["experts"])) + ["shared"]:
                q = f"{p}mlp.e{e}." if e != "shared" else p + "mlp.shared."
                n = f["expert"]["ff"] if e != "shared" else f["shared"]["ff"]
                W[q + "gate"] = torch.randn(n, w, generator=g); W[q + "up"] = torch.randn(n, w, generator=g); W[q + "down"] = torch.randn(w, n, generator=g)
            W[p + "mlp.shared.sg"] = torch.randn(1, w, generator=g)
            W[p + "mlp.router"] = torch.randn(f["router"]["experts"], w, generator=g); W[p + "mlp.correction"] = torch.randn(f["router"]["experts"], generator=g)
    return W


def test_model_from_a_written_checkpoint_on_the_cpu(tmp_path):
    """Loading needs no GPU: tensors land where the mechanisms expect them, a borrowing layer IS the lender's block, and every layer has a state of its own."""
    from safetensors.torch import save_file
    from exllamav3_amd import registry
    cfg = dict(BASE, layers=LAYERS)
    W = _weights(cfg, torch.Generator().manual_seed(0))
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    m = registry.load_model(str(tmp_path), "cpu", torch.float32)
    assert m.architecture == "Dikopel" and m.vocab == 10 and len(m.blocks) == 4 and m.blocks[2] is m.blocks[0] and m.blocks[3] is not m.blocks[1]
    assert torch.equal(m.final_w, torch.full((16,), 0.75)) and torch.equal(m.final_b, torch.full((16,), -0.25))
    par = m.blocks[0].mixer
    assert par.inp.weight.shape == (32 + 16 + 12 + 8 + 8 + 20 + 2 + 2 + 20, 16)          # ONE input product for both mixers
    assert par.inp.offsets["right.k"][0] == par.inp.offsets["right.q"][0] + 8 and par.inp.offsets["right.v"][0] == par.inp.offsets["right.k"][0] + 8
    assert par.right.conv.shape == (3, 36) and torch.equal(par.right.conv[:, 8:16].t(), W["l0.mix.right.k.conv"].to(torch.bfloat16).float())
    assert m.blocks[1].mlp.shared.inp.weight.shape == (12 + 12 + 1, 16) and m.blocks[1].mlp.w_gate.shape == (4, 8, 16)
    assert abs(float(m.pos_freq[1]) - 10000.0 ** (-2.0 / 16)) < 1e-7 and m.pos_freq.numel() == 8
    cache = m.new_cache(slots=3, tokens=100)
    assert len(cache.layers) == 4 and set(cache.layers[0]) == {"left.k", "left.v", "page_table", "right.S", "right.conv", "canon1"} and set(cache.layers[1]) == {"S", "n", "m", "canon1"}
    assert cache.layers[0]["left.k"].shape[1:] == (m.PAGE_SIZE, 16) and cache.layers[0]["left.k"].data_ptr() != cache.layers[2]["left.k"].data_ptr()
    assert cache.layers[0]["page_table"] is cache.layers[2]["page_table"] and cache.layers[2]["right.S"].shape == (3, 2, 10, 8)


def test_pages_of_the_slot_state_manager():
    from exllamav3_amd.state_cache import PagedSpec, SlotStateCache, StateSpec
    c = SlotStateCache([[StateSpec("S", (2,), torch.float32), PagedSpec("k", (3,), torch.float32)], [StateSpec("r", (1,), torch.float32)], [PagedSpec("k", (5,), torch.bfloat16)]],
                       "cpu", slots=2, page_size=4, tokens=20)
    assert c.num_pages == 5 + 2 and c.layers[0]["k"].shape == (7, 4, 3) and c.layers[2]["k"].shape == (7, 4, 5) and "page_table" not in c.layers[1]
    a, b = c.alloc(), c.alloc()
    c.begin_step([(a, [1] * 9), (b, [2] * 4)])
    assert c.pages_of == {a: [0, 1, 2], b: [3]} and c.page_table[a, :3].tolist() == [0, 1, 2] and c.page_table[b, 0].item() == 3 and c.pages_in_use() == 4
    gen = c.generation
    c.begin_step([(a, [1]), (b, [2])])                                       # a stays inside its third page, b opens a second one
    assert c.pages_of[a] == [0, 1, 2] and c.pages_of[b] == [3, 4] and c.generation == gen
    c.layers[0]["k"][4, 0, 0] = 7.0
    c.release(a)
    assert c.pages_in_use() == 2 and c.free_pages[-3:] == [2, 1, 0]
    d = c.alloc()
    assert d == a
    c.begin_step([(d, [3] * 30)])                                            # more pages than the pool has, more than the table is wide: both grow, contents stay
    assert c.generation > gen and len(c.pages_of[d]) == 8 and c.pages_of[d][:3] == [0, 1, 2] and c.num_pages >= 10 and c.table_width >= 8
    assert c.page_table[d, :8].tolist() == c.pages_of[d] and c.page_table[b, :2].tolist() == [3, 4] and c.layers[0]["k"][4, 0, 0].item() == 7.0
    assert c.layers[0]["page_table"] is c.page_table and c.layers[2]["page_table"] is c.page_table
    e = c.alloc()                                                            # a third slot: the pool of slots doubles, the table follows
    c.begin_step([(e, [1])])
    assert c.page_table.shape[0] == c.capacity == 4 and c.page_table[d, :8].tolist() == c.pages_of[d] and len(set(c.pages_of[d] + c.pages_of[b] + c.pages_of[e])) == 11
    for s in (b, d, e):
        c.release(s)
    assert c.pages_in_use() == 0 and c.in_use() == 0
    with pytest.raises(RuntimeError):
        c.release(b)
    plain = SlotStateCache([[StateSpec("S", (2,), torch.float32)]], "cpu")
    assert not plain.paged and plain.page_table is None
    plain.reserve([(plain.alloc(), [1, 2, 3])])                              # nothing to do without pages


def test_registered_and_declared():
    from exllamav3_amd import _lib, registry
    assert "Dikopel" in registry.architectures() and registry.native_libraries("Dikopel") == ("mix",)
    names = _lib.mix_declared_symbols()
    for n in ("exl3_mix_embed_sinusoid", "exl3_mix_layer_norm_rows", "exl3_mix_residual_norm_conv", "exl3_mix_glu_act_rowgate", "exl3_mix_topk_grouped_ex", "exl3_mix_paged_store",
              "exl3_mix_sigattn_prefill", "exl3_mix_sigattn_decode", "exl3_mix_sigattn_prefill_mfma", "exl3_mix_mlstm_scan", "exl3_mix_delta_prep", "exl3_mix_delta_scan",
              "exl3_mix_head_norm_gate", "exl3_mix_rms_pair"):
        assert n in names
    assert _lib.check_mix_symbols()
