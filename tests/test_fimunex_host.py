"""CPU tests around the Fimunex design: the oracle's own closed forms (input convolution, rotate-half rotation, chunk mask, grouped router, identity
experts), the order of layer runs, the configuration reader's defaults and refusals, a model built on the CPU from a written checkpoint (weights reach
the right places, state per layer run), the registry and the declared C symbols."""
import json
import math
import os
import pytest
import torch
import fimunex_oracle as fo

F64 = torch.float64


def test_oracle_input_convolution_and_norm():
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=F64)
    w = torch.tensor([[1.0, 0.0, 0.5], [0.0, 2.0, 0.0]], dtype=F64)          # channel 0: h_(t-2) + 0.5 h_t; channel 1: 2 h_(t-1)
    o = fo.causal_taps(h, w)
    assert torch.allclose(o[:, 0], torch.tensor([1.5, 3.0, 5.5, 8.0], dtype=F64))
    assert torch.allclose(o[:, 1], torch.tensor([10.0, 40.0, 70.0, 100.0], dtype=F64))
    assert torch.equal(fo.causal_taps(h, torch.zeros(2, 1, dtype=F64)), h)
    x = torch.tensor([[3.0, -4.0]], dtype=F64)
    assert torch.allclose(fo.norm_one_plus(x, torch.tensor([0.0, 1.0], dtype=F64), 0.0), torch.tensor([[3.0, -8.0]], dtype=F64) / math.sqrt(12.5))


def test_oracle_rotation_pairs_halves_and_composes():
    v = torch.randn(12, 2, 10, dtype=F64)
    c, s = fo.rotary_half_tables(12, 6, 100.0)
    r = fo.rotate_half(v, c, s, 6)
    assert torch.equal(r[..., 6:], v[..., 6:])
    for i in range(3):                                           # entry i turns with entry i + 3 and the pair keeps its length
        assert torch.allclose(r[..., i] ** 2 + r[..., i + 3] ** 2, v[..., i] ** 2 + v[..., i + 3] ** 2)
    # the score of a rotated query and key depends on the distance only
    q, k = torch.randn(1, 6, dtype=F64), torch.randn(1, 6, dtype=F64)
    rq, rk = fo.rotate_half(q.expand(12, 6), c, s, 6), fo.rotate_half(k.expand(12, 6), c, s, 6)
    assert abs(float(rq[7] @ rk[3]) - float(rq[11] @ rk[7])) < 1e-12
    sc = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    c, s = fo.rotary_half_tables(2, 16, 10000.0, sc)
    mag = 0.1 * math.log(4.0) + 1
    f = lambda i: 10000.0 ** (-2.0 * i / 16)
    assert abs(float(c[1, 0] ** 2 + s[1, 0] ** 2) - mag ** 2) < 1e-12
    assert abs(float(torch.atan2(s[1, 0], c[1, 0])) - f(0)) < 1e-12 and abs(float(torch.atan2(s[1, 7], c[1, 7])) - f(7) / 4.0) < 1e-12


def test_oracle_chunk_mask_and_softcap():
    T = 7
    q = torch.zeros(T, 2, dtype=F64); k = torch.zeros(T, 2, dtype=F64)
    v = torch.arange(T, dtype=F64).reshape(T, 1)
    o = fo.chunk_softmax_attention(q, k, v, 1.0, 0.0, 3)         # equal scores: the mean over the row's own chunk up to itself
    assert torch.allclose(o[:, 0], torch.tensor([0.0, 0.5, 1.0, 3.0, 3.5, 4.0, 6.0], dtype=F64))
    q = torch.tensor([[1.0], [1.0]], dtype=F64); k = torch.tensor([[0.0], [1000.0]], dtype=F64)
    o = fo.chunk_softmax_attention(q, k, torch.tensor([[0.0], [1.0]], dtype=F64), 1.0, 2.0, 8)
    assert abs(float(o[1, 0]) - 1.0 / (1.0 + math.exp(-2.0))) < 1e-9          # the score 1000 is capped to 2


def test_oracle_grouped_router_and_identity_experts():
    z = torch.log(torch.tensor([[0.05, 0.30, 0.10, 0.15, 0.22, 0.18]], dtype=F64))          # softmax gives these scores back
    none = torch.zeros(6, dtype=F64)
    idx, w = fo.grouped_router(z, none, 2, 1, 1)
    assert sorted(idx[0].tolist()) == [1, 4] and abs(float(w.sum()) - 1) < 1e-12
    idx, w = fo.grouped_router(z, none, 2, 3, 1)                 # groups {0,1} {2,3} {4,5}: only the group of the best single expert
    assert sorted(idx[0].tolist()) == [0, 1]
    assert abs(float(w[0, idx[0].tolist().index(1)]) - 0.30 / 0.35) < 1e-12
    # the correction moves the choice, not the weights.  Choice scores 0.05 -0.9 | -0.9 -0.85 | -0.78 -1.02: groups 0 and 2 are kept, and expert 4 at
    # -0.78 is taken although the experts of the group that is left out would count as 0 if they were not taken out altogether
    corr = torch.tensor([0.0, -1.2, -1.0, -1.0, -1.0, -1.2], dtype=F64)
    idx, w = fo.grouped_router(z, corr, 2, 3, 2)
    assert sorted(idx[0].tolist()) == [0, 4]
    assert abs(float(w[0, idx[0].tolist().index(4)]) - 0.22 / 0.27) < 1e-12
    # an identity expert returns its input with its weight
    W = {"router": torch.tensor([[0.0], [5.0]], dtype=F64), "e0.up": torch.ones(1, 1, dtype=F64), "e0.down": torch.ones(1, 1, dtype=F64)}
    f = {"expert": {"ff": 1}, "router": {"experts": 1, "identity": 1, "top": 2}}
    h = torch.tensor([[2.0]], dtype=F64)
    s = torch.softmax(torch.tensor([0.0, 10.0], dtype=F64), 0)
    assert abs(float(fo.expert_mixture(h, W, "", f)) - float(s[0] * 4.0 + s[1] * 2.0)) < 1e-12


LAYER = {"type": "attention", "mlp": None,
         "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 4, "scale": 0.3, "diff": 0.4, "mask": {"size": 6}, "rot": {"base": 100.0, "dims": 4}}}


def test_layer_runs_of_config_and_oracle_agree():
    from exllamav3_amd.fimunex import FimunexConfig
    base = {"vocab": 8, "width": 8, "norm": {"eps": 1e-5}, "canon": {"taps": 2}, "layers": [LAYER] * 5}
    for loop, want in ((None, [0, 1, 2, 3, 4]), ((0, 2, 3), [0, 1, 0, 1, 0, 1, 2, 3, 4]), ((1, 4, 2), [0, 1, 2, 3, 1, 2, 3, 4]), ((4, 5, 1), [0, 1, 2, 3, 4]), ((0, 5, 2), list(range(5)) * 2)):
        cfg = dict(base)
        if loop:
            cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
        assert FimunexConfig(cfg).runs() == want == fo.layer_runs(cfg)
    for bad in ((3, 2, 1), (0, 6, 1), (0, 2, 0)):
        with pytest.raises(RuntimeError):
            FimunexConfig(dict(base, loop=dict(zip(("start", "stop", "times"), bad))))


def test_config_defaults_and_refusals():
    from exllamav3_amd.fimunex import FimunexConfig
    from exllamav3_amd.modules import SparseExperts
    cfg = FimunexConfig({"vocab": 8, "width": 16, "norm": {"eps": 1e-6}, "canon": {"taps": 3}, "layers": [LAYER]})
    blk = cfg.build_layers()[0]
    assert cfg.logit_softcap == 0.0 and cfg.loop is None and blk.mlp is None and blk.in2 is None and blk.in1.taps == 3
    assert blk.mixer.softcap == 0.0 and blk.mixer.rot_dims == 4 and blk.mixer.span == 6 and blk.mixer.kv_heads == 1
    assert [s.name for s in blk.state_specs()] == ["ring_k", "ring_v", "canon1"]
    assert blk.state_specs()[0].shape == (6, 2, 8) and blk.state_specs()[1].shape == (6, 1, 4) and blk.state_specs()[2].shape == (2, 16)
    with pytest.raises(RuntimeError):
        FimunexConfig({"vocab": 8, "width": 16, "norm": {"eps": 1e-6}, "layers": [dict(LAYER, type="gla")]}).build_layers()
    with pytest.raises(RuntimeError):
        FimunexConfig({"vocab": 8, "width": 16, "norm": {"eps": 1e-6}, "layers": [dict(LAYER, mixer={k: v for k, v in LAYER["mixer"].items() if k != "mask"})]}).build_layers()
    with pytest.raises(RuntimeError):                            # three choices cannot come out of one kept group of two
        SparseExperts(16, 8, 3, 3, router="softmax_all", gated=False, act="relu2", identity=1, groups=2, keep_groups=1)
    with pytest.raises(RuntimeError):
        SparseExperts(16, 8, 4, 2, router="softmax", identity=2)


def test_model_from_a_written_checkpoint_on_the_cpu(tmp_path):
    """Loading needs no GPU: the tensors land where the mechanisms expect them, the norm weights w of the checkpoint are held as 1 + w, the state of
    a looped layer exists once per pass."""
    from safetensors.torch import save_file
    from exllamav3_amd import registry
    g = torch.Generator().manual_seed(0)
    moe = {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "identity": 1, "top": 2, "groups": {"count": 2, "keep": 1}}}
    cfg = {"architecture": "Fimunex", "vocab": 10, "width": 16, "norm": {"eps": 1e-5}, "canon": {"taps": 3}, "logit_softcap": 9.0,
           "loop": {"start": 0, "stop": 1, "times": 2}, "layers": [dict(LAYER, mlp=moe), LAYER]}
    W = {"embed": torch.randn(10, 16, generator=g), "head": torch.randn(10, 16, generator=g), "final.norm": torch.full((16,), 0.25)}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        W[p + "norm1"] = torch.full((16,), -0.5); W[p + "canon1"] = torch.randn(16, 3, generator=g)
        for nm, rows in (("q", 32), ("k", 16), ("v", 4)):
            W[p + "mix." + nm] = torch.randn(rows, 16, generator=g); W[p + "mix." + nm + ".b"] = torch.randn(rows, generator=g)
        W[p + "mix.q.norm"] = torch.ones(8); W[p + "mix.k.norm"] = torch.ones(8)
        for nm, val in (("lq1", 0.5), ("lk1", 0.25), ("lq2", 0.0), ("lk2", 7.0)):
            W[p + "mix." + nm] = torch.full((8,), val)
        W[p + "mix.g"] = torch.randn(2, 16, generator=g); W[p + "mix.o"] = torch.randn(16, 8, generator=g); W[p + "mix.o.b"] = torch.randn(16, generator=g)
        if L["mlp"]:
            W[p + "norm2"] = torch.zeros(16); W[p + "canon2"] = torch.randn(16, 3, generator=g)
            for e in range(3):
                W[f"{p}mlp.e{e}.up"] = torch.randn(8, 16, generator=g); W[f"{p}mlp.e{e}.down"] = torch.randn(16, 8, generator=g)
            W[p + "mlp.router"] = torch.randn(4, 16, generator=g); W[p + "mlp.correction"] = torch.randn(4, generator=g)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    m = registry.load_model(str(tmp_path), "cpu", torch.float32)
    assert m.architecture == "Fimunex" and m.runs == [0, 0, 1] and m.vocab == 10
    assert torch.equal(m.final_norm, torch.full((16,), 1.25)) and torch.equal(m.blocks[0].in1.w, torch.full((16,), 0.5))
    assert abs(m.blocks[0].mixer.lam - (math.exp(1.0) - 1.0 + 0.4)) < 1e-12                  # exp(8 * 0.5 * 0.25) - exp(0) + diff
    assert m.blocks[0].mixer.inp.weight.shape == (32 + 16 + 4 + 2, 16) and m.blocks[0].mlp.w_up.shape == (3, 8, 16) and m.blocks[0].mlp.w_gate is None
    cache = m.new_cache(slots=3)
    assert len(cache.layers) == 3 and set(cache.layers[0]) == {"ring_k", "ring_v", "canon1", "canon2"} and set(cache.layers[2]) == {"ring_k", "ring_v", "canon1"}
    assert cache.layers[1]["ring_k"].shape == (3, 6, 2, 8) and cache.layers[0]["ring_k"].data_ptr() != cache.layers[1]["ring_k"].data_ptr()


def test_registered_and_declared():
    from exllamav3_amd import _lib, registry
    assert "Fimunex" in registry.architectures() and registry.native_libraries("Fimunex") == ("mix",)
    names = _lib.mix_declared_symbols()
    for n in ("exl3_mix_attn_prefill_ex", "exl3_mix_attn_prefill_mfma_ex", "exl3_mix_attn_decode_ex", "exl3_mix_qk_prep", "exl3_mix_diff_combine", "exl3_mix_residual_rms",
              "exl3_mix_canon", "exl3_mix_topk_grouped", "exl3_mix_moe_up_act", "exl3_mix_moe_expert_major_plain", "exl3_mix_moe_down_id", "exl3_mix_moe_combine_id"):
        assert n in names
    assert _lib.check_mix_symbols()
