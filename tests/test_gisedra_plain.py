"""The plain Gisedra implementation pinned by closed forms, and the package's configuration, registry,
schedule and cache layout for the architecture (no GPU)."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_gisedra as plain
import tiny_gisedra as tiny

F64 = torch.float64


def _w64(cfg, seed=1):
    return {k: v.to(torch.bfloat16).to(F64) for k, v in tiny.make_weights(cfg, seed).items()}


# ------------------------------------------------------------------ mechanisms by hand
def test_dynamic_tanh_takes_no_statistics():
    x = torch.tensor([[0.5, -2.0, 30.0]], dtype=F64)
    y = plain.dynamic_tanh(x, torch.tensor([2.0, 1.0, 3.0], dtype=F64), torch.tensor([0.1, 0.0, -1.0], dtype=F64), 0.5)
    assert y[0, 0].item() == pytest.approx(math.tanh(0.25) * 2 + 0.1)
    assert y[0, 1].item() == pytest.approx(math.tanh(-1.0))
    assert y[0, 2].item() == pytest.approx(3.0 - 1.0)            # saturated
    two = plain.dynamic_tanh(torch.cat([x, x * 0 + 7.0]), torch.ones(3, dtype=F64), torch.zeros(3, dtype=F64), 0.5)
    assert torch.equal(two[0], plain.dynamic_tanh(x, torch.ones(3, dtype=F64), torch.zeros(3, dtype=F64), 0.5)[0])


def test_rotation_layouts_by_hand():
    x = torch.arange(1.0, 7.0, dtype=F64).reshape(1, 1, 6).repeat(3, 1, 1)
    pos = torch.arange(3)
    f = plain.rotary_frequencies(4, 100.0)
    assert f == pytest.approx([1.0, 0.1])
    half = plain.rotate(x, pos, f, False)
    inter = plain.rotate(x, pos, f, True)
    assert torch.equal(half[0], x[0]) and torch.equal(inter[0], x[0])          # position 0: no turn
    assert torch.equal(half[..., 4:], x[..., 4:]) and torch.equal(inter[..., 4:], x[..., 4:])
    a0, a1 = 2.0 * 1.0, 2.0 * 0.1
    assert half[2, 0, 0].item() == pytest.approx(1 * math.cos(a0) - 3 * math.sin(a0))     # pairs (0, 2) and (1, 3)
    assert half[2, 0, 2].item() == pytest.approx(3 * math.cos(a0) + 1 * math.sin(a0))
    assert half[2, 0, 3].item() == pytest.approx(4 * math.cos(a1) + 2 * math.sin(a1))
    assert inter[2, 0, 0].item() == pytest.approx(1 * math.cos(a0) - 2 * math.sin(a0))    # pairs (0, 1) and (2, 3)
    assert inter[2, 0, 1].item() == pytest.approx(2 * math.cos(a0) + 1 * math.sin(a0))
    assert inter[2, 0, 3].item() == pytest.approx(4 * math.cos(a1) + 3 * math.sin(a1))


def test_rescaled_frequencies_by_wavelength():
    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f = plain.rotary_frequencies(16, 1000.0, sc)
    raw = [1000.0 ** (-2.0 * i / 16) for i in range(8)]
    kinds = set()
    for fi, ri in zip(f, raw):
        wave = 2 * math.pi / ri
        if wave < 64 / 4.0:
            assert fi == pytest.approx(ri)
            kinds.add("kept")
        elif wave > 64 / 1.0:
            assert fi == pytest.approx(ri / 8.0)
            kinds.add("slowed")
        else:
            s = (64 / wave - 1.0) / 3.0
            assert fi == pytest.approx((1 - s) * ri / 8.0 + s * ri) and ri / 8.0 < fi < ri
            kinds.add("blended")
    assert kinds == {"kept", "slowed", "blended"}
    # the package's table is the same one, and its other rule is still there
    from swifttransformer_amd.parts.position import rotary_frequencies
    g, mult = rotary_frequencies(16, 1000.0, sc)
    assert mult == 1.0 and np.allclose(g, f)
    _, mult2 = rotary_frequencies(16, 1000.0, {"factor": 8.0, "original": 32, "fast": 2.0, "slow": 0.5})
    assert mult2 == pytest.approx(0.1 * math.log(8.0) + 1.0)


def test_the_window_keeps_the_first_tokens():
    seen = plain.visible(10, 3, 2)
    assert seen[9].tolist() == [True, True, False, False, False, False, False, True, True, True]
    assert seen[2].tolist() == [True, True, True] + [False] * 7
    assert plain.visible(10, 3)[9].sum() == 3 and plain.visible(10, 0)[9].all()
    # equal scores: every visible key weighs the same
    q = torch.zeros(10, 1, 4, dtype=F64)
    v = torch.arange(10.0, dtype=F64).reshape(10, 1, 1)
    o = plain.softmax_attention(q, q, v, 1.0, seen)
    assert o[9, 0, 0].item() == pytest.approx((0 + 1 + 7 + 8 + 9) / 5)


def test_retention_by_hand_and_a_decay_of_one_sums():
    W = {"m.q": torch.eye(2, dtype=F64), "m.k": torch.eye(2, dtype=F64) * math.sqrt(2.0), "m.v": torch.eye(2, dtype=F64),
         "m.g": torch.zeros(2, 2, dtype=F64), "m.o": torch.eye(2, dtype=F64)}
    h = torch.tensor([[1.0, 0.0], [1.0, 1.0], [0.0, 2.0]], dtype=F64)
    c = {"heads": 1, "dim": 2, "vdim": 2, "decay": [0.5]}
    # the gate silu(0) = 0 hides everything: look at the state's read-out through a gate of one instead
    W["m.g"] = torch.full((2, 2), 50.0, dtype=F64)          # silu(large) ~ its argument; the unit norm is what is checked
    out = plain.retention(h, W, "m", c, 0.0)
    # S_0 = h0 h0^T; o_0 = S_0^T h0 = h0;  S_1 = 0.5 S_0 + h1 h1^T; o_1 = 0.5 h0 (h0.h1) + h1 (h1.h1) = [2.5, 2]
    o1 = torch.tensor([2.5, 2.0], dtype=F64)
    gate1 = plain.silu(torch.tensor([100.0, 100.0], dtype=F64))
    assert torch.allclose(out[1], o1 / torch.sqrt((o1 * o1).mean()) * gate1)
    c1 = dict(c, decay=[1.0])
    W["m.g"] = torch.eye(2, dtype=F64)
    a = plain.retention(h, W, "m", c1, 1e-6)
    b = plain.retention(torch.flip(h[:2], [0]), W, "m", c1, 1e-6)     # without decay the state is a plain sum
    assert a.shape == (3, 2) and torch.isfinite(a).all() and torch.isfinite(b).all()


def test_latent_attention_first_token_and_its_window():
    cfg = tiny.CONFIGS["A"]
    w = _w64(cfg)
    c = cfg["layers"][0]["mixer"]
    h = torch.randn(12, cfg["width"], dtype=F64, generator=torch.Generator().manual_seed(0))
    out = plain.latent_attention(h, w, "l0.mix", c, 1e-6)
    # the first token sees itself alone: its result is Wo Wuv c_0
    lat = plain.unit_rms(h[:1] @ w["l0.mix.dkv"].T[:, :c["kv_rank"]], 1e-6) * w["l0.mix.dkv.norm"]
    assert torch.allclose(out[0], (lat @ w["l0.mix.uv"].T @ w["l0.mix.o"].T)[0])
    wider = copy.deepcopy(c)
    wider["mask"]["size"] += 1
    other = plain.latent_attention(h, w, "l0.mix", wider, 1e-6)
    assert torch.allclose(out[:9], other[:9]) and not torch.allclose(out[9:], other[9:])


def test_experts_weights_are_a_softmax_over_the_chosen_alone():
    g = torch.Generator().manual_seed(3)
    W = {"m.router": torch.zeros(3, 4, dtype=F64), "m.router.b": torch.tensor([2.0, 1.0, -50.0], dtype=F64)}
    for e in range(3):
        W[f"m.e{e}.gate"] = torch.randn(5, 4, generator=g, dtype=F64)
        W[f"m.e{e}.up"] = torch.randn(5, 4, generator=g, dtype=F64)
        W[f"m.e{e}.down"] = torch.randn(4, 5, generator=g, dtype=F64)
    h = torch.randn(2, 4, generator=g, dtype=F64)
    one = lambda e: (plain.silu(h @ W[f"m.e{e}.gate"].T) * (h @ W[f"m.e{e}.up"].T)) @ W[f"m.e{e}.down"].T
    two = plain.routed_experts(h, W, "m", {"router": {"experts": 3, "top": 2}})
    p = math.exp(2.0) / (math.exp(2.0) + math.exp(1.0))
    assert torch.allclose(two, p * one(0) + (1 - p) * one(1))
    assert torch.allclose(plain.routed_experts(h, W, "m", {"router": {"experts": 3, "top": 1}}), one(0))


def test_filter_uses_the_last_column_for_the_token_itself():
    u = torch.tensor([[1.0], [10.0], [100.0]], dtype=F64)
    y = plain.causal_filter(u, torch.tensor([[3.0, 2.0]], dtype=F64))
    assert y[:, 0].tolist() == [2.0, 23.0, 230.0]


def test_side_input_enters_at_unit_root_mean_square():
    cfg = tiny.CONFIGS["A"]
    w = _w64(cfg)
    x = torch.randn(5, cfg["width"], dtype=F64, generator=torch.Generator().manual_seed(1))
    tokens = torch.tensor([3, 9, 3, 50, 96])
    s = plain.side_input(x, tokens, w, 1, 8, 1e-6)
    gain = w["l1.side.norm"]
    live = gain != 0
    assert torch.allclose(((s[:, live] / gain[live]) ** 2).sum(-1) / cfg["width"] +
                          ((s[:, ~live]) ** 2).sum(-1), torch.ones(5, dtype=F64) * live.sum() / cfg["width"], atol=0.35)
    # the layer's own columns of the table: another layer's part gives another result
    assert not torch.allclose(s, plain.side_input(x, tokens, {**w, "l1.side.gate": w["l1.side.gate"], "side.embed":
                              torch.roll(w["side.embed"], 8, dims=1)}, 1, 8, 1e-6))


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_prefix_invariance_and_pass_order(name):
    cfg = tiny.CONFIGS[name]
    w = _w64(cfg)
    seq = tiny.prompt(30, cfg["vocab"], 2)
    full = plain.logits(cfg, w, seq)
    assert torch.allclose(plain.logits(cfg, w, seq[:17]), full[:17], atol=1e-9)
    order = plain.run_order(cfg)
    loop = cfg.get("loop")
    if loop:
        a, b, n = loop["start"], loop["stop"], loop["times"]
        assert len(order) == len(cfg["layers"]) + (n - 1) * (b - a)
        assert [p for _, p in order if p is not None] == list(range(n))
        assert all(i == a for i, p in order if p is not None)
    else:
        assert order == [(i, None) for i in range(len(cfg["layers"]))]
    streams = plain.residual_streams(cfg, w, seq)
    assert len(streams) == len(order)


def test_the_embedding_comes_back_from_the_second_pass_on():
    cfg = copy.deepcopy(tiny.CONFIGS["A"])
    w = _w64(cfg)
    seq = tiny.prompt(9, cfg["vocab"], 4)
    base = plain.logits(cfg, w, seq)
    moved = dict(w)
    moved["loop.step"] = w["loop.step"].clone()
    moved["loop.step"][2] += 1.0
    assert not torch.allclose(plain.logits(cfg, moved, seq), base)
    # one pass only: neither the embedding nor the later passes' vectors matter
    cfg["loop"]["times"] = 1
    w1 = dict(w)
    w1["loop.step"] = w["loop.step"][:1]
    once = plain.logits(cfg, w1, seq)
    first = x = w["embed"][torch.tensor(seq)]
    x = plain.layer(x, torch.tensor(seq), w, cfg, 0)
    x = x + w["loop.step"][0]
    for i in (1, 2):
        x = plain.layer(x, torch.tensor(seq), w, cfg, i)
    assert torch.allclose(once, plain._norm(x, w, "final.norm") @ w["head"].T)


# ------------------------------------------------------------------ the package's side, without a GPU
def test_config_errors_name_their_key():
    from swifttransformer_amd.config.gisedra_param import GisedraHyperParam
    from swifttransformer_amd.config.hyper_param import ConfigError
    good = tiny.CONFIGS["A"]
    GisedraHyperParam.from_dict(good)

    def broken(change):
        cfg = copy.deepcopy(good)
        change(cfg)
        return cfg
    cases = {
        "kv_rank": lambda c: c["layers"][0]["mixer"].pop("kv_rank"),
        "rot_dim": lambda c: c["layers"][0]["mixer"].update(rot_dim=7),
        "decay": lambda c: c["layers"][1]["mixer"]["right"].update(decay=[0.5]),
        "kv_heads": lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3),
        "conv": lambda c: c["layers"][1]["mixer"]["left"].update(conv=9),
        "top": lambda c: c["layers"][0]["mlp"]["router"].update(top=5),
        "kind": lambda c: c["layers"][0]["mlp"].update(kind="dense"),
        "loop": lambda c: c["loop"].update(stop=4),
        "type": lambda c: c["layers"][2].update(type="attention"),
        "left_scale": lambda c: c["layers"][1]["mixer"].pop("left_scale"),
        "high": lambda c: c["layers"][1]["mixer"]["left"]["rot"]["scaling"].update(high=0.5),
    }
    for key, change in cases.items():
        with pytest.raises(ConfigError, match=key):
            GisedraHyperParam.from_dict(broken(change))


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_schedule_caches_and_tensor_declaration(name, tmp_path):
    from swifttransformer_amd.config.registry import hyper_param_from_dir
    from swifttransformer_amd.models import build_model
    cfg = tiny.CONFIGS[name]
    folder = tiny.write_folder(cfg, str(tmp_path / name), 5)
    arch, hp = hyper_param_from_dir(folder)
    assert arch.name == "Gisedra" and hp.to_config_dict()["layers"] == cfg["layers"]
    model = build_model(hp, torch.float32)
    order = plain.run_order(cfg)
    assert [e.layer for e in model.schedule] == [i for i, _ in order]
    assert [e.enter is not None for e in model.schedule] == [p is not None for _, p in order]
    assert len(model.entries) == (cfg["loop"]["times"] if cfg.get("loop") else 0)
    assert [e.add_first for e in model.entries] == [t > 0 for t in range(len(model.entries))]
    # every run has caches of its own: a latent run one paged cache, a parallel run pages, a filter state (with
    # more than one tap) and the retention's state
    needs = model.cache_needs()
    for run, (i, _) in enumerate(order):
        L = cfg["layers"][i]
        if L["type"] == "latent_attention":
            need = needs[run]
            m = L["mixer"]
            assert need.kind == "paged_kv" and not need.values and need.num_kv_heads == 1
            assert need.head_dim == -(-(m["kv_rank"] + m["rot_dim"]) // 16) * 16
            assert need.window == (m.get("mask") or {}).get("size", 0)
        else:
            left, right = L["mixer"]["left"], L["mixer"]["right"]
            kv = needs[(run, "left.kv")]
            mask = left.get("mask") or {}
            assert (kv.num_kv_heads, kv.head_dim, kv.window) == (left["kv_heads"], left["dim"], mask.get("size", 0))
            assert kv.keep_first == (mask.get("keep_first", 0) if mask.get("size") else 0)
            assert ((run, "left.conv") in needs) == (left.get("conv", 0) > 1)
            assert needs[(run, "right")].state_shape == (right["heads"], right["dim"], right["vdim"])
    _, w = plain.load_folder(folder)
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == {k: tuple(v.shape) for k, v in w.items()}


def test_kept_first_pages_are_never_given_back():
    from swifttransformer_amd.cache.manager import CacheManager
    from swifttransformer_amd.parts.base import CacheNeed
    needs = {0: CacheNeed("paged_kv", num_kv_heads=1, head_dim=16, window=8, keep_first=5),
             1: CacheNeed("paged_kv", num_kv_heads=1, head_dim=16, window=8)}
    m = CacheManager(needs, page_size=4, num_pages=16, max_seqs=2, max_pages_per_seq=64)
    assert len(m.paged_groups) == 2                       # the kept tokens make a group of its own
    m.admit("r")
    m.extend("r", 40)
    m.release_behind_window("r", 40)
    kept, plain_group = (m.requests["r"].tables[g.index] for g in m.paged_groups)
    assert [p >= 0 for p in kept] == [True, True] + [False] * 6 + [True, True]      # 5 tokens: two pages stay
    assert [p >= 0 for p in plain_group] == [False] * 8 + [True, True]
    m.check_invariants()
    m.finish("r")
    assert all(g.pool.num_free == 16 for g in m.paged_groups)


def test_named_sizes():
    from swifttransformer_amd.config.registry import hyper_param_by_name
    hp = hyper_param_by_name("gisedra_1.3b", num_layers=8)
    assert hp.width == 2048 and [L["type"] for L in hp.layers].count("parallel") == 2
    assert hp.loop == {"start": 0, "stop": 2, "times": 2} and hp.token_side_dim == 16
    with pytest.raises(KeyError, match="gisedra_"):
        hyper_param_by_name("gisedra_77b")
