"""The plain Pupalix pinned by hand-made cases and closed forms, its configuration and what the engine makes of it
(parts, tensor names, schedule, caches); no GPU."""
import copy
import math

import pytest
import torch

import plain_pupalix as plain
import tiny_pupalix as tiny

F = torch.float64


def test_pair_rows_by_hand():
    assert plain.bigram_rows([3, 4, 0, 4], 7, 2, 3) == [7, (3 * 2 + 4 * 3) % 7, (4 * 2) % 7, (0 + 12) % 7]
    assert plain.bigram_rows([9], 5, 1, 1) == [5]
    table, pairs = torch.arange(12, dtype=F).view(6, 2), torch.arange(100, 108, dtype=F).view(4, 2)
    x = plain.embed([5, 1], table, 2.0, pairs, {"buckets": 3, "mul_prev": 1, "mul_cur": 1})
    assert x.tolist() == [[2 * 10 + 106, 2 * 11 + 107], [2 * 2 + 100, 2 * 3 + 101]]


def test_rescaled_frequencies_keep_the_fast_pairs_and_divide_the_slow_ones():
    f, mult = plain.yarn_frequencies(8, 100.0, None)
    assert mult == 1.0 and f == [100.0 ** (-2 * i / 8) for i in range(4)]
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    g, mult = plain.yarn_frequencies(8, 100.0, sc)
    assert mult == pytest.approx(0.1 * math.log(4.0) + 1.0)
    d = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(d(8.0)), 0), min(math.ceil(d(1.0)), 7)
    for i in range(4):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0), 1)
        assert g[i] == pytest.approx(f[i] / 4.0 * ramp + f[i] * (1 - ramp))
    assert g[0] == f[0] and g[3] == pytest.approx(f[3] / 4.0)        # the first pair keeps its own, the last is slowed
    # both borders between the two pairs: the first keeps its frequency, the second takes the whole factor
    g2, _ = plain.yarn_frequencies(4, 10.0, {"factor": 2.0, "original": 7, "fast": 1.0, "slow": 1.0})
    assert g2[0] == 1.0 and g2[1] == pytest.approx(10.0 ** -0.5 / 2.0)


def test_turned_pairs_are_neighbours_and_scores_depend_on_the_distance_only():
    f, mult = [0.3, 0.05], 1.2
    x = torch.tensor([[1.0, 0.0, 0.0, 2.0, 9.0]], dtype=F)
    y = plain.turn_pairs(x, [5], f, mult)[0]
    assert y[0] == pytest.approx(mult * math.cos(1.5)) and y[1] == pytest.approx(mult * math.sin(1.5))
    assert y[2] == pytest.approx(-2.0 * mult * math.sin(0.25)) and y[3] == pytest.approx(2.0 * mult * math.cos(0.25))
    assert y[4] == 9.0
    g = torch.Generator().manual_seed(0)
    a, b = torch.randn(1, 4, generator=g, dtype=F), torch.randn(1, 4, generator=g, dtype=F)
    s1 = plain.turn_pairs(a, [7], f, mult) @ plain.turn_pairs(b, [3], f, mult).T
    s2 = plain.turn_pairs(a, [104], f, mult) @ plain.turn_pairs(b, [100], f, mult).T
    assert s1.item() == pytest.approx(s2.item())


def test_chunks_are_counted_from_the_start_and_values_are_the_raw_keys():
    g = torch.Generator().manual_seed(1)
    T, W, H, d = 9, 6, 2, 4
    h = torch.randn(T, W, generator=g, dtype=F)
    w = {"q": torch.randn(H * d, W, generator=g, dtype=F), "k": torch.randn(d, W, generator=g, dtype=F),
         "q.norm": torch.ones(H * d, dtype=F), "k.norm": torch.full((d,), 2.0, dtype=F),
         "o": torch.eye(H * d, dtype=F)}
    m = {"heads": H, "kv_heads": 1, "dim": d, "scale": 0.0, "mask": {"size": 4}}
    out = plain.tied_attention(h, w, m, 1e-6).view(T, H, d)
    k_raw = h @ w["k"].T
    # with a scale of zero every visible key weighs the same: the mean of the raw keys of the row's own chunk
    for t in range(T):
        lo = t - t % 4
        assert torch.allclose(out[t, 0], k_raw[lo:t + 1].mean(0)) and torch.allclose(out[t, 1], k_raw[lo:t + 1].mean(0))
    m2 = dict(m, scale=3.0, softcap=0.5)
    capped = plain.tied_attention(h, w, m2, 1e-6)
    m3 = dict(m, scale=3.0)
    assert not torch.allclose(capped, plain.tied_attention(h, w, m3, 1e-6))
    # a cap far above the scores changes nothing
    assert torch.allclose(plain.tied_attention(h, w, dict(m3, softcap=1e6), 1e-6), plain.tied_attention(h, w, m3, 1e-6))


def test_lightning_closed_form_for_constant_inputs():
    T, d, vd, decay = 7, 3, 2, 0.8
    h = torch.ones(T, 1, dtype=F)
    w = {"q": torch.full((d, 1), 1.0, dtype=F), "k": torch.full((d, 1), 2.0, dtype=F), "v": torch.full((vd, 1), -1.0, dtype=F),
         "g": torch.zeros(vd, 1, dtype=F), "norm": torch.ones(vd, dtype=F), "o": torch.eye(vd, dtype=F)}
    out = plain.lightning(h, w, {"heads": 1, "dim": d, "vdim": vd, "decay": [decay]}, 1e-12)
    # o_t = (sum_j decay^(t-j)) * (q . k) * v, the same in both value channels: after the norm it is +-1, times sigmoid(0)
    v = plain.silu(torch.tensor(-1.0, dtype=F))
    assert torch.allclose(out, torch.full((T, vd), 0.5 * math.copysign(1.0, v.item()), dtype=F), atol=1e-9)


def test_experts_only_from_the_best_groups():
    s = torch.tensor([0.05, 0.30, 0.02, 0.03, 0.25, 0.20, 0.10, 0.05], dtype=F)
    assert plain.route(s, 2, 1, 1) == [1, 4]
    assert plain.route(s, 3, 4, 2) == [1, 4, 5]                 # groups (0,1) and (4,5): 0.30 and 0.25
    assert plain.route(s, 2, 4, 1) == [1, 0]                    # only the group of the best expert
    assert sorted(plain.route(s, 4, 2, 1)) == [0, 1, 2, 3]      # the first half holds the best expert
    # the weights are the shares of the softmax over all experts, not renormalised
    h = torch.zeros(1, 3, dtype=F)
    w = {"router": torch.zeros(4, 3, dtype=F)}
    for e in range(4):
        w.update({f"e{e}.gate": torch.zeros(2, 3, dtype=F), f"e{e}.up": torch.zeros(2, 3, dtype=F), f"e{e}.down": torch.zeros(3, 2, dtype=F)})
    assert plain.moe_ff(h, w, {"router": {"experts": 4, "top": 2}}).abs().sum() == 0


def test_streams_with_identity_weights_are_the_plain_residual_sum():
    g = torch.Generator().manual_seed(2)
    S, T, W = 3, 5, 4
    x = torch.randn(T, W, generator=g, dtype=F)
    xs = torch.stack([x] * S)
    hc = {"in": torch.tensor([1.0, 0.0, 0.0], dtype=F), "out": torch.tensor([1.0, 0.0, 0.0], dtype=F), "mix": torch.eye(S, dtype=F)}
    f = lambda h: 2.0 * h
    new = plain.hyper_step(xs, hc, f, torch.ones(W, dtype=F), 1e-6)
    assert torch.allclose(new[0], x + 2.0 * plain.rms(x, 1e-6)) and torch.allclose(new[1], x) and torch.allclose(new[2], x)
    # the mixing matrix is indexed [from, to]
    hc["mix"] = torch.tensor([[1.0, 1.0, 0.0], [0.0, 1.0, 0.0], [0.0, 0.0, 1.0]], dtype=F)
    hc["out"] = torch.zeros(S, dtype=F)
    new = plain.hyper_step(torch.stack([x, 2 * x, 3 * x]), hc, f, torch.ones(W, dtype=F), 1e-6)
    assert torch.allclose(new[1], 3 * x) and torch.allclose(new[0], x)


def test_head_is_the_table_without_its_factor_and_limits_smoothly():
    x = torch.tensor([[3.0, 4.0]], dtype=F)
    table = torch.tensor([[1.0, 0.0], [0.0, 100.0]], dtype=F)
    z = plain.head(x, table, torch.ones(2, dtype=F), 1e-12, 2.0, 5.0)
    r = math.sqrt(12.5)
    assert z[0, 0].item() == pytest.approx(5.0 * math.tanh(2.0 * 3.0 / r / 5.0)) and z[0, 1].item() == pytest.approx(5.0, abs=1e-6)


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_configuration_round_trip_spec_and_caches(name):
    from swifttransformer_amd.config.pupalix_param import PupalixHyperParam
    from swifttransformer_amd.models import build_model
    cfg = tiny.CONFIGS[name]
    hp = PupalixHyperParam.from_dict(cfg)
    assert PupalixHyperParam.from_dict(hp.to_config_dict()) == hp
    assert hp.run_order() == plain.run_order(cfg)
    model = build_model(hp, torch.float32)
    w = tiny.make_weights(cfg, 0)
    specs = {s.name: tuple(s.shape) for s in model.tensor_specs() if not s.optional}
    assert specs == {k: tuple(v.shape) for k, v in w.items()}
    needs = model.cache_needs()
    runs = hp.run_order()
    assert [k for k in needs if isinstance(k, int)] == list(range(len(runs)))        # a cache or state a run of a layer
    assert (("embedding",) in needs) == bool(cfg["embedding"].get("bigram"))
    for run, i in enumerate(runs):
        kind = cfg["layers"][i]["type"]
        assert needs[run].kind == ("state" if kind == "lightning" else "paged_kv")
        if kind == "latent_attention":
            m = cfg["layers"][i]["mixer"]
            assert needs[run].num_kv_heads == 1 and needs[run].head_dim >= m["kv_rank"] + m["rot_dim"] and not needs[run].values
    assert model.streams == cfg.get("streams", 0)


def test_configuration_errors_name_the_key():
    from swifttransformer_amd.config.hyper_param import ConfigError
    from swifttransformer_amd.config.pupalix_param import PupalixHyperParam
    base = tiny.CONFIGS["A"]

    def broken(change):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError) as e:
            PupalixHyperParam.from_dict(cfg)
        return str(e.value)
    assert "layers[1].mixer.heads" in broken(lambda c: c["layers"][1]["mixer"].update(heads=3))
    assert "vdim" in broken(lambda c: c["layers"][1]["mixer"].update(vdim=8))
    assert "groups" in broken(lambda c: c["layers"][1]["mlp"]["router"].update(groups={"count": 4, "keep": 2}))
    assert "top" in broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=5))
    assert "decay" in broken(lambda c: c["layers"][2]["mixer"].update(decay=[0.5]))
    assert "loop" in broken(lambda c: c.update(loop={"start": 2, "stop": 2, "times": 1}))
    assert "type" in broken(lambda c: c["layers"][0].update(type="other"))
    assert "kind" in broken(lambda c: c["layers"][0]["mlp"].update(kind="sparse"))
    assert "rot_dim" in broken(lambda c: c["layers"][0]["mixer"].update(rot_dim=7))
    assert "buckets" in broken(lambda c: c["embedding"]["bigram"].update(buckets=0))
    assert "streams" in broken(lambda c: c.update(streams=0))


def test_a_layer_without_feed_forward_may_keep_its_second_norm_in_the_file():
    from swifttransformer_amd.config.pupalix_param import PupalixHyperParam
    from swifttransformer_amd.models import build_model
    from swifttransformer_amd.weights.loader import match_specs
    cfg = tiny.CONFIGS["A"]
    model = build_model(PupalixHyperParam.from_dict(cfg), torch.float32)
    shapes = {k: tuple(v.shape) for k, v in tiny.make_weights(cfg, 0).items()}
    match_specs(model.tensor_specs(), shapes)
    S, W = cfg["streams"], cfg["width"]
    shapes.update({"l2.norm2": (W,), "l2.hc2.in": (S,), "l2.hc2.out": (S,), "l2.hc2.mix": (S, S)})
    match_specs(model.tensor_specs(), shapes)
