"""Gisedra on the GPU against the plain implementation: each new or extended kernel alone, then the engine on
small models in float32 and bfloat16: every layer run, whole prompts, decoding through state and cache,
portions down to two tokens, unequal batches with slots and pages used again, first tokens, keys just inside
and just outside a window, kept first tokens, page borders, keys far back, long decoding, greedy generation
through ``Engine``, the replay loop and a named size."""
import copy
import os

import numpy as np
import pytest
import torch

import plain_gisedra as plain
import tiny_gisedra as tiny
from test_zimorax_gpu import DEV, DTYPES, F64, check, dev, items_ctx, make_runner, rounded, run_schedule

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", list(DTYPES))
def test_dynamic_tanh_unit_add_and_row_add(dtype):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(1)
    T, W = 13, 70
    x = torch.randn(T, W, generator=g) * 2.0
    w, b, base = 1.0 + 0.2 * torch.randn(W, generator=g), 0.1 * torch.randn(W, generator=g), torch.randn(T, W, generator=g)
    alpha = torch.tensor([0.8])
    ref = plain.dynamic_tanh(x.to(F64), w.to(F64), b.to(F64), 0.8)
    dt = DTYPES[dtype]
    out_t, out32 = torch.empty(T, W, dtype=dt, device=DEV), torch.empty(T, W, device=DEV)
    K.dynamic_tanh(dev(x), dev(w), dev(b), dev(alpha), out_t=out_t, out_f32=out32)
    check(out32, ref.numpy(), torch.float32, "dynamic tanh")
    check(out_t, ref.numpy(), dt, "dynamic tanh, storage type")
    rows = torch.tensor([5, -1, 0, 12], dtype=torch.int32, device=DEV)          # picked rows, one skipped
    picked = torch.full((4, W), 3.0, device=DEV)
    K.dynamic_tanh(dev(x), dev(w), None, dev(alpha), rows=rows, out_f32=picked)
    want = plain.dynamic_tanh(x.to(F64), w.to(F64), 0.0, 0.8)[[5, 0, 0, 12]].numpy()
    want[1] = 3.0
    check(picked, want, torch.float32, "picked rows")
    onto = torch.empty(T, W, device=DEV)
    K.dynamic_tanh(dev(x), dev(w), dev(b), dev(alpha), out_f32=onto, base=dev(base))
    check(onto, (ref + base.to(F64)).numpy(), torch.float32, "onto a stream")
    y = torch.randn(T, W, generator=g) * 3.0
    got = K.unit_add(dev(base).clone(), dev(y), dev(w), 1e-3)
    check(got, (base.to(F64) + plain.unit_rms(y.to(F64), 1e-3) * w.to(F64)).numpy(), torch.float32, "unit add")
    check(K.row_add(dev(x), dev(base), dev(b)), (x + base + b).to(F64).numpy(), torch.float32, "row add")
    check(K.row_add(dev(x), None, dev(b)), (x + b).to(F64).numpy(), torch.float32, "row add without the second stream")
    a = torch.randn(T, W, generator=g)
    got = K.activation_multiply(dev(a, dt), dev(x, dt), "sigmoid")
    check(got, (torch.sigmoid(rounded(a, dtype)) * rounded(x, dtype)).numpy(), dt, "sigmoid gate")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_rotary_interleaved_from_an_offset_and_latent_write_with_a_turned_tail(dtype):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(2)
    dt = DTYPES[dtype]
    T, heads, hd, off, dims = 9, 3, 48, 20, 12
    pos = torch.tensor([0, 1, 2, 40, 41, 300, -1, 7, 1000], dtype=torch.int32)
    freq = torch.tensor(plain.rotary_frequencies(dims, 50.0), dtype=F64)
    q = rounded(torch.randn(T, heads, hd, generator=g, dtype=F64), dtype)
    ref = q.clone()
    ref[..., off:off + dims] = plain.rotate(q[..., off:off + dims], pos.clamp(min=0), freq.tolist(), True)
    ref[6] = q[6]                                        # a padding row stays as it is
    wide = torch.zeros(T, heads * hd + 8, dtype=dt, device=DEV)
    wide[:, :heads * hd] = q.reshape(T, -1).to(dt).to(DEV)
    K.rotary(wide[:, :heads * hd], None, hd, dev(freq), 1.0, pos.to(DEV), offset=off, interleaved=True)
    check(wide[:, :heads * hd], ref.reshape(T, -1).numpy(), dt, "interleaved rotation from an offset")
    # the latent write: rank 20 normalised, a tail of 8 turned, an entry of 32 with 4 cleared
    rank, tail, entry, ps = 20, 8, 32, 4
    x = torch.randn(T, rank + tail, generator=g)
    gain = 1.0 + 0.2 * torch.randn(rank, generator=g)
    f2 = plain.rotary_frequencies(tail, 30.0)
    cache = torch.full((5, 1, ps, entry), float("nan"), dtype=dt, device=DEV)
    bt = torch.tensor([[3, 1, 4, 0]], dtype=torch.int32, device=DEV)
    p2 = torch.tensor([0, 1, 2, 3, 4, 5, -1, 14, 15], dtype=torch.int32)
    item = torch.tensor([0] * 6 + [-1, 0, 0], dtype=torch.int32, device=DEV)
    K.latent_write(cache, dev(x), dev(gain), 1e-4, item, p2.to(DEV), bt, tail=tail, tail_freq=dev(torch.tensor(f2)))
    lat = plain.unit_rms(x[:, :rank].to(F64), 1e-4) * gain.to(F64)
    turned = plain.rotate(x[:, rank:].to(F64).view(T, 1, tail), p2.clamp(min=0), f2, True).view(T, tail)
    pages = [3, 1, 4, 0]
    for t in range(T):
        if t == 6:
            continue
        got = cache[pages[int(p2[t]) // ps], 0, int(p2[t]) % ps]
        want = torch.cat([lat[t], turned[t], torch.zeros(entry - rank - tail, dtype=F64)]).numpy()
        check(got[None], want[None], dt, f"entry of token {t}")
    K.latent_write(cache, dev(x), dev(gain), 1e-4, item, p2.to(DEV), bt, tail=tail)       # a tail that does not turn
    check(cache[3, 0, 1][None, rank:rank + tail], x[1, rank:][None].to(F64).numpy(), dt, "plain tail")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("W,dim,parts,index", [(64, 8, 3, 1), (72, 6, 2, 1), (100, 2, 1, 0), (2048, 16, 4, 3), (328, 20, 2, 0)])
def test_token_side_input_in_one_kernel(dtype, W, dim, parts, index):
    """Lookup, gate product, GELU, projection, unit norm and the sum into the stream: against the plain function, on
    columns of a wider table, with a padding row, a token outside the table and sizes that no vector load divides."""
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(W + dim)
    dt = DTYPES[dtype]
    T, V, eps = 11, 37, 1e-5
    x = torch.randn(T, W, generator=g) * 1.5
    tokens = torch.randint(0, V, (T,), generator=g)
    weights = {"side.embed": rounded(torch.randn(V, parts * dim, generator=g), dtype),
               f"l{index}.side.gate": rounded(torch.randn(dim, W, generator=g) / W ** 0.5, dtype),
               f"l{index}.side.proj": rounded(torch.randn(W, dim, generator=g) / dim ** 0.5, dtype),
               f"l{index}.side.norm": 0.5 + 0.1 * torch.randn(W, generator=g).to(F64)}
    ref = x.to(F64) + plain.side_input(x.to(F64), tokens, weights, index, dim, eps)
    ref[4] = x[4].to(F64)                       # a padding row stays as it is
    item = torch.zeros(T, dtype=torch.int32)
    item[4] = -1
    ids = tokens.to(torch.int32)
    ids[9] = V + 3                              # outside the table: gated with zeros, so y = 0 and x stays
    ref[9] = x[9].to(F64)
    table = dev(weights["side.embed"], dt)[:, index * dim:(index + 1) * dim]
    got = K.token_side(dev(x).clone(), ids.to(DEV), item.to(DEV), table, dev(weights[f"l{index}.side.gate"], dt),
                       dev(weights[f"l{index}.side.proj"], dt), dev(weights[f"l{index}.side.norm"]), eps)
    check(got, ref.numpy(), dt, f"token side input, width {W}, {dim} of {parts * dim} columns", loosen=2.0)


def plain_kept_window(q, k, v, scale, window, keep_first):
    T = q.shape[0]
    return plain.softmax_attention(q, k, v, scale, plain.visible(T, window, keep_first))


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("H,G,dk,dv,window,keep,ps", [
    (4, 2, 16, 24, 12, 3, 4), (3, 3, 10, 6, 70, 0, 2), (8, 1, 32, 32, 64, 70, 16), (2, 2, 48, 16, 9, 130, 8),
    (6, 3, 8, 40, 65, 64, 16), (1, 1, 24, 8, 1, 1, 4)])
def test_window_attention_that_keeps_the_first_tokens(dtype, H, G, dk, dv, window, keep, ps):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(H * 100 + dk)
    lens = [200, 3, 67]
    dt = DTYPES[dtype]
    pages_per = [-(-n // ps) for n in lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    k_cache = torch.full((num_pages, G, ps, dk), float("nan"), dtype=dt, device=DEV)
    v_cache = torch.full((num_pages, G, ps, dv), float("nan"), dtype=dt, device=DEV)
    bt = torch.full((len(lens), max(pages_per) + 2), -1, dtype=torch.int32)
    qs, refs, tok_item, positions = [], [], [], []
    nxt = 0
    for b, n in enumerate(lens):
        q = rounded(torch.randn(n, H, dk, generator=g, dtype=F64) * 1.5, dtype)
        k = rounded(torch.randn(n, G, dk, generator=g, dtype=F64), dtype)
        v = rounded(torch.randn(n, G, dv, generator=g, dtype=F64), dtype)
        # keys that stand out: the last kept one, the first that is not kept, and one in the middle
        for j in (keep - 1, keep, n // 2):
            if 0 <= j < n:
                k[j] *= 3.0
        refs.append(plain_kept_window(q, k, v, 0.3, window, keep).reshape(n, H * dv))
        pg = perm[nxt:nxt + pages_per[b]]
        nxt += pages_per[b]
        bt[b, :len(pg)] = torch.tensor(pg, dtype=torch.int32)
        for t in range(n):
            k_cache[pg[t // ps], :, t % ps] = k[t].to(dt).to(DEV)
            v_cache[pg[t // ps], :, t % ps] = v[t].to(dt).to(DEV)
        qs.append(q.reshape(n, H * dk))
        tok_item += [b] * n
        positions += list(range(n))
    q_all, ref = torch.cat(qs), torch.cat(refs).numpy()
    mk = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    for splits in (1, 3):
        out = K.sink_attention(dev(q_all, dt), k_cache, v_cache, mk(tok_item), mk(positions), bt.to(DEV), H, 0.3,
                               window=window, keep_first=keep, sink=False, num_splits=splits)
        check(out, ref, dt, f"kept window, {splits} splits", loosen=2.0 if dtype == "bfloat16" else 1.0)


@pytest.mark.parametrize("heads,kd,vd", [(2, 12, 20), (1, 5, 18), (4, 64, 16), (3, 32, 64)])
def test_retention_scan_with_constant_gates(heads, kd, vd):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(kd + vd)
    T = 41
    q, k, v = (torch.randn(T, heads * n, generator=g) for n in (kd, kd, vd))
    decay = [1.0, 0.5, 0.97, 0.9990234375][:heads]
    ref = torch.zeros(T, heads, vd, dtype=F64)
    S = torch.zeros(heads, kd, vd, dtype=F64)
    for h in range(heads):
        for t in range(T):
            S[h] = decay[h] * S[h] + torch.outer(k[t, h * kd:(h + 1) * kd].to(F64) * kd ** -0.5, v[t, h * vd:(h + 1) * vd].to(F64))
            ref[t, h] = S[h].T @ q[t, h * kd:(h + 1) * kd].to(F64)
    ref = ref.reshape(T, heads * vd).numpy()
    factor = torch.full((1, heads), kd ** -0.5, device=DEV)
    decays = torch.tensor([decay], dtype=torch.float32, device=DEV)
    for cuts in ([T], [1] * T, [2, 9, 1, 2, 20, 7]):
        state = torch.full((3, heads, kd, vd), float("nan"), device=DEV)
        state[2].zero_()
        outs, t0 = [], 0
        for n in cuts:
            outs.append(K.state_scan(dev(q[t0:t0 + n]), dev(k[t0:t0 + n]), dev(v[t0:t0 + n]), factor, decays, state,
                                     items_ctx([n], [2]), heads, "additive", max_item_rows=1 if n == 1 else 0))
            t0 += n
        check(torch.cat(outs), ref, torch.float32, f"retention cut {cuts[:3]}", loosen=3.0)
        check(state[2], S.numpy(), torch.float32, "final state", loosen=3.0)


@pytest.mark.parametrize("heads,kd,vd", [(2, 12, 20), (1, 5, 18), (4, 64, 16), (3, 32, 64), (2, 128, 40), (1, 200, 33),
                                         (4, 64, 128)])
def test_retention_in_chunks(heads, kd, vd):
    """The chunked kernels against the recurrence written out: unequal items in one launch (longer than a chunk, a
    chunk exactly, one row, a chunk and one row), an item that is skipped, states that are not zero, a request cut
    into portions at and off the chunks' borders, a decay of one and a fast one."""
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(3 * kd + vd)
    decay = [1.0, 0.5, 0.97, 0.9990234375][:heads]
    lens = [200, 64, 1, 65, 0, 130]
    slots = [3, 0, 5, 1, -1, 4]
    T = sum(lens)
    q, k, v = (torch.randn(T, heads * n, generator=g) for n in (kd, kd, vd))
    start = torch.randn(6, heads, kd, vd, generator=g)
    ref = torch.zeros(T, heads, vd, dtype=F64)
    S = start.to(F64).clone()
    t0 = 0
    for n, slot in zip(lens, slots):
        for h in range(heads):
            for t in range(t0, t0 + n):
                S[slot, h] = decay[h] * S[slot, h] + torch.outer(k[t, h * kd:(h + 1) * kd].to(F64) * kd ** -0.5,
                                                                 v[t, h * vd:(h + 1) * vd].to(F64))
                ref[t, h] = S[slot, h].T @ q[t, h * kd:(h + 1) * kd].to(F64)
        t0 += n
    ref = ref.reshape(T, heads * vd).numpy()
    decays = torch.tensor(decay, dtype=torch.float32, device=DEV)
    state = dev(start).clone()
    # q, k, v as columns of one wider tensor, as the mixer's product leaves them
    wide = torch.cat([q, k, v], dim=1).to(DEV)
    qk = heads * kd
    out = K.retention_chunks(wide[:, :qk], wide[:, qk:2 * qk], wide[:, 2 * qk:], decays, kd ** -0.5, state,
                             items_ctx(lens, slots), heads)
    check(out, ref, torch.float32, "items of unequal lengths", loosen=3.0)
    check(state, S.numpy(), torch.float32, "states after the launch", loosen=3.0)
    # one request in portions: every cut gives the recurrence's values
    n0 = lens[0]
    for cuts in ([n0], [64, 64, 72], [3, 61, 1, 70, 65]):
        state = dev(start).clone()
        outs, t0 = [], 0
        for n in cuts:
            outs.append(K.retention_chunks(dev(q[t0:t0 + n]), dev(k[t0:t0 + n]), dev(v[t0:t0 + n]), decays, kd ** -0.5,
                                           state, items_ctx([n], [3]), heads))
            t0 += n
        check(torch.cat(outs), ref[:n0], torch.float32, f"portions {cuts}", loosen=3.0)
        check(state[3], S[3].numpy(), torch.float32, f"state after portions {cuts}", loosen=3.0)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("T,E,top,W,F", [(5, 4, 2, 64, 24), (70, 3, 3, 72, 20), (9, 5, 1, 72, 50), (700, 8, 2, 128, 40)])
def test_experts_weighted_by_the_softmax_over_the_chosen(dtype, T, E, top, W, F):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(T + E)
    dt = DTYPES[dtype]
    x = rounded(torch.randn(T, W, generator=g, dtype=F64), dtype)
    names = {f"m.e{e}.{n}": rounded(torch.randn(*s, generator=g, dtype=F64) * s[1] ** -0.5, dtype)
             for e in range(E) for n, s in (("gate", (F, W)), ("up", (F, W)), ("down", (W, F)))}
    # logits with wide gaps, so that the choice rests on no close call; one row is a padding row
    logits = torch.stack([torch.randperm(E, generator=g).to(F64) * 0.7 for _ in range(T)]) + 0.1 * torch.randn(T, E, generator=g, dtype=F64)
    logits = logits.to(torch.float32)
    names["m.router"], names["m.router.b"] = torch.zeros(E, W, dtype=F64), torch.zeros(E, dtype=F64)
    ref = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        best = sorted(range(E), key=lambda e: (-float(logits[t, e]), e))[:top]
        wts = torch.softmax(logits[t, best].to(F64), dim=0)
        for wi, e in zip(wts, best):
            y = plain.silu(names[f"m.e{e}.gate"] @ x[t]) * (names[f"m.e{e}.up"] @ x[t])
            ref[t] += wi * (names[f"m.e{e}.down"] @ y)
    item = torch.zeros(T, dtype=torch.int32)
    item[T // 2] = -1
    ref[T // 2] = 0.0
    stack = lambda n: dev(torch.stack([names[f"m.e{e}.{n}"] for e in range(E)]), dt)
    got = K.routed_experts(dev(x, dt), dev(logits), stack("gate"), stack("up"), stack("down"), None, top=top,
                           token_item=item.to(DEV), style="softmax_output")
    check(got, ref.numpy(), dt, "the weighted sum alone", loosen=2.0 if dtype == "bfloat16" else 1.0)
    res = torch.randn(T, W, generator=g)
    got = K.routed_experts(dev(x, dt), dev(logits), stack("gate"), stack("up"), stack("down"), dev(res), top=top,
                           token_item=item.to(DEV), style="softmax_output", out_scale=0.5)
    check(got, (res.to(F64) + 0.5 * ref).numpy(), dt, "onto a stream", loosen=2.0 if dtype == "bfloat16" else 1.0)


# ------------------------------------------------------------------ the engine on small models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("gisedra")
    out = {}
    for name, cfg in tiny.CONFIGS.items():
        d = tiny.write_folder(cfg, str(root / name), 11)
        out[name] = (d,) + plain.load_folder(d)
    return out


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_every_layer_run_against_the_plain_residual_stream(models, name, dtype):
    from swifttransformer_amd.engine.step import StepEntry
    folder, cfg, w = models[name]
    seq = tiny.prompt(23, cfg["vocab"], 1)
    want = plain.residual_streams(cfg, w, seq)
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 8 + 23 // ps, record_after=0)
    seen = []
    for layer in runner.model.layers:
        inner = layer.arrangement.forward

        def spy(*a, _inner=inner, **k):
            out = _inner(*a, **k)
            seen.append(out.detach().clone())
            return out
        layer.arrangement.forward = spy
    runner.admit(0)
    runner.step([StepEntry(0, seq, [])])
    assert len(seen) == len(want) == len(runner.model.schedule)
    for run, (got, ref) in enumerate(zip(seen, want)):
        check(got, ref.numpy(), DTYPES[dtype], f"{name} run {run}", loosen=2.0 if dtype == "float32" else 4.0)


@pytest.mark.parametrize("recording", [2, 1])
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_whole_decoded_and_in_portions(models, name, dtype, recording):
    folder, cfg, w = models[name]
    seq = tiny.prompt(61, cfg["vocab"], 3)
    ref = plain.logits(cfg, w, seq).numpy()
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, -(-61 // ps) + 1, record_after=recording)
    what = f"{name} {dtype} recording {recording}"
    for k in range(2):                                # twice: the second time on slots and pages used before
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, 61)]], dtype, what + " whole")
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, 27)]] + [[(0, 1)]] * 34, dtype, what + " decoded")
        portions = [2, 3, 2, 9, 1, 2, 17, 2, 5, 1, 1, 2, 14]
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, n)] for n in portions], dtype, what + " portions")
    if recording == 1:
        assert runner.graph_replays == runner.steps_run, "a step ran unrecorded"


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_first_tokens_and_unequal_batches_with_slots_and_pages_used_again(models, name, dtype):
    folder, cfg, w = models[name]
    lens = {"a": 1, "b": 2, "c": 3, "d": 40, "e": 9, "f": 33, "g": 5}
    seqs = {r: tiny.prompt(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 4 * (-(-40 // ps)), record_after=2)
    schedule = [[("a", 1), ("d", 7), ("b", 1)],                    # first tokens beside a portion
                [("b", 1), ("d", 2), ("c", 2)],
                [("c", 1), ("d", 1), ("e", 9), ("f", 3)],           # a and b have ended: their slots go to e and f
                [("d", 20), ("f", 1)],
                [("f", 2), ("d", 1), ("g", 2)],
                [("d", 9), ("g", 1), ("f", 17)],
                [("g", 2), ("f", 10)]]
    run_schedule(runner, seqs, refs, schedule, dtype, f"{name} {dtype} mixed")
    assert runner.manager.num_free_slots == 4
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)
    run_schedule(runner, seqs, refs, [[("d", 40)], [("f", 33)]], dtype, f"{name} {dtype} alone")


def _single_layer(cfg0, w0, index, tmp_path, boost_names, boost, change):
    """A model made of layer ``index`` of ``cfg0`` alone (as its layer 0), without feed-forward, token input
    and passes, its query matrices scaled up so that the softmax picks single keys."""
    cfg = copy.deepcopy(cfg0)
    cfg["layers"] = [dict(cfg["layers"][index], mlp=None)]
    cfg.pop("loop", None)
    cfg.pop("token_side", None)
    change(cfg["layers"][0]["mixer"])
    pre = f"l{index}."
    w = {("l0." + k[len(pre):] if k.startswith(pre) else k): v.to(torch.float32).clone() for k, v in w0.items()
         if (k.startswith(pre) and ".mlp." not in k and ".side." not in k and "norm2" not in k)
         or k in ("embed", "head") or k.startswith("final")}
    for n in boost_names:
        w[n] *= boost
    folder = tiny.write_folder(cfg, str(tmp_path / "peaked"), 0, weights=w)
    return (folder,) + plain.load_folder(folder)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("window,keep", [(12, 3), (64, 20), (100, 0), (0, 0)])
def test_peaked_window_attention_at_its_edges_kept_tokens_page_borders_and_far_back(models, tmp_path, dtype, window, keep):
    """The left attention alone with scaled-up queries: a key that is wrongly seen or wrongly missed moves the
    row.  The plain model's own parts say which key each late query weighs most; among them must be the
    oldest key of the window, kept first tokens far behind the window, page borders and (without a window)
    keys hundreds of tokens back."""
    _, cfg0, w0 = models["A"]
    boost = 6.0 if dtype == "float32" else 0.6

    def change(m):
        m["right_scale"] = 0.05                      # the retention stays in, small
        if window:
            m["left"]["mask"] = {"size": window, "keep_first": keep}
        else:
            del m["left"]["mask"]
    folder, cfg, w = _single_layer(cfg0, w0, 1, tmp_path, ["l0.mix.left.q"], boost, change)
    T, ps = 330, 16
    seq = tiny.prompt(T, cfg["vocab"], 5)
    ref = plain.logits(cfg, w, seq).numpy()
    c = cfg["layers"][0]["mixer"]["left"]
    h = plain.dynamic_tanh(w["embed"][torch.tensor(seq)], w["l0.norm1"], w["l0.norm1.b"], w["l0.norm1.alpha"])
    q, k = (plain.causal_filter(h @ w[f"l0.mix.left.{n}"].T, w[f"l0.mix.left.{n}.conv"]) for n in "qk")
    f = plain.rotary_frequencies(c["rot"]["dims"], c["rot"]["base"], c["rot"].get("scaling"))
    pos = torch.arange(T)
    q = plain.rotate(q.view(T, c["heads"], c["dim"]), pos, f, False)
    k = plain.rotate(k.view(T, c["kv_heads"], c["dim"]), pos, f, False)
    seen = plain.visible(T, window, keep)
    best = []
    for head in range(c["heads"]):
        s = (q[:, head] @ k[:, head // (c["heads"] // c["kv_heads"])].T).masked_fill(~seen, float("-inf"))
        best += [(i, int(s[i].argmax())) for i in range(200, T)]
    gaps = [i - b for i, b in best]
    if window:
        assert window - 1 in gaps, "no query weighs the oldest key of its window most"
        if keep:
            assert any(b < keep for i, b in best), "no late query weighs a kept first token most"
    else:
        assert max(gaps) > 150
    assert any(b % ps in (0, ps - 1) for _, b in best)
    # with a short window the pool is too small for the whole sequence: pages behind the window must come back
    # while the request is live, except those of the kept tokens
    pages = -(-(window + 230) // ps) + 2 + -(-keep // ps) if window else -(-T // ps) + 2
    runner = make_runner(folder, dtype, ps, pages, record_after=2, max_seqs=2)
    loosen = max(boost, 1.0) * (2.0 if dtype == "bfloat16" else 1.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 230)]] + [[(0, 1)]] * 100, dtype, f"window {window} decoded", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 f"window {window} portions", loosen)
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("window", [9, 64, 0])
def test_peaked_latent_attention_at_window_edges_page_borders_and_far_back(models, tmp_path, dtype, window):
    _, cfg0, w0 = models["A"]
    boost = 6.0 if dtype == "float32" else 0.6

    def change(m):
        if window:
            m["mask"] = {"size": window}
        else:
            m.pop("mask", None)
    folder, cfg, w = _single_layer(cfg0, w0, 0, tmp_path, ["l0.mix.q"], boost, change)
    T, ps = 330, 16
    seq = tiny.prompt(T, cfg["vocab"], 6)
    ref = plain.logits(cfg, w, seq).numpy()
    c = cfg["layers"][0]["mixer"]
    H, d, r, R = c["heads"], c["dim"], c["rot_dim"], c["kv_rank"]
    h = plain.dynamic_tanh(w["embed"][torch.tensor(seq)], w["l0.norm1"], w["l0.norm1.b"], w["l0.norm1.alpha"])
    q = (h @ w["l0.mix.q"].T).view(T, H, d + r)
    down = h @ w["l0.mix.dkv"].T
    lat = plain.unit_rms(down[:, :R], cfg["norm"]["eps"]) * w["l0.mix.dkv.norm"]
    f = plain.rotary_frequencies(r, c["rot"]["base"])
    pos = torch.arange(T)
    k_rot, q_rot = plain.rotate(down[:, R:].view(T, 1, r), pos, f, True), plain.rotate(q[..., d:], pos, f, True)
    k_plain = (lat @ w["l0.mix.uk"].T).view(T, H, d)
    seen = plain.visible(T, window)
    best = []
    for n in range(H):
        s = (q[:, n, :d] @ k_plain[:, n].T + q_rot[:, n] @ k_rot[:, 0].T).masked_fill(~seen, float("-inf"))
        best += [(i, int(s[i].argmax())) for i in range(200, T)]
    gaps = [i - b for i, b in best]
    if window:
        assert window - 1 in gaps, "no query weighs the oldest key of its window most"
    else:
        assert max(gaps) > 150
    assert any(b % ps in (0, ps - 1) for _, b in best)
    pages = -(-(window + 230) // ps) + 2 if window else -(-T // ps) + 2
    runner = make_runner(folder, dtype, ps, pages, record_after=2, max_seqs=2)
    loosen = max(boost, 1.0) * (2.0 if dtype == "bfloat16" else 1.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 230)]] + [[(0, 1)]] * 100, dtype, f"latent window {window} decoded", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 f"latent window {window} portions", loosen)
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)


def test_the_step_that_is_recorded_gives_its_own_result_also_where_its_tensors_left_the_arena(models, dtype="float32"):
    """A step's bucket of rows may be larger than the most tokens the runner was built for, and a tensor that
    does not fit the arena comes from the ordinary allocator: the batch whose step is recorded must read the
    result of its own run, not the recording's untouched memory."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.batch import token_bucket
    from swifttransformer_amd.engine.step import ModelRunner
    from swifttransformer_amd.models import load_model
    folder, cfg, w = models["A"]
    seqs = {0: tiny.prompt(70, cfg["vocab"], 21), 1: tiny.prompt(66, cfg["vocab"], 22)}      # one bucket: 128 rows
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    ps = tiny.PAGE_SIZE["A"]
    model = load_model(folder, DTYPES[dtype], DEV)
    runner = ModelRunner(model, CacheParam(page_size=ps, num_pages=40, max_seqs=4), DEV, record_after=2, max_batched_tokens=70)
    assert runner.arena_rows == token_bucket(70) == 128
    run_schedule(runner, seqs, refs, [[(0, 70)], [(1, 66)], [(0, 70)], [(1, 66)]], dtype, f"{dtype} in the arena")
    assert runner.arena.overflows == 0 and runner.graph_replays == 3
    # nothing fits: every tensor of the first run and of the recording comes from elsewhere
    runner = ModelRunner(model, CacheParam(page_size=ps, num_pages=40, max_seqs=4), DEV, record_after=2, max_batched_tokens=70)
    runner.arena.resize(256)
    run_schedule(runner, seqs, refs, [[(0, 70)], [(1, 66)], [(0, 70)], [(1, 66)]], dtype, f"{dtype} outside the arena")
    assert runner.arena.overflows > 0 and runner.graph_replays == 3


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_long_portions_take_the_chunked_retention_and_short_ones_the_scan_on_one_state(models, name, dtype, monkeypatch):
    folder, cfg, w = models[name]
    seq = tiny.prompt(150, cfg["vocab"], 7)
    ref = plain.logits(cfg, w, seq).numpy()
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, -(-150 // ps) + 2, record_after=2)
    what = f"{name} {dtype}"
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 150)]], dtype, what + " whole", loosen=2.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 100)]] + [[(0, 1)]] * 50, dtype, what + " decoded", loosen=2.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, n)] for n in (70, 3, 64, 13)], dtype, what + " portions", loosen=2.0)
    # every step with a portion in chunks, down to two rows, beside single tokens of another request
    from swifttransformer_amd.parts.retention import Retention
    monkeypatch.setattr(Retention, "chunked_from", 2)
    other = tiny.prompt(30, cfg["vocab"], 8)
    refs = {0: ref, 1: plain.logits(cfg, w, other).numpy()}
    runner = make_runner(folder, dtype, ps, -(-150 // ps) + -(-30 // ps) + 2, record_after=2)
    schedule = [[(0, 2), (1, 20)], [(1, 1), (0, 65)], [(0, 3), (1, 1)], [(1, 1), (0, 64)], [(0, 16), (1, 7)]]
    run_schedule(runner, {0: seq, 1: other}, refs, schedule, dtype, what + " mixed", loosen=2.0)


def test_greedy_generation_through_the_engine(models):
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    folder, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab"], 40 + i) for i, n in enumerate((1, 7, 19, 30, 4, 12))]
    eng = Engine(folder, dtype="fp32", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain.generate(cfg, w, p, 12), f"prompt of {len(p)} tokens"
    assert eng.runner.manager.num_free_slots == 3
    # bfloat16: every chosen token is the plain model's best for the engine's own sequence, up to rounding
    eng = Engine(folder, dtype="bf16", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts[:3], SamplingParams(max_new_tokens=8, ignore_eos=True))
    for p, o in zip(prompts, outs):
        logits = plain.logits(cfg, w, list(p) + list(o)).numpy()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert row.max() - row[tok] <= 0.05 * row.std() + 0.02 * abs(row.max())


def test_trace_replay_command_line_and_a_named_size(models, tmp_path):
    import io
    import json
    import subprocess
    import sys
    folder, cfg, w = models["B"]
    seqs = {"x": tiny.prompt(21, cfg["vocab"], 60), "y": tiny.prompt(9, cfg["vocab"], 61)}
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": seqs["x"][:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": seqs["y"][:8], "want": []},
                                     {"id": "x", "tokens": seqs["x"][13:15], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": seqs["x"][15:], "want": [5]},
                                     {"id": "y", "tokens": seqs["y"][8:], "want": [0]}], "end": ["x", "y"]}]
    out = str(tmp_path / "out")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", out, "--max-tokens", "64", "--page-size", "2"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = cfg["vocab"]
    got = {n: np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4").reshape(-1, V) for n in (0, 1, 2)}
    check(torch.from_numpy(got[0]), refs["x"][[0, 12]], torch.float32, "step 0")
    check(torch.from_numpy(got[1]), refs["x"][[14]], torch.float32, "step 1")
    check(torch.from_numpy(got[2]), np.stack([refs["x"][20], refs["y"][8]]), torch.float32, "step 2")
    inp = tmp_path / "prompts.txt"
    inp.write_text(" ".join(map(str, seqs["y"])) + "\n")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "run_opt"), folder, "auto", "fp32", str(inp),
                        "--max-new-tokens", "5", "--ignore-eos", "--block-size", "2", "--num-blocks", "64", "--max-seqs", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = plain.generate(cfg, w, seqs["y"], 5)
    assert ")" + "".join(f"{t} " for t in want) in r.stdout
    # a named size with random weights, from its folder: the same logits as the plain model
    from swifttransformer_amd.config.registry import hyper_param_by_name
    from swifttransformer_amd.weights import write_random_model
    hp = hyper_param_by_name("gisedra_125m", num_layers=4, vocab=211, max_positions=128, window=24)
    d = write_random_model(hp, str(tmp_path / "named"), seed=3)
    cfg3, w3 = plain.load_folder(d)
    seq = tiny.prompt(40, 211, 8)
    runner = make_runner(d, "float32", 16, 8)
    run_schedule(runner, {0: seq}, {0: plain.logits(cfg3, w3, seq).numpy()}, [[(0, 33)]] + [[(0, 1)]] * 7, "float32",
                 "named size")
