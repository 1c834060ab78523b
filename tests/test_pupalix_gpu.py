"""Pupalix on the GPU against the plain implementation: each new or extended kernel alone, then the engine on
small models in float32 and bfloat16: every layer run, whole prompts, decoding through state and cache,
portions down to two tokens, unequal batches with slots and pages used again, first tokens, keys just inside
and just outside a chunk, page borders, keys far back, long decoding, greedy generation through ``Engine``,
the replay loop and a named size."""
import copy
import os

import numpy as np
import pytest
import torch

import plain_pupalix as plain
import tiny_pupalix as tiny
from test_zimorax_gpu import DEV, DTYPES, F64, check, dev, items_ctx, make_runner, rounded, run_schedule

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("S,W", [(1, 64), (3, 90), (4, 328), (5, 72), (8, 2048)])
def test_streams_read_write_expand_and_sum(dtype, S, W):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(S * 1000 + W)
    dt = DTYPES[dtype]
    T, eps = 11, 1e-5
    xs = torch.randn(S, T, W, generator=g, dtype=F64) * 3.0
    hc = {"in": torch.rand(S, generator=g, dtype=F64) + 0.2, "out": torch.randn(S, generator=g, dtype=F64),
          "mix": torch.eye(S, dtype=F64) + 0.3 * torch.randn(S, S, generator=g, dtype=F64)}
    hc2_in = torch.randn(S, generator=g, dtype=F64)
    gain, gain2 = 1.0 + 0.2 * torch.randn(W, generator=g, dtype=F64), 1.0 + 0.2 * torch.randn(W, generator=g, dtype=F64)
    x_dev = dev(xs.permute(1, 0, 2).reshape(T, S * W))
    f32 = lambda t: dev(t)
    u = torch.einsum("s,stw->tw", hc["in"], xs)
    check(K.streams_read(x_dev, f32(hc["in"]), f32(gain), eps, dt), (plain.rms(u, eps) * gain).numpy(), dt, "read")
    check(K.streams_read(x_dev, f32(hc["in"]), None, 0.0, torch.float32), u.numpy(), torch.float32, "read without norm")
    y = torch.randn(T, W, generator=g, dtype=F64) * 2.0
    new = plain.hyper_step(xs, hc, lambda h: y, torch.ones(W, dtype=F64), eps)
    x1 = x_dev.clone()
    assert K.streams_write(x1, f32(y), f32(hc["mix"]), f32(hc["out"])) is None
    check(x1, new.permute(1, 0, 2).reshape(T, S * W).numpy(), torch.float32, "write")
    x2 = x_dev.clone()
    nxt = K.streams_write(x2, f32(y), f32(hc["mix"]), f32(hc["out"]), then=(f32(hc2_in), f32(gain2), eps), out_dtype=dt)
    assert torch.equal(x1, x2)
    u2 = torch.einsum("s,stw->tw", hc2_in, new)
    check(nxt, (plain.rms(u2, eps) * gain2).numpy(), dt, "write and the next read")
    one = torch.randn(T, W, generator=g)
    ex = K.streams_expand(dev(one), S)
    assert torch.equal(ex.view(T, S, W).cpu(), one[:, None, :].expand(T, S, W))
    rows = torch.tensor([T - 1, -1, 0, 3], dtype=torch.int32, device=DEV)
    want = xs.sum(0)[[T - 1, 0, 0, 3]].numpy()
    want[1] = 0.0
    check(K.streams_sum(x_dev, S, rows), want, torch.float32, "sum of picked rows")
    check(K.streams_sum(x_dev, S), xs.sum(0).numpy(), torch.float32, "sum")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(53, 5, 11), (7, 1, 1), (1, 3, 2), (65521, 36313, 27191)])
def test_hashed_pair_embedding_carries_the_last_token_between_steps(dtype, buckets, mul_prev, mul_cur):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(buckets)
    dt = DTYPES[dtype]
    V, W, scale = 50000 if buckets > 1000 else 97, 40, 2.5
    table = rounded(torch.randn(V, W, generator=g), dtype)
    pairs = rounded(torch.randn(buckets + 1, W, generator=g), dtype)
    seqs = {3: torch.randint(0, V, (9,), generator=g).tolist(), 0: torch.randint(0, V, (6,), generator=g).tolist()}
    refs = {s: plain.embed(seq, table, scale, pairs, {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur})
            for s, seq in seqs.items()}
    state = torch.full((4, 1), 77, dtype=torch.int32, device=DEV)       # whatever a slot's last request left
    done = {3: 0, 0: 0}
    for step in ([(3, 4), (0, 1)], [(0, 2), (3, 1)], [(3, 4), (0, 3)]):
        ids, pos, lens, slots, want = [], [], [], [], []
        for slot, n in step:
            a = done[slot]
            ids += seqs[slot][a:a + n]
            pos += list(range(a, a + n))
            lens.append(n)
            slots.append(slot)
            want.append(refs[slot][a:a + n])
            done[slot] = a + n
        ids.append(5), pos.append(-1)                       # a padding row
        ti, il, off, sl = items_ctx(lens, slots)
        ti = torch.cat([ti, torch.tensor([-1], dtype=torch.int32, device=DEV)])
        mk = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
        got = K.hashed_embed(mk(ids), mk(pos), (ti, il, off, sl), state, dev(table, dt), dev(pairs, dt), mul_prev, mul_cur,
                             scale)
        check(got[:-1], torch.cat(want).numpy(), torch.float32, f"step {step}")
        assert float(got[-1].abs().max()) == 0.0
    assert state[3, 0].item() == seqs[3][-1] and state[0, 0].item() == seqs[0][-1] and state[1, 0].item() == 77
    got = K.hashed_embed(mk(ids), mk(pos), (ti, il, off, sl), None, dev(table, dt), None, 0, 0, scale)
    check(got[:-1], (table[torch.tensor(ids[:-1])] * scale).numpy(), torch.float32, "without a pair table")


def _paged(lens, ps, g):
    """Block tables over shuffled pages for requests of these lengths: (tables [B, width], pages)."""
    per = [-(-n // ps) for n in lens]
    num_pages = sum(per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    bt = torch.full((len(lens), max(per) + 2), -1, dtype=torch.int32)
    at = 0
    for b, n in enumerate(per):
        bt[b, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    return bt, num_pages


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("H,G,d,chunk,cap,ps", [(4, 2, 16, 12, 5.0, 4), (3, 3, 10, 0, 0.0, 2), (8, 1, 32, 64, 30.0, 16),
                                              (2, 1, 64, 100, 0.0, 16), (6, 2, 48, 7, 2.0, 8), (2, 2, 24, 1, 4.0, 4)])
def test_normed_queries_and_keys_into_pages_and_capped_chunked_attention_rows(dtype, H, G, d, chunk, cap, ps):
    """The norm over the whole projections, normalised keys and raw keys into their pools (in two portions, heads
    padded to the kernels' sizes), then every row's attention over its chunk through the row kernel with and
    without key splits, against the plain function of the same inputs."""
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(H * 100 + d + chunk)
    dt = DTYPES[dtype]
    lens, eps, scale = [150, 3, 67], 1e-5, 0.4
    pad = -(-d // 16) * 16
    bt, num_pages = _paged(lens, ps, g)
    k_cache = torch.full((num_pages, G, ps, pad), float("nan"), dtype=dt, device=DEV)
    v_cache = torch.full((num_pages, G, ps, pad), float("nan"), dtype=dt, device=DEV)
    gq, gk = 1.0 + 0.3 * torch.randn(H * d, generator=g), 1.0 + 0.3 * torch.randn(G * d, generator=g)
    outs, refs = [], []
    for b, n in enumerate(lens):
        qk = torch.randn(n, (H + G) * d + 5, generator=g) * 2.0          # rows wider than q and k: a slice of a product
        qs = []
        for a, e in ((0, n // 2), (n // 2, n)):                           # two portions
            if e == a:
                continue
            item = torch.full((e - a,), b, dtype=torch.int32, device=DEV)
            pos = torch.arange(a, e, dtype=torch.int32, device=DEV)
            qs.append(K.qk_norm_write(dev(qk)[a:e, :(H + G) * d], dev(gq), dev(gk), eps, H, G, d, k_cache, v_cache, item, pos,
                                      bt.to(DEV)))
        q_dev = torch.cat(qs)
        q64, k64 = qk[:, :H * d].to(F64), qk[:, H * d:(H + G) * d].to(F64)
        qn = (plain.rms(q64, eps) * gq.to(F64)).view(n, H, d)
        check(q_dev.view(n, H, pad)[:, :, :d].reshape(n, H * d), qn.reshape(n, H * d).numpy(), dt, f"queries of request {b}")
        assert float(q_dev.view(n, H, pad)[:, :, d:].abs().sum()) == 0.0
        # the plain attention on what the pools hold (rounded to the storage type)
        kn = rounded((plain.rms(k64, eps) * gk.to(F64)), dtype).view(n, G, d).repeat_interleave(H // G, dim=1)
        vv = rounded(k64, dtype).view(n, G, d).repeat_interleave(H // G, dim=1)
        s = torch.einsum("ihd,jhd->hij", rounded(qn, dtype), kn) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
        seen = (j <= i) & ((i // chunk == j // chunk) if chunk else True)
        refs.append(torch.einsum("hij,jhd->ihd", plain.softmax_rows(s, seen[None]), vv))
        outs.append(q_dev)
    q_all = torch.cat(outs)
    ti = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    pos = torch.tensor([p for n in lens for p in range(n)], dtype=torch.int32, device=DEV)
    ref = torch.cat(refs)
    for splits in (1, 3):
        got = K.attention_rows(q_all, k_cache, v_cache, ti, pos, bt.to(DEV), H, scale, window=-chunk, num_splits=splits,
                               softcap=cap)
        check(got.view(-1, H, pad)[:, :, :d].reshape(-1, H * d), ref.reshape(-1, H * d).numpy(), dt,
              f"rows, {splits} splits", loosen=2.0)
    # tiles of the matrix-core kernel over the same pools
    from swifttransformer_amd.parts.attention import plan_tiles
    from swifttransformer_amd.engine.batch import StepItem
    items = [StepItem(slot=b, start=0, tokens=[0] * n) for b, n in enumerate(lens)]
    plan = plan_tiles(items, 8)
    mk = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    off = np.concatenate([[0], np.cumsum(lens)[:-1]])
    out = torch.zeros_like(q_all)
    K.attention_prefill(q_all, k_cache, v_cache, mk(plan.arrays["tile_item"]), mk(plan.arrays["tile_q0"]), mk(off),
                        mk([0] * len(lens)), mk(lens), bt.to(DEV), H, scale, window=-chunk, out=out, softcap=cap)
    long_rows = [t for t, b in enumerate(ti.tolist()) if lens[b] >= 8]
    check(out[long_rows].view(-1, H, pad)[:, :, :d].reshape(-1, H * d), ref[long_rows].reshape(-1, H * d).numpy(), dt,
          "tiles", loosen=2.0)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("E,top,groups,keep,W,F", [(6, 2, 3, 2, 64, 24), (8, 4, 4, 3, 72, 20), (5, 5, 1, 1, 40, 50), (8, 1, 4, 1, 128, 40),
                                                  (12, 3, 2, 1, 64, 16)])
def test_experts_chosen_within_the_best_groups_and_weighted_by_the_softmax_over_all(dtype, E, top, groups, keep, W, F):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(E * 10 + top)
    dt = DTYPES[dtype]
    T = 37
    x = rounded(torch.randn(T, W, generator=g), dtype)
    w = {f"e{e}.{n}": rounded(torch.randn(*shape, generator=g) / shape[1] ** 0.5, dtype)
         for e in range(E) for n, shape in (("gate", (F, W)), ("up", (F, W)), ("down", (W, F)))}
    # logits a permutation of well separated levels a row: no choice is a close call
    logits = torch.stack([torch.randperm(E, generator=g).to(torch.float32) * 0.37 for _ in range(T)])
    ref = torch.zeros(T, W, dtype=F64)
    s = torch.softmax(logits.to(F64), dim=-1)
    for t in range(T):
        for e in plain.route(s[t], top, groups, keep):
            h = x[t]
            ref[t] += s[t, e] * ((plain.silu(h @ w[f"e{e}.gate"].T) * (h @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T)
    stack = lambda n: dev(torch.stack([w[f"e{e}.{n}"] for e in range(E)]), dt)
    item = torch.zeros(T, dtype=torch.int32, device=DEV)
    got = K.routed_experts(dev(x, dt), dev(logits), stack("gate"), stack("up"), stack("down"), None, top=top,
                           token_item=item, style="softmax_all", groups=groups, keep=keep)
    check(got, ref.numpy(), dt, "experts of the best groups", loosen=2.0)
    base = torch.randn(T, W, generator=g)
    got = K.routed_experts(dev(x, dt), dev(logits), stack("gate"), stack("up"), stack("down"), dev(base), top=top,
                           token_item=item, style="softmax_all", groups=groups, keep=keep)
    check(got, (ref + base.to(F64)).numpy(), dt, "onto a stream", loosen=2.0)


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_norm_over_all_heads_with_a_sigmoid_gate_the_limit_on_logits_and_a_scaled_turned_tail(dtype):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(4)
    dt = DTYPES[dtype]
    T, W = 9, 90
    o, gate = torch.randn(T, W, generator=g) * 3.0, rounded(torch.randn(T, W, generator=g), dtype)
    gain = 1.0 + 0.2 * torch.randn(W, generator=g)
    got = K.gated_group_norm(dev(o), dev(gate, dt), dev(gain), 1, 1e-5, dt, gate_kind="sigmoid")
    check(got, (plain.rms(o.to(F64), 1e-5) * gain.to(F64) * torch.sigmoid(gate)).numpy(), dt, "norm over all heads, sigmoid gate")
    got = K.gated_group_norm(dev(o), dev(gate, dt), dev(gain[:30]), 3, 1e-5, dt)
    want = plain.rms(o.to(F64).view(T, 3, 30), 1e-5) * gain[:30].to(F64) * plain.silu(gate).view(T, 3, 30)
    check(got, want.reshape(T, W).numpy(), dt, "norm a head, silu gate")
    z = torch.randn(T, W, generator=g) * 20.0
    check(K.scale_softcap(dev(z).clone(), 1.5, 8.0), (8.0 * torch.tanh(z.to(F64) * 1.5 / 8.0)).numpy(), torch.float32, "limit")
    check(K.scale_softcap(dev(z).clone(), 0.5, 0.0), (z.to(F64) * 0.5).numpy(), torch.float32, "factor alone")
    # the latent write with a tail whose cosine and sine carry a factor
    rank, tail, entry, ps = 20, 8, 32, 4
    x = torch.randn(T, rank + tail, generator=g)
    f2, mult = plain.yarn_frequencies(tail, 30.0, {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0})
    assert mult > 1.1
    cache = torch.full((5, 1, ps, entry), float("nan"), dtype=dt, device=DEV)
    bt = torch.tensor([[3, 1, 4, 0]], dtype=torch.int32, device=DEV)
    pos = torch.tensor([0, 1, 2, 3, 4, 5, 13, 14, 15], dtype=torch.int32)
    K.latent_write(cache, dev(x), dev(gain[:rank]), 1e-4, torch.zeros(T, dtype=torch.int32, device=DEV), pos.to(DEV), bt,
                   tail=tail, tail_freq=dev(torch.tensor(f2)), tail_mult=mult)
    turned = plain.turn_pairs(x[:, rank:].to(F64), pos.tolist(), f2, mult)
    pages = [3, 1, 4, 0]
    for t in range(T):
        got = cache[pages[int(pos[t]) // ps], 0, int(pos[t]) % ps]
        check(got[None, rank:rank + tail], turned[t][None].numpy(), dt, f"tail of token {t}")


# ------------------------------------------------------------------ the engine on small models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("pupalix")
    out = {}
    for name, cfg in tiny.CONFIGS.items():
        d = tiny.write_folder(cfg, str(root / name), 13)
        out[name] = (d,) + plain.load_folder(d)
    return out


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_every_layer_run_against_the_plain_residual_stream(models, name, dtype):
    from swifttransformer_amd.engine.batch import pack_batch
    from swifttransformer_amd.engine.step import StepEntry
    from swifttransformer_amd.ops import kernels as K
    folder, cfg, w = models[name]
    seq = tiny.prompt(23, cfg["vocab"], 1)
    want = plain.residual_streams(cfg, w, seq)
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 8 + 23 // ps, record_after=0)
    model = runner.model
    runner.admit(0)
    items = runner.prepare([StepEntry(0, seq, [])])
    ctx = pack_batch(items, runner.paged_group_ids, runner.max_pages_per_seq, ps, DEV, vocab_size=cfg["vocab"],
                     max_positions=model.max_positions, planners=runner.planners)
    seen = []
    for layer in model.layers:
        arr, orig = layer.arrangement, layer.arrangement.forward

        def fwd(x32, *a, _orig=orig, **kw):
            out = _orig(x32, *a, **kw)
            seen.append(K.streams_sum(out, model.streams).clone() if model.streams else out.clone())
            return out
        arr.forward = fwd
    model.forward_layers(ctx, runner.cache.views)
    assert len(seen) == want.shape[0] == len(plain.run_order(cfg))
    for run, got in enumerate(seen):
        check(got, want[run].numpy(), DTYPES[dtype], f"{name} {dtype} after run {run}", loosen=2.0)


@pytest.mark.parametrize("recording", [0, 2])
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_whole_decoded_and_in_portions(models, name, dtype, recording):
    folder, cfg, w = models[name]
    seq = tiny.prompt(150, cfg["vocab"], 2)
    ref = plain.logits(cfg, w, seq).numpy()
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, -(-150 // ps) + 2, record_after=recording)
    what = f"{name} {dtype}"
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 150)]], dtype, what + " whole", loosen=2.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 90)]] + [[(0, 1)]] * 60, dtype, what + " decoded", loosen=2.0)
    run_schedule(runner, {0: seq[:40]}, {0: ref[:40]}, [[(0, 1)]] * 40, dtype, what + " token by token", loosen=2.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, n)] for n in (11, 2, 13, 64, 3, 2, 40, 15)], dtype, what + " portions",
                 loosen=2.0)
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_first_tokens_and_unequal_batches_with_slots_and_pages_used_again(models, name, dtype):
    folder, cfg, w = models[name]
    lens = {0: 70, 1: 1, 2: 33, 3: 9, 4: 26, 5: 2, 6: 41}
    seqs = {r: tiny.prompt(n, cfg["vocab"], 10 + r) for r, n in lens.items()}
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 3 * (-(-70 // ps)) + 4, record_after=2, max_seqs=3)
    schedule = [[(0, 30), (1, 1), (2, 2)],              # a request of one token ends at once: its slot comes back
                [(2, 1), (0, 2), (3, 9)],               # a new request in the freed slot beside portions
                [(0, 1), (2, 30)],                      # request 2 ends
                [(4, 13), (0, 1)], [(0, 36), (4, 1)],   # request 0 ends
                [(5, 1), (4, 12), (6, 3)], [(5, 1), (6, 2)], [(6, 36)]]
    run_schedule(runner, seqs, refs, schedule, dtype, f"{name} {dtype} mixed", loosen=2.0)
    assert runner.manager.num_free_slots == 3
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)


def _single_layer(cfg0, w0, index, tmp_path, change):
    """A model made of layer ``index`` of ``cfg0`` alone (as its layer 0), without feed-forward and passes."""
    cfg = copy.deepcopy(cfg0)
    cfg["layers"] = [dict(cfg["layers"][index], mlp=None)]
    cfg.pop("loop", None)
    change(cfg["layers"][0]["mixer"])
    pre = f"l{index}."
    w = {("l0." + k[len(pre):] if k.startswith(pre) else k): v.to(torch.float32).clone() for k, v in w0.items()
         if (k.startswith(pre) and ".mlp." not in k and "norm2" not in k and ".hc2." not in k)
         or k in ("embed", "bigram") or k.startswith("final")}
    folder = tiny.write_folder(cfg, str(tmp_path / "peaked"), 0, weights=w)
    return (folder,) + plain.load_folder(folder)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("chunk,ps", [(12, 4), (64, 16), (100, 16), (33, 8), (0, 16)])
def test_peaked_attention_at_chunk_edges_page_borders_and_far_back(models, tmp_path, dtype, chunk, ps):
    """The attention with tied keys and values alone, its scores scaled up (and its cap raised) so that the
    softmax picks single keys: a key that is wrongly seen or wrongly missed moves the row.  The plain model's own
    parts say which key each query weighs most: among them must be the first key of a chunk, and a key just
    before a chunk must be what some query would weigh most if it saw it."""
    _, cfg0, w0 = models["A"]
    boost = 40.0 if dtype == "float32" else 6.0

    def change(m):
        m["scale"] = boost
        m["softcap"] = 3.0 * boost
        if chunk:
            m["mask"] = {"size": chunk}
        else:
            m.pop("mask", None)
    folder, cfg, w = _single_layer(cfg0, w0, 1, tmp_path, change)
    T = 330
    seq = tiny.prompt(T, cfg["vocab"], 5)
    ref = plain.logits(cfg, w, seq).numpy()
    c, eps, S = cfg["layers"][0]["mixer"], cfg["norm"]["eps"], cfg["streams"]
    e = plain.embed(seq, w["embed"], cfg["embedding"]["scale"], w["bigram"], cfg["embedding"]["bigram"])
    h = plain.rms(e * w["l0.hc1.in"].sum(), eps) * w["l0.norm1"]
    q = (plain.rms(h @ w["l0.mix.q"].T, eps) * w["l0.mix.q.norm"]).view(T, c["heads"], c["dim"])
    k = (plain.rms(h @ w["l0.mix.k"].T, eps) * w["l0.mix.k.norm"]).view(T, c["kv_heads"], c["dim"])
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    causal = j <= i
    seen = causal & ((i // chunk == j // chunk) if chunk else True)
    best, blind = [], []
    for head in range(c["heads"]):
        s = q[:, head] @ k[:, head // (c["heads"] // c["kv_heads"])].T
        best += [(r, int(s[r].masked_fill(~seen[r], float("-inf")).argmax())) for r in range(T)]
        blind += [(r, int(s[r].masked_fill(~causal[r], float("-inf")).argmax())) for r in range(T)]
    if chunk:
        assert any(b == r - r % chunk and r % chunk >= 3 for r, b in best), "no query weighs its chunk's first key most"
        assert any(b == r - r % chunk - 1 for r, b in blind), "no query would weigh the key just before its chunk most"
    else:
        assert max(r - b for r, b in best) > 150
    assert any(b % ps in (0, ps - 1) for _, b in best)
    runner = make_runner(folder, dtype, ps, -(-T // ps) + 2, record_after=2, max_seqs=2)
    loosen = 4.0
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, T)]], dtype, f"chunk {chunk} whole", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 230)]] + [[(0, 1)]] * 100, dtype, f"chunk {chunk} decoded", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 f"chunk {chunk} portions", loosen)
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_peaked_latent_attention_far_back_and_at_page_borders(models, tmp_path, dtype):
    _, cfg0, w0 = models["A"]
    boost = 8.0 if dtype == "float32" else 1.5

    def change(m):
        m["scale"] = m["scale"] * boost
    folder, cfg, w = _single_layer(cfg0, w0, 0, tmp_path, change)
    T, ps = 330, 16
    seq = tiny.prompt(T, cfg["vocab"], 6)
    ref = plain.logits(cfg, w, seq).numpy()
    c, eps = cfg["layers"][0]["mixer"], cfg["norm"]["eps"]
    H, d, r, R = c["heads"], c["dim"], c["rot_dim"], c["kv_rank"]
    e = plain.embed(seq, w["embed"], cfg["embedding"]["scale"], w["bigram"], cfg["embedding"]["bigram"])
    h = plain.rms(e * w["l0.hc1.in"].sum(), eps) * w["l0.norm1"]
    q = (h @ w["l0.mix.q"].T).view(T, H, d + r)
    down = h @ w["l0.mix.dkv"].T
    lat = plain.rms(down[:, :R], eps) * w["l0.mix.dkv.norm"]
    f, mult = plain.yarn_frequencies(r, c["rot"]["base"], c["rot"].get("scaling"))
    pos = list(range(T))
    k_rot = plain.turn_pairs(down[:, R:], pos, f, mult)
    k_plain = (lat @ w["l0.mix.uk"].T).view(T, H, d)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    best = []
    for n in range(H):
        q_rot = plain.turn_pairs(q[:, n, d:], pos, f, mult)
        s = (q[:, n, :d] @ k_plain[:, n].T + q_rot @ k_rot.T).masked_fill(j > i, float("-inf"))
        best += [(t, int(s[t].argmax())) for t in range(200, T)]
    assert max(t - b for t, b in best) > 150
    assert any(b % ps in (0, ps - 1) for _, b in best)
    runner = make_runner(folder, dtype, ps, -(-T // ps) + 2, record_after=2, max_seqs=2)
    loosen = 4.0
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 230)]] + [[(0, 1)]] * 100, dtype, "latent decoded", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 "latent portions", loosen)


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_long_portions_take_the_chunked_recurrence_and_short_ones_the_scan_on_one_state(models, dtype, monkeypatch):
    folder, cfg, w = models["C"]
    seq = tiny.prompt(200, cfg["vocab"], 7)
    ref = plain.logits(cfg, w, seq).numpy()
    ps = tiny.PAGE_SIZE["C"]
    from swifttransformer_amd.parts.retention import Retention
    monkeypatch.setattr(Retention, "chunked_from", 2)
    other = tiny.prompt(30, cfg["vocab"], 8)
    refs = {0: ref, 1: plain.logits(cfg, w, other).numpy()}
    runner = make_runner(folder, dtype, ps, -(-200 // ps) + -(-30 // ps) + 2, record_after=2)
    schedule = [[(0, 2), (1, 20)], [(1, 1), (0, 65)], [(0, 3), (1, 1)], [(1, 1), (0, 64)], [(0, 16), (1, 7)]] + [[(0, 1)]] * 50
    run_schedule(runner, {0: seq, 1: other}, refs, schedule, dtype, f"C {dtype} mixed", loosen=2.0)


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


def test_a_request_that_loses_its_pages_starts_again_from_cleared_state(models):
    """A pool that cannot hold the requests together: the scheduler takes pages back from a running request, which is
    computed again later in a slot that held another request's recurrent state and last token."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    folder, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab"], 70 + i) for i, n in enumerate((30, 26, 21, 5))]
    sp = SamplingParams(max_new_tokens=20, ignore_eos=True)
    tight = Engine(folder, dtype="fp32", page_size=4, num_pages=19, max_seqs=2, max_batched_tokens=64, prefill_chunk=9)
    outs = tight.generate(prompts, sp)
    assert tight.stats.preemptions >= 1, "the pool was meant to run out"
    for p, o in zip(prompts, outs):
        assert o == plain.generate(cfg, w, p, 20), f"prompt of {len(p)} tokens"
    tight.runner.manager.check_invariants()
    assert tight.runner.manager.num_free_slots == 2


def test_trace_replay_command_line_and_a_named_size(models, tmp_path):
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
    hp = hyper_param_by_name("pupalix_125m", num_layers=4, vocab=211, max_positions=128, chunk=24)
    d = write_random_model(hp, str(tmp_path / "named"), seed=3)
    cfg3, w3 = plain.load_folder(d)
    seq = tiny.prompt(40, 211, 8)
    runner = make_runner(d, "float32", 16, 8)
    run_schedule(runner, {0: seq}, {0: plain.logits(cfg3, w3, seq).numpy()}, [[(0, 33)]] + [[(0, 1)]] * 7, "float32",
                 "named size", loosen=3.0)
