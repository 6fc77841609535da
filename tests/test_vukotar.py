"""Vukotar on the engine against the plain float64 oracle (vukotar_oracle.py).

Every test builds its own small configuration and random checkpoint, loads it
through the framework's config reader and weight loader, runs it through the
engine (scheduler, paged cache, decode graphs on the GPU) and compares logits
with the oracle run on whole sequences; the mechanisms are also tested alone
at the level of the ops. The CPU cases run the torch reference ops; the `gpu`
cases run the HIP kernels in fp32 and bf16.
"""

import json
import random

import pytest
import torch

import vukotar_oracle as O
from sutro_amd.engine.config import EngineConfig
from sutro_amd.engine.engine import LLMEngine
from sutro_amd.engine.request import SamplingParams
from sutro_amd.models.registry import spec_from_dir
from sutro_amd.ops import hybrid as hops

BACKENDS = [
    pytest.param(("cpu", torch.float32), id="cpu"),
    pytest.param(("cuda", torch.float32), id="gpu-fp32", marks=pytest.mark.gpu),
    pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu),
]


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def row_errors(got, want):
    """Per position: root mean square of the difference (mean over the
    vocabulary taken off), relative to the spread of the expected logits."""
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()


def rel_err(got, want):
    return float(row_errors(got, want).max())


# ------------------------------------------------------------- configs ------

def config_a():
    """Key and value sizes that differ, three groups of which two stay, a
    layer without feed-forward, a layer with one group (no restriction), and
    two layers that borrow the parameters of others, one of them of a LATER
    layer; sizes that are multiples of 8 nowhere."""
    a = O.attn_cfg(4, 2, 12, 20, 0.3)
    b = O.attn_cfg(3, 3, 10, 6, 0.45)
    c = O.attn_cfg(2, 1, 14, 14, 0.25)
    m1 = O.moe_cfg(20, 6, 3, 3, 2)
    m2 = O.moe_cfg(12, 5, 2, 1, 1)
    return O.make_config(44, 270, [
        O.layer(a, m1),
        O.layer(c, m2, weights_of=4),
        O.layer(b, None),
        O.layer(a, m1, weights_of=0),
        O.layer(c, m2),
    ], eps=1e-5, embed_scale=0.7, softcap=12.0)


def config_b():
    """One head, groups of one expert (a group's worth is its only score),
    every group kept, one expert a token, a vocabulary below the byte
    alphabet, an embedding scale of one."""
    return O.make_config(36, 50, [
        O.layer(O.attn_cfg(1, 1, 10, 18, 0.5), O.moe_cfg(28, 4, 1, 4, 4)),
        O.layer(O.attn_cfg(2, 2, 6, 10, 0.4), O.moe_cfg(8, 6, 6, 2, 2)),
        O.layer(O.attn_cfg(1, 1, 10, 18, 0.5), O.moe_cfg(28, 4, 1, 4, 4),
                weights_of=0),
    ], eps=2e-4, embed_scale=1.0, softcap=50.0)


def config_c():
    """Sizes the matrix-core kernels take (pages of 32, head sizes multiples
    of 8, width and expert width multiples of 64), eight groups of two, a
    loop over three layers run twice."""
    a = O.attn_cfg(4, 2, 32, 16, 0.18)
    b = O.attn_cfg(2, 2, 64, 64, 0.12)
    m = O.moe_cfg(64, 16, 4, 8, 3)
    return O.make_config(128, 300, [
        O.layer(a, m), O.layer(b, None), O.layer(a, O.moe_cfg(128, 4, 2, 2, 1)),
        O.layer(a, m, weights_of=0), O.layer(b, None, weights_of=1),
        O.layer(a, O.moe_cfg(128, 4, 2, 2, 1), weights_of=2),
    ], eps=1e-6, embed_scale=0.4, softcap=25.0)


_CACHE = {}


def checkpoint(tmp_path_factory, name, cfg_fn, seed=0, tweak=None):
    key = (name, seed)
    if key not in _CACHE:
        cfg = cfg_fn()
        w = O.make_weights(cfg, seed=seed)
        if tweak:
            tweak(w)
            w = {k: v.to(torch.bfloat16).to(O.F64) for k, v in w.items()}
        path = O.save_checkpoint(str(tmp_path_factory.mktemp(name)), cfg, w)
        _CACHE[key] = (path, cfg, w, {})
    return _CACHE[key]


def oracle_logits(ck, tokens):
    path, cfg, w, memo = ck
    key = tuple(tokens)
    if key not in memo:
        memo[key] = O.forward(cfg, w, list(tokens))
    return memo[key]


def engine(ck, backend, page=8, blocks=64, max_seqs=4, budget=4096, **kw):
    device, dtype = backend
    spec = spec_from_dir(ck[0])
    cfg = EngineConfig(spec=spec, device=device, dtype=dtype,
                       kv_block_size=page, max_model_len=page * (blocks - 1),
                       max_num_seqs=max_seqs, num_kv_blocks=blocks,
                       max_tokens_per_step=budget, **kw)
    return LLMEngine(cfg)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(3, cfg["vocab"], (n,), generator=g).tolist()


def clear_tokens(ck, n, seed, gap=0.03):
    """Tokens whose routing rests on no close call: the first drawn sequence
    for which every choice of the oracle's routers is at least `gap` (in
    sigmoid score) from another outcome. For short sequences only."""
    for k in range(200):
        toks = tokens_for(ck[1], n, seed + 1000 * k)
        gaps = []
        O.forward(ck[1], ck[2], toks, gaps=gaps)
        if not gaps or min(gaps) > gap:
            return toks
    raise AssertionError("no sequence without close routing calls")


def replay(eng, seqs, schedule):
    """Run `schedule` (a list of steps, each a list of (name, count)) and
    return name -> logits of every position [len, vocab]."""
    live, at, out = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in schedule:
        entries = []
        for name, n in step:
            if name not in live:
                live[name] = eng.new_replay_request()
            lo = at[name]
            entries.append((live[name], seqs[name][lo:lo + n], list(range(n))))
            at[name] = lo + n
        logits = eng.replay_step(entries)
        k = 0
        for name, n in step:
            out[name].append(logits[k:k + n])
            k += n
        for name, _ in step:
            if at[name] == len(seqs[name]) and name in live:
                eng.finish_replay_request(live.pop(name))
    return {k: torch.cat(v) for k, v in out.items() if v}


def check(ck, got, seqs, dtype, names=None):
    """fp32: every position within the limit. bf16: rounding alone can hand a
    token of these tiny models to another expert (two router scores next to
    each other), which moves that position by far more than rounding does
    elsewhere; so the limit holds for the median position, and at most one
    position in ten (or one) may be beyond five times it. Faults of masks,
    pages or routing show in the fp32 runs of the same kernels."""
    for name in names or got:
        want = oracle_logits(ck, seqs[name])
        assert got[name].shape == want.shape
        rows = row_errors(got[name], want)
        if dtype == torch.float32:
            assert float(rows.max()) < limit(dtype), \
                f"{name}: relative error {float(rows.max())}"
        else:
            assert float(rows.median()) < limit(dtype), \
                f"{name}: median relative error {float(rows.median())}"
            far_off = int((rows > 5 * limit(dtype)).sum())
            assert far_off <= max(1, len(rows) // 10), \
                f"{name}: {far_off} of {len(rows)} positions far off"


def page_of(cfg_fn):
    return 32 if cfg_fn is config_c else 8


# ------------------------------------------------ whole prompts, decoding ---

@pytest.mark.parametrize("cfg_fn", [config_a, config_b, config_c])
def test_whole_prompt(tmp_path_factory, backend, cfg_fn):
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page_of(cfg_fn), blocks=24)
    seqs = {"s": tokens_for(ck[1], 90 if cfg_fn is config_c else 45, 1)}
    got = replay(eng, seqs, [[("s", len(seqs["s"]))]])
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn", [config_a, config_c])
def test_layer_streams_match(tmp_path_factory, backend, cfg_fn):
    """The fp32 stream after every layer against the oracle's: a fault shows
    in the layer that makes it (a borrowed layer counts like any other)."""
    device, dtype = backend
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page_of(cfg_fn))
    toks = tokens_for(ck[1], 23, 9)
    want = []
    O.forward(ck[1], ck[2], toks, streams=want)
    eng.model.layer_taps = []
    replay(eng, {"s": toks}, [[("s", 23)]])
    taps = eng.model.layer_taps
    eng.model.layer_taps = None
    assert len(taps) == len(want) == len(ck[1]["layers"])
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    for i, (g, e) in enumerate(zip(taps, want)):
        err = float((g.double().cpu() - e).abs().max() / e.abs().max())
        assert err < tol, f"layer {i}: {err}"


@pytest.mark.parametrize("cfg_fn", [config_a, config_b])
def test_first_tokens(tmp_path_factory, backend, cfg_fn):
    """Sequences of one, two and three tokens (a first token attends to
    itself and the sink only), alone and decoded one by one."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend)
    seqs = {f"n{n}": clear_tokens(ck, n, 10 + n) for n in (1, 2, 3)}
    got = replay(eng, seqs, [[("n1", 1)], [("n2", 2)], [("n3", 3)]])
    check(ck, got, seqs, backend[1])
    got = replay(eng, seqs, [[("n3", 1), ("n2", 1)], [("n3", 1), ("n2", 1)],
                             [("n3", 1)]])
    check(ck, got, seqs, backend[1], names=["n2", "n3"])


@pytest.mark.parametrize("cfg_fn", [config_a, config_b, config_c])
def test_prefill_then_token_by_token(tmp_path_factory, backend, cfg_fn):
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page_of(cfg_fn), blocks=24)
    seqs = {"s": tokens_for(ck[1], 45, 1)}
    got = replay(eng, seqs, [[("s", 9)]] + [[("s", 1)]] * 36)
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_a, 32),
                                         (config_c, 32)])
def test_portions_of_many_sizes(tmp_path_factory, backend, cfg_fn, page):
    """Prompt pieces of 2, 3, 1, 11, 2, 5 ... tokens: cuts inside pages; a
    piece attends to everything the pieces before it left in the pages. With
    pages of 32 the bf16 prompt pieces take the matrix-core attention
    kernel."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"s": tokens_for(ck[1], 62, 2)}
    sizes = [2, 3, 1, 11, 2, 5, 1, 1, 13, 2, 8, 7, 2, 4]
    assert sum(sizes) == 62
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


def test_long_decoding(tmp_path_factory, backend):
    """A short prompt and 150 decoded tokens: many page borders pass under
    single-token steps and every decoded token sees all earlier ones."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend)
    seqs = {"s": tokens_for(ck[1], 154, 3)}
    got = replay(eng, seqs, [[("s", 4)]] + [[("s", 1)]] * 150)
    check(ck, got, seqs, backend[1])


# ------------------------------------------------ random configurations -----

def random_config(seed):
    """Widths, head counts, key and value sizes, expert counts, groups and how
    many stay, choices a token, the number of layers, which of them have a
    feed-forward and which borrow another's parameters: all drawn."""
    rnd = random.Random(seed)
    n = rnd.randint(2, 6)
    own = []
    for i in range(n):
        G = rnd.choice([1, 2, 4])
        mixer = O.attn_cfg(G * rnd.choice([1, 2, 3]), G,
                           rnd.choice([16, 24, 32, 40, 20]),
                           rnd.choice([16, 8, 48, 36]),
                           rnd.choice([0.1, 0.2, 0.35]))
        mlp = None
        if rnd.random() < 0.8:
            groups = rnd.choice([1, 2, 3, 4])
            size = rnd.choice([1, 2, 3, 5])
            keep = rnd.randint(1, groups)
            top = rnd.randint(1, keep * size)
            mlp = O.moe_cfg(rnd.choice([24, 40, 64, 72]), groups * size, top,
                            groups, keep)
        own.append(O.layer(mixer, mlp))
    order = [("own", k) for k in range(n)]
    for _ in range(rnd.randint(0, 3)):      # before or after the owner
        order.insert(rnd.randint(0, len(order)), ("borrow", rnd.randrange(n)))
    final = []
    for kind, k in order:
        if kind == "own":
            final.append(own[k])
        else:
            final.append(O.layer(own[k]["mixer"], own[k]["mlp"],
                                 weights_of=order.index(("own", k))))
    return O.make_config(rnd.choice([64, 96, 136, 50]),
                         rnd.choice([300, 512, 777]), final,
                         eps=rnd.choice([1e-6, 1e-5]),
                         embed_scale=rnd.choice([0.25, 1.0, 1.5]),
                         softcap=rnd.choice([8.0, 30.0, 100.0]))


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5])
def test_random_configurations(tmp_path_factory, backend, seed):
    """A drawn configuration through a mixed schedule (portions beside single
    tokens, pages of 32, a pool smaller than the sum of the requests)."""
    ck = checkpoint(tmp_path_factory, f"random{seed}",
                    lambda: random_config(seed), seed=seed)
    eng = engine(ck, backend, page=32, blocks=8, max_seqs=3)
    seqs = {"a": tokens_for(ck[1], 90, seed), "b": tokens_for(ck[1], 31, seed + 1),
            "c": tokens_for(ck[1], 47, seed + 2)}
    schedule = [[("a", 40), ("b", 3)], [("a", 1), ("b", 20), ("c", 2)],
                [("a", 30), ("b", 1), ("c", 1)], [("a", 2), ("b", 1), ("c", 40)],
                [("a", 1), ("b", 1), ("c", 1)], [("a", 1), ("b", 1), ("c", 1)],
                [("a", 15), ("b", 4), ("c", 2)]]
    got = replay(eng, seqs, schedule)
    for k in seqs:
        rows = row_errors(got[k], oracle_logits(ck, seqs[k]))
        if backend[1] == torch.float32:
            assert float(rows.max()) < limit(backend[1]), (k, float(rows.max()))
        else:   # single positions of a drawn model can be ill-conditioned
            assert float(rows.median()) < 6e-2, (k, float(rows.median()))


# ----------------------------------------------------- batches, reuse -------

@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_c, 32)])
def test_mixed_batch_equals_each_alone(tmp_path_factory, backend, cfg_fn, page):
    """Unequal requests in one batch (prompt pieces beside single tokens,
    requests that sit out a step) give what each gives alone: the experts'
    segments mix rows of all requests, the result of a row must not depend on
    its neighbours."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"a": tokens_for(ck[1], 40, 4), "b": tokens_for(ck[1], 17, 5),
            "c": tokens_for(ck[1], 9, 6), "d": tokens_for(ck[1], 26, 7)}
    schedule = [
        [("a", 13), ("b", 1)],
        [("a", 1), ("b", 1), ("c", 2)],
        [("b", 6), ("c", 1), ("d", 20), ("a", 1)],
        [("a", 20), ("c", 1), ("d", 1)],
        [("b", 9), ("d", 1), ("c", 5), ("a", 5)],
        [("d", 4)],
    ]
    got = replay(eng, seqs, schedule)
    check(ck, got, seqs, backend[1])
    alone = replay(engine(ck, backend, page=page, blocks=24), seqs,
                   [[(k, len(v))] for k, v in seqs.items()])
    for k in seqs:
        e = rel_err(got[k], alone[k].double().cpu())
        assert e < (limit(backend[1]) if backend[1] == torch.float32 else 0.3)


def test_pages_are_reused(tmp_path_factory, backend):
    """Two sequence slots and a pool of six pages serve eight requests one
    after another; a freed page's keys and values (of a layer's own pages and
    of the pages of the layers that borrow its parameters) must not leak into
    the next request."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, page=8, blocks=7, max_seqs=2)
    seqs = {f"r{i}": tokens_for(ck[1], 9 + 3 * (i % 4), 20 + i) for i in range(8)}
    names = list(seqs)
    schedule = []
    for i in range(0, 8, 2):
        a, b = names[i], names[i + 1]
        la, lb = len(seqs[a]), len(seqs[b])
        schedule += [[(a, 5), (b, 2)], [(a, la - 5), (b, 1)], [(b, lb - 3)]]
    got = replay(eng, seqs, schedule)
    check(ck, got, seqs, backend[1])
    assert eng.kv.allocator.num_free == 6
    with pytest.raises(MemoryError):
        replay(eng, {"x": [3] * 8, "y": [4] * 8, "z": [5] * 8},
               [[("x", 2), ("y", 2), ("z", 2)]])


def test_borrowed_layers_keep_pages_of_their_own(tmp_path_factory):
    """A layer that runs another layer's parameters sees other inputs, so its
    keys differ: the cache must hold one set of pages per layer, not per
    parameter set."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, ("cpu", torch.float32))
    kv, st = eng.model.cache_layout()
    assert kv == [(2, 12, 20), (1, 14, 14), (3, 10, 6), (2, 12, 20), (1, 14, 14)]
    assert all(s is None for s in st) and eng.kv.state is None
    assert len(eng.model.blocks) == 3
    replay(eng, {"s": tokens_for(ck[1], 12, 1)}, [[("s", 12)]])
    k0, k3 = eng.kv.k_cache[0], eng.kv.k_cache[3]
    assert float(k0.abs().max()) > 0 and float(k3.abs().max()) > 0
    assert float((k0 - k3).abs().max()) > 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_graph_replays_equal_eager_steps(tmp_path_factory, dtype):
    """Single-token steps run as captured hipGraphs (router, dispatch, expert
    GEMMs and the gather inside). Many replays with prompt pieces of other
    requests and host synchronisation between them must give, every time,
    what an engine that captures nothing gives (up to rounding: a graph pads
    its batch and its block tables, so GEMMs and the decode attention may sum
    in another order)."""
    ck = checkpoint(tmp_path_factory, "config_c", config_c)
    seqs = {"a": tokens_for(ck[1], 60, 1), "b": tokens_for(ck[1], 45, 2),
            "c": tokens_for(ck[1], 38, 3)}
    schedule = [[("a", 20)], [("a", 1)], [("a", 1), ("b", 30)],
                [("a", 1), ("b", 1)], [("c", 33), ("a", 1)]]
    schedule += [[("a", 1), ("b", 1), ("c", 1)]] * 5 + [[("a", 31), ("b", 8)]]
    graphs = engine(ck, ("cuda", dtype), page=32, blocks=24)
    assert graphs.graph_runner is not None
    eager = engine(ck, ("cuda", dtype), page=32, blocks=24, enforce_eager=True)
    assert eager.graph_runner is None
    got, want = replay(graphs, seqs, schedule), replay(eager, seqs, schedule)
    for k in seqs:
        rows = row_errors(got[k], want[k].double().cpu())
        if dtype == torch.float32:
            assert float(rows.max()) < 1e-5, (k, float(rows.max()))
        else:
            assert float(rows.median()) < 2e-2, (k, float(rows.median()))
            assert int((rows > 0.3).sum()) <= max(1, len(rows) // 10), k


@pytest.mark.gpu
def test_no_cyclic_collection_inside_graph_captures(tmp_path_factory, monkeypatch):
    """Python's cyclic collector must be off while a stream captures: it runs
    at arbitrary allocations, and freeing an unreferenced engine's graphs and
    events inside a capture is refused by the runtime. After the captures it
    is on again."""
    import gc

    from sutro_amd.models.vukotar import VukotarModel

    seen = []
    plain = VukotarModel.forward

    def watched(self, fb, kv):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return plain(self, fb, kv)

    monkeypatch.setattr(VukotarModel, "forward", watched)
    ck = checkpoint(tmp_path_factory, "config_b", config_b)
    assert gc.isenabled()
    eng = engine(ck, ("cuda", torch.float32))
    assert eng.graph_runner is not None and gc.isenabled()
    captured = [on for capturing, on in seen if capturing]
    assert captured and not any(captured)


# ------------------------------------------------- mechanisms on their own --

def _paged_attention(device, dtype, q, k, v, scale, page, pieces, sink=True,
                     seed=0):
    """Run q, k, v [T, H|G, d] of one sequence through attn_prep-free paging
    and `local_attention` piece by piece, pages handed out in a scrambled
    order. Returns [T, H, dv] fp32 on the CPU."""
    T, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    g = torch.Generator().manual_seed(seed)
    n_blocks = T // page + 3
    order = torch.randperm(n_blocks - 1, generator=g) + 1
    table = order[: (T + page - 1) // page].to(torch.int32)
    kc = torch.zeros(n_blocks, G, page, dk, dtype=dtype, device=device)
    vc = torch.zeros(n_blocks, G, page, dv, dtype=dtype, device=device)
    got, done = [], 0
    for n in pieces:
        pos = torch.arange(done, done + n)
        blk, off = table[pos // page].long(), pos % page
        kc[blk.to(device), :, off.to(device)] = k[done:done + n].to(dtype).to(device)
        vc[blk.to(device), :, off.to(device)] = v[done:done + n].to(dtype).to(device)
        qq = q[done:done + n].to(dtype).to(device).contiguous()
        out = torch.zeros(n, H * dv, dtype=dtype, device=device)
        done += n
        tiles = {}
        if n > 1:      # prompt pieces carry the 32-row tile map
            tiles = dict(
                tile_seq=torch.zeros((n + 31) // 32, dtype=torch.int32, device=device),
                tile_q0=torch.arange(0, n, 32, dtype=torch.int32, device=device),
                prefill_rows=n)
        hops.local_attention(
            qq, kc, vc, table[None].to(device),
            torch.tensor([done], dtype=torch.int32, device=device),
            torch.tensor([0, n], dtype=torch.int32, device=device), scale, 0,
            0, qq.view(n, -1), -1, out, 0, 1.0,
            token_seq=torch.zeros(n, dtype=torch.int32, device=device),
            sink=sink, **tiles)
        got.append(out.float().cpu())
    return torch.cat(got).view(T, H, dv)


@pytest.mark.parametrize("mode", ["prompt", "pieces", "decoded"])
@pytest.mark.parametrize("page,dk,dv", [(4, 12, 20), (8, 16, 8), (32, 32, 64)])
def test_far_keys_and_the_sink_stand_out(backend, mode, page, dk, dv):
    """Scores are made so that single things decide rows: (1) one key far
    back, at or next to a page border, scores far above all others, so the
    row's output must be (nearly) that key's value, among hundreds of keys,
    in prompts and in decoding; (2) rows whose scores are all far below zero
    must give (nearly) nothing, because the sink takes the weight (a plain
    softmax would return an average of the values instead); (3) the first
    token of the sequence shares its weight with the sink."""
    device, dtype = backend
    T, H, G = 300, 4, 2
    g = torch.Generator().manual_seed(page)
    q = torch.randn(T, H, dk, generator=g) * 0.1
    k = torch.randn(T, G, dk, generator=g) * 0.1
    v = torch.randn(T, G, dv, generator=g)
    probes, quiet = [], []
    # keys to single out, each once: the first two, then both sides of every
    # page border; when those run out, keys just behind the query
    cand = [0, 1] + [m * page + o for m in range(1, T) for o in (-1, 0, 1)]
    used = set()
    n = 0
    for i in range(40, T, 7):
        far = cand[n] if cand[n] < i - 3 else i - 1 - (n % 3)
        if n % 5 == 4:          # a row that likes nothing it sees (kv head 1)
            h, ch = 2 + n % 2, n % dk
            q[i, h] = 0.0
            q[i, h, ch] = 6.0
            k[: i + 1, 1, ch] = -5.0 - torch.rand(i + 1, generator=g)
            quiet.append((i, h))
        elif far not in used:   # one key in a direction of its own (kv head 0)
            used.add(far)
            h = n % 2
            u = torch.randn(dk, generator=g)
            u = u / u.norm()
            k[far, 0] += 9.0 * u
            q[i, h] += 9.0 * u
            probes.append((i, far, h))
        n += 1
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    scale = 0.8
    want = torch.stack([O.sink_attention(q[:, h].double(), k[:, h // 2].double(),
                                         v[:, h // 2].double(), scale)
                        for h in range(H)], 1)
    pieces = {"prompt": [T], "pieces": [37, 2, 90, 1, 33, 64, 3, 70],
              "decoded": [6] + [1] * (T - 6)}[mode]
    got = _paged_attention(device, dtype, q, k, v, scale, page, pieces)
    tol = 1e-4 if dtype == torch.float32 else 4e-2
    assert float((got.double() - want).abs().max()) < tol
    # the oracle itself shows the three effects
    assert len(probes) >= 20 and len(quiet) >= 5
    for i, j, h in probes:
        assert float((want[i, h] - v[j, h // 2].double()).abs().max()) < 0.05
    for i, h in quiet:
        assert float(want[i, h].abs().max()) < 1e-3
        plain = _paged_attention("cpu", torch.float32, q[: i + 1], k[: i + 1],
                                 v[: i + 1], scale, page, [i + 1], sink=False)
        assert float(plain[i, h].abs().max()) > 0.05
    s0 = float(q[0, 0].double() @ k[0, 0].double()) * scale
    first = torch.tensor(s0).exp() / (1 + torch.tensor(s0).exp())
    assert float((got[0, 0].double() - first * v[0, 0].double()).abs().max()) < tol


@pytest.mark.parametrize("E,top,groups,keep", [
    (8, 3, 4, 2), (6, 6, 1, 1), (12, 1, 12, 5), (9, 4, 3, 2), (64, 8, 8, 4),
    (130, 6, 10, 3), (4, 2, 2, 2)])
def test_router_choice_and_weights(backend, E, top, groups, keep):
    """Chosen experts and weights of 200 tokens against the oracle's router:
    only experts of the kept groups, groups worth their two best scores (one
    if a group has one expert), weights that sum to one."""
    device, dtype = backend
    if dtype != torch.float32:
        pytest.skip("the router is fp32 in every mode")
    g = torch.Generator().manual_seed(E * 7 + top)
    z = torch.randn(200, E, generator=g) * 2.0
    z[0] = -30.0           # every score tiny: the weights still sum to one
    z[0, :top] = -29.0
    idx, w = hops.moe_route(z.to(device), top, groups, keep)
    idx, w = idx.cpu(), w.cpu()
    assert idx.dtype == torch.int32 and w.dtype == torch.float32
    size = E // groups
    for t in range(z.shape[0]):
        chosen, weights = O.route(z[t].double(), top, groups, keep)
        assert sorted(idx[t].tolist()) == sorted(chosen), t
        by = dict(zip(idx[t].tolist(), w[t].tolist()))
        for e, x in zip(chosen, weights):
            assert abs(by[e] - x) < 1e-5
        assert len({e // size for e in chosen}) <= keep
        assert abs(float(w[t].sum()) - 1.0) < 1e-5


@pytest.mark.parametrize("T,W,ff,E,top", [(37, 44, 20, 6, 3), (5, 64, 128, 4, 2),
                                          (300, 128, 64, 16, 4), (1, 36, 8, 3, 3),
                                          (700, 64, 64, 2, 1),
                                          (1100, 128, 128, 2, 2)])
def test_expert_segments_and_gather(backend, T, W, ff, E, top):
    """Dispatch into padded per-expert segments, both expert GEMMs and the
    weighted gather inside the residual kernel against the oracle's experts,
    token by token; sizes the matrix-core kernel takes (64- and 128-row
    tiles, 64 and 128 columns a workgroup) and sizes it does not, segments
    longer than one tile, experts nobody chose."""
    device, dtype = backend
    g = torch.Generator().manual_seed(T + W)
    h = (torch.randn(T, W, generator=g) * 0.7).to(dtype)
    up = (torch.randn(E, ff, W, generator=g) * W ** -0.5).to(dtype)
    down = (torch.randn(E, W, ff, generator=g) * ff ** -0.5).to(dtype)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)])
    if E > 2:
        idx[idx == E - 1] = (E - 2 if top < E - 1 else E - 1)  # an idle expert
        for t in range(T):                                     # no repeats
            if len(set(idx[t].tolist())) < top:
                idx[t] = torch.arange(top)
    wts = torch.rand(T, top, generator=g) + 0.1
    wts = wts / wts.sum(-1, keepdim=True)
    x0 = torch.randn(T, W, generator=g)
    y1 = (torch.randn(T, W, generator=g) * 0.5).to(dtype)
    ls1, ls2 = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    alpha = torch.tensor(0.6)
    nw, nb = torch.rand(W, generator=g) + 0.5, torch.randn(W, generator=g) * 0.1

    d = lambda t: t.to(device)
    bm = hops.expert_gemm_tile(d(h), d(up), T * top)
    row_tok, tile_off, counts, padpos = hops.moe_dispatch(
        d(idx.to(torch.int32)), E, bm)
    assert row_tok.numel() % bm == 0
    cnt = torch.bincount(idx.reshape(-1), minlength=E)
    assert counts.cpu().tolist() == cnt.tolist()
    starts = (tile_off.cpu().long() * bm).tolist()
    for e in range(E):
        assert starts[e + 1] - starts[e] >= int(cnt[e])
        seg = row_tok.cpu()[starts[e]:starts[e + 1]].tolist()
        assert sorted(x for x in seg if x >= 0) == sorted(
            t for t in range(T) if e in idx[t].tolist())
    for t in range(T):
        for j in range(top):
            r = int(padpos[t, j])
            assert starts[int(idx[t, j])] <= r < starts[int(idx[t, j]) + 1]
            assert int(row_tok[r]) == t
    n = row_tok.numel()
    act = torch.zeros(n, ff, dtype=dtype, device=device)
    hops.expert_gemm(act, d(h), d(up), row_tok, tile_off, counts,
                     hops.ACT_RELU2, bm)
    rows = torch.zeros(n, W, dtype=dtype, device=device)
    hops.expert_gemm(rows, act, d(down), None, tile_off, counts,
                     hops.ACT_NONE, bm)
    x = d(x0.clone())
    h_out = torch.empty(T, W, dtype=dtype, device=device)
    hops.dyt_residual(x, d(y1), d(ls1), None, d(ls2), rows, padpos, d(wts),
                      norm=(d(alpha), d(nw), d(nb)), h_out=h_out)
    want = x0.double() + ls1.double() * y1.double()
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            want[t] += ls2.double() * wts[t, j].double() * O.expert(
                h[t].double(), up[e].double(), down[e].double())
    tol = 2e-4 if dtype == torch.float32 else 6e-2
    assert float((x.double().cpu() - want).abs().max()) < tol * float(want.abs().max())
    hn = O.dynamic_tanh(x.double().cpu(), alpha.double(), nw.double(), nb.double())
    assert float((h_out.double().cpu() - hn).abs().max()) < (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("W", [44, 15, 1024, 2050])
def test_dynamic_tanh_and_layer_scales(backend, W):
    """The residual kernel in its other forms: the norm alone (stream
    untouched), one branch, two dense branches; widths that take the 16-byte
    form and widths that do not."""
    device, dtype = backend
    T = 7
    g = torch.Generator().manual_seed(W)
    x0 = torch.randn(T, W, generator=g) * 3
    y1 = torch.randn(T, W, generator=g).to(dtype)
    y2 = torch.randn(T, W, generator=g).to(dtype)
    ls1, ls2 = torch.randn(W, generator=g), torch.randn(W, generator=g)
    alpha = torch.tensor(0.37)
    nw, nb = torch.randn(W, generator=g), torch.randn(W, generator=g)
    d = lambda t: t.to(device)
    norm = (d(alpha), d(nw), d(nb))
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    x = d(x0.clone())
    h = torch.empty(T, W, dtype=dtype, device=device)
    hops.dyt_residual(x, norm=norm, h_out=h)
    assert torch.equal(x.cpu(), x0)
    want = O.dynamic_tanh(x0.double(), alpha.double(), nw.double(), nb.double())
    assert float((h.double().cpu() - want).abs().max()) < tol
    hops.dyt_residual(x, d(y1), d(ls1), norm=norm, h_out=h)
    x1 = x0.double() + ls1.double() * y1.double()
    assert float((x.double().cpu() - x1).abs().max()) < 1e-5
    want = O.dynamic_tanh(x1, alpha.double(), nw.double(), nb.double())
    assert float((h.double().cpu() - want).abs().max()) < tol
    hops.dyt_residual(x, d(y1), d(ls1), d(y2), d(ls2))
    x2 = x1 + ls1.double() * y1.double() + ls2.double() * y2.double()
    assert float((x.double().cpu() - x2).abs().max()) < 2e-5


@pytest.mark.parametrize("W", [24, 15])
def test_scaled_embedding_and_positions(backend, W):
    """The embedding alone: the token row times the scale plus the sinusoid,
    at positions far from zero, an odd width (the last column has a sine and
    no cosine)."""
    device, dtype = backend
    g = torch.Generator().manual_seed(W)
    table = torch.randn(30, W, generator=g).to(dtype)
    ids = torch.tensor([3, 29, 0, 7, 7, 12])
    pos = torch.tensor([0, 1, 2, 700, 701, 4000])
    inv = hops.sinusoid_inv_freq(W, 10000.0)
    got = hops.token_embed(ids.to(device), None, pos.to(device),
                           table.to(device), None, 0, 0, 0, inv.to(device),
                           scale=0.35)
    full = O.sinusoid(4001, W)
    want = table[ids].double() * 0.35 + full[pos]
    assert float((got.double().cpu() - want).abs().max()) < 2e-3


def test_logit_softcap(backend):
    device, dtype = backend
    z = (torch.linspace(-90, 90, 77).view(7, 11)).to(dtype)
    got = hops.softcap(z.to(device), 20.0)
    assert got.dtype == torch.float32
    want = 20.0 * torch.tanh(z.double() / 20.0)
    assert float((got.double().cpu() - want).abs().max()) < 1e-4


def test_engine_picks_the_oracles_experts(tmp_path_factory, backend):
    """The experts the engine's router picks in the first layer, token by
    token, against the oracle's."""
    device, dtype = backend
    ck = checkpoint(tmp_path_factory, "config_c", config_c)
    eng = engine(ck, backend, page=32)
    toks = tokens_for(ck[1], 40, 5)
    picks = []
    O.forward(ck[1], ck[2], toks, picks=picks)
    blk = eng.model.block_of(0)
    x = hops.token_embed(
        torch.tensor(toks, device=device), None,
        torch.arange(len(toks), device=device), eng.model.embed_tokens.weight,
        None, 0, 0, 0, eng.model.pos_inv_freq, scale=eng.spec.embed_scale)
    h = torch.empty(x.shape, dtype=dtype, device=device)
    hops.dyt_residual(x, norm=blk.norm.parts(), h_out=h)
    idx, w, _ = blk.experts.route(h)
    same = sum(sorted(idx[t].tolist()) == sorted(picks[0][t])
               for t in range(len(toks)))
    assert same >= (len(toks) if dtype == torch.float32 else len(toks) - 3)


# -------------------------------------------- through the serving entry -----

def test_greedy_generation_through_scheduler(tmp_path_factory, backend):
    """Requests go through add_request / step(): the scheduler cuts prompts by
    its own token budget, batches prefill with decode and samples greedily.
    Every generated token must be the oracle's argmax given the same prefix
    (ties within rounding excepted)."""
    device, dtype = backend
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, budget=16, blocks=40)
    prompts = [tokens_for(ck[1], n, 30 + n) for n in (21, 5, 34, 2, 13)]
    reqs = [eng.add_request(p, SamplingParams(max_tokens=12, temperature=0.0))
            for p in prompts]
    steps = 0
    while eng.has_work():
        eng.step()
        steps += 1
        assert steps < 400
    checked = 0
    for p, r in zip(prompts, reqs):
        assert r.finished and len(r.output_token_ids) >= 1
        seq = p + r.output_token_ids
        logits = oracle_logits(ck, seq[:-1])
        for n, tok in enumerate(r.output_token_ids):
            row = logits[len(p) - 1 + n, :eng.tokenizer.vocab_size]
            best = int(row.argmax())
            margin = float(row[best] - row[tok])
            assert tok == best or margin < 20 * limit(dtype), (n, tok, best)
            checked += 1
    assert checked >= 20


def test_service_job_on_a_checkpoint_directory(tmp_path_factory, local_client):
    """A checkpoint directory is a model name for the job service too."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    job = local_client.infer(["alpha", "beta gamma"], model=ck[0],
                             sampling_params={"max_tokens": 4, "temperature": 0},
                             stay_attached=False)
    out = local_client.await_job_completion(job, timeout=120)
    assert out is not None and len(out) == 2


def test_cli_generates_from_a_checkpoint_directory(tmp_path_factory):
    from click.testing import CliRunner

    from sutro_amd.cli import cli

    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    res = CliRunner().invoke(cli, ["generate", "--model", ck[0], "--prompt",
                                   "hello there", "--prompt", "two",
                                   "--max-tokens", "5", "--temperature", "0",
                                   "--device", "cpu", "--max-model-len", "256"])
    assert res.exit_code == 0, res.output
    lines = [json.loads(x) for x in res.output.strip().splitlines()]
    assert [x["prompt"] for x in lines] == ["hello there", "two"]


def test_registry_reads_every_size_from_the_config(tmp_path_factory):
    from sutro_amd.models.hybrid_spec import (AttnMixerSpec, HybridSpec,
                                              vukotar_spec)
    from sutro_amd.models.registry import get_model_spec

    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    spec = get_model_spec(ck[0])
    assert isinstance(spec, HybridSpec) and spec.arch == "vukotar"
    assert all(isinstance(l.mixer, AttnMixerSpec) and l.mixer.sink
               and not l.mixer.qk_norm and l.mixer.rot_dims == 0
               for l in spec.layers)
    assert [l.weights_of for l in spec.layers] == [None, 4, None, 0, None]
    assert spec.layers[0].moe.groups == 3 and spec.layers[0].moe.keep == 2
    assert spec.layers[0].moe.top == 3 and spec.layers[0].moe.experts == 6
    assert spec.layers[2].moe is None and spec.layers[4].moe.ff == 12
    assert spec.layers[0].mixer.dim == 12 and spec.layers[0].mixer.vdim == 20
    assert spec.embed_scale == 0.7 and spec.logit_softcap == 12.0
    assert spec.norm_eps == 1e-5 and spec.tie_embeddings
    # parameters of borrowed layers are counted once: the count is the
    # checkpoint's; a token uses fewer (its chosen experts only), but passes
    # borrowed layers again
    assert spec.param_count() == sum(v.numel() for v in ck[2].values())
    assert spec.active_param_count() != spec.param_count()
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][1]["mixer"]["dim"] = 16        # borrows, but another shape
    with pytest.raises(ValueError):
        vukotar_spec(bad)
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][0]["mlp"]["router"]["top"] = 5  # two groups of two hold four
    with pytest.raises(ValueError):
        vukotar_spec(bad)
