"""Nosalorn on the engine against the plain float64 oracle (nosalorn_oracle.py).

Every test builds its own small configuration and random checkpoint, loads it
through the framework's config reader and weight loader, runs it through the
engine (scheduler, paged cache, state slots, decode graphs on the GPU) and
compares logits with the oracle run on whole sequences; the mechanisms are
also tested alone at the level of the ops. The CPU cases run the torch
reference ops; the `gpu` cases run the HIP kernels in fp32 and bf16.
"""

import json
import math
import random

import pytest
import torch

import nosalorn_oracle as O
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

YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def config_a():
    """Sizes that are multiples of 8 nowhere. Attention with two key heads,
    split key / value sizes, a rotated prefix with YaRN frequencies, a window
    of 7 that keeps 3 first tokens, blended values in layers 1, 3 and 5 (layer
    4 does not blend and has no window); a state-space mixer with three
    groups and three norm parts and one with one of each; decay attention;
    dense, routed (identity experts, groups, shared expert; or none of
    these) and absent feed-forwards."""
    a = O.attn_cfg(4, 2, 12, 20, 0.3, size=7, keep_first=3, rot_dims=8,
                   base=500.0, scaling=YARN, v_mix=True)
    b = O.attn_cfg(6, 2, 10, 20, 0.4, size=5, keep_first=0, rot_dims=10,
                   base=100.0, v_mix=True)
    c = O.attn_cfg(3, 3, 14, 6, 0.25)
    m1 = O.moe_cfg(20, 5, 3, identity=4, groups=3, keep=2, scale=1.7,
                   limit=1.5, shared_ff=12, shared_limit=0.8)
    m2 = O.moe_cfg(12, 6, 2, limit=3.0)
    return O.make_config(44, 270, [
        O.layer("mamba2", O.mamba2_cfg(3, 10, 12, 3, 3, 3), O.dense_cfg(52)),
        O.layer("attention", a, m1),
        O.layer("lightning", O.lightning_cfg(2, 10, 14, [0.7, 0.97]), m2),
        O.layer("attention", b, None),
        O.layer("attention", c, m1),
        O.layer("attention", a, O.dense_cfg(20)),
        O.layer("mamba2", O.mamba2_cfg(4, 6, 9, 1, 2, 1), None),
    ], eps=1e-5, embed_scale=3.0, logit_scale=0.5)


def config_b():
    """One head, a window of one, more kept tokens than the window is long, a
    fully rotated head without scaling, a filter of one tap and one of five,
    one expert a token, only identity experts beside one expert, embedding
    and logit scales of one, a vocabulary below the byte alphabet."""
    return O.make_config(36, 50, [
        O.layer("attention", O.attn_cfg(1, 1, 10, 18, 0.5, size=1,
                                        keep_first=0, rot_dims=10),
                O.moe_cfg(28, 4, 1, groups=4, keep=4)),
        O.layer("mamba2", O.mamba2_cfg(2, 8, 6, 2, 1, 2),
                O.moe_cfg(8, 1, 2, identity=3, groups=2, keep=1, scale=0.5,
                          shared_ff=20, shared_limit=5.0)),
        O.layer("lightning", O.lightning_cfg(1, 6, 10, [1.0]), None),
        O.layer("attention", O.attn_cfg(2, 1, 6, 10, 0.4, size=3,
                                        keep_first=9, rot_dims=2, base=7.0,
                                        scaling={"factor": 1.5, "original": 16,
                                                 "fast": 2.0, "slow": 0.5},
                                        v_mix=True), O.dense_cfg(40)),
        O.layer("mamba2", O.mamba2_cfg(1, 12, 10, 1, 5, 1), None),
    ], eps=2e-4, embed_scale=1.0, logit_scale=1.0)


def config_c():
    """Sizes the matrix-core kernels take (pages of 32, head sizes multiples
    of 8, widths multiples of 64); windows shorter and longer than a page and
    kept tokens beyond the first page."""
    a = O.attn_cfg(4, 2, 32, 16, 0.18, size=44, keep_first=19, rot_dims=16,
                   scaling={"factor": 3.0, "original": 32, "fast": 4.0,
                            "slow": 1.0}, v_mix=True)
    b = O.attn_cfg(2, 1, 64, 32, 0.12, size=9, keep_first=35, rot_dims=64,
                   v_mix=True)
    m = O.moe_cfg(64, 13, 4, identity=3, groups=4, keep=3, scale=1.8,
                  limit=2.4, shared_ff=64, shared_limit=1.6)
    return O.make_config(128, 300, [
        O.layer("attention", a, m),
        O.layer("mamba2", O.mamba2_cfg(4, 32, 16, 2, 3, 4), O.dense_cfg(192)),
        O.layer("attention", b, O.moe_cfg(128, 4, 2, limit=4.0)),
        O.layer("lightning", O.lightning_cfg(2, 64, 32, [0.6, 0.995]), m),
        O.layer("attention", O.attn_cfg(2, 2, 64, 64, 0.12, rot_dims=32), None),
    ], eps=1e-6, embed_scale=8.0, logit_scale=0.3)


_CACHE = {}


def checkpoint(tmp_path_factory, name, cfg_fn, seed=0):
    key = (name, seed)
    if key not in _CACHE:
        cfg = cfg_fn()
        w = O.make_weights(cfg, seed=seed)
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


def clear_tokens(ck, n, seed, gap=0.003):
    """Tokens whose routing rests on no close call (for short sequences)."""
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
    token of these tiny models to another expert (two choice scores next to
    each other), which moves that position by far more than rounding does
    elsewhere; so the limit holds for the median position, and at most one
    position in ten (or one) may be beyond five times it. Faults of masks,
    pages, state or routing show in the fp32 runs of the same kernels."""
    for name in names or got:
        want = oracle_logits(ck, seqs[name])
        assert got[name].shape == want.shape
        rows = row_errors(got[name], want)
        if dtype == torch.float32:
            assert float(rows.max()) < limit(dtype), \
                f"{name}: relative error {float(rows.max())} at " \
                f"{int(rows.argmax())}"
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


@pytest.mark.parametrize("cfg_fn", [config_a, config_b, config_c])
def test_layer_streams_match(tmp_path_factory, backend, cfg_fn):
    """The fp32 stream after every layer against the oracle's: a fault shows
    in the layer that makes it."""
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
    tol = 2e-5 if dtype == torch.float32 else 5e-2
    for i, (g, e) in enumerate(zip(taps, want)):
        err = (g.double().cpu() - e).abs().max(-1).values / e.abs().max()
        # in bf16 a token's close routing call may fall the other way
        worst = float(err.max() if dtype == torch.float32 else err.median())
        assert worst < tol, f"layer {i}: {worst}"


@pytest.mark.parametrize("cfg_fn", [config_a, config_b])
def test_first_tokens(tmp_path_factory, backend, cfg_fn):
    """Sequences of one, two and three tokens (zero filter history, zero
    state, a window that is not yet full), alone and decoded one by one."""
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
    n = 75 if cfg_fn is config_c else 45
    seqs = {"s": tokens_for(ck[1], n, 1)}
    got = replay(eng, seqs, [[("s", 9)]] + [[("s", 1)]] * (n - 9))
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_a, 32),
                                         (config_b, 4), (config_c, 32)])
def test_portions_of_many_sizes(tmp_path_factory, backend, cfg_fn, page):
    """Prompt pieces of 2, 3, 1, 11, 2, 5 ... tokens: cuts inside pages,
    windows and filter histories; a piece continues from the pages, the
    filter inputs and the memories the pieces before it left. With pages of
    32 the bf16 prompt pieces take the matrix-core attention kernel."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"s": tokens_for(ck[1], 62, 2)}
    sizes = [2, 3, 1, 11, 2, 5, 1, 1, 13, 2, 8, 7, 2, 4]
    assert sum(sizes) == 62
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn", [config_a, config_c])
def test_long_decoding(tmp_path_factory, backend, cfg_fn):
    """A short prompt and 150 decoded tokens: many page borders and whole
    windows pass under single-token steps; the recurrent layers carry their
    memory through every step."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page_of(cfg_fn), blocks=24)
    seqs = {"s": tokens_for(ck[1], 154, 3)}
    got = replay(eng, seqs, [[("s", 4)]] + [[("s", 1)]] * 150)
    check(ck, got, seqs, backend[1])


# ------------------------------------------------ random configurations -----

def random_config(seed):
    """Widths, the order and number of layers, head counts, key, value and
    state sizes, windows and kept tokens, rotation, filters, decays, expert
    counts, identity experts, groups, choices: all drawn."""
    rnd = random.Random(seed)
    n = rnd.randint(3, 6)
    layers = []
    mix_cols = rnd.choice([16, 24, 40])     # blended values share a width
    for i in range(n):
        kind = rnd.choice(["attention", "attention", "lightning", "mamba2"])
        if kind == "attention":
            G = rnd.choice([1, 2])
            v_mix = rnd.random() < 0.6
            dv = mix_cols // G if v_mix else rnd.choice([8, 12, 36])
            dk = rnd.choice([16, 24, 32, 20])
            rot = rnd.choice([0, 4, dk // 2 * 2, 8])
            mixer = O.attn_cfg(
                G * rnd.choice([1, 2, 3]), G, dk, dv, rnd.choice([0.1, 0.2, 0.35]),
                size=rnd.choice([0, 1, 6, 33, 50]),
                keep_first=rnd.choice([0, 1, 5, 34]), rot_dims=rot,
                base=rnd.choice([50.0, 10000.0]),
                scaling=rnd.choice([None, YARN]), v_mix=v_mix)
        elif kind == "lightning":
            H = rnd.choice([1, 2, 3])
            mixer = O.lightning_cfg(H, rnd.choice([8, 12, 32]),
                                    rnd.choice([8, 20, 32]),
                                    [rnd.choice([0.5, 0.9, 0.99, 1.0])
                                     for _ in range(H)])
        else:
            G = rnd.choice([1, 2])
            H = G * rnd.choice([1, 2, 3])
            dv = rnd.choice([4, 8, 10])
            parts = rnd.choice([p for p in (1, 2, H) if (H * dv) % p == 0])
            mixer = O.mamba2_cfg(H, dv, rnd.choice([4, 16, 24]), G,
                                 rnd.choice([1, 2, 4]), parts)
        mlp = None
        r = rnd.random()
        if r < 0.25:
            mlp = O.dense_cfg(rnd.choice([24, 64, 100]))
        elif r < 0.85:
            groups = rnd.choice([1, 2, 3, 4])
            size = rnd.choice([1, 2, 3, 5])
            total = groups * size
            ident = rnd.randint(0, total - 1)
            keep = rnd.randint(1, groups)
            top = rnd.randint(1, keep * size)
            mlp = O.moe_cfg(rnd.choice([24, 40, 64, 72]), total - ident, top,
                            identity=ident, groups=groups, keep=keep,
                            scale=rnd.choice([1.0, 1.8]),
                            limit=rnd.choice([1.0, 7.0]),
                            shared_ff=rnd.choice([0, 16, 64]),
                            shared_limit=rnd.choice([0.5, 7.0]))
        layers.append(O.layer(kind, mixer, mlp))
    return O.make_config(rnd.choice([64, 96, 136, 50]),
                         rnd.choice([300, 512, 777]), layers,
                         eps=rnd.choice([1e-6, 1e-5]),
                         embed_scale=rnd.choice([0.5, 1.0, 6.0]),
                         logit_scale=rnd.choice([0.3, 1.0, 2.0]))


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_configurations(tmp_path_factory, backend, seed):
    """A drawn configuration through a mixed schedule (portions beside single
    tokens, pages of 32, a pool smaller than the sum of the requests, three
    state slots)."""
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
            assert float(rows.max()) < limit(backend[1]), \
                (k, float(rows.max()), int(rows.argmax()))
        else:   # single positions of a drawn model can be ill-conditioned
            assert float(rows.median()) < 6e-2, (k, float(rows.median()))


# ----------------------------------------------------- batches, reuse -------

@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_c, 32)])
def test_mixed_batch_equals_each_alone(tmp_path_factory, backend, cfg_fn, page):
    """Unequal requests in one batch (prompt pieces beside single tokens,
    requests that sit out a step) give what each gives alone: expert segments
    mix rows of all requests, recurrences run side by side, and the result of
    a row must not depend on its neighbours."""
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


def test_pages_and_slots_are_reused(tmp_path_factory, backend):
    """Two sequence slots and a pool of six pages serve eight requests one
    after another; a freed page's keys and values, a freed slot's filter
    history and memories must not leak into the next request."""
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
    assert eng.kv.state.num_free == 2
    with pytest.raises(MemoryError):
        replay(eng, {"x": [3] * 8, "y": [4] * 8, "z": [5] * 8},
               [[("x", 2), ("y", 2), ("z", 2)]])


def test_cache_layout(tmp_path_factory):
    """Attention layers hold pages, recurrent layers hold state, by layer."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, ("cpu", torch.float32))
    kv, st = eng.model.cache_layout()
    assert kv == [None, (2, 12, 20), None, (2, 10, 20), (3, 14, 6),
                  (2, 12, 20), None]
    assert st[0] == (30 + 72, 3, 3, 12, 10) and st[1] is None
    assert st[2] == {"mem": (2, 10, 14)} and st[6] == (24 + 18, 2, 4, 9, 6)
    assert eng.kv.state.ssm[0].shape[1:] == (3, 12, 10)
    assert eng.kv.state.conv[6].shape[1:] == (1, 42)
    assert eng.kv.state.named[2]["mem"].dtype == torch.float32


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_graph_replays_equal_eager_steps(tmp_path_factory, dtype):
    """Single-token steps run as captured hipGraphs. Many replays with prompt
    pieces of other requests and host synchronisation between them must give,
    every time, what an engine that captures nothing gives (up to rounding: a
    graph pads its batch and its block tables)."""
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


# ------------------------------------------------- mechanisms on their own --

def _paged_attention(device, dtype, q, k, v, scale, page, pieces, window,
                     keep_first, seed=0):
    """Run q, k, v [T, H|G, d] of one sequence through `local_attention` piece
    by piece, pages handed out in a scrambled order. Returns [T, H, dv] fp32
    on the CPU."""
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
            window, qq.view(n, -1), -1, out, 0, 1.0,
            token_seq=torch.zeros(n, dtype=torch.int32, device=device),
            keep_first=keep_first, **tiles)
        got.append(out.float().cpu())
    return torch.cat(got).view(T, H, dv)


@pytest.mark.parametrize("mode", ["prompt", "pieces", "decoded"])
@pytest.mark.parametrize("page,dk,dv,window,keep", [
    (4, 12, 20, 7, 3), (8, 16, 8, 41, 17), (32, 32, 64, 36, 21),
    (32, 64, 32, 33, 70), (8, 16, 8, 1, 0), (32, 32, 16, 64, 32)])
def test_window_edges_and_kept_tokens_stand_out(backend, mode, page, dk, dv,
                                                window, keep):
    """One key is made to score far above all others, so a row's output is
    (nearly) that key's value if and only if the row sees it. The key sits
    just inside the kept first tokens, just outside them, and in the middle
    of the sequence, where it is the window's last key for one row and just
    outside for the next; prompts, portions (cuts at and next to the edges)
    and single-token steps."""
    device, dtype = backend
    T, H, G = 150, 4, 2
    g = torch.Generator().manual_seed(page + window)
    scale = 0.25
    for star in sorted({max(keep - 1, 0), keep, 77}):
        q = torch.randn(T, H, dk, generator=g, dtype=torch.float64) * 0.5
        k = torch.randn(T, G, dk, generator=g, dtype=torch.float64) * 0.5
        v = torch.randn(T, G, dv, generator=g, dtype=torch.float64)
        u = torch.zeros(dk, dtype=torch.float64)
        u[star % dk] = 1.0
        k[star] += 12.0 * u
        q += 6.0 * u
        q, k, v = (z.to(torch.bfloat16).double() for z in (q, k, v))
        if mode == "prompt":
            pieces = [T]
        elif mode == "pieces":
            cuts = sorted({2, max(star, 3), star + 1, star + window - 1,
                           star + window, star + window + 2, 120} - {0})
            cuts = [c for c in cuts if 0 < c < T]
            pieces = [b - a for a, b in zip([0] + cuts, cuts + [T])]
        else:
            pieces = [5] + [1] * (T - 5)
        got = _paged_attention(device, dtype, q, k, v, scale, page, pieces,
                               window, keep, seed=star)
        want = torch.stack([
            O.windowed_attention(q[:, a], k[:, a // (H // G)],
                                 v[:, a // (H // G)], scale, window, keep)
            for a in range(H)], dim=1)
        err = float((got.double() - want).abs().max())
        assert err < (1e-4 if dtype == torch.float32 else 4e-2), (star, err)
        # the rows around the edge really differ
        sees = [i for i in range(star, T) if i - star < window or star < keep]
        if len(sees) < T - star:
            i = sees[-1]
            assert float((want[i, 0] - v[star, 0]).abs().max()) < 0.05
            assert float((want[i + 1, 0] - v[star, 0]).abs().max()) > 0.05


def _meta(device, lens_new, lens_total):
    qlocs = [0]
    for n in lens_new:
        qlocs.append(qlocs[-1] + n)
    i32 = dict(dtype=torch.int32, device=device)
    token_seq = torch.tensor([s for s, n in enumerate(lens_new)
                              for _ in range(n)], **i32)
    return (torch.tensor(qlocs, **i32), torch.tensor(lens_total, **i32),
            token_seq)


@pytest.mark.parametrize("H,G,dk,dv", [(2, 1, 12, 10), (4, 2, 32, 32),
                                       (3, 3, 70, 20), (2, 2, 130, 72),
                                       (1, 1, 6, 200)])
def test_decay_scan_far_memory_and_slots(backend, H, G, dk, dv):
    """Two sequences side by side, in portions and single tokens, through
    state slots that hold stale numbers; decays near one keep the first
    tokens' keys readable hundreds of tokens later; gains, skips and grouped
    keys as the state-space mixer uses them, constant decays as decay
    attention does."""
    device, dtype = backend
    g = torch.Generator().manual_seed(H * dk)
    lens = [210, 37]
    f64 = torch.float64
    data = []
    for T in lens:
        q = torch.randn(T, G, dk, generator=g, dtype=f64) * 0.3
        k = torch.randn(T, G, dk, generator=g, dtype=f64) * 0.3
        v = torch.randn(T, H, dv, generator=g, dtype=f64)
        k[1, :, 0] += 3.0          # a key far back that late queries ask for
        q[T - 3:, :, 0] += 3.0
        data.append((q, k, v))
    for per_token in (True, False):
        decay_h = torch.tensor([0.999, 0.9, 1.0, 0.5][:H], dtype=f64)
        state = torch.full((3, H, dk, dv), 7.0, dtype=torch.float32,
                           device=device)
        slots = torch.tensor([2, 1], dtype=torch.int32, device=device)
        skip = torch.randn(H, generator=g, dtype=f64) if per_token else None
        want, dec, gain = [], [], []
        for (q, k, v), T in zip(data, lens):
            if per_token:
                d = torch.rand(T, H, generator=g, dtype=f64) * 0.05 + 0.95
                b = torch.rand(T, H, generator=g, dtype=f64) + 0.2
            else:
                d, b = decay_h.expand(T, H), torch.ones(T, H, dtype=f64)
            dec.append(d)
            gain.append(b)
            o = torch.stack([
                O.decay_memory(q[:, a // (H // G)], k[:, a // (H // G)],
                               v[:, a], d[:, a], b[:, a])
                + (skip[a] * v[:, a] if skip is not None else 0.0)
                for a in range(H)], dim=1)
            want.append(o)
        at = [0, 0]
        steps = [(150, 2), (1, 1), (1, 30), (58, 1), (0, 3)]
        got = [[], []]
        for na, nb in steps:
            new = [na, nb]
            parts = [[z[at[s]:at[s] + new[s]] for z in data[s]] for s in (0, 1)]
            cat = [torch.cat([parts[0][j], parts[1][j]]).float().to(device)
                   for j in range(3)]
            for s in (0, 1):
                at[s] += new[s]
            qlocs, seq_lens, _ = _meta(device, new, at)
            if per_token:
                d = torch.cat([dec[s][at[s] - new[s]:at[s]] for s in (0, 1)])
                b = torch.cat([gain[s][at[s] - new[s]:at[s]] for s in (0, 1)])
                o = hops.decay_scan(cat[0], cat[1], cat[2],
                                    d.float().to(device).contiguous(),
                                    b.float().to(device).contiguous(),
                                    skip.float().to(device), state, slots,
                                    qlocs, seq_lens)
            else:
                o = hops.decay_scan(cat[0], cat[1], cat[2],
                                    decay_h.float().to(device), None, None,
                                    state, slots, qlocs, seq_lens)
            got[0].append(o[:na].cpu())
            got[1].append(o[na:].cpu())
        for s in (0, 1):
            o = torch.cat(got[s]).double()
            err = float((o - want[s]).abs().max() / want[s].abs().max())
            assert err < 2e-5, (per_token, s, err)
        assert float(state[0].min()) == 7.0      # the scratch slot is untouched


@pytest.mark.parametrize("taps,H,dv,G,N", [(4, 3, 10, 3, 12), (1, 2, 8, 1, 5),
                                           (5, 4, 32, 2, 32), (2, 1, 3, 1, 2)])
def test_filter_history_across_pieces(backend, taps, H, dv, G, N):
    """The short causal filter over pieces as short as one token (shorter
    than the filter), from a slot with stale history, beside a second
    sequence; steps and decays against their formulas."""
    device, dtype = backend
    g = torch.Generator().manual_seed(taps)
    C = H * dv + 2 * G * N
    f64 = torch.float64
    lens = [23, 9]
    w = torch.randn(C, taps, generator=g, dtype=f64).to(torch.bfloat16).double()
    b = torch.randn(C, generator=g, dtype=f64).to(torch.bfloat16).double()
    dtb = torch.randn(H, generator=g, dtype=f64)
    alog = torch.randn(H, generator=g, dtype=f64) * 0.5
    pad = 5                                     # columns before the section
    raws = [torch.randn(T, pad + C + H, generator=g, dtype=f64)
            .to(torch.bfloat16).double() for T in lens]
    conv_state = torch.full((3, max(1, taps - 1), C), 9.0, dtype=torch.float32,
                            device=device)
    slots = torch.tensor([1, 2], dtype=torch.int32, device=device)
    at = [0, 0]
    outs = [[], []]
    dts = [[], []]
    for na, nb in [(2, 1), (1, 1), (1, 3), (11, 1), (8, 3)]:
        new = [na, nb]
        proj = torch.cat([raws[s][at[s]:at[s] + new[s]] for s in (0, 1)])
        proj = proj.to(dtype).to(device)
        for s in (0, 1):
            at[s] += new[s]
        qlocs, seq_lens, token_seq = _meta(device, new, at)
        x, B, Cc, decay, dt = hops.ssd_prep(
            proj, pad, pad + C, H, dv, G, N, w.float().to(device),
            b.float().to(device), dtb.float().to(device),
            alog.float().to(device), conv_state, slots, qlocs, seq_lens,
            token_seq=token_seq)
        T = na + nb
        y = torch.cat([x.reshape(T, -1), B.reshape(T, -1), Cc.reshape(T, -1)],
                      dim=1).cpu()
        outs[0].append(y[:na])
        outs[1].append(y[na:])
        dts[0].append(torch.stack([dt[:na].cpu(), decay[:na].cpu()]))
        dts[1].append(torch.stack([dt[na:].cpu(), decay[na:].cpu()]))
    for s in (0, 1):
        want = O.silu(O.causal_filter(raws[s][:, pad:pad + C], w, b))
        err = float((torch.cat(outs[s]).double() - want).abs().max())
        assert err < 1e-4, (s, err)
        d = O.softplus(raws[s][:, pad + C:] + dtb)
        got = torch.cat(dts[s], dim=1).double()
        assert float((got[0] - d).abs().max()) < 1e-5
        assert float((got[1] - torch.exp(-torch.exp(alog) * d)).abs().max()) < 1e-5


@pytest.mark.parametrize("n,ident,top,groups,keep", [
    (12, 3, 5, 3, 2), (6, 0, 2, 1, 1), (4, 3, 2, 2, 1), (16, 0, 6, 8, 3),
    (9, 8, 1, 9, 9), (70, 5, 8, 7, 4), (130, 2, 3, 2, 2)])
def test_router_choice_and_weights(backend, n, ident, top, groups, keep):
    """Choice by score + correction (negative choice scores included), groups
    by their largest member, dropped groups out whatever their sign, weights
    from the plain scores times the scale, identity experts folded."""
    device, dtype = backend
    g = torch.Generator().manual_seed(n + top)
    T = 37
    z = torch.randn(T, n, generator=g) * 2.0
    corr = torch.randn(n, generator=g) * 0.3 - 0.2
    idx, w, idw = hops.moe_route_softmax(z.to(device), corr.to(device), top,
                                         groups, keep, n - ident, 1.7)
    idx, w, idw = idx.cpu(), w.cpu(), idw.cpu()
    for t in range(T):
        chosen = O.route(z[t].double(), corr.double(), top, groups, keep, 1.7)
        real = sorted((j, wt) for j, wt in chosen if j < n - ident)
        want_id = sum(wt for j, wt in chosen if j >= n - ident)
        got = sorted((int(j), float(x)) for j, x in zip(idx[t], w[t])
                     if int(j) < n - ident)
        assert [j for j, _ in got] == [j for j, _ in real], t
        for (_, a), (_, b) in zip(got, real):
            assert abs(a - b) < 1e-5
        assert abs(float(idw[t]) - want_id) < 1e-5
        spare = [(int(j), float(x)) for j, x in zip(idx[t], w[t])
                 if int(j) >= n - ident]
        assert all(j == n - ident and x == 0.0 for j, x in spare)
        assert len(spare) + len(real) == top


@pytest.mark.parametrize("T,W,ff,E,ident,top", [
    (50, 44, 20, 5, 4, 3), (9, 36, 28, 4, 0, 1), (300, 128, 64, 12, 4, 4),
    (1, 64, 64, 3, 2, 2)])
def test_expert_segments_identity_and_shared(backend, T, W, ff, E, ident, top):
    """Dispatch, both expert GEMMs with the clamped unit, and the fused sum of
    expert rows, identity share, gated shared expert, residual and norm
    against the per-token formulas."""
    device, dtype = backend
    from sutro_amd.models.hybrid_spec import RoutedExpertsSpec
    from sutro_amd.models.layers import RoutedExperts

    g = torch.Generator().manual_seed(T + W)
    n = E + ident
    groups = 1
    spec = RoutedExpertsSpec(ff=ff, experts=E, top=top, groups=groups, keep=1,
                             group_rank=1, router="softmax", act="clamped_glu",
                             identity=ident, route_scale=1.4, correction=True,
                             limit=1.2, shared_ff=24, shared_limit=0.9)
    mod = RoutedExperts(spec, W, dtype).to(device).requires_grad_(False)
    w = {}

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"] = rnd(ff, W, std=1.5 * W ** -0.5), \
            rnd(ff, W, std=1.5 * W ** -0.5)
        w[f"e{e}.down"] = rnd(W, ff, std=ff ** -0.5)
    w["shared.gate"], w["shared.up"] = rnd(24, W, std=W ** -0.5), \
        rnd(24, W, std=W ** -0.5)
    w["shared.down"], w["shared.sg"] = rnd(W, 24, std=0.2), rnd(1, W, std=0.3)
    w["router"], w["correction"] = rnd(n, W, std=3 * W ** -0.5), rnd(n, std=0.05)
    params = dict(mod.named_parameters())
    with torch.no_grad():
        for ck, (pname, dim, start, length, _) in \
                mod.param_targets("", "").items():
            src = w[ck.lstrip(".")].float()
            dst = params[pname].narrow(dim, start, length)
            if dst.dim() == src.dim() + 1:
                dst = dst.squeeze(dim)
            dst.copy_(src.to(dst.dtype))
    h = (torch.randn(T, W, generator=g)).to(torch.bfloat16)
    x0 = torch.randn(T, W, generator=g)
    nw = torch.rand(W, generator=g) + 0.5
    hd = h.to(dtype).to(device)
    rows, padpos, wts, idw = mod(hd)
    y2, proj2, sg = mod.shared_forward(hd)
    x = x0.clone().to(device)
    h_out = hd.clone()
    hops.add_rmsnorm(x, None, rows, padpos, wts, idw, h_out, y2, proj2, sg,
                     nw.to(device), 1e-5, h_out)
    w64 = {"m." + k: v.double() for k, v in w.items()}
    fc = {"router": {"experts": E, "identity": ident, "top": top, "scale": 1.4,
                     "groups": {"count": 1, "keep": 1}},
          "expert": {"limit": 1.2}, "shared": {"limit": 0.9}}
    gaps = []
    want = x0.double() + O.moe_ff(h.double(), w64, "m.", fc, gaps=gaps)
    err = (x.double().cpu() - want).abs().max(-1).values / want.abs().max()
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    # a token whose choice is a close call may go to another expert in bf16
    assert float(err.median()) < tol
    assert int((err > tol).sum()) <= (0 if dtype == torch.float32 else T // 10)
    hn = O.rms_norm(x.double().cpu(), nw.double(), 1e-5)
    assert float((h_out.double().cpu() - hn).abs().max()) < \
        (1e-4 if dtype == torch.float32 else 5e-2)


@pytest.mark.parametrize("n,parts", [(40, 1), (30, 3), (256, 2), (1100, 4)])
def test_gated_norms_and_units(backend, n, parts):
    """Gate-before-norm in parts, norm-then-gate over all heads, the three
    gated units, and the rotation frequencies against their formulas."""
    device, dtype = backend
    g = torch.Generator().manual_seed(n)
    T = 13
    o = torch.randn(T, n, generator=g)
    proj = torch.randn(T, 2 * n + 8, generator=g).to(torch.bfloat16)
    nw = torch.rand(n, generator=g) + 0.5
    pd = proj.to(dtype).to(device)
    z = proj[:, 8:8 + n].double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    out = torch.zeros(T, n + 8, dtype=dtype, device=device)
    hops.gated_group_norm(o.to(device), pd, 8, nw.to(device), 1e-5, parts,
                          True, out, 8)
    y = o.double() * O.silu(z)
    want = O.rms_norm(y.view(T, parts, n // parts), torch.ones((), dtype=O.F64),
                      1e-5).reshape(T, n) * nw.double()
    assert float((out[:, 8:].double().cpu() - want).abs().max()) < tol * 4
    assert float(out[:, :8].abs().max()) == 0.0
    hops.gated_group_norm(o.to(device), pd, 8, nw.to(device), 1e-5, 1, False,
                          out, 0)
    want = O.rms_norm(o.double(), nw.double(), 1e-5) * torch.sigmoid(z)
    assert float((out[:, :n].double().cpu() - want).abs().max()) < tol * 4
    gte, up = proj[:, 8:8 + n].double(), proj[:, 8 + n:8 + 2 * n].double()
    got = hops.glu_mul(pd, 8, 8 + n, n, hops.GLU_SILU).double().cpu()
    assert float((got - O.silu(gte) * up).abs().max()) < tol * 8
    got = hops.glu_mul(pd, 8, 8 + n, n, hops.GLU_CLAMPED, 0.7).double().cpu()
    gc = gte.clamp(max=0.7)
    want = gc * torch.sigmoid(1.702 * gc) * (up.clamp(-0.7, 0.7) + 1.0)
    assert float((got - want).abs().max()) < tol * 4


@pytest.mark.parametrize("rot", [
    {"dims": 48, "base": 30000.0,
     "scaling": {"factor": 3.0, "original": 1024, "fast": 16.0, "slow": 2.0}},
    {"dims": 8, "base": 500.0, "scaling": YARN},
    {"dims": 2, "base": 7.0,
     "scaling": {"factor": 1.5, "original": 16, "fast": 2.0, "slow": 0.5}},
    {"dims": 10, "base": 100.0}])
def test_rotation_frequencies(rot):
    sc = rot.get("scaling")
    f, amp = hops.yarn_inv_freq(
        rot["dims"], rot["base"],
        (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None)
    wf, wamp = O.rot_frequencies(rot)
    assert float((f.double() - wf).abs().max() / wf.abs().max()) < 1e-6
    assert abs(amp - wamp) < 1e-12
    if sc:
        assert amp == pytest.approx(0.1 * math.log(sc["factor"]) + 1.0)


def test_value_blending_reaches_the_cache(tmp_path_factory, backend):
    """The cached values of a blending layer are the blend, the first
    blending layer's are its own: decoding a token after a prompt (which
    reads the cache) equals the whole prompt (which the oracle blends)."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend)
    toks = tokens_for(ck[1], 12, 77)
    replay(eng, {"s": toks}, [[("s", 12)]])
    v1, v5 = eng.kv.v_cache[1], eng.kv.v_cache[5]
    assert float((v1.float() - v5.float()).abs().max()) > 1e-3
    lam = float(ck[2]["l5.mix.vmix"])
    assert 0.05 < lam < 0.95


def test_unused_blend_weight_may_be_present(tmp_path_factory):
    """A layer that does not blend may carry the blend weight all the same;
    the loader takes it and the model ignores it."""
    cfg = config_a()
    w = O.make_weights(cfg, seed=3)
    assert "l4.mix.vmix" not in w
    w["l4.mix.vmix"] = torch.tensor(0.75, dtype=O.F64)
    path = O.save_checkpoint(str(tmp_path_factory.mktemp("extra")), cfg, w)
    ck = (path, cfg, w, {})
    eng = engine(ck, ("cpu", torch.float32))
    seqs = {"s": tokens_for(cfg, 20, 5)}
    check(ck, replay(eng, seqs, [[("s", 20)]]), seqs, torch.float32)


# ------------------------------------------------ the framework's own path --

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
    from sutro_amd.models.hybrid_spec import (AttnMixerSpec, DecayAttnMixerSpec,
                                              HybridSpec, SSDMixerSpec,
                                              nosalorn_spec)
    from sutro_amd.models.registry import get_model_spec

    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    spec = get_model_spec(ck[0])
    assert isinstance(spec, HybridSpec) and spec.arch == "nosalorn"
    kinds = [type(l.mixer) for l in spec.layers]
    assert kinds == [SSDMixerSpec, AttnMixerSpec, DecayAttnMixerSpec,
                     AttnMixerSpec, AttnMixerSpec, AttnMixerSpec, SSDMixerSpec]
    a = spec.layers[1].mixer
    assert (a.window, a.keep_first, a.rot_dims, a.rot_base) == (7, 3, 8, 500.0)
    assert a.rot_scaling == (4.0, 64.0, 8.0, 1.0) and a.v_mix and a.bias
    assert not a.qk_norm and not a.out_gate and not a.sink
    assert spec.layers[3].mixer.rot_scaling is None
    assert spec.layers[4].mixer.window == 0 and not spec.layers[4].mixer.v_mix
    assert spec.layers[2].mixer.decay == (0.7, 0.97)
    s0 = spec.layers[0].mixer
    assert (s0.heads, s0.vdim, s0.state, s0.groups, s0.conv, s0.norm_groups) \
        == (3, 10, 12, 3, 3, 3)
    m = spec.layers[1].moe
    assert (m.experts, m.identity, m.top, m.groups, m.keep) == (5, 4, 3, 3, 2)
    assert (m.route_scale, m.limit, m.shared_ff, m.shared_limit) == \
        (1.7, 1.5, 12, 0.8)
    assert spec.layers[0].ff == 52 and spec.layers[3].ff == 0
    assert spec.layers[3].moe is None and spec.layers[2].moe.shared_ff == 0
    assert spec.embed_scale == 3.0 and spec.logit_scale == 0.5
    assert spec.norm_eps == 1e-5 and not spec.tie_embeddings
    assert spec.param_count() == sum(v.numel() for v in ck[2].values())
    assert spec.active_param_count() < spec.param_count()
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][3]["mixer"]["vdim"] = 16       # blends, but another width
    with pytest.raises(ValueError):
        nosalorn_spec(bad)
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][1]["mlp"]["router"]["top"] = 7  # two groups of three hold six
    with pytest.raises(ValueError):
        nosalorn_spec(bad)
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][2]["type"] = "unheard_of"
    with pytest.raises(ValueError):
        nosalorn_spec(bad)
