"""GPU: the Nodutar design on the layered engine tier (block-local grouped-query attention with
turned values beside a gated linear recurrence, distance-biased attention whose values are its
keys, softmax-routed experts, sandwich norms, a repeated layer group) against the plain numpy
restatement in tests/nodutar_oracle.py, on small random models of several shapes.

fp32 engines are held to REL32 of the logits' spread, bf16 engines to REL16.  Weights are made
peaky where a fault would otherwise hide: large attention scales make single keys carry the
softmax, forget gates near one make far tokens live on in the state.
"""
import numpy as np
import pytest

import nodutar_oracle as O
from nodutar_oracle import dist, par

pytestmark = pytest.mark.gpu

REL32 = 2e-4
REL16 = 5e-2


def words(a):
    """float32 values that are exact bf16 -> bf16 words"""
    return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(np.shape(a))


MIXED = [par(size=9), dist(), par(heads=2, kv_heads=2, dim=8, vdim=16, rot_dims=8, size=33, rheads=2, rdim=40, rvdim=70, mlp=None),
         dist(heads=6, kv_heads=3, dim=6, mlp=("moe", 10, 3, 1))]


class Model:
    def __init__(self, layers, seed=0, vocab=101, width=40, dtype="float32", max_ctx=512, slots=4, page_tokens=16,
                 n_pages=0, eps=1e-5, loop=None, tweak=None):
        import qwen_inference_engine_amd as q
        self.rng = np.random.default_rng(seed)
        self.cfg, self.T = O.random_model(self.rng, vocab=vocab, width=width, layers=layers, loop=loop, eps=eps)
        if tweak is not None:
            tweak(self.T, self.cfg)             # values must stay exact bf16
        self.spec = q.spec_from_config(self.cfg)
        self.eng = q.Engine(self.spec, max_ctx=max_ctx, dtype=dtype).load_tensors({k: words(v) for k, v in self.T.items()})
        self.batch = self.eng.batch(slots, max_ctx, page_tokens=page_tokens, n_pages=n_pages)
        self.vocab, self.dtype = vocab, dtype
        self.tol = REL32 if dtype == "float32" else REL16

    def tokens(self, n):
        return [int(t) for t in self.rng.integers(0, self.vocab, n)]

    def ref(self, toks, layers_out=None):
        return O.forward(self.cfg, self.T, toks, layers_out)

    def close(self):
        self.batch.close()
        self.eng.close()


def rel(got, want):
    d = np.asarray(got, dtype=np.float64) - want
    return float(np.abs(d).max() / (np.std(want) + 1e-30))


def rel_most(got, want, q=0.9):
    """The q-quantile over rows of the per-row root-mean-square error: a bf16 engine may pick another expert than
    the oracle on a near-tie of router logits, which moves single rows by much more than rounding."""
    d = np.sqrt(((np.asarray(got, dtype=np.float64) - want) ** 2).mean(axis=1))
    return float(np.quantile(d, q) / (np.std(want) + 1e-30))


def feed(m, slot, toks, cuts):
    """Feeds toks to `slot` in portions of the sizes in `cuts` (then one by one); logits of all rows."""
    out, pos = [], 0
    sizes = list(cuts)
    while pos < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - pos)
        out.append(m.batch.step([(slot, toks[pos:pos + n])], range(n)))
        pos += n
    return np.concatenate(out)


@pytest.fixture
def model():
    made = []

    def make(*a, **k):
        made.append(Model(*a, **k))
        return made[-1]
    yield make
    for m in made:
        m.close()


def with_mask(cfg, delta):
    """The same config with every block-local mask `delta` positions longer."""
    out = {**cfg, "layers": []}
    for L in cfg["layers"]:
        if L["type"] == "parallel":
            left = {**L["mixer"]["left"], "mask": {"size": L["mixer"]["left"]["mask"]["size"] + delta}}
            L = {**L, "mixer": {**L["mixer"], "left": left}}
        out["layers"].append(L)
    return out


# ------------------------------------------------------------------ mechanisms, one at a time
@pytest.mark.parametrize("layers,loop", [
    ([par(right_scale=0.0, mlp=None)], None),                       # block-local attention with turned values alone
    ([par(right_scale=0.0, rot_dims=12, vdim=12, kv_heads=4, mlp=None)], None),   # every coordinate turns, one key head per query head
    ([par(right_scale=0.0, rot_dims=0, mlp=None)], None),           # no rotation of queries and keys; the values still turn
    ([par(left_scale=0.0, mlp=None)], None),                        # the recurrence alone
    ([par(left_scale=0.0, rheads=1, rdim=70, rvdim=130, mlp=None)], None),   # three row groups, three column tiles
    ([par(mlp=None)], None),
    ([dist(mlp=None)], None),
    ([dist(heads=6, kv_heads=3, mlp=None)], None),
    ([par(mlp=("moe", 14, 5, 2))], None),
    ([dist(mlp=("moe", 14, 4, 4))], None),                          # every expert chosen
    ([dist(mlp=("moe", 14, 6, 1))], None),                          # one expert: its weight is 1
    ([par(mlp=None), dist(mlp=None)], (0, 2, 3)),                   # the whole stack three times
    ([dist(mlp=None), par(), dist()], (1, 2, 2)),                   # a single repeated layer
    ([par(), dist()], (0, 1, 1)),                                   # a group that runs once
], ids=["chunk-attn", "full-rot-mha", "no-qk-rot", "recurrence", "recurrence-wide", "parallel", "distance", "distance-gqa",
        "moe-top2", "moe-all", "moe-top1", "loop-all-x3", "loop-one-x2", "loop-x1"])
def test_mechanism_streams_match_oracle(model, layers, loop):
    m = model(layers, seed=len(layers) + 3, loop=loop)
    toks = m.tokens(29)
    m.batch.keep_layers(True)
    got = m.batch.step([(0, toks)], range(len(toks)))
    want_layers = []
    want = m.ref(toks, want_layers)
    assert len(want_layers) == m.spec.n_runs
    streams = m.batch.step_layers(len(toks))
    for i, w in enumerate(want_layers):
        assert rel(streams[i], w) < REL32, f"stream after layer run {i}"
    assert rel(got, want) < REL32


def test_router_bias_and_ties(model):
    """Identical router rows with equal biases tie: the lower index wins; a bias alone changes the choice."""
    def tw(T, cfg):
        T["l0.mlp.router"][2] = T["l0.mlp.router"][0]
        T["l0.mlp.router.b"][2] = T["l0.mlp.router.b"][0]
        T["l0.mlp.router"][3] = T["l0.mlp.router"][1]
        T["l0.mlp.router.b"][3] = O.bf(T["l0.mlp.router.b"][1] + np.float32(2.0))
    m = model([dist(mlp=("moe", 14, 5, 2))], seed=5, tweak=tw)
    toks = m.tokens(16)
    assert rel(m.batch.step([(0, toks)], range(16)), m.ref(toks)) < REL32


# ------------------------------------------------------------------ prompts, portions, decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree(model, dtype):
    # bf16: an expert chosen differently on a near-tie changes that row's keys for every later query of the causal
    # layers, so only the last layer routes there; fp32 keeps every feed-forward
    layers = MIXED if dtype == "float32" else [{**L, "mlp": None} for L in MIXED[:3]] + MIXED[3:]
    m = model(layers, seed=11, dtype=dtype, loop=(1, 3, 2))
    toks = m.tokens(90)
    want = m.ref(toks)
    err = rel if dtype == "float32" else rel_most
    whole = m.batch.step([(0, toks)], range(len(toks)))
    assert err(whole, want) < m.tol
    single = feed(m, 1, toks, [])               # token by token from the first token on
    assert err(single, want) < m.tol
    parts = feed(m, 2, toks, [2, 3, 11, 2, 17, 16, 2, 30])   # cut inside pages and blocks, down to two tokens
    assert err(parts, want) < m.tol
    bound = 5e-5 if dtype == "float32" else 2e-2
    assert err(single, whole) < bound and err(parts, whole) < bound


def test_unequal_requests_in_one_step_equal_each_alone(model):
    m = model(MIXED, seed=12, slots=4, loop=(0, 2, 2))
    reqs = [m.tokens(n) for n in (41, 7, 64, 18)]
    want = [m.ref(t) for t in reqs]
    pos = [0, 0, 0, 0]
    plan = [[(0, 16), (1, 7), (2, 33), (3, 2)], [(0, 1), (2, 31), (3, 16)], [(0, 24)]]
    for step in plan:
        entries = [(r, reqs[r][pos[r]:pos[r] + n]) for r, n in step]
        got = m.batch.step(entries, range(sum(n for _, n in step)))
        row = 0
        for r, n in step:
            assert rel(got[row:row + n], want[r][pos[r]:pos[r] + n]) < REL32, (r, pos[r], n)
            row += n
            pos[r] += n


def long_memory(T, cfg):
    """Forget gates close to one: what the state took in long ago still shapes the output."""
    for k in T:
        if k.endswith("right.lower"):
            T[k][:] = O.bf(0.97 + 0.029 * np.linspace(0, 1, T[k].size))


def test_slots_pages_and_states_are_reused(model):
    """A pool smaller than the sum of all requests: finished requests give pages and slots back, later ones take
    them; neither stale rows nor the previous owner's recurrent state may leak."""
    m = model([par(size=13, left_scale=0.3, right_scale=1.0), par(size=5, left_scale=0.3, right_scale=1.0, mlp=None)], seed=13, slots=2,
              page_tokens=16, n_pages=8, tweak=long_memory)
    free0, _, pt = m.batch.page_stats()
    assert (free0, pt) == (7, 16)
    # the oracle itself must carry the first token to the last row, which only the state can do here
    a = m.tokens(60)
    a2 = [(a[0] + 1) % m.vocab] + a[1:]
    assert rel(m.ref(a2)[-1:], m.ref(a)[-1:]) > 50 * REL32
    for round_ in range(4):
        a, b = m.tokens(60 + round_), m.tokens(37)
        ga = m.batch.step([(0, a[:50]), (1, b)], range(50 + 37))
        gb = m.batch.step([(0, a[50:])], range(len(a) - 50))
        assert rel(np.concatenate([ga[:50], gb]), m.ref(a)) < REL32
        assert rel(ga[50:], m.ref(b)) < REL32
        with pytest.raises(Exception):
            m.batch.step([(1, m.tokens(40))])         # 4 + 3 pages held: no room for 2 more
        m.batch.release(0)
        m.batch.release(1)
        assert m.batch.page_stats()[0] == 7


# ------------------------------------------------------------------ block edges, far keys
def test_block_edges_in_prompt_and_decoding(model):
    """Peaky attention: the first key of a block is seen by its last query and by nothing after it, for blocks
    shorter than, equal to and longer than a page, in prompts and while decoding."""
    for size in (3, 16, 21):
        m = model([par(size=size, scale=4.0, right_scale=0.05, mlp=None), par(size=size + 2, scale=4.0, right_scale=0.05, mlp=None)],
                  seed=20 + size, page_tokens=16)
        toks = m.tokens(3 * size + 19)
        want = m.ref(toks)
        for delta in (1, -1):                   # the oracle itself reacts to the edge
            assert rel(O.forward(with_mask(m.cfg, delta), m.T, toks), want) > 50 * REL32
        assert rel(m.batch.step([(0, toks)], range(len(toks))), want) < REL32
        assert rel(feed(m, 1, toks, [size + 5]), want) < REL32     # block edges pass while decoding
        assert rel(feed(m, 2, toks, [size - 1, 2, size, 2]), want) < REL32


def test_far_key_dominates_across_pages(model):
    """Distance-biased causal attention with a large score scale and a weak bias: single keys many pages back carry
    the softmax; prompts and 90 decoded tokens follow the oracle."""
    def tw(T, cfg):
        T["l0.mix.r1"][:] = O.bf(0.05 * np.ones_like(T["l0.mix.r1"]))
    m = model([dist(heads=2, kv_heads=1, dim=8, scale=5.0, mlp=None)], seed=31, width=24, page_tokens=16, max_ctx=256, tweak=tw)
    toks = m.tokens(150)
    want = m.ref(toks)
    assert rel(m.batch.step([(0, toks)], range(150)), want) < REL32
    assert rel(feed(m, 1, toks, [60]), want) < REL32


def test_distance_bias_shapes_the_scores(model):
    """A strong bias: leaving it out, or measuring the distance one off, moves the oracle far more than the
    engine is allowed to differ."""
    def tw(T, cfg):
        T["l0.mix.r1"][:] = O.bf(np.array([3.0, 0.5, 2.0, 1.0]))
        T["l0.mix.r2"][:] = O.bf(np.array([0.25, 4.0, 1.0, 0.125]))
    m = model([dist(mlp=None)], seed=33, tweak=tw)
    toks = m.tokens(70)
    want = m.ref(toks)
    T0 = {**m.T, "l0.mix.r1": np.zeros_like(m.T["l0.mix.r1"])}
    assert rel(O.forward(m.cfg, T0, toks), want) > 50 * REL32
    assert rel(m.batch.step([(0, toks)], range(70)), want) < REL32
    assert rel(feed(m, 1, toks, [17, 2]), want) < REL32


def test_first_tokens_and_single_token_request(model):
    m = model(MIXED, seed=41, loop=(1, 3, 2))
    for n in (1, 2, 3):
        toks = m.tokens(n)
        assert rel(m.batch.step([(0, toks)], range(n)), m.ref(toks)) < REL32
        m.batch.release(0)


def test_long_decoding_over_many_pages(model):
    m = model([par(size=19, mlp=("moe", 14, 6, 2)), dist(mlp=None), par(size=40, heads=3, kv_heads=1)], seed=51, page_tokens=16,
              max_ctx=400, loop=(0, 2, 2), tweak=long_memory)
    toks = m.tokens(330)
    assert rel(feed(m, 0, toks, [9]), m.ref(toks)) < REL32


def test_long_portions_scan_in_pieces(model):
    """Entries of more than 128 rows run the recurrence in pieces of 64 rows side by side and carry the states
    across afterwards: from a fresh state, from a state left by an earlier portion, beside short entries of other
    requests, with gates close to one so that every piece's incoming state matters."""
    m = model([par(size=50, left_scale=0.2, right_scale=1.0, rheads=2, rdim=40, rvdim=70), dist(mlp=None),
               par(size=7, left_scale=0.2, right_scale=1.0, mlp=None)], seed=55, page_tokens=16, max_ctx=512, loop=(0, 2, 2),
              tweak=long_memory)
    toks, other, third = m.tokens(400), m.tokens(30), m.tokens(140)
    want, want_o, want_t = m.ref(toks), m.ref(other), m.ref(third)
    assert rel(m.batch.step([(0, toks)], range(400)), want) < REL32                      # 7 pieces from zero
    a = m.batch.step([(1, toks[:150])], range(150))                                      # 3 pieces, the last one short
    b1 = m.batch.step([(2, other[:29])], range(29))
    b = m.batch.step([(1, toks[150:379]), (2, other[29:]), (3, third)], range(229 + 1 + 140))   # pieces from a kept state
    c = feed(m, 1, toks[379:], [2])
    assert rel(np.concatenate([a, b[:229], c]), want) < REL32
    assert rel(np.concatenate([b1, b[229:230]]), want_o) < REL32
    assert rel(b[230:], want_t) < REL32


def test_other_sizes(model):
    """Sizes and constants unlike the shapes above: odd head sizes, one head, many heads, vdim above and below
    dim, a rotary extent of 2, top 3 of 7, different scales per side."""
    layers = [par(heads=5, kv_heads=5, dim=14, vdim=6, rot_dims=2, base=50.0, size=12, rheads=5, rdim=3, rvdim=5,
                  left_scale=1.3, right_scale=0.2, mlp=("moe", 9, 7, 3)),
              dist(heads=1, kv_heads=1, dim=33, mlp=("moe", 130, 2, 2)),
              par(heads=8, kv_heads=2, dim=4, vdim=30, rot_dims=4, base=1e6, size=64, rheads=1, rdim=33, rvdim=64, mlp=None)]
    m = model(layers, seed=61, vocab=67, width=52)
    toks = m.tokens(70)
    assert rel(feed(m, 0, toks, [33, 2, 20]), m.ref(toks)) < REL32


@pytest.mark.parametrize("hd,size,page", [(32, 21, 32), (64, 40, 64), (128, 70, 32), (64, 33, 16)],
                         ids=["hd32", "hd64", "hd128", "hd64-page16"])
def test_bf16_matrix_shapes(model, hd, size, page):
    """Sizes that take the bf16 matrix kernels (pages of 32 or more tokens: attention on the matrix cores over
    transposed value rows, key splits while decoding; pages of 16: the plain attention): whole prompts, portions
    and single tokens against the oracle, beside another request, with more than 256 routed rows in one step."""
    # pages of 64: 8 heads over 2 key heads (the four waves of a workgroup share their key head's tiles); else 4 over 2
    layers = [par(heads=8 if page == 64 else 4, kv_heads=2, dim=hd, vdim=hd, rot_dims=hd // 2, size=size, scale=0.5, rheads=2, rdim=32,
                  rvdim=64, mlp=("moe", 32, 4, 2)),
              dist(heads=4, kv_heads=1, dim=hd, scale=1.0, mlp=("moe", 96, 4, 2))]
    m = model(layers, seed=hd, vocab=160, width=64, dtype="bfloat16", page_tokens=page, max_ctx=512, loop=(0, 1, 2))
    toks = m.tokens(150)
    want = m.ref(toks)
    assert rel_most(O.forward(with_mask(m.cfg, 1), m.T, toks), want, 0.97) > 2 * REL16
    whole = m.batch.step([(0, toks)], range(len(toks)))
    assert rel_most(whole, want) < REL16
    parts = feed(m, 1, toks, [2, 45, 19, 64])
    assert rel_most(parts, want) < REL16
    other = m.tokens(140)
    got = m.batch.step([(2, other), (3, toks[:130])], range(140 + 130))
    assert rel_most(got[:140], m.ref(other)) < REL16
    assert rel_most(got[140:], want[:130]) < REL16
    rest = feed(m, 3, toks[130:], [])
    assert rel_most(rest, want[130:]) < REL16


# ------------------------------------------------------------------ generation through the scheduler
def oracle_greedy(m, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(m.ref(toks)[-1]))
        out.append(t)
        toks.append(t)
    return out


def test_greedy_generation_through_the_batcher(model):
    """Five requests through ContinuousBatcher (two slots, a small page pool, 24-row steps): prompts are read in
    portions beside decoding requests, finished requests free their slot, pages and state for the waiting ones."""
    from qwen_inference_engine_amd.scheduler import ContinuousBatcher
    m = model(MIXED, seed=71, dtype="float32", loop=(1, 3, 2))
    m.batch.close()
    cb = ContinuousBatcher(m.eng, slots=2, max_ctx=128, page_tokens=16, n_pages=9, chunk_tokens=24, keep_logits=True)
    m.batch = cb.batch
    prompts = [m.tokens(n) for n in (30, 5, 50, 1, 17)]
    gens = [6, 9, 4, 7, 5]
    rids = [cb.submit(p, g) for p, g in zip(prompts, gens)]
    out = cb.run()
    for p, g, rid in zip(prompts, gens, rids):
        want = oracle_greedy(m, p, g)
        got = out[rid]
        assert len(got) == g
        if got != want:   # a near-tie may flip: the logits must then be within rounding of the oracle's
            k = next(i for i in range(g) if got[i] != want[i])
            lg = m.ref(list(p) + want[:k])[-1]
            assert abs(lg[got[k]] - lg[want[k]]) < 1e-4 * np.std(lg), (rid, k)
    assert cb.batch.page_stats()[0] == 8


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_steps_replay_graphs_equal_eager(dtype):
    """Decoding steps of one shape are captured once and replayed, with eager work of other shapes and a release
    in between; every replayed step's logits equal those of an engine without graphs bit for bit."""
    import qwen_inference_engine_amd as q
    layers = MIXED if dtype == "float32" else [{**L, "mlp": None} for L in MIXED[:3]] + MIXED[3:]
    a = Model(layers, seed=91, dtype=dtype, loop=(1, 3, 2))
    b = Model(layers, seed=91, dtype=dtype, loop=(1, 3, 2))
    b.batch.close()
    b.eng.close()
    b.eng = q.Engine(b.spec, max_ctx=512, dtype=dtype, use_graph=False).load_tensors({k: words(v) for k, v in b.T.items()})
    b.batch = b.eng.batch(4, 512, page_tokens=16)
    try:
        toks, other = a.tokens(60), a.tokens(40)
        for m in (a, b):
            m.out, m.tail = [m.batch.step([(0, toks[:20]), (1, other[:11])], [19, 30])], []
            for i in range(20, 60):
                if i % 7 == 0:
                    m.out.append(m.batch.step([(2, other[:5])], [4]))
                    m.batch.release(2)
                if i < 40:
                    entries, want = [(0, [toks[i]]), (1, [other[i - 9]])], [0, 1]
                else:
                    entries, want = [(0, [toks[i]])], [0]
                m.out.append(m.batch.step(entries, want))
                if i >= 40:
                    m.tail.append(m.out[-1][0])
        assert a.batch.graph_stats()[0] >= 2 and a.batch.graph_stats()[1] >= 30
        assert b.batch.graph_stats() == (0, 0)
        for x, y in zip(a.out, b.out):
            assert np.array_equal(x, y)
        assert (rel if dtype == "float32" else rel_most)(np.stack(a.tail), a.ref(toks)[40:60]) < a.tol
    finally:
        a.close()
        b.close()


# ------------------------------------------------------------------ the command-line programs
def write_model_dir(path, cfg, T):
    import json
    import struct
    hdr, blob = {}, b""
    for name, v in T.items():
        raw = words(v).tobytes()
        hdr[name] = {"dtype": "BF16", "shape": list(np.shape(v)), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    hj = json.dumps(hdr).encode()
    (path / "config.json").write_text(json.dumps(cfg))
    (path / "model.safetensors").write_bytes(struct.pack("<Q", len(hj)) + hj + blob)


def test_trace_replay_and_generate_programs(tmp_path):
    """bin/trace_run replays interleaved requests (portions beside single tokens, a slot, its pages and its state
    used again) and writes the wanted logits; bin/qie generates greedily: both equal the oracle."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    rng = np.random.default_rng(81)
    cfg, T = O.random_model(rng, vocab=89, width=40, layers=MIXED, loop=(1, 3, 2))
    write_model_dir(tmp_path, cfg, T)
    reqs = {k: [int(t) for t in rng.integers(0, 89, n)] for k, n in (("a", 70), ("b", 9), ("c", 33), ("d", 50), ("e", 64))}
    want = {k: O.forward(cfg, T, v) for k, v in reqs.items()}
    plan = [[("a", 0, 40), ("b", 0, 9)], [("a", 40, 2), ("c", 0, 33), ("d", 0, 17)], [("a", 42, 1), ("d", 17, 33)],
            [("a", 43, 27), ("e", 0, 64)]]
    last = {k: max(p[1] + p[2] for st in plan for p in st if p[0] == k) for k in reqs}
    lines, rows = [], []
    for n, st in enumerate(plan):
        entries, end, r = [], [], []
        for k, lo, cnt in st:
            w = list(range(0, cnt, 3)) + ([cnt - 1] if (cnt - 1) % 3 else [])
            entries.append({"id": k, "tokens": reqs[k][lo:lo + cnt], "want": w})
            r += [(k, lo + i) for i in w]
            if lo + cnt == last[k]:
                end.append(k)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        rows.append(r)
    for dtype, tol, err in (("float32", REL32, rel), ("bfloat16", REL16, rel_most)):
        out = tmp_path / ("out_" + dtype)
        r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "256"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
        for n, rr in enumerate(rows):
            got = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rr), 89)
            ref = np.stack([want[k][i] for k, i in rr])
            assert err(got, ref) < tol, (dtype, n)
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "qie"), "--model", str(tmp_path), "--dtype", "float32", "--gen", "5",
                        "--prompt", ",".join(map(str, reqs["b"])), "--prompt", " ".join(map(str, reqs["c"])), "--slots", "2",
                        "--chunk-tokens", "16"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    got = {l.split(":")[0]: [int(t) for t in l.split(":")[1].split()] for l in r.stdout.splitlines() if l.startswith("tokens[")}

    class M:
        ref = staticmethod(lambda toks: O.forward(cfg, T, toks))
    assert got["tokens[0]"] == oracle_greedy(M, reqs["b"], 5)
    assert got["tokens[1]"] == oracle_greedy(M, reqs["c"], 5)
