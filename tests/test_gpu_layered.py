"""GPU: the layered engine tier (latent attention, routed experts, output-side scalar norms,
depth-weighted residuals; ragged paged steps) against the plain numpy restatement in
tests/layered_oracle.py, on small random models of several shapes.

fp32 engines are held to REL32 of the logits' spread, bf16 engines to REL16 (bf16 operand
rounding over a few layers).  Random weights are made peaky where a fault would otherwise hide:
a larger attention scale or boosted queries make single keys carry visible weight.
"""
import numpy as np
import pytest

import layered_oracle as O

pytestmark = pytest.mark.gpu

REL32 = 2e-4
REL16 = 5e-2


def words(a):
    """float32 values that are exact bf16 -> bf16 words"""
    return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(np.shape(a))


def att(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=20, window=7, kv_from=None, mlp=None, base=100.0, scale=None):
    d = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, window=window, kv_from=kv_from, mlp=mlp,
             base=base)
    if scale is not None:
        d["scale"] = scale
    return d


MIXED = [att(window=9, mlp=("dense", 28)),
         att(window=5, kv_from=0, mlp=("moe", 14, 5, 2)),
         att(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=24, window=33, mlp=None),
         att(heads=2, dim=8, rot_dim=8, vdim=6, kv_rank=24, window=4, kv_from=2, mlp=("moe", 10, 3, 1))]


class Model:
    def __init__(self, layers, seed=0, vocab=101, width=40, dtype="float32", max_ctx=512, slots=4, page_tokens=16,
                 n_pages=0, eps=1e-5, tweak=None):
        import qwen_inference_engine_amd as q
        self.rng = np.random.default_rng(seed)
        self.cfg, self.T = O.random_model(self.rng, vocab=vocab, width=width, layers=layers, eps=eps)
        if tweak is not None:
            tweak(self.T)                       # values must stay exact bf16
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
    the oracle on a near-tie of router scores, which moves single rows by much more than rounding."""
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


# ------------------------------------------------------------------ mechanisms, one at a time
@pytest.mark.parametrize("layers", [
    [att(mlp=None)],                                        # attention, output norm, depth mix alone
    [att(rot_dim=0, mlp=None)],                             # no rotated part at all
    [att(mlp=("dense", 28))],
    [att(mlp=("moe", 14, 5, 2))],
    [att(mlp=("moe", 14, 4, 4))],                           # every expert chosen
    [att(mlp=None), att(kv_from=0, window=3, vdim=4, mlp=None)],   # borrowed cache rows, own window
], ids=["attention", "no-rotary", "dense", "moe-top2", "moe-all", "kv-from"])
def test_mechanism_streams_match_oracle(model, layers):
    m = model(layers, seed=len(layers) + layers[0]["rot_dim"])
    toks = m.tokens(23)
    m.batch.keep_layers(True)
    got = m.batch.step([(0, toks)], range(len(toks)))
    want_layers = []
    want = m.ref(toks, want_layers)
    streams = m.batch.step_layers(len(toks))
    for i, w in enumerate(want_layers):
        assert rel(streams[i], w) < REL32, f"stream after layer {i}"
    assert rel(got, want) < REL32


def test_router_prefers_lower_index_on_equal_scores(model):
    """Two identical router rows give equal scores: the lower expert index is chosen."""
    def same_rows(T):
        T["l0.mlp.router"][2] = T["l0.mlp.router"][0]
        T["l0.mlp.router"][3] = T["l0.mlp.router"][1]
    m = model([att(mlp=("moe", 14, 4, 1))], seed=5, tweak=same_rows)
    toks = m.tokens(12)
    assert rel(m.batch.step([(0, toks)], range(12)), m.ref(toks)) < REL32


# ------------------------------------------------------------------ prompts, portions, decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree(model, dtype):
    m = model(MIXED, seed=11, dtype=dtype)
    toks = m.tokens(90)
    want = m.ref(toks)
    err = rel if dtype == "float32" else rel_most
    whole = m.batch.step([(0, toks)], range(len(toks)))
    assert err(whole, want) < m.tol
    # token by token from the first token on
    single = feed(m, 1, toks, [])
    assert err(single, want) < m.tol
    # portions of changing size, down to two tokens, cut inside pages and windows
    parts = feed(m, 2, toks, [2, 3, 11, 2, 17, 16, 2, 30])
    assert err(parts, want) < m.tol
    # the same position must not depend on the cut beyond rounding
    # (few rows and many rows take kernels that sum in different orders)
    bound = 5e-5 if dtype == "float32" else 2e-2
    assert err(single, whole) < bound and err(parts, whole) < bound


def test_unequal_requests_in_one_step_equal_each_alone(model):
    m = model(MIXED, seed=12, slots=4)
    reqs = [m.tokens(n) for n in (41, 7, 64, 18)]
    want = [m.ref(t) for t in reqs]
    # step 1: portions of different sizes; later steps: one decoding beside prompt portions
    pos = [0, 0, 0, 0]
    plan = [[(0, 16), (1, 7), (2, 33), (3, 2)], [(0, 1), (2, 31), (3, 16)], [(0, 24)]]
    for step in plan:
        entries, rows = [], []
        for r, n in step:
            entries.append((r, reqs[r][pos[r]:pos[r] + n]))
        got = m.batch.step(entries, range(sum(n for _, n in step)))
        row = 0
        for r, n in step:
            assert rel(got[row:row + n], want[r][pos[r]:pos[r] + n]) < REL32, (r, pos[r], n)
            row += n
            pos[r] += n


def test_slots_and_pages_are_reused(model):
    """A pool smaller than the sum of all requests: finished requests give their pages back
    and later ones take the same slots and pages; stale rows must not leak."""
    m = model(MIXED, seed=13, slots=2, page_tokens=16, n_pages=8)   # 7 pages = 112 tokens
    free0, _, pt = m.batch.page_stats()
    assert (free0, pt) == (7, 16)
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


# ------------------------------------------------------------------ window edges, far keys
def test_window_edges_in_prompt_and_decoding(model):
    """Peaky attention (scale x 6): the key at distance window - 1 is seen, the one at distance
    window is not — for windows shorter than, equal to and longer than a page."""
    for window in (3, 16, 21):
        layers = [att(window=window, scale=1.5, mlp=None), att(window=window + 2, scale=1.5, kv_from=0, mlp=None)]
        m = model(layers, seed=20 + window, page_tokens=16)
        toks = m.tokens(3 * window + 19)
        want = m.ref(toks)
        # the oracle itself must react to the edge (else this test shows nothing)
        cfg2 = {**m.cfg, "layers": [{**L, "mixer": {**L["mixer"], "mask": {"size": L["mixer"]["mask"]["size"] + 1}}}
                                    for L in m.cfg["layers"]]}
        assert rel(O.forward(cfg2, m.T, toks), want) > 50 * REL32
        assert rel(m.batch.step([(0, toks)], range(len(toks))), want) < REL32
        cut = window + 5
        assert rel(feed(m, 1, toks, [cut]), want) < REL32          # the window passes over decoded tokens


def test_far_key_dominates_across_pages(model):
    """Queries boosted 4x make single far keys dominate the softmax: the logits follow the
    oracle while such a key is inside the window (several pages back) and after it has left."""
    def boost(T):
        T["l0.mix.q"] *= 4.0                    # a power of two keeps the values exact bf16
    layers = [att(heads=2, dim=8, rot_dim=0, vdim=8, kv_rank=16, window=70, scale=1.0, mlp=None)]
    m = model(layers, seed=31, width=24, page_tokens=16, max_ctx=256, tweak=boost)
    toks = m.tokens(150)
    want = m.ref(toks)
    assert rel(m.batch.step([(0, toks)], range(150)), want) < REL32
    assert rel(feed(m, 1, toks, [60]), want) < REL32           # 90 decoded tokens, the window leaves the prompt


def test_first_tokens_and_single_token_request(model):
    m = model(MIXED, seed=41)
    for n in (1, 2, 3):
        toks = m.tokens(n)
        assert rel(m.batch.step([(0, toks)], range(n)), m.ref(toks)) < REL32
        m.batch.release(0)


def test_long_decoding_over_many_pages(model):
    m = model([att(window=19, mlp=("moe", 14, 6, 2)), att(window=40, kv_from=0, mlp=("dense", 20))], seed=51,
              page_tokens=16, max_ctx=400)
    toks = m.tokens(330)
    want = m.ref(toks)
    assert rel(feed(m, 0, toks, [9]), want) < REL32


def test_other_sizes_wide_latent_and_many_heads(model):
    layers = [att(heads=5, dim=16, rot_dim=4, vdim=7, kv_rank=300, window=12, mlp=("moe", 9, 7, 3), base=50.0),
              att(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5, window=64, mlp=("dense", 130))]
    m = model(layers, seed=61, vocab=67, width=52)
    toks = m.tokens(70)
    assert rel(feed(m, 0, toks, [33, 2, 20]), m.ref(toks)) < REL32


# ------------------------------------------------------------------ bf16 engines on the matrix cores
@pytest.mark.parametrize("heads,kv_rank,rot_dim,window", [(4, 32, 8, 21), (16, 144, 16, 40), (20, 272, 8, 33), (3, 48, 0, 37)],
                         ids=["4h-r32", "16h-r144", "20h-r272", "3h-r48-norot"])
def test_bf16_matrix_core_shapes(model, heads, kv_rank, rot_dim, window):
    """Sizes that take the bf16 MFMA kernels (products through the GEMM / GEMV kernels, attention
    on the matrix cores with the key-interleaved cache copy): whole prompts, portions and single
    tokens against the oracle, with a peaky softmax so that a wrong edge or a lost key shows."""
    layers = [att(heads=heads, dim=16, rot_dim=rot_dim, vdim=8, kv_rank=kv_rank, window=window, scale=0.6,
                  mlp=("moe", 32, 4, 2)),
              att(heads=heads, dim=16, rot_dim=rot_dim, vdim=24, kv_rank=kv_rank, window=window // 2 + 1, scale=0.6, kv_from=0,
                  mlp=("dense", 96))]
    m = model(layers, seed=heads + kv_rank, vocab=160, width=64, dtype="bfloat16", page_tokens=16, max_ctx=512)
    toks = m.tokens(150)
    want = m.ref(toks)
    cfg2 = {**m.cfg, "layers": [{**L, "mixer": {**L["mixer"], "mask": {"size": L["mixer"]["mask"]["size"] + 1}}}
                                for L in m.cfg["layers"]]}
    assert rel_most(O.forward(cfg2, m.T, toks), want, 0.97) > 2 * REL16   # the oracle itself reacts to the edge
    whole = m.batch.step([(0, toks)], range(len(toks)))
    assert rel_most(whole, want) < REL16
    parts = feed(m, 1, toks, [2, 45, 19, 64])                          # then 20 single tokens
    assert rel_most(parts, want) < REL16
    # beside another request, with a step of more than 256 routed rows (experts on the MFMA kernels)
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
    """Five requests through ContinuousBatcher (two slots, a small page pool, 24-row steps):
    prompts are read in portions beside decoding requests, finished requests free their slot
    and pages for the waiting ones; greedy tokens equal the oracle's."""
    from qwen_inference_engine_amd.scheduler import ContinuousBatcher
    m = model(MIXED, seed=71, dtype="float32")
    m.batch.close()
    cb = ContinuousBatcher(m.eng, slots=2, max_ctx=128, page_tokens=16, n_pages=9, chunk_tokens=24, keep_logits=True)
    m.batch = cb.batch                          # closed with the model, before its engine
    prompts = [m.tokens(n) for n in (30, 5, 50, 1, 17)]
    gens = [6, 9, 4, 7, 5]
    rids = [cb.submit(p, g) for p, g in zip(prompts, gens)]
    out = cb.run()
    for p, g, rid in zip(prompts, gens, rids):
        want = oracle_greedy(m, p, g)
        got = out[rid]
        assert len(got) == g
        if got != want:   # a near-tie may flip: the kept logits must then be within rounding of the oracle's
            k = next(i for i in range(g) if got[i] != want[i])
            lg = m.ref(list(p) + want[:k])[-1]
            assert abs(lg[got[k]] - lg[want[k]]) < 1e-4 * np.std(lg), (rid, k)
    assert cb.batch.page_stats()[0] == 8


# ------------------------------------------------------------------ graph replays of small steps
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_steps_replay_graphs_equal_eager(dtype):
    """Decoding steps of one shape are captured once and replayed; between the replays the
    program does its own eager work (a prompt portion of another request, a release, a step of
    another shape).  Every replayed step's logits equal the eager engine's bit for bit."""
    a = Model(MIXED, seed=91, dtype=dtype)
    b = Model(MIXED, seed=91, dtype=dtype)
    b.batch.close()
    b.eng.close()
    import qwen_inference_engine_amd as q
    b.eng = q.Engine(b.spec, max_ctx=512, dtype=dtype, use_graph=False).load_tensors({k: words(v) for k, v in b.T.items()})
    b.batch = b.eng.batch(4, 512, page_tokens=16)
    try:
        toks = a.tokens(60)
        other = a.tokens(40)
        for m in (a, b):
            m.out, m.tail = [m.batch.step([(0, toks[:20]), (1, other[:11])], [19, 30])], []
            for i in range(20, 60):
                if i % 7 == 0:                     # eager work between replays: another shape
                    m.out.append(m.batch.step([(2, other[:5])], [4]))
                    m.batch.release(2)
                if i < 40:
                    entries, want = [(0, [toks[i]]), (1, [other[i - 9]])], [0, 1]
                else:                              # then single-row steps (a second graph)
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
    """config.json + model.safetensors (8-byte header length, JSON header, bf16 data)."""
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
    """bin/trace_run replays interleaved requests (portions beside single tokens, a slot and its
    pages used again) and writes the wanted logits; bin/qie generates greedily: both equal the oracle."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    rng = np.random.default_rng(81)
    cfg, T = O.random_model(rng, vocab=89, width=40, layers=MIXED)
    write_model_dir(tmp_path, cfg, T)
    reqs = {k: [int(t) for t in rng.integers(0, 89, n)] for k, n in (("a", 70), ("b", 9), ("c", 33), ("d", 50), ("e", 64))}
    want = {k: O.forward(cfg, T, v) for k, v in reqs.items()}
    plan = [[("a", 0, 40), ("b", 0, 9)], [("a", 40, 2), ("c", 0, 33), ("d", 0, 17)], [("a", 42, 1), ("d", 17, 33)],
            [("a", 43, 27), ("e", 0, 64)]]            # 'e' takes the slot and pages that 'b' or 'c' gave back
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
    lines.insert(2, json.dumps({"step": 77, "entries": [], "end": []}))      # a step that brings nothing
    for dtype, tol, err in (("float32", REL32, rel), ("bfloat16", REL16, rel_most)):
        out = tmp_path / ("out_" + dtype)
        r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "256"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 77", "done 2", "done 3"]
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
