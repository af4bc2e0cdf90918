"""CPU: the host side of the layered engine tier — config reader and model registry, checkpoint
tensor names, the safetensors reader, the ragged planner of ContinuousBatcher (on a fake batch),
and the oracle's own algebra (the absorbed form of latent attention that the engine runs equals
the expanded form the oracle states)."""
import json
import struct

import numpy as np
import pytest

import layered_oracle as O
from qwen_inference_engine_amd import spec as S
from qwen_inference_engine_amd.scheduler import ContinuousBatcher
from qwen_inference_engine_amd.weights import read_safetensors


def small_cfg():
    rng = np.random.default_rng(3)
    layers = [dict(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=20, window=7, mlp=("dense", 28)),
              dict(heads=3, dim=12, rot_dim=6, vdim=5, kv_rank=20, window=4, kv_from=0, mlp=("moe", 14, 5, 2)),
              dict(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, window=11, mlp=None)]
    return O.random_model(rng, vocab=61, width=24, layers=layers)


def test_config_reader_and_registry():
    cfg, T = small_cfg()
    spec = S.spec_from_config(json.loads(json.dumps(cfg)), name="t")
    assert isinstance(spec, S.LayeredSpec) and spec.n_layers == 3 and (spec.width, spec.vocab) == (24, 61)
    m0, m1, m2 = (L.mixer for L in spec.layers)
    assert (m0.kv_from, m1.kv_from, m1.window, m1.vdim) == (None, 0, 4, 5)
    assert m0.rot_dims == 6 and m2.rot_base == 10000.0
    assert spec.layers[0].mlp == S.FeedForward("dense", 28)
    assert spec.layers[1].mlp == S.FeedForward("moe", 14, 5, 2)
    assert spec.layers[2].mlp is None
    # every checkpoint tensor the oracle model has is named with its shape, and nothing else
    shapes = spec.tensor_shapes()
    assert set(shapes) == set(T)
    for k, v in T.items():
        assert list(np.shape(v)) == shapes[k], k
    assert "l1.mix.dkv" not in shapes and "l2.norm2" not in shapes
    arch, keep = spec.to_c()
    assert arch.n_layers == 3 and keep[1].kv_from == 0 and keep[0].kv_from == -1 and keep[2].ff_kind == 0
    assert spec.cache_row_elems() == 26 + 20
    with pytest.raises(ValueError):
        S.spec_from_config({"architecture": "Nonesuch"})
    with pytest.raises(ValueError):
        S.spec_from_config({**cfg, "layers": [{**cfg["layers"][0], "type": "other"}]})
    # a HuggingFace Qwen config still gives the Qwen decoder spec
    hf = dict(model_type="qwen2", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
              intermediate_size=128, vocab_size=100)
    assert isinstance(S.spec_from_config(hf), S.ModelSpec)


def test_safetensors_reader(tmp_path):
    a = np.arange(12, dtype=np.uint16).reshape(3, 4)
    b = np.asarray(7, dtype=np.uint16)
    c = np.arange(5, dtype=np.int32)
    hdr, blob = {}, b""
    for name, arr, dt in (("a", a, "BF16"), ("s", b, "BF16"), ("t", c, "I32")):
        raw = arr.tobytes()
        hdr[name] = {"dtype": dt, "shape": list(arr.shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    hj = json.dumps({"__metadata__": {"x": "y"}, **hdr}).encode()
    p = tmp_path / "m.safetensors"
    p.write_bytes(struct.pack("<Q", len(hj)) + hj + blob)
    got = read_safetensors(str(p))
    assert set(got) == {"a", "s", "t"}
    assert got["a"][0] == 0 and np.array_equal(got["a"][1], a)
    assert got["s"][1].shape == () and int(got["s"][1]) == 7
    assert got["t"][0] == 1 and np.array_equal(got["t"][1], c)


# ------------------------------------------------------------------ the ragged planner
class FakeBatch:
    def __init__(self, slots, max_ctx, page_tokens, n_pages):
        self.B, self.max_ctx, self.pt, self.free = slots, max_ctx, page_tokens, n_pages - 1
        self.steps, self.released = [], []

    def page_stats(self):
        return self.free, np.zeros(self.B, np.int32), self.pt

    def step(self, entries, want, fetch=True):
        self.steps.append(([(s, list(t)) for s, t in entries], list(want)))
        self.n = len(want)
        return None

    def step_sample(self, sampling):
        return [1000 + len(self.steps)] * self.n

    def release(self, slot):
        self.released.append(slot)

    def close(self):
        pass


class FakeEngine:
    layered = True

    def batch(self, slots, max_ctx, page_tokens=None, n_pages=0):
        self.b = FakeBatch(slots, max_ctx, page_tokens, n_pages)
        return self.b


def test_ragged_planner_budget_order_and_completion():
    eng = FakeEngine()
    cb = ContinuousBatcher(eng, slots=2, max_ctx=256, page_tokens=16, n_pages=12, chunk_tokens=10)
    r0 = cb.submit(list(range(100, 123)), 3)       # 23-token prompt
    r1 = cb.submit([7, 8, 9], 2)
    r2 = cb.submit([5], 2)                          # waits for a slot
    out = cb.run()
    # steps 1-2 read 20 tokens of r0; step 3 ends both prompts; r2 takes r1's slot once r1 is done
    assert out == {r0: [1003, 1004, 1005], r1: [1003, 1004], r2: [1005, 1006]}
    steps = eng.b.steps
    # step 1: both prompts are new; the budget of 10 rows goes to slot 0 first, nothing is left for slot 1
    assert steps[0] == ([(0, list(range(100, 110)))], [])
    # every step stays within 10 rows, entries in slot order
    for entries, want in steps:
        assert sum(len(t) for _, t in entries) <= 10
        assert [s for s, _ in entries] == sorted(s for s, _ in entries)
    fed = {0: [], 1: []}
    for entries, _ in steps:
        for s, t in entries:
            fed[s] += t
    assert fed[0][:23] == list(range(100, 123))
    # slot 1 served r1 (prompt, then its first token fed back), then r2 after r1 finished
    assert fed[1][:3] == [7, 8, 9] and 5 in fed[1]
    assert sorted(eng.b.released) == [0, 1, 1]
    assert cb.idle()


def test_ragged_planner_wants_last_rows_only():
    eng = FakeEngine()
    cb = ContinuousBatcher(eng, slots=3, max_ctx=128, page_tokens=16, n_pages=30, chunk_tokens=64)
    cb.submit([1, 2, 3, 4], 2)
    cb.submit([9], 2)
    cb.step()
    entries, want = eng.b.steps[0]
    assert entries == [(0, [1, 2, 3, 4]), (1, [9])] and want == [3, 4]
    cb.step()
    entries, want = eng.b.steps[1]
    assert entries == [(0, [1001]), (1, [1001])] and want == [0, 1]


# ------------------------------------------------------------------ the oracle's algebra
def test_absorbed_latent_attention_equals_expanded():
    """score_h(i, j) = q_nope . (W_uk,h c_j) = (W_uk,h^T q_nope) . c_j and
    out_h = W_uv,h sum_j p_j c_j: the form the engine runs, restated here on the oracle's tensors."""
    cfg, T = small_cfg()
    T = {k: np.asarray(v, np.float64) for k, v in T.items()}
    m, pfx, eps = cfg["layers"][0]["mixer"], "l0.mix.", cfg["norm"]["eps"]
    rng = np.random.default_rng(1)
    n = 19
    h = rng.standard_normal((n, cfg["width"]))
    pos = np.arange(n)
    kv = O.latent_kv(h, m, T, pfx, pos, eps)
    want = O.latent_attention(h, m, T, pfx, pos, kv, eps)
    H, dim, rot, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = kv
    q = (h @ T[pfx + "q"].T).reshape(n, H, dim + rot)
    qr = O.rotate_half(q[:, :, dim:].transpose(1, 0, 2), pos, m["rot"]["dims"], m["rot"]["base"]).transpose(1, 0, 2)
    uk = T[pfx + "uk"].reshape(H, dim, R)
    uv = T[pfx + "uv"].reshape(H, vd, R)
    gate = 1 / (1 + np.exp(-(h @ T[pfx + "g"].T)))
    out = np.zeros((n, H, vd))
    for i in range(n):
        lo = max(0, i - m["mask"]["size"] + 1)
        for hh in range(H):
            qa = q[i, hh, :dim] @ uk[hh]
            s = (c[lo:i + 1] @ qa + kr[lo:i + 1] @ qr[i, hh]) * m["scale"]
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, hh] = uv[hh] @ (p @ c[lo:i + 1]) * gate[i, hh]
    got = out.reshape(n, H * vd) @ T[pfx + "o"].T
    assert np.abs(got - want).max() < 1e-10 * (1 + np.abs(want).max())


def test_oracle_window_is_exact():
    """A token outside every layer's reach leaves later logits untouched; one step closer changes them."""
    rng = np.random.default_rng(2)
    layers = [dict(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, window=4, mlp=None)]
    cfg, T = O.random_model(rng, vocab=31, width=16, layers=layers)
    toks = [int(t) for t in rng.integers(0, 31, 12)]
    base = O.forward(cfg, T, toks)
    other = list(toks)
    other[5] = (toks[5] + 1) % 31
    moved = O.forward(cfg, T, other)
    assert np.abs(moved[9:] - base[9:]).max() == 0.0          # 9 - 5 = 4 = window: not seen
    assert np.abs(moved[8] - base[8]).max() > 1e-6            # 8 - 5 = 3 < window: seen
