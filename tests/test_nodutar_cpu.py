"""CPU: the Nodutar config reader and registry entry, tensor names, layer runs, and the plain
restatement's own mechanisms checked against their defining properties."""
import numpy as np
import pytest

import nodutar_oracle as O
from nodutar_oracle import dist, par


def small(loop=(1, 3, 2)):
    rng = np.random.default_rng(3)
    return O.random_model(rng, vocab=31, width=24, layers=[par(), dist(), par(mlp=None), dist(heads=6, kv_heads=3)], loop=loop)


def test_config_reader_and_registry():
    import qwen_inference_engine_amd as q
    from qwen_inference_engine_amd import spec as S
    cfg, T = small()
    sp = q.spec_from_config(cfg)
    assert isinstance(sp, S.LayeredSpec) and sp.block == "sandwich" and sp.tied_head and not sp.depth_mix
    assert sp.loop == (1, 3, 2) and sp.runs() == [0, 1, 2, 1, 2, 3] and sp.n_runs == 6
    m0, m1 = sp.layers[0].mixer, sp.layers[1].mixer
    assert isinstance(m0, S.AttentionWithRecurrence) and isinstance(m1, S.GqaAttention)
    a = m0.attn
    assert (a.qk_norm, a.rot_layout, a.rot_values, a.mask, a.mask_size) == ("weight", "interleaved", True, "chunk", 7)
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims) == (4, 2, 12, 10, 8)
    assert (m0.rec.heads, m0.rec.dim, m0.rec.vdim, m0.attn_scale, m0.rec_scale) == (3, 6, 8, 0.7, 0.6)
    assert (m1.qk_norm, m1.values_are_keys, m1.dist_bias, m1.mask, m1.rot_dims) == ("plain", True, True, "causal", 0)
    assert sp.layers[0].mlp.router == "softmax_out" and sp.layers[2].mlp is None
    # every checkpoint tensor is named with its shape, and nothing else
    shapes = sp.tensor_shapes()
    assert set(shapes) == set(T)
    for k, v in T.items():
        assert list(np.shape(v)) == shapes[k], k
    # cached elements per token and state per slot count every run
    per_run = {0: 2 * (12 + 10), 1: 1 * 20, 2: 2 * (12 + 10), 3: 3 * 20}
    assert sp.cache_row_elems() == sum(per_run[i] for i in sp.runs())
    assert sp.state_elems() == 3 * 3 * 6 * 8
    arch, keep = sp.to_c()
    assert (arch.loop_start, arch.loop_stop, arch.loop_times, arch.tied_head) == (1, 3, 2, 1)
    assert sp.step_flops(8, 100) > 0


def test_reader_refuses_what_the_design_does_not_have():
    import qwen_inference_engine_amd as q
    cfg, _ = small()
    bad = {**cfg, "layers": [{**cfg["layers"][0], "type": "convolution"}]}
    with pytest.raises(ValueError):
        q.spec_from_config(bad)
    bad = {**cfg, "layers": [{**cfg["layers"][0], "mlp": {"kind": "dense", "ff": 8}}]}
    with pytest.raises(ValueError):
        q.spec_from_config(bad)
    with pytest.raises(ValueError):
        q.spec_from_config({**cfg, "loop": {"start": 2, "stop": 9, "times": 2}})
    sp = q.spec_from_config({k: v for k, v in cfg.items() if k != "loop"})
    assert sp.runs() == [0, 1, 2, 3]
    assert q.spec_from_config({**cfg, "loop": {"start": 0, "stop": 4, "times": 3}}).n_runs == 12


def test_layer_runs_of_the_restatement():
    cfg, _ = small()
    assert O.layer_runs(cfg) == [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]
    assert O.layer_runs({**cfg, "loop": None}) == [(i, False) for i in range(4)]


def test_turned_values_are_a_relative_rotation():
    """Turning value j by j and the sum back by i equals turning every value by j - i before the sum."""
    rng = np.random.default_rng(0)
    n, vd = 9, 8
    v = rng.standard_normal((n, 1, vd))
    p = rng.random(n)
    p /= p.sum()
    pos = np.arange(n)
    i = n - 1
    direct = O.rotate_pairs((p[:, None, None] * O.rotate_pairs(v, pos, vd, 100.0)).sum(0, keepdims=True), [i], vd, 100.0, sign=-1.0)
    relative = (p[:, None, None] * O.rotate_pairs(v, pos - i, vd, 100.0)).sum(0, keepdims=True)
    assert np.allclose(direct, relative, atol=1e-12)
    # pairs are neighbours: coordinates 2m, 2m + 1 keep their joint length, position 0 turns nothing
    r = O.rotate_pairs(v, pos, vd, 100.0)
    assert np.allclose(r[..., 0::2] ** 2 + r[..., 1::2] ** 2, v[..., 0::2] ** 2 + v[..., 1::2] ** 2)
    assert np.array_equal(r[0], v[0])
    # only the first `dims` coordinates turn
    assert np.array_equal(O.rotate_pairs(v, pos, 4, 100.0)[..., 4:], v[..., 4:])


def test_recurrence_equals_its_unrolled_sum():
    """S_t = sum_j (prod_{j < s <= t} f_s) (1 - f_j) v_j^T per row of the state."""
    rng = np.random.default_rng(1)
    cfg, T = O.random_model(rng, vocab=11, width=16, layers=[par(rheads=2, rdim=3, rvdim=4, mlp=None)])
    T = {k: np.asarray(v, dtype=np.float64) for k, v in T.items()}
    m, pfx = cfg["layers"][0]["mixer"]["right"], "l0.mix.right."
    h = rng.standard_normal((7, 16))
    got = O.gated_recurrence(h, m, T, pfx, 1e-5)
    q = O.silu(h @ T[pfx + "q"].T).reshape(7, 2, 3)
    v = (h @ T[pfx + "v"].T).reshape(7, 2, 4)
    low = T[pfx + "lower"]
    f = (low + (1 - low) * O.sigmoid(h @ T[pfx + "f"].T + T[pfx + "f.b"])).reshape(7, 2, 3)
    o = np.zeros((7, 2, 4))
    for t in range(7):
        for j in range(t + 1):
            decay = np.prod(f[j + 1:t + 1], axis=0)                    # [heads, dim]
            o[t] += np.einsum("hd,hv->hv", q[t] * decay * (1 - f[j]), v[j])
    want = (O.rms(o, 1e-5) * T[pfx + "norm"]).reshape(7, 8) @ T[pfx + "o"].T
    assert np.allclose(got, want, atol=1e-10)
    assert f.min() > low.min() - 1e-12 and f.max() < 1.0


def test_block_mask_and_router_of_the_restatement():
    rng = np.random.default_rng(2)
    cfg, T = O.random_model(rng, vocab=11, width=16, layers=[par(size=4, mlp=("moe", 6, 5, 2))])
    T64 = {k: np.asarray(v, dtype=np.float64) for k, v in T.items()}
    h = rng.standard_normal((10, 16))
    left = cfg["layers"][0]["mixer"]["left"]
    a = O.chunk_attention(h, left, T64, "l0.mix.left.", 1e-5)
    # rows of one block do not change when another block's inputs change
    h2 = h.copy()
    h2[:4] += 1.0
    b = O.chunk_attention(h2, left, T64, "l0.mix.left.", 1e-5)
    assert np.allclose(a[4:], b[4:]) and not np.allclose(a[:4], b[:4])
    # router: weights of the chosen experts sum to one, a large bias forces the choice
    T64["l0.mlp.router.b"] = np.array([0.0, 50.0, 0.0, 40.0, 0.0])
    f = O.moe_ff(h, cfg["layers"][0]["mlp"], T64, "l0.mlp.")
    e1 = (O.silu(h @ T64["l0.mlp.e1.gate"].T) * (h @ T64["l0.mlp.e1.up"].T)) @ T64["l0.mlp.e1.down"].T
    assert np.allclose(f, e1, atol=1e-3 * np.abs(e1).max())
