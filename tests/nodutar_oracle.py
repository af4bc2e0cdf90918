"""Plain, slow restatement of the Nodutar decoder in numpy float64.

One function per mechanism, written from the equations only; it shares no code with the
engine.  A model is (cfg, tensors): cfg the dict of config.json, tensors {name: ndarray}.

Notation (x_t the residual row of token t, position t counted from 0 in its sequence):
  rms(v)      = v / sqrt(mean(v^2) + eps)
  N_w(v)      = rms(v) * (1 + w)                      the block norms: weights stored around zero
  block       x <- x + N_1b(mixer(N_1(x)));  x <- x + N_2b(ff(N_2(x)))     (ff may be absent)
  layer runs  layers [start, stop) are run `times` times in a row with the same weights; every
              run has its own keys / values / state; before run 2, 3, ... of the group starts,
              the embedding rows are added to x
  logits      = E N_final(x), E the embedding table
"""
import numpy as np


def rms(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def norm_one_plus(v, w, eps):
    return rms(v, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotate_pairs(v, pos, dims, base, sign=1.0):
    """v [n, ..., d]; row t turns by sign * pos[t]: inside the first `dims` coordinates of the last
    axis, coordinate 2i is paired with 2i + 1 and turned by the angle pos * base^(-2i / dims)."""
    out = np.array(v, dtype=np.float64, copy=True)
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = sign * np.asarray(pos, dtype=np.float64)[:, None] * f[None, :]
    a = a.reshape((len(pos),) + (1,) * (v.ndim - 2) + (half,))
    c, s = np.cos(a), np.sin(a)
    u, w = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - w * s
    out[..., 1:dims:2] = w * c + u * s
    return out


def softmax_rows(s):
    p = np.exp(s - s.max())
    return p / p.sum()


def chunk_attention(h, m, T, pfx, eps):
    """Grouped-query attention whose query i sees key j <= i of its own block of mask.size
    positions only.  Queries and keys: per-head rms with a plain weight, then the pair rotation on
    the first rot.dims coordinates.  Values: turned by their own position over all vdim
    coordinates; the head's weighted sum is turned back by the query's position."""
    n = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(n)
    q = (h @ T[pfx + "q"].T).reshape(n, H, d)
    k = (h @ T[pfx + "k"].T).reshape(n, G, d)
    v = (h @ T[pfx + "v"].T).reshape(n, G, vd)
    q = rms(q, eps) * T[pfx + "q.norm"]
    k = rms(k, eps) * T[pfx + "k.norm"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q = rotate_pairs(q, pos, dims, base)
    k = rotate_pairs(k, pos, dims, base)
    v = rotate_pairs(v, pos, vd, base)
    size = m["mask"]["size"]
    out = np.zeros((n, H, vd))
    for i in range(n):
        lo = (i // size) * size
        for hh in range(H):
            g = hh // (H // G)
            p = softmax_rows((k[lo:i + 1, g] @ q[i, hh]) * m["scale"])
            out[i, hh] = p @ v[lo:i + 1, g]
    out = rotate_pairs(out, pos, vd, base, sign=-1.0)
    return out.reshape(n, H * vd) @ T[pfx + "o"].T


def gated_recurrence(h, m, T, pfx, eps):
    """Linear attention whose forget gate also writes: per head, with f in (lower, 1),
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,  o_t = S_t^T q_t,  q = silu(W_q h),
    f = lower + (1 - lower) * sigmoid(W_f h + b); o is rms-normed per head with a plain weight."""
    n = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ T[pfx + "q"].T).reshape(n, H, d)
    v = (h @ T[pfx + "v"].T).reshape(n, H, vd)
    low = T[pfx + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ T[pfx + "f"].T + T[pfx + "f.b"])).reshape(n, H, d)
    S = np.zeros((H, d, vd))
    o = np.zeros((n, H, vd))
    for t in range(n):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = rms(o, eps) * T[pfx + "norm"]
    return o.reshape(n, H * vd) @ T[pfx + "o"].T


def parallel_mixer(h, m, T, pfx, eps):
    return (m["left_scale"] * chunk_attention(h, m["left"], T, pfx + "left.", eps)
            + m["right_scale"] * gated_recurrence(h, m["right"], T, pfx + "right.", eps))


def distance_attention(h, m, T, pfx, eps):
    """Causal grouped-query attention without rotation: the values are the projected keys as they
    leave W_k; queries and keys are rms-normed per head without a weight; the score loses
    r1_h * ln(1 + r2_h * (i - j))."""
    n = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ T[pfx + "q"].T).reshape(n, H, d)
    v = (h @ T[pfx + "k"].T).reshape(n, G, d)
    q, k = rms(q, eps), rms(v, eps)
    r1, r2 = T[pfx + "r1"], T[pfx + "r2"]
    out = np.zeros((n, H, d))
    for i in range(n):
        dist = i - np.arange(i + 1)
        for hh in range(H):
            g = hh // (H // G)
            s = (k[:i + 1, g] @ q[i, hh]) * m["scale"] - r1[hh] * np.log1p(r2[hh] * dist)
            out[i, hh] = softmax_rows(s) @ v[:i + 1, g]
    return out.reshape(n, H * d) @ T[pfx + "o"].T


def moe_ff(h, mlp, T, pfx):
    """Router logits z = W_r h + b; the `top` largest are chosen and weighted by the softmax over
    those alone; the weights multiply the experts' outputs."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ T[pfx + "router"].T + T[pfx + "router.b"]
    out = np.zeros((h.shape[0], T[pfx + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        # ranked on logits rounded far below any real difference: rows of W_r that are equal give
        # equal logits here, whatever order the matrix product summed them in
        idx = np.argsort(-np.round(z[t], 10), kind="stable")[:top]
        w = softmax_rows(z[t, idx])
        for wt, e in zip(w, idx):
            p = f"{pfx}e{e}."
            x = h[t:t + 1]
            out[t] += wt * ((silu(x @ T[p + "gate"].T) * (x @ T[p + "up"].T)) @ T[p + "down"].T)[0]
    return out


def layer_runs(cfg):
    """[(layer index, starts a repeated pass)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    if b <= a or times <= 1:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(a)]
    for r in range(times):
        runs += [(i, r > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, T, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence; layers_out receives the stream after every run."""
    T = {k: np.asarray(v, dtype=np.float64) for k, v in T.items()}
    eps = cfg["norm"]["eps"]
    x0 = T["embed"][np.asarray(tokens)]
    x = x0.copy()
    for i, again in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if again:
            x = x + x0
        h = norm_one_plus(x, T[p + "norm1"], eps)
        if L["type"] == "parallel":
            y = parallel_mixer(h, L["mixer"], T, p + "mix.", eps)
        elif L["type"] == "attention":
            y = distance_attention(h, L["mixer"], T, p + "mix.", eps)
        else:
            raise ValueError(L["type"])
        x = x + norm_one_plus(y, T[p + "norm1b"], eps)
        if L.get("mlp") is not None:
            f = moe_ff(norm_one_plus(x, T[p + "norm2"], eps), L["mlp"], T, p + "mlp.")
            x = x + norm_one_plus(f, T[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm_one_plus(x, T["final.norm"], eps) @ T["embed"].T


# ------------------------------------------------------------------ random models
def bf(a):
    """values rounded to bfloat16, as float32"""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def par(heads=4, kv_heads=2, dim=12, vdim=10, rot_dims=8, base=100.0, size=7, scale=None, rheads=3, rdim=6, rvdim=8,
        left_scale=0.7, right_scale=0.6, mlp=("moe", 14, 5, 2)):
    return dict(type="parallel", heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=rot_dims, base=base, size=size,
                scale=scale, rheads=rheads, rdim=rdim, rvdim=rvdim, left_scale=left_scale, right_scale=right_scale, mlp=mlp)


def dist(heads=4, kv_heads=1, dim=10, scale=None, mlp=("moe", 14, 5, 2)):
    return dict(type="attention", heads=heads, kv_heads=kv_heads, dim=dim, scale=scale, mlp=mlp)


def random_model(rng, *, vocab=97, width=48, layers=None, loop=None, eps=1e-5):
    """cfg + tensors with random weights that are exact bfloat16 values.  `layers`: dicts made by
    par() / dist(); loop: (start, stop, times) or None."""
    def lin(o, i, s=1.0):
        return bf(rng.standard_normal((o, i)) * (s / np.sqrt(i)))

    def small(n, s=0.2):
        return bf(s * rng.standard_normal(n))

    cfg = {"architecture": "Nodutar", "layers": [], "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    T = {"embed": bf(rng.standard_normal((vocab, width))), "final.norm": small(width)}
    for i, L in enumerate(layers):
        p = f"l{i}."
        T[p + "norm1"], T[p + "norm1b"] = small(width), small(width)
        if L["type"] == "parallel":
            H, G, d, vd = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            left = {"heads": H, "kv_heads": G, "dim": d, "vdim": vd, "mask": {"size": L["size"]},
                    "rot": {"base": L["base"], "dims": L["rot_dims"]}, "scale": L["scale"] or d ** -0.5 * 3.0}
            q = p + "mix.left."
            T[q + "q"], T[q + "k"], T[q + "v"] = lin(H * d, width, 2.0), lin(G * d, width, 2.0), lin(G * vd, width)
            T[q + "q.norm"], T[q + "k.norm"] = bf(1.0 + 0.2 * rng.standard_normal(d)), bf(1.0 + 0.2 * rng.standard_normal(d))
            T[q + "o"] = lin(width, H * vd)
            RH, rd, rv = L["rheads"], L["rdim"], L["rvdim"]
            right = {"heads": RH, "dim": rd, "vdim": rv}
            r = p + "mix.right."
            T[r + "q"], T[r + "f"], T[r + "v"] = lin(RH * rd, width, 2.0), lin(RH * rd, width, 2.0), lin(RH * rv, width)
            T[r + "f.b"] = bf(1.0 + rng.standard_normal(RH * rd))
            T[r + "lower"] = bf(0.05 + 0.9 * rng.random(RH * rd))
            T[r + "norm"] = bf(1.0 + 0.2 * rng.standard_normal(rv))
            T[r + "o"] = lin(width, RH * rv)
            mixer = {"left": left, "right": right, "left_scale": L["left_scale"], "right_scale": L["right_scale"]}
        else:
            H, G, d = L["heads"], L["kv_heads"], L["dim"]
            mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": L["scale"] or 2.0}
            q = p + "mix."
            T[q + "q"], T[q + "k"], T[q + "o"] = lin(H * d, width, 2.0), lin(G * d, width, 2.0), lin(width, H * d)
            T[q + "r1"] = bf(0.3 + 1.5 * rng.random(H))
            T[q + "r2"] = bf(0.05 + 0.5 * rng.random(H))
        mlp = L.get("mlp")
        if mlp is None:
            mc = None
        else:
            _, ff, E, top = mlp
            mc = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top}}
            T[p + "norm2"], T[p + "norm2b"] = small(width), small(width)
            T[p + "mlp.router"] = lin(E, width, 3.0)
            T[p + "mlp.router.b"] = small(E, 0.5)
            for e in range(E):
                for nm, o, ii in (("gate", ff, width), ("up", ff, width), ("down", width, ff)):
                    T[f"{p}mlp.e{e}.{nm}"] = lin(o, ii, 1.5)
        cfg["layers"].append({"type": L["type"], "mixer": mixer, "mlp": mc})
    return cfg, T
