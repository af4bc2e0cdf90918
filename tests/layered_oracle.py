"""Plain, slow restatement of the layered decoder family (Tivazen) in numpy float64.

One function per mechanism, written from the equations only; it shares no code with the
engine.  A model is (cfg, tensors): cfg the dict of config.json, tensors {name: ndarray}.

Notation: x_t the residual row of token t (position t, counted from 0 per sequence),
X_0 the embedding rows, X_(i+1) the result of layer i.
  layer i:   y = x + g1 * rms(mixer(x));  X_(i+1) = y + g2 * rms(ff(y))   (ff may be absent)
             next x = sum_{j <= i+1} a_i[j] X_j
  rms(v) = v / sqrt(mean(v^2) + eps)
"""
import numpy as np


def rms(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def scalar_norm(v, g, eps):
    return rms(v, eps) * float(g)


def rotate_half(v, pos, dims, base):
    """v [..., n, d] with n positions `pos`; the first `dims` coordinates of the last axis are
    rotated, coordinate i paired with i + dims/2, angle pos * base^(-2i/dims)."""
    out = v.copy()
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = np.asarray(pos, dtype=np.float64)[:, None] * f[None, :]
    c, s = np.cos(a), np.sin(a)
    u, w = v[..., :half], v[..., half:dims]
    out[..., :half] = u * c - w * s
    out[..., half:dims] = w * c + u * s
    return out


def latent_kv(h, m, T, pfx, pos, eps):
    """The cached part of a latent-attention mixer: (c [n, r], k_rot [n, rot] rotated)."""
    r, rot = m["kv_rank"], m["rot_dim"]
    d = h @ T[pfx + "dkv"].T
    c = rms(d[:, :r], eps) * T[pfx + "dkv.norm"]
    kr = rotate_half(d[:, r:r + rot], pos, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, m, T, pfx, pos, kv, eps):
    """h [n, W] -> mixer output [n, W].  kv = (c, k_rot) of this layer or of the layer it
    borrows from.  Non-absorbed form: keys and values are expanded per head."""
    H, dim, rot, vd, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    c, kr = kv
    q = (h @ T[pfx + "q"].T).reshape(n, H, dim + rot)
    qn, qr = q[:, :, :dim], q[:, :, dim:]
    qr = rotate_half(qr.transpose(1, 0, 2), pos, m["rot"]["dims"], m["rot"]["base"]).transpose(1, 0, 2)
    kn = (c @ T[pfx + "uk"].T).reshape(n, H, dim)
    v = (c @ T[pfx + "uv"].T).reshape(n, H, vd)
    gate = 1.0 / (1.0 + np.exp(-(h @ T[pfx + "g"].T)))          # [n, H]
    win = m["mask"]["size"]
    out = np.zeros((n, H, vd))
    for i in range(n):
        lo = max(0, i - win + 1)
        for hh in range(H):
            s = (kn[lo:i + 1, hh] @ qn[i, hh] + kr[lo:i + 1] @ qr[i, hh]) * m["scale"]
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, hh] = (p @ v[lo:i + 1, hh]) * gate[i, hh]
    return out.reshape(n, H * vd) @ T[pfx + "o"].T


def silu(z):
    return z / (1.0 + np.exp(-z))


def gated_ff(h, Wg, Wu, Wd):
    return (silu(h @ Wg.T) * (h @ Wu.T)) @ Wd.T


def moe_ff(h, mlp, T, pfx):
    """Sigmoid router, `top` largest scores, the score scales the expert's INPUT."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = 1.0 / (1.0 + np.exp(-(h @ T[pfx + "router"].T)))
    out = np.zeros((h.shape[0], T[pfx + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e in np.argsort(-s[t], kind="stable")[:top]:
            p = f"{pfx}e{e}."
            out[t] += gated_ff(s[t, e] * h[t:t + 1], T[p + "gate"], T[p + "up"], T[p + "down"])[0]
    return out


def forward(cfg, T, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence.  layers_out: list that receives the stream
    after every layer (after the depth average)."""
    T = {k: np.asarray(v, dtype=np.float64) for k, v in T.items()}
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    pos = np.arange(n)
    x = T["embed"][np.asarray(tokens)]
    X = [x]
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        m, pfx = L["mixer"], f"l{i}.mix."
        assert L["type"] == "latent_attention"
        if m.get("kv_from") is None:
            kvs[i] = latent_kv(x, m, T, pfx, pos, eps)
            kv = kvs[i]
        else:
            kv = kvs[m["kv_from"]]
        y = x + scalar_norm(latent_attention(x, m, T, pfx, pos, kv, eps), T[f"l{i}.norm1"], eps)
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                f = gated_ff(y, T[f"l{i}.mlp.gate"], T[f"l{i}.mlp.up"], T[f"l{i}.mlp.down"])
            else:
                f = moe_ff(y, mlp, T, f"l{i}.mlp.")
            y = y + scalar_norm(f, T[f"l{i}.norm2"], eps)
        X.append(y)
        a = T[f"l{i}.dwa"]
        x = sum(a[j] * X[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x.copy())
    return scalar_norm(x, T["final.norm"], eps) @ T["head"].T


# ------------------------------------------------------------------ random models
def random_model(rng, *, vocab=97, width=48, layers=None, eps=1e-5, wscale=None):
    """cfg + tensors with random weights.  `layers`: list of dicts
    {heads, dim, rot_dim, vdim, kv_rank, window, kv_from (None), mlp: None | ("dense", ff) |
    ("moe", ff, experts, top), base, scale}; weights are rounded to bfloat16 values."""
    def bf(a):
        b = np.asarray(a, dtype=np.float32).view(np.uint32)
        b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
        return b.astype(np.uint32).view(np.float32)

    def lin(o, i, s=1.0):
        return bf(rng.standard_normal((o, i)) * (s / np.sqrt(i)))

    cfg = {"architecture": "Tivazen", "layers": [], "norm": {"eps": eps}, "vocab": vocab, "width": width}
    T = {"embed": bf(rng.standard_normal((vocab, width))), "head": lin(vocab, width),
         "final.norm": bf(np.float32(1.0 + 0.1 * rng.standard_normal()))}
    for i, L in enumerate(layers):
        H, dim, rot, vd, r = L["heads"], L["dim"], L["rot_dim"], L["vdim"], L["kv_rank"]
        m = {"heads": H, "dim": dim, "rot_dim": rot, "vdim": vd, "kv_rank": r, "mask": {"size": L["window"]},
             "rot": {"base": L.get("base", 10000.0), "dims": rot}, "scale": L.get("scale", (dim + rot) ** -0.5)}
        p = f"l{i}.mix."
        T[p + "q"] = lin(H * (dim + rot), width, 2.0)
        if L.get("kv_from") is None:
            T[p + "dkv"] = lin(r + rot, width, 2.0)
            T[p + "dkv.norm"] = bf(1.0 + 0.2 * rng.standard_normal(r))
        else:
            m["kv_from"] = L["kv_from"]
        T[p + "uk"] = lin(H * dim, r, 2.0)
        T[p + "uv"] = lin(H * vd, r)
        T[p + "g"] = lin(H, width, 2.0)
        T[p + "o"] = lin(width, H * vd)
        T[f"l{i}.norm1"] = bf(np.float32(0.7 + 0.2 * rng.random()))
        mlp = L.get("mlp")
        if mlp is None:
            mc = None
        elif mlp[0] == "dense":
            mc = {"kind": "dense", "ff": mlp[1]}
            for nm, o, ii in (("gate", mlp[1], width), ("up", mlp[1], width), ("down", width, mlp[1])):
                T[f"l{i}.mlp.{nm}"] = lin(o, ii)
        else:
            _, ff, E, top = mlp
            mc = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top}}
            T[f"l{i}.mlp.router"] = lin(E, width, 3.0)
            for e in range(E):
                for nm, o, ii in (("gate", ff, width), ("up", ff, width), ("down", width, ff)):
                    T[f"l{i}.mlp.e{e}.{nm}"] = lin(o, ii, 1.5)
        if mc is not None:
            T[f"l{i}.norm2"] = bf(np.float32(0.7 + 0.2 * rng.random()))
        T[f"l{i}.dwa"] = bf(np.concatenate([0.15 * rng.standard_normal(i + 1), [1.0]]))
        cfg["layers"].append({"type": "latent_attention", "mixer": m, "mlp": mc})
    return cfg, T
