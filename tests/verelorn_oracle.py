"""The Verelorn design restated in numpy float64, one function per mechanism.

Slow and plain on purpose: whole sequences at once, explicit loops over positions where a
recurrence runs, no cache and no batching.  Shares no code with the engine.  ``cfg`` is a
config dictionary in the layout of a Verelorn config.json, ``W`` maps tensor names to arrays.

Notation: T tokens, h the input of a mixer (after the layer's norm and input convolution).
"""
from __future__ import annotations

import math

import numpy as np


def f64(a):
    return np.asarray(a, dtype=np.float64)


def rms_unit(x, eps):
    """x over its root mean square, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_offset(x, w, eps):
    """Norm of the layers, the embedding and the output: weights stored around zero."""
    return rms_unit(x, eps) * (1.0 + f64(w))


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * f64(w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(x, w):
    """x [T, C], w [C, taps]: out_t = sum_j w[:, j] x_(t - taps + 1 + j); zeros before the start."""
    x, w = f64(x), f64(w)
    T, taps = x.shape[0], w.shape[1]
    out = np.zeros_like(x)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += w[:, j][None, :] * x[:T - back]
    return out


def rotary_freqs(rot):
    """f_i = base^(-2i / dims), then the wavelength-dependent scaling when rot has 'scaling'."""
    dims = int(rot["dims"])
    f = np.array([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = f.copy()
        for i, fi in enumerate(f):
            lam = 2.0 * math.pi / fi
            if lam < orig / high:
                out[i] = fi
            elif lam > orig / low:
                out[i] = fi / factor
            else:
                s = (orig / lam - low) / (high - low)
                out[i] = (1.0 - s) * fi / factor + s * fi
        f = out
    return f


def rotate(x, pos, rot, layout):
    """x [T, ..., D]: the first rot['dims'] coordinates of the last axis turn by pos * f_i.
    layout 'halves': i pairs with i + dims / 2; 'interleaved': 2i with 2i + 1."""
    if not rot or int(rot.get("dims", 0)) == 0:
        return x
    dims = int(rot["dims"])
    f = rotary_freqs(rot)
    ang = f64(pos)[:, None] * f[None, :]                      # [T, dims / 2]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    out = x.copy()
    if layout == "halves":
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * c - b * s
        out[..., dims // 2:dims] = b * c + a * s
    else:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    return out


def softmax_causal(scores, sink=None):
    """scores [H, T, T] -> weights; position i sees j <= i; sink [H]: exp(sink) joins the denominator."""
    H, T, _ = scores.shape
    mask = np.tril(np.ones((T, T), dtype=bool))
    s = np.where(mask[None], scores, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, f64(sink)[:, None, None])
    e = np.exp(s - m)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(f64(sink)[:, None, None] - m)
    return e / den


def sink_attention(m, W, p, h):
    """Grouped-query attention whose values are its keys as projected, with biases on q and k, a
    partial rotate-half rotary, a sink in the softmax and an element-wise output gate."""
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    pos = np.arange(T)
    q = (h @ f64(W[p + "q"]).T + f64(W[p + "q.b"])).reshape(T, H, D)
    k = (h @ f64(W[p + "k"]).T + f64(W[p + "k.b"])).reshape(T, G, D)
    v = k.copy()
    q = rotate(q, pos, m.get("rot"), "halves")
    k = rotate(k, pos, m.get("rot"), "halves")
    rep = H // G
    scores = np.stack([q[:, hh] @ k[:, hh // rep].T for hh in range(H)]) * float(m["scale"])
    wts = softmax_causal(scores, W[p + "sink"])
    o = np.stack([wts[hh] @ v[:, hh // rep, :Dv] for hh in range(H)], axis=1)       # [T, H, Dv]
    gate = sigmoid(h @ f64(W[p + "g"]).T)
    return (o.reshape(T, H * Dv) * gate) @ f64(W[p + "o"]).T


def latent_kv(m, W, p, h, eps):
    """(c [T, kv_rank], rotated shared key part [T, rot_dim]) of a layer that owns W_dkv."""
    R = int(m["kv_rank"])
    T = h.shape[0]
    kv = h @ f64(W[p + "dkv"]).T
    c = norm_plain(kv[:, :R], W[p + "dkv.norm"], eps)
    kr = rotate(kv[:, R:], np.arange(T), m.get("rot"), "interleaved")
    return c, kr


def latent_attention(m, W, p, h, eps, kv):
    """Attention through a compressed row: queries through a latent of their own, per-head keys and
    values expanded from c, one rotated key part shared by the heads (expanded form)."""
    H, D, Dr, Dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    T = h.shape[0]
    c, kr = kv
    cq = norm_plain(h @ f64(W[p + "dq"]).T, W[p + "dq.norm"], eps)
    q = (cq @ f64(W[p + "uq"]).T).reshape(T, H, D + Dr)
    qn = q[..., :D]
    qr = rotate(q[..., D:], np.arange(T), m.get("rot"), "interleaved")
    kn = (c @ f64(W[p + "uk"]).T).reshape(T, H, D)
    vv = (c @ f64(W[p + "uv"]).T).reshape(T, H, Dv)
    scores = np.stack([qn[:, hh] @ kn[:, hh].T + qr[:, hh] @ kr.T for hh in range(H)]) * float(m["scale"])
    wts = softmax_causal(scores)
    o = np.stack([wts[hh] @ vv[:, hh] for hh in range(H)], axis=1)
    return o.reshape(T, H * Dv) @ f64(W[p + "o"]).T


def unit_vectors(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def channel_delta(m, W, p, h, eps):
    """Gated delta rule with one decay per head and key channel."""
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = silu(causal_conv(h @ f64(W[p + "q"]).T, W[p + "q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ f64(W[p + "k"]).T, W[p + "k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ f64(W[p + "v"]).T, W[p + "v.conv"])).reshape(T, H, Dv)
    q = unit_vectors(q) * D ** -0.5
    k = unit_vectors(k)
    beta = sigmoid(h @ f64(W[p + "b"]).T)                                              # [T, H]
    a = (h @ f64(W[p + "a1"]).T) @ f64(W[p + "a2"]).T + f64(W[p + "dt_bias"])
    g = np.exp(-np.exp(f64(W[p + "A_log"]))[None, :, None] * softplus(a).reshape(T, H, D))
    o = np.zeros((T, H, Dv))
    rep = H // G
    for hh in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            kt, qt = k[t, hh // rep], q[t, hh // rep]
            S = g[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ kt)
            S = S + np.outer(kt, u)
            o[t, hh] = S.T @ qt
    o = rms_unit(o, eps) * f64(W[p + "norm"])
    gate = sigmoid((h @ f64(W[p + "g1"]).T) @ f64(W[p + "g2"]).T).reshape(T, H, Dv)
    return (o * gate).reshape(T, H * Dv) @ f64(W[p + "o"]).T


def dense_ff(W, p, h):
    return (gelu_tanh(h @ f64(W[p + "gate"]).T) * (h @ f64(W[p + "up"]).T)) @ f64(W[p + "down"]).T


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence.  layers_out (a list) receives the sum of the streams
    after every layer."""
    eps = float(cfg["norm"]["eps"])
    tokens = np.asarray(tokens)
    x = norm_offset(f64(W["embed"])[tokens], W["embed.norm"], eps)
    n_str = int(cfg.get("streams") or 0)
    X = np.stack([x] * max(n_str, 1))                    # [streams, T, width]
    taps = int((cfg.get("canon") or {}).get("taps", 0))
    kvs = {}

    def sublayer(X, i, q, fn):
        pl = f"l{i}."
        if n_str:
            u = np.tensordot(f64(W[f"{pl}hc{q}.in"]), X, axes=(0, 0))
        else:
            u = X[0]
        y = fn(norm_offset(u, W[f"{pl}norm{q}"], eps))
        if n_str:
            mix, out = f64(W[f"{pl}hc{q}.mix"]), f64(W[f"{pl}hc{q}.out"])
            return np.einsum("st,srw->trw", mix, X) + out[:, None, None] * y[None]
        return X + y[None]

    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}.mix."

        def mixer(h):
            if taps:
                h = h + causal_conv(h, W[f"l{i}.canon1"])
            if L["type"] == "attention":
                return sink_attention(m, W, p, h)
            if L["type"] == "channel_delta":
                return channel_delta(m, W, p, h, eps)
            if L["type"] == "latent_attention":
                if m.get("kv_from") is None:
                    kvs[i] = latent_kv(m, W, p, h, eps)
                    return latent_attention(m, W, p, h, eps, kvs[i])
                return latent_attention(m, W, p, h, eps, kvs[int(m["kv_from"])])
            raise ValueError(L["type"])

        X = sublayer(X, i, 1, mixer)
        if L.get("mlp") is not None:
            X = sublayer(X, i, 2, lambda h: dense_ff(W, f"l{i}.mlp.", h))
        if layers_out is not None:
            layers_out.append(X.sum(axis=0))
    x = norm_offset(X.sum(axis=0), W["final.norm"], eps)
    return x @ f64(W["head"]).T


# ---------------------------------------------------------------- small configurations and random weights
def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def attn(heads=4, kv_heads=2, dim=16, rot_dims=8, base=10000.0, scaling=None, scale=None, mlp="dense"):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if rot_dims:
        m["rot"] = rot
    return {"type": "attention", "mixer": m, "mlp": dense() if mlp == "dense" else mlp}


def latent(heads=2, dim=8, rot_dim=4, vdim=12, kv_rank=16, q_rank=24, base=10000.0, kv_from=None, scale=None, mlp="dense"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": dense() if mlp == "dense" else mlp}


def delta(heads=2, kv_heads=1, dim=8, vdim=12, conv=3, ranks=(6, 5), mlp=None):
    """ranks: rows of a1 / g1 - sizes only the tensors carry."""
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": dense() if mlp == "dense" else mlp, "_ranks": ranks}


def config(layers, vocab=101, width=40, eps=1e-5, streams=3, taps=3):
    cfg = {"architecture": "Verelorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [{k: v for k, v in L.items() if k != "_ranks"} for L in layers]}
    if streams:
        cfg["streams"] = streams
    if taps:
        cfg["canon"] = {"taps": taps}
    cfg["_ranks"] = [L.get("_ranks") for L in layers]
    return cfg


def to_bf16_exact(a):
    """float32 values rounded to the nearest bf16 (kept as float32)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & np.uint32(0xFFFF0000)
    return u.view(np.float32).reshape(np.shape(a))


def random_weights(cfg, seed=0, qk_gain=2.0):
    """{name: float32 array of exact bf16 values} for a config made by config().  The branches' output projections
    are small beside the residual rows, as in a trained model: a rounding error then shrinks from layer to layer
    instead of doubling.  qk_gain: how sharp the softmaxes are (scores of a few units at 2, which a tight fp32
    comparison wants; 1 for comparisons of bf16 engines, whose rounded keys move sharp weights by percents)."""
    rng = np.random.default_rng(seed)
    W, V, T = cfg["width"], cfg["vocab"], {}

    def lin(o, i, gain=1.0):
        return rng.normal(0.0, gain / math.sqrt(i), (o, i))

    def vec(n, sd=0.2, mean=0.0):
        return mean + rng.normal(0.0, sd, n)

    T["embed"], T["embed.norm"], T["final.norm"], T["head"] = rng.normal(0, 1, (V, W)), vec(W), vec(W), lin(V, W)
    n = int(cfg.get("streams") or 0)
    taps = int((cfg.get("canon") or {}).get("taps", 0))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        subs = (1, 2) if L.get("mlp") is not None else (1,)
        for q in subs:
            T[f"{p}norm{q}"] = vec(W)
            if n:
                T[f"{p}hc{q}.in"] = vec(n, 0.2, 1.0 / n)
                T[f"{p}hc{q}.out"] = vec(n, 0.3, 0.7)
                T[f"{p}hc{q}.mix"] = np.eye(n) * 0.8 + rng.normal(0, 0.15, (n, n))
        if taps:
            T[p + "canon1"] = rng.normal(0, 0.4, (W, taps))
        x = p + "mix."
        if L["type"] == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            T[x + "q"], T[x + "k"], T[x + "g"], T[x + "o"] = lin(H * D, W, qk_gain), lin(G * D, W, qk_gain), lin(H * D, W), lin(W, H * D, 0.5)
            T[x + "q.b"], T[x + "k.b"], T[x + "sink"] = vec(H * D, 0.5), vec(G * D, 0.5), vec(H, 1.0, 1.0)
        elif L["type"] == "latent_attention":
            H, D, Dr, Dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            T[x + "dq"], T[x + "dq.norm"], T[x + "uq"] = lin(Q, W), vec(Q, 0.2, 1.0), lin(H * (D + Dr), Q, qk_gain)
            if m.get("kv_from") is None:
                T[x + "dkv"], T[x + "dkv.norm"] = lin(R + Dr, W, qk_gain), vec(R, 0.2, 1.0)
            T[x + "uk"], T[x + "uv"], T[x + "o"] = lin(H * D, R, qk_gain), lin(H * Dv, R), lin(W, H * Dv, 0.5)
        else:
            H, G, D, Dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            ra, rg = cfg["_ranks"][i]
            T[x + "q"], T[x + "k"], T[x + "v"], T[x + "b"] = lin(G * D, W, 2.0), lin(G * D, W, 2.0), lin(H * Dv, W, 2.0), lin(H, W, 2.0)
            for t, c in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                T[f"{x}{t}.conv"] = rng.normal(0, 0.6, (c, K))
            T[x + "A_log"], T[x + "dt_bias"], T[x + "norm"] = vec(H, 0.7, -1.0), vec(H * D, 1.0), vec(Dv, 0.2, 1.0)
            T[x + "a1"], T[x + "a2"], T[x + "g1"], T[x + "g2"] = lin(ra, W), lin(H * D, ra, 2.0), lin(rg, W), lin(H * Dv, rg, 2.0)
            T[x + "o"] = lin(W, H * Dv, 0.5)
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            T[p + "mlp.gate"], T[p + "mlp.up"], T[p + "mlp.down"] = lin(ff, W, 1.5), lin(ff, W), lin(W, ff, 0.5)
    return {k: to_bf16_exact(v) for k, v in T.items()}
