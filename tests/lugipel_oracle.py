"""Plain numpy (float64) restatement of the Lugipel design, one function per mechanism.

A decoder whose layers are x <- x + mixer(N(x)), x <- x + ff(N(x)) with N(v) = v / sqrt(mean(v^2) + eps) * w.
Shares no code with the engine; slow on purpose (loops over positions and keys).

Model description (a dict, the shape of the design's config.json):
  {"architecture": "Lugipel", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"},
   "layers": [{"type": "attention" | "mingru", "mixer": {...}, "mlp": {...} | None}, ...]}
Weights: a dict name -> float64 array, with the checkpoint's tensor names.
"""
import math

import numpy as np


def rms(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def silu(z):
    return z * sigmoid(z)


def position_vector(p, width):
    """Entry 2i = sin(p * 10000^(-2i / width)), entry 2i + 1 = cos of the same angle."""
    out = np.zeros(width)
    for i in range((width + 1) // 2):
        ang = p * 10000.0 ** (-2.0 * i / width)
        out[2 * i] = math.sin(ang)
        if 2 * i + 1 < width:
            out[2 * i + 1] = math.cos(ang)
    return out


def embed(tokens, table, scale, first_pos=0):
    width = table.shape[1]
    return np.stack([table[t] * scale + position_vector(first_pos + n, width) for n, t in enumerate(tokens)])


def query_temperature(p, coef, every):
    return 1.0 + coef * math.log((p + 1) // every + 1)


def head_slopes(heads):
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def sigmoid_attention(h, w, pre, m, eps):
    """h [T, width] (positions 0 .. T-1 of one sequence).  Every visible key gets the weight
    sigmoid(score + pb_head); the weights are not normalised."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D)
    k = (h @ w[pre + "k"].T).reshape(T, G, D)
    v = (h @ w[pre + "v"].T).reshape(T, G, V)
    q = rms(q, eps) * w[pre + "q.norm"]
    k = rms(k, eps) * w[pre + "k.norm"]
    gate = sigmoid(h @ w[pre + "g"].T)                       # [T, H]
    slopes = head_slopes(H)
    size = m["mask"]["size"]
    out = np.zeros((T, H, V))
    for i in range(T):
        temp = query_temperature(i, m["q_temp"]["coef"], m["q_temp"]["every"])
        for hd in range(H):
            g = hd // (H // G)
            js = np.arange(max(0, i - size + 1), i + 1)          # the visible keys: 0 <= i - j < size
            s = (k[js, g] @ q[i, hd]) * temp * m["scale"] - slopes[hd] * (i - js)
            out[i, hd] = (sigmoid(s + w[pre + "pb"][hd]) @ v[js, g]) * gate[i, hd]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def min_gru(h, w, pre, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t, element by element; returns (outputs, last state)."""
    z = sigmoid(h @ w[pre + "z"].T + w[pre + "z.b"])
    u = h @ w[pre + "x"].T + w[pre + "x.b"]
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    gate = silu(h @ w[pre + "g"].T)
    S = np.zeros(z.shape[1]) if state is None else state.copy()
    out = np.zeros_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        out[t] = S * gate[t]
    return out @ w[pre + "o"].T, S


def xielu(z, p, q):
    ap, aq = softplus(p), 0.5 + softplus(q)
    return np.where(z > 0, ap * z * z + 0.5 * z, aq * (np.expm1(np.minimum(z, 0.0)) - z) + 0.5 * z)


def dense_ff(h, w, pre):
    a = w[pre + "act"]
    return xielu(h @ w[pre + "up"].T, a[0], a[1]) @ w[pre + "down"].T


def route(h_row, w, pre, r):
    """(chosen expert ids, their weights) of one row.  Experts experts .. experts + identity - 1 are
    identity experts."""
    n = r["experts"] + r["identity"]
    z = np.array([float(row @ h_row) for row in w[pre + "router"]])   # row by row: equal rows give equal logits
    s = np.exp(z - z.max())
    s = s / s.sum()
    choice = s + w[pre + "correction"]
    count, keep = r["groups"]["count"], r["groups"]["keep"]
    per = n // count
    best = [choice[g * per:(g + 1) * per].max() for g in range(count)]
    kept = sorted(range(count), key=lambda g: (-best[g], g))[:keep]
    allowed = [e for e in range(n) if e // per in kept]
    chosen = sorted(allowed, key=lambda e: (-choice[e], e))[:r["top"]]
    ws = np.array([s[e] for e in chosen])
    ws = ws / (ws.sum() + 1e-20) * r["scale"]
    return chosen, ws


def moe_ff(h, w, pre, f):
    r = f["router"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, ws = route(h[t], w, pre, r)
        for e, wt in zip(chosen, ws):
            if e >= r["experts"]:
                out[t] += wt * h[t]
            else:
                p = f"{pre}e{e}."
                out[t] += wt * ((silu(w[p + "gate"] @ h[t]) * (w[p + "up"] @ h[t])) @ w[p + "down"].T)
    return out


def forward(cfg, w, tokens, want_layers=False):
    """Logits [T, vocab] of one sequence fed whole (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, w["embed"], cfg["embedding"]["scale"])
    kept = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps) * w[p + "norm1"]
        if L["type"] == "attention":
            x = x + sigmoid_attention(h, w, p + "mix.", L["mixer"], eps)
        elif L["type"] == "mingru":
            x = x + min_gru(h, w, p + "mix.")[0]
        else:
            raise ValueError(L["type"])
        f = L.get("mlp")
        if f is not None:
            h = rms(x, eps) * w[p + "norm2"]
            x = x + (dense_ff(h, w, p + "mlp.") if f["kind"] == "dense" else moe_ff(h, w, p + "mlp.", f))
        kept.append(x.copy())
    logits = (rms(x, eps) * w["final.norm"]) @ w["head"].T
    return (logits, np.stack(kept)) if want_layers else logits


def tensor_shapes(cfg):
    W, out = cfg["width"], {"embed": [cfg["vocab"], cfg["width"]]}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = [W]
        if L["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": [H * D, W], p + "mix.k": [G * D, W], p + "mix.v": [G * V, W], p + "mix.q.norm": [D],
                        p + "mix.k.norm": [D], p + "mix.pb": [H], p + "mix.g": [H, W], p + "mix.o": [W, H * V]})
        else:
            n = m["width"]
            out.update({p + "mix.z": [n, W], p + "mix.z.b": [n], p + "mix.x": [n, W], p + "mix.x.b": [n], p + "mix.g": [n, W],
                        p + "mix.o": [W, n]})
        f = L.get("mlp")
        if f is None:
            continue
        out[p + "norm2"] = [W]
        if f["kind"] == "dense":
            out.update({p + "mlp.up": [f["ff"], W], p + "mlp.down": [W, f["ff"]], p + "mlp.act": [2]})
        else:
            r, ff = f["router"], f["expert"]["ff"]
            for e in range(r["experts"]):
                q = f"{p}mlp.e{e}."
                out.update({q + "gate": [ff, W], q + "up": [ff, W], q + "down": [W, ff]})
            out[p + "mlp.router"] = [r["experts"] + r["identity"], W]
            out[p + "mlp.correction"] = [r["experts"] + r["identity"]]
    out["final.norm"] = [W]
    out["head"] = [cfg["vocab"], W]
    return out


def attn(heads=4, kv_heads=2, dim=8, vdim=8, size=11, coef=0.3, every=4, scale=None, mlp="dense"):
    """A layer with the attention mixer; mlp: None, "dense", a dict, or moe(...)."""
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size},
                      "q_temp": {"coef": coef, "every": every}, "scale": float(scale if scale is not None else dim ** -0.5)},
            "mlp": dense() if mlp == "dense" else mlp}


def gru(width=24, mlp="dense"):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": dense() if mlp == "dense" else mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, identity=2, top=2, count=2, keep=1, scale=1.5, ff=16):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": count, "keep": keep}, "scale": scale}}


def config(layers, vocab=101, width=40, eps=1e-5, embed_scale=0.5):
    return {"architecture": "Lugipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
            "layers": layers}


def bf16_round(a):
    """float -> nearest-even bfloat16 value (as float32)."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def random_weights(cfg, seed=0, scale=None):
    """bf16-representable random weights (float32 arrays): matrices ~ N(0, 1 / fan_in), norm weights
    around one, small biases."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 2 and name != "embed":
            a = rng.standard_normal(shape) / math.sqrt(shape[1])
        elif name == "embed":
            a = rng.standard_normal(shape)
        elif name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif name.endswith("correction"):
            a = 0.1 * rng.standard_normal(shape)
        elif name.endswith("pb"):
            a = -1.0 + 0.5 * rng.standard_normal(shape)
        else:
            a = 0.3 * rng.standard_normal(shape)
        w[name] = bf16_round(a)
    return w
