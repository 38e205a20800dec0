"""CPU: the Verelorn design's configuration reader and registry, its tensor names and sizes, and properties of the
plain restatement in tests/verelorn_oracle.py that the GPU tests lean on."""
import math

import numpy as np
import pytest

import verelorn_oracle as O
from verelorn_oracle import attn, delta, latent

from qwen_inference_engine_amd import spec as S


def public(cfg):
    return {k: v for k, v in cfg.items() if not k.startswith("_")}


LAYERS = [latent(), attn(scaling=(8.0, 1.0, 4.0, 64)), delta(), latent(kv_from=0, mlp=None), delta(heads=4, kv_heads=2, ranks=(3, 7), mlp="dense")]


def test_config_reader_and_registry():
    cfg = O.config(LAYERS, vocab=77, width=24, streams=5, taps=2)
    sp = S.spec_from_config(public(cfg))
    assert isinstance(sp, S.LayeredSpec) and "Verelorn" in S.ARCHITECTURES
    assert (sp.block, sp.norm_offset, sp.streams, sp.canon_taps, sp.embed_norm, sp.tied_head) == ("prenorm", 1.0, 5, 2, True, False)
    a, l0, d = sp.layers[1].mixer, sp.layers[0].mixer, sp.layers[2].mixer
    assert isinstance(a, S.GqaAttention) and a.values_are_keys and a.qk_bias and a.sink and a.out_gate and a.mask == "causal"
    assert a.rot_layout == "halves" and a.rot_scaling == (8.0, 1.0, 4.0, 64.0)
    assert isinstance(l0, S.LatentAttention) and l0.q_rank == 24 and l0.rot_layout == "interleaved" and not l0.head_gate and l0.window == 0
    assert sp.layers[3].mixer.kv_from == 0 and sp.layers[3].mlp is None
    assert isinstance(d, S.ChannelDelta) and d.rank_a == 0        # the config does not carry the ranks
    assert sp.layers[1].mlp.act == "gelu_tanh_gated"
    plain = S.spec_from_config(public(O.config([attn()], streams=0, taps=0)))
    assert plain.streams == 0 and plain.canon_taps == 0
    arch, _keep = sp.to_c()
    assert (arch.streams, arch.canon_taps, arch.embed_norm) == (5, 2, 1) and arch.layers[2].delta.conv == 3


def test_tensor_names_and_sizes_from_the_tensors():
    cfg = O.config(LAYERS, vocab=77, width=24, streams=5, taps=2)
    T = O.random_weights(cfg)
    sp = S.with_tensor_sizes(S.spec_from_config(public(cfg)), {k: list(v.shape) for k, v in T.items()})
    assert (sp.layers[2].mixer.rank_a, sp.layers[2].mixer.rank_g) == (6, 5)
    assert (sp.layers[4].mixer.rank_a, sp.layers[4].mixer.rank_g) == (3, 7)
    shapes = sp.tensor_shapes()
    assert set(shapes) == set(T)
    assert all(list(T[k].shape) == shapes[k] for k in shapes)
    assert "l3.mix.dkv" not in shapes and "l3.hc2.in" not in shapes and shapes["l1.mix.g"] == [4 * 16, 24]
    # per token: two latent rows and the attention's keys twice; per slot: the input taps, the delta states and their taps
    assert sp.cache_row_elems() == (16 + 4) + 2 * 2 * 16
    assert sp.state_elems() == 5 * 1 * 24 + (2 * 8 * 12 + 2 * (2 * 8 + 24)) + (4 * 8 * 12 + 2 * (2 * 16 + 48))
    with pytest.raises(ValueError):
        S.with_tensor_sizes(S.spec_from_config(public(cfg)), {})


def test_refusals():
    cfg = public(O.config([attn()]))
    cfg["layers"][0]["type"] = "window_attention"
    with pytest.raises(ValueError):
        S.spec_from_config(cfg)
    cfg = public(O.config([attn()]))
    cfg["layers"][0]["mixer"]["vdim"] = 8
    with pytest.raises(ValueError):
        S.spec_from_config(cfg)
    cfg = public(O.config([attn()], streams=33))
    with pytest.raises(ValueError):
        S.spec_from_config(cfg)


def test_scaled_frequencies_have_three_regimes():
    rot = {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    f0 = O.rotary_freqs({"base": 10000.0, "dims": 16})
    f = O.rotary_freqs(rot)
    lam = 2 * math.pi / f0
    kept, slowed = lam < 16, lam > 64
    assert kept.any() and slowed.any() and (~kept & ~slowed).any()
    assert np.allclose(f[kept], f0[kept]) and np.allclose(f[slowed], f0[slowed] / 4)
    mid = ~kept & ~slowed
    assert np.all(f[mid] < f0[mid]) and np.all(f[mid] > f0[mid] / 4)


def test_rotary_layouts_are_relative():
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(1, 12)), rng.normal(size=(1, 12))
    for layout in ("halves", "interleaved"):
        rot = {"base": 50.0, "dims": 8}
        d = [(O.rotate(q, np.array([p + 5]), rot, layout) @ O.rotate(k, np.array([p]), rot, layout).T).item() for p in (0, 9, 40)]
        assert np.allclose(d, d[0])
        assert np.array_equal(O.rotate(q, np.array([7]), rot, layout)[:, 8:], q[:, 8:])       # the rest passes unchanged
    a, b = O.rotate(q, np.array([3]), {"base": 50.0, "dims": 8}, "halves"), O.rotate(q, np.array([3]), {"base": 50.0, "dims": 8}, "interleaved")
    assert not np.allclose(a, b)


def test_causal_conv_reaches_back_taps_minus_one():
    x = np.zeros((6, 2))
    x[1] = 1.0
    w = np.array([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    y = O.causal_conv(x, w)
    assert np.array_equal(y[:, 0], [0, 3, 2, 1, 0, 0]) and np.array_equal(y[:, 1], [0, 6, 5, 4, 0, 0])


def test_sink_only_joins_the_denominator():
    s = np.zeros((1, 3, 3))
    s[0, 1, 1] = math.log(3.0)
    w = O.softmax_causal(s, sink=np.array([math.log(4.0)]))
    assert np.allclose(w[0, 0], [0.2, 0, 0]) and np.allclose(w[0, 1], [1 / 8, 3 / 8, 0]) and np.allclose(w[0, 2], [1 / 7] * 3)


def test_delta_rule_equals_its_unrolled_form_and_carries_its_state():
    cfg = O.config([delta(heads=2, kv_heads=1, dim=4, vdim=3, conv=2)], width=16, streams=0, taps=0)
    T = O.random_weights(cfg, seed=2)
    T["l0.mix.A_log"][:] = -6.0
    W = {k: v.astype(np.float64) for k, v in T.items()}
    rng = np.random.default_rng(1)
    h = rng.normal(size=(9, 16))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    out = O.channel_delta(m, W, p, h, 1e-5)
    # the same rule as one matrix recurrence: S_t = (I - beta k k^T) diag(g) S_(t-1) + beta k v^T
    q = O.unit_vectors(O.silu(O.causal_conv(h @ W[p + "q"].T, W[p + "q.conv"]))) * 4 ** -0.5
    k = O.unit_vectors(O.silu(O.causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])))
    v = O.silu(O.causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(9, 2, 3)
    beta = O.sigmoid(h @ W[p + "b"].T)
    g = np.exp(-np.exp(W[p + "A_log"])[None, :, None] * O.softplus((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).reshape(9, 2, 4))
    o = np.zeros((9, 2, 3))
    for hh in range(2):
        S = np.zeros((4, 3))
        for t in range(9):
            A = (np.eye(4) - beta[t, hh] * np.outer(k[t], k[t])) @ np.diag(g[t, hh])
            S = A @ S + beta[t, hh] * np.outer(k[t], v[t, hh])
            o[t, hh] = S.T @ q[t]
    gate = O.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).reshape(9, 2, 3)
    want = ((O.rms_unit(o, 1e-5) * W[p + "norm"]) * gate).reshape(9, 6) @ W[p + "o"].T
    assert np.allclose(out, want, rtol=1e-9, atol=1e-12)
    h2 = h.copy()
    h2[0] += 1.0
    assert np.abs(O.channel_delta(m, W, p, h2, 1e-5)[-1] - out[-1]).max() > 1e-4     # row 0 lives on in the state


def test_identity_hyper_connections_are_the_plain_residual():
    layers = [attn(), delta(mlp="dense")]
    c1, c0 = O.config(layers, streams=1, taps=2), O.config(layers, streams=0, taps=2)
    T = O.random_weights(c1, seed=4)
    for k in T:
        if ".hc" in k:
            T[k][...] = 1.0
    W = {k: v.astype(np.float64) for k, v in T.items()}
    toks = list(range(12))
    assert np.allclose(O.forward(c1, W, toks), O.forward(c0, W, toks), rtol=1e-10, atol=1e-12)
    c3 = O.config(layers, streams=3, taps=2)
    T3 = O.random_weights(c3, seed=4)
    l3, l1 = [], []
    O.forward(c3, {k: v.astype(np.float64) for k, v in T3.items()}, toks, l3)
    assert l3[0].shape == (12, 40)


def test_borrowed_latent_rows_are_the_owner_s():
    cfg = O.config([latent(), latent(heads=3, dim=5, vdim=9, q_rank=10, kv_from=0)], streams=2, taps=0)
    W = {k: v.astype(np.float64) for k, v in O.random_weights(cfg, seed=6).items()}
    assert "l1.mix.dkv" not in W
    a = O.forward(cfg, W, list(range(10)))
    W2 = dict(W, **{"l0.mix.dkv.norm": W["l0.mix.dkv.norm"] * 1.5})
    assert np.abs(O.forward(cfg, W2, list(range(10))) - a).max() > 1e-3
