"""CPU: the Lugipel config reader and registry, tensor names, and the plain restatement's own properties."""
import numpy as np
import pytest

import lugipel_oracle as O
from lugipel_oracle import attn, dense, gru, moe

from qwen_inference_engine_amd import spec as S

LAYERS = [attn(size=9), gru(mlp=moe()), attn(heads=6, kv_heads=3, dim=6, vdim=10, size=33, every=7, mlp=moe(5, 1, 3, 3, 2, 0.75)),
          gru(width=70, mlp=None)]


def test_config_reader_and_registry():
    cfg = O.config(LAYERS, vocab=77, width=24, eps=2e-6, embed_scale=0.25)
    sp = S.spec_from_config(cfg)
    assert isinstance(sp, S.LayeredSpec) and sp.block == "prenorm" and sp.pos_embed == "sinusoid" and not sp.tied_head
    assert sp.embed_scale == 0.25 and sp.norm_eps == 2e-6 and sp.width == 24 and sp.vocab == 77 and sp.n_runs == 4
    a = sp.layers[2].mixer
    assert isinstance(a, S.GqaAttention) and (a.heads, a.kv_heads, a.dim, a.vdim) == (6, 3, 6, 10)
    assert a.mask == "window" and a.mask_size == 33 and a.weights == "sigmoid" and a.slope_bias and a.head_gate
    assert a.q_temp_every == 7 and a.q_temp_coef == 0.3 and a.qk_norm == "weight" and a.rot_dims == 0
    assert isinstance(sp.layers[1].mixer, S.MinGru) and sp.layers[3].mixer.width == 70 and sp.layers[3].mlp is None
    f = sp.layers[2].mlp
    assert (f.kind, f.experts, f.identity, f.top, f.groups, f.groups_keep, f.route_scale) == ("moe", 5, 1, 3, 3, 2, 0.75)
    assert f.router == "softmax_all" and sp.layers[0].mlp.act == "xielu"
    assert sp.state_elems() == 24 + 70
    assert sp.cache_row_elems() == 2 * (8 + 8) + 3 * (6 + 10)
    assert sp.tensor_shapes() == O.tensor_shapes(cfg)
    arch, keep = sp.to_c()
    assert arch.n_layers == 4 and arch.layers[1].mingru.width == 24 and arch.layers[2].identity == 1


def test_config_reader_refuses_what_it_does_not_know():
    with pytest.raises(ValueError):
        S.spec_from_config(O.config([{"type": "conv", "mixer": {}, "mlp": None}]))
    with pytest.raises(ValueError):
        S.spec_from_config(O.config([gru(mlp=moe(5, 2, 2, 2, 1))]))          # 7 outputs do not form 2 groups
    with pytest.raises(ValueError):
        S.spec_from_config(O.config([gru(mlp=moe(6, 2, 5, 2, 1))]))          # top above the kept group's experts
    with pytest.raises(ValueError):
        S.spec_from_config(O.config([gru(mlp={"kind": "glu", "ff": 8})]))


def weights(cfg, seed=0):
    return {k: np.asarray(v, dtype=np.float64) for k, v in O.random_weights(cfg, seed).items()}


def test_min_gru_is_its_unrolled_sum_and_carries_its_state():
    cfg = O.config([gru(width=12, mlp=None)], width=16)
    w = weights(cfg, 1)
    h = np.random.default_rng(2).standard_normal((9, 16))
    out, S_end = O.min_gru(h, w, "l0.mix.")
    z = O.sigmoid(h @ w["l0.mix.z"].T + w["l0.mix.z.b"])
    u = h @ w["l0.mix.x"].T + w["l0.mix.x.b"]
    c = np.where(u >= 0, u + 0.5, O.sigmoid(u))
    S = sum(z[j] * c[j] * np.prod(1 - z[j + 1:], axis=0) for j in range(9))
    assert np.allclose(S, S_end)
    a, Sa = O.min_gru(h[:4], w, "l0.mix.")
    b, Sb = O.min_gru(h[4:], w, "l0.mix.", Sa)
    assert np.allclose(np.concatenate([a, b]), out) and np.allclose(Sb, S_end)
    assert np.all(c > 0)                                                     # the candidate is positive on both branches


def test_attention_window_and_weights():
    cfg = O.config([attn(heads=2, kv_heads=1, dim=4, vdim=4, size=3, mlp=None)], width=8)
    w = weights(cfg, 3)
    h = np.random.default_rng(4).standard_normal((7, 8))
    full = O.sigmoid_attention(h, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    h2 = h.copy()
    h2[1] += 1.0                                                             # position 1 is seen by 1, 2, 3 only
    moved = O.sigmoid_attention(h2, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    changed = np.abs(moved - full).max(axis=1) > 1e-12
    assert list(changed) == [False, True, True, True, False, False, False]
    assert O.head_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]
    assert O.query_temperature(6, 0.5, 4) == 1 + 0.5 * np.log(2) and O.query_temperature(2, 0.5, 4) == 1.0


def test_router_weights_sum_to_the_scale_and_stay_in_the_kept_groups():
    cfg = O.config([gru(mlp=moe(6, 2, 3, 4, 2, 1.5))], width=16)
    w = weights(cfg, 5)
    r = cfg["layers"][0]["mlp"]["router"]
    rng = np.random.default_rng(6)
    for _ in range(20):
        chosen, ws = O.route(rng.standard_normal(16), w, "l0.mlp.", r)
        assert len(set(chosen)) == 3 and abs(ws.sum() - 1.5) < 1e-12
        assert len({e // 2 for e in chosen}) <= 2
    # an identity expert passes its input through with its weight
    w["l0.mlp.correction"][:] = [-9, -9, -9, -9, -9, -9, 5, 4]
    h = rng.standard_normal((1, 16))
    r1 = {**r, "top": 2, "groups": {"count": 4, "keep": 1}}
    assert np.allclose(O.moe_ff(h, w, "l0.mlp.", {**cfg["layers"][0]["mlp"], "router": r1}), 1.5 * h)


def test_xielu_is_continuous_with_slope_one_half_at_zero():
    z = np.array([-1e-6, 0.0, 1e-6])
    y = O.xielu(z, 0.3, -0.2)
    assert y[1] == 0 and np.allclose(np.diff(y) / 1e-6, 0.5, atol=1e-5)
    assert np.isclose(O.xielu(np.array([2.0]), 0.3, -0.2)[0], O.softplus(0.3) * 4 + 1)


def test_position_vector_pairs():
    v = O.position_vector(5, 7)
    assert np.isclose(v[0], np.sin(5)) and np.isclose(v[1], np.cos(5)) and np.isclose(v[6], np.sin(5 * 10000 ** (-6 / 7)))
