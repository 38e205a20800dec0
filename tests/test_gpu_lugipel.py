"""GPU: the Lugipel design on the layered engine tier (sliding-window attention with sigmoid weights, a query
temperature, head slopes and a head gate; the minGRU recurrence; xIELU; the grouped softmax router with identity
experts; pre-norm blocks over a scaled embedding with sinusoidal positions) against the plain numpy restatement
in tests/lugipel_oracle.py, on small random models of several shapes.

fp32 engines are held to REL32 of the logits' spread, bf16 engines to REL16.  Weights are made peaky where a
fault would otherwise hide: beacon tokens whose keys alone carry weight sit at the windows' edges and far back,
update gates near zero make early tokens live on in the recurrent state.
"""
import numpy as np
import pytest

import lugipel_oracle as O
from lugipel_oracle import attn, dense, gru, moe

pytestmark = pytest.mark.gpu

REL32 = 2e-4
REL16 = 5e-2


def words(a):
    """float32 values that are exact bf16 -> bf16 words"""
    return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(np.shape(a))


MIXED = [attn(size=9), gru(mlp=moe()), attn(heads=6, kv_heads=3, dim=6, vdim=10, size=33, every=7, mlp=moe(5, 1, 3, 3, 2, 0.75)),
         gru(width=70, mlp=None), attn(heads=2, kv_heads=2, dim=12, vdim=4, size=200, mlp=dense(24))]


class Model:
    def __init__(self, layers, seed=0, vocab=101, width=40, dtype="float32", max_ctx=512, slots=4, page_tokens=16,
                 n_pages=0, eps=1e-5, embed_scale=0.5, tweak=None, use_graph=True):
        import qwen_inference_engine_amd as q
        self.rng = np.random.default_rng(seed)
        self.cfg = O.config(layers, vocab=vocab, width=width, eps=eps, embed_scale=embed_scale)
        self.T = O.random_weights(self.cfg, seed=seed)
        if tweak is not None:
            tweak(self.T, self.cfg)             # values must stay exact bf16
        self.spec = q.spec_from_config(self.cfg)
        self.eng = q.Engine(self.spec, max_ctx=max_ctx, dtype=dtype, use_graph=use_graph).load_tensors(
            {k: words(v) for k, v in self.T.items()})
        self.batch = self.eng.batch(slots, max_ctx, page_tokens=page_tokens, n_pages=n_pages)
        self.vocab, self.dtype = vocab, dtype
        self.tol = REL32 if dtype == "float32" else REL16
        self.W64 = {k: np.asarray(v, dtype=np.float64) for k, v in self.T.items()}

    def tokens(self, n):
        return [int(t) for t in self.rng.integers(0, self.vocab, n)]

    def ref(self, toks, want_layers=False, cfg=None):
        return O.forward(cfg or self.cfg, self.W64, toks, want_layers)

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


def err_of(m):
    return rel if m.dtype == "float32" else rel_most


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


def rows_rms(a, b):
    return np.sqrt(((np.asarray(a, dtype=np.float64) - b) ** 2).mean(axis=1))


def assert_right_window(got, want, wrong, tol, min_rows=3):
    """`wrong`: the oracle's logits with other window sizes.  Every row that tells the sizes apart (by more than
    four times the tolerance) must lie much closer to the right size's logits than the wrong size's do, and there
    must be such rows; all rows together stay within the tolerance in the 0.9-quantile."""
    std = np.std(want)
    e = rows_rms(got, want)
    for other in wrong:
        d = rows_rms(other, want)
        tells = d > 4 * tol * std
        assert tells.sum() >= min_rows
        assert np.all(e[tells] < 0.34 * d[tells])
    assert np.quantile(e, 0.9) < tol * std


def beacon(T, cfg, beta=4.0, out_gain=8.0):
    """Makes the last token id a beacon for the attention of layer 0: its key is aligned with every other token's
    query, all other keys are opposed to them, so a visible beacon gets a weight near one and everything else a
    weight near zero.  The last coordinate of the stream is the slowest cosine of the position vector, close to one
    at every position used here: the query and key projections read a fixed head direction `a` from it with
    opposite signs; the beacon's large embedding flips that coordinate's sign after the norm."""
    W, X = cfg["width"], cfg["vocab"] - 1
    m = cfg["layers"][0]["mixer"]
    rng = np.random.default_rng(7)
    r = np.where(rng.random(W) < 0.5, -1.0, 1.0).astype(np.float32)
    r[W - 1] = -1.0
    T["embed"][:, W - 1] = 0.0
    T["embed"][X] = 8.0 * r
    a = np.where(rng.random(m["dim"]) < 0.5, -1.0, 1.0).astype(np.float32)
    T["l0.mix.q"][:, W - 1] = beta * np.tile(a, m["heads"])
    T["l0.mix.k"][:, W - 1] = -beta * np.tile(a, m["kv_heads"])
    for name in ("l0.mix.q.norm", "l0.mix.k.norm"):
        T[name][:] = 1.0
    T["l0.norm1"][W - 1] = 1.0
    T["l0.mix.pb"][:] = 0.0
    T["l0.mix.o"] *= np.float32(out_gain)


def beacon_tokens(m, n, at):
    toks = [t % (m.vocab - 1) for t in m.tokens(n)]
    for p in at:
        if p < n:
            toks[p] = m.vocab - 1
    return toks


def with_window(cfg, delta):
    """The same config with every attention window `delta` positions longer."""
    out = {**cfg, "layers": []}
    for L in cfg["layers"]:
        if L["type"] == "attention":
            L = {**L, "mixer": {**L["mixer"], "mask": {"size": L["mixer"]["mask"]["size"] + delta}}}
        out["layers"].append(L)
    return out


# ------------------------------------------------------------------ mechanisms, one at a time
@pytest.mark.parametrize("layers,kw", [
    ([attn(mlp=None)], {}),
    ([attn(heads=3, kv_heads=3, dim=10, vdim=6, size=5, mlp=None)], {}),          # one key head per query head, dim != vdim
    ([attn(heads=5, kv_heads=1, dim=4, vdim=20, size=64, every=1, coef=1.5, mlp=None)], {}),   # one key head; a temperature that moves at every position
    ([attn(coef=0.0, every=1000, size=1, mlp=None)], {}),                         # no temperature; a window of the token itself
    ([gru(mlp=None)], {}),
    ([gru(width=300, mlp=None)], {"width": 24}),                                  # wider than the stream, two channel blocks
    ([attn(mlp=dense(56))], {}),
    ([gru(mlp=moe(6, 2, 2, 2, 1, 1.5))], {}),
    ([attn(mlp=moe(8, 0, 3, 1, 1, 1.0))], {}),                                    # no identity experts, one group, scale 1
    ([gru(mlp=moe(4, 4, 1, 4, 2, 2.5))], {}),                                     # one expert chosen: its weight is the scale
    ([attn(mlp=moe(3, 3, 4, 3, 2, 0.5))], {}),                                    # every expert of the kept groups chosen
    ([attn(mlp=moe(1, 5, 2, 2, 2, 1.0))], {}),                                    # mostly identity experts, every group kept
    (MIXED, {}),
    (MIXED, {"width": 37, "embed_scale": 1.0, "vocab": 33}),                      # an odd width, unscaled embedding
], ids=["attn", "attn-mha", "attn-mqa-temp", "attn-self-only", "mingru", "mingru-wide", "xielu", "moe", "moe-plain", "moe-top1",
        "moe-all-kept", "moe-identity", "mixed", "mixed-odd"])
def test_mechanism_streams_match_oracle(model, layers, kw):
    m = model(layers, seed=len(layers) + 3, **kw)
    toks = m.tokens(29)
    m.batch.keep_layers(True)
    got = m.batch.step([(0, toks)], range(len(toks)))
    want, want_layers = m.ref(toks, want_layers=True)
    assert len(want_layers) == m.spec.n_runs
    streams = m.batch.step_layers(len(toks))
    for i, w in enumerate(want_layers):
        assert rel(streams[i], w) < REL32, f"stream after layer {i}"
    assert rel(got, want) < REL32


def test_xielu_both_branches_and_its_two_numbers(model):
    """Large pre-activations of both signs: the square branch, the exponential branch and both numbers show."""
    def tw(T, cfg):
        T["l0.mlp.up"] *= np.float32(4.0)
        T["l0.mlp.act"][:] = O.bf16_round(np.array([1.25, -0.75]))
    m = model([gru(mlp=dense(40))], seed=5, tweak=tw)
    toks = m.tokens(20)
    want = m.ref(toks)
    assert rel(m.batch.step([(0, toks)], range(20)), want) < REL32
    other = {**m.W64, "l0.mlp.act": np.array([1.25, 0.75])}
    assert rel(O.forward(m.cfg, other, toks), want) > 1e-2          # the oracle itself feels the second number


def test_router_correction_groups_and_negative_choice_scores(model):
    """A correction far below zero makes every choice score negative: the experts outside the kept group must
    be excluded outright (a masked score of zero would win against them); the correction picks the experts but the weights are the plain scores."""
    def tw(T, cfg):
        T["l0.mlp.correction"][:] = np.array([-5.0, -6.25, -7.5, -3.0, -6.0, -6.5, -7.0, -4.5], dtype=np.float32)
    m = model([gru(mlp=moe(6, 2, 2, 2, 1, 1.5))], seed=6, tweak=tw)
    toks = m.tokens(24)
    W = m.W64
    x0 = O.embed(toks, W["embed"], 0.5)
    x1 = x0 + O.min_gru(O.rms(x0, 1e-5) * W["l0.norm1"], W, "l0.mix.")[0]
    h = O.rms(x1, 1e-5) * W["l0.norm2"]
    chosen = [O.route(r, W, "l0.mlp.", m.cfg["layers"][0]["mlp"]["router"])[0] for r in h]
    assert all(c == [3, 0] for c in chosen)                          # the group that holds the -3, its two best
    assert rel(m.batch.step([(0, toks)], range(24)), m.ref(toks)) < REL32


def test_router_ties_go_to_the_lower_index(model):
    def tw(T, cfg):
        T["l0.mlp.router"][4] = T["l0.mlp.router"][1]
        T["l0.mlp.correction"][4] = T["l0.mlp.correction"][1]
        T["l0.mlp.router"][3] = T["l0.mlp.router"][0]
        T["l0.mlp.correction"][3] = T["l0.mlp.correction"][0]
    m = model([attn(mlp=moe(6, 0, 2, 1, 1, 1.0))], seed=8, tweak=tw)
    toks = m.tokens(31)
    assert rel(m.batch.step([(0, toks)], range(31)), m.ref(toks)) < REL32


# ------------------------------------------------------------------ prompts, portions, decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_equals_token_by_token_and_portions(model, dtype):
    m = model(MIXED, seed=11, dtype=dtype)
    toks = m.tokens(75)
    want = m.ref(toks)
    err = err_of(m)
    whole = m.batch.step([(0, toks)], range(75))
    assert err(whole, want) < m.tol
    one = feed(m, 1, toks, [])
    assert err(one, want) < m.tol
    m.batch.release(0)
    for slot, cuts in ((2, [2, 2, 3, 16, 17, 2, 30]), (3, [40, 33]), (0, [1, 2, 63, 2])):
        assert err(feed(m, slot, toks, cuts), want) < m.tol, cuts
    if dtype == "float32":
        assert rel(one, whole) < REL32


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_step_equal_each_alone(model, dtype):
    m = model(MIXED, seed=12, dtype=dtype, slots=4)
    seqs = [m.tokens(n) for n in (50, 3, 21, 34)]
    want = [m.ref(s) for s in seqs]
    err = err_of(m)
    # step 1: portions of unequal size; step 2: a single token beside portions; step 3: the rest
    cuts = [(30, 1, 20, 2), (1, 1, 1, 30), (19, 1, 0, 2)]
    pos = [0, 0, 0, 0]
    got = [[] for _ in seqs]
    for cut in cuts:
        entries, want_rows, row = [], [], 0
        for i, n in enumerate(cut):
            if n == 0:
                continue
            entries.append((i, seqs[i][pos[i]:pos[i] + n]))
            want_rows.append((i, row, n))
            row += n
        lg = m.batch.step(entries, range(row))
        for i, r0, n in want_rows:
            got[i].append(lg[r0:r0 + n])
            pos[i] += n
    for i in range(4):
        assert pos[i] == len(seqs[i])
        assert err(np.concatenate(got[i]), want[i]) < m.tol, i


def test_pages_slots_and_states_are_used_again(model):
    """A pool smaller than the traffic: requests come and go through two slots.  Update gates near zero make the
    state remember its first tokens, so a state left behind by the slot's previous request would show."""
    def tw(T, cfg):
        T["l1.mix.z.b"][:] = np.float32(-4.0)
        T["l3.mix.z.b"][:] = np.float32(-4.0)
    m = model(MIXED, seed=13, slots=2, n_pages=8, max_ctx=64, tweak=tw)
    # the oracle carries token 0 to the last row through the state
    a = m.tokens(40)
    b2 = [(a[0] + 1) % m.vocab] + a[1:]
    assert rel(m.ref(b2)[-1:], m.ref(a)[-1:]) > 1e-3
    free0 = m.batch.page_stats()[0]
    for k, n in enumerate((40, 64, 17, 33, 64, 5)):
        slot = k % 2
        toks = m.tokens(n)
        got = feed(m, slot, toks, [n // 2, 2, n])
        assert rel(got, m.ref(toks)) < REL32, k
        m.batch.release(slot)
        assert m.batch.page_stats()[0] == free0
    # seven pages of 16: four held by slot 0 leave three, a request of 49 tokens is refused with nothing run
    m.batch.step([(0, m.tokens(64))], [])
    toks = m.tokens(49)
    with pytest.raises(Exception):
        m.batch.step([(1, toks)], [])
    assert rel(m.batch.step([(1, toks[:48])], range(48)), m.ref(toks[:48])) < REL32
    assert m.batch.page_stats()[0] == 0


@pytest.mark.parametrize("size", [7, 16, 17, 40])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edges_in_prompts_and_decoding(model, size, dtype):
    """Windows shorter than, equal to and longer than a page, with beacon tokens (see beacon()) a little more than a
    window apart: a row sees one beacon or none, so the row at which a beacon is the last key the window holds, and
    the next row, which has lost it, tell the window's size: the oracle with a window one key shorter or longer
    differs there far beyond the tolerance (asserted first); the engine must agree with the right size for whole
    prompts, portions cut around the window's length, and decoding."""
    m = model([attn(heads=2, kv_heads=1, dim=8, vdim=8, size=size, coef=0.0, scale=1.5, mlp=None), gru(mlp=None)], seed=size,
              dtype=dtype, tweak=beacon)
    n = 3 * size + 30
    toks = beacon_tokens(m, n, range(2, n, size + 3))
    want = m.ref(toks)
    wrong = [m.ref(toks, cfg=with_window(m.cfg, d)) for d in (-1, 1)]
    assert_right_window(m.batch.step([(0, toks)], range(n)), want, wrong, m.tol)
    assert_right_window(feed(m, 1, toks, [size - 1, 2, size, 3]), want, wrong, m.tol)
    assert_right_window(feed(m, 2, toks, [size + 1]), want, wrong, m.tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_key_across_pages(model, dtype):
    """A window of 300 keys over pages of 16 with one beacon token near the start of the sequence: it is the only key
    that carries weight, up to 299 positions and 18 pages back; the row at which it leaves the window is among
    those decoded one by one."""
    m = model([attn(heads=2, kv_heads=2, dim=8, vdim=8, size=300, coef=0.2, every=50, scale=1.5, mlp=dense(24))], seed=21,
              dtype=dtype, max_ctx=512, tweak=beacon)
    toks = beacon_tokens(m, 330, (5,))
    want = m.ref(toks)
    wrong = [m.ref(toks, cfg=with_window(m.cfg, -250)), m.ref(toks, cfg=with_window(m.cfg, -1)), m.ref(toks, cfg=with_window(m.cfg, 1))]
    assert_right_window(m.batch.step([(0, toks)], range(330)), want, wrong, m.tol, min_rows=1)
    assert_right_window(feed(m, 1, toks, [295]), want, wrong, m.tol, min_rows=1)   # 35 tokens decoded one by one over the window's edge


def test_first_tokens_of_a_sequence(model):
    m = model(MIXED, seed=31)
    for n in (1, 2, 3):
        toks = m.tokens(n)
        assert rel(m.batch.step([(0, toks)], range(n)), m.ref(toks)) < REL32
        m.batch.release(0)
        assert rel(feed(m, 0, toks, []), m.ref(toks)) < REL32
        m.batch.release(0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model, dtype):
    m = model(MIXED, seed=41, dtype=dtype)
    toks = m.tokens(340)
    want = m.ref(toks)
    got = feed(m, 0, toks, [10])
    assert err_of(m)(got, want) < m.tol
    if dtype == "float32":
        assert rel(got[-20:], want[-20:]) < REL32


def test_long_portions_run_the_recurrence_in_pieces(model):
    """Portions above 128 rows are scanned in pieces with a carry pass: from a fresh state and from a kept one,
    beside short entries of other slots; update gates near zero keep the early tokens alive."""
    def tw(T, cfg):
        T["l0.mix.z.b"][:] = np.float32(-3.0)
    m = model([gru(width=50, mlp=None), attn(size=20, mlp=dense(24)), gru(mlp=None)], seed=51, max_ctx=1024, tweak=tw)
    a, b2, c = m.tokens(900), m.tokens(140), m.tokens(9)
    wa, wb, wc = m.ref(a), m.ref(b2), m.ref(c)
    g1 = m.batch.step([(0, a[:400]), (1, b2[:3]), (2, c)], range(412))
    assert rel(g1[:400], wa[:400]) < REL32 and rel(g1[400:403], wb[:3]) < REL32 and rel(g1[403:], wc) < REL32
    g2 = m.batch.step([(1, b2[3:]), (0, a[400:])], range(637))
    assert rel(g2[:137], wb[3:]) < REL32 and rel(g2[137:], wa[400:]) < REL32


# ------------------------------------------------------------------ the matrix-core attention (bf16 caches)
@pytest.mark.parametrize("heads,kv,dim,vdim,pt,size", [
    (4, 1, 32, 32, 32, 50),      # four heads of one key head share its tiles
    (8, 2, 64, 32, 64, 200),
    (2, 1, 128, 64, 32, 33),     # head ratio 2: heads packed into a wave's columns
    (3, 3, 32, 128, 64, 90),
    (8, 1, 32, 32, 32, 70),      # eight heads of one key head: two workgroups share its tiles
    (6, 2, 64, 32, 64, 45),      # head ratio 3: packed
    (4, 4, 64, 64, 16, 40),      # pages too small for the matrix-core form: the plain kernel on bf16 rows
])
def test_bf16_attention_shapes(model, heads, kv, dim, vdim, pt, size):
    m = model([attn(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, size=size, every=16, mlp=None), gru(width=64, mlp=dense(64))],
              seed=heads * dim, width=64, dtype="bfloat16", page_tokens=pt, max_ctx=512)
    toks = m.tokens(260)
    want = m.ref(toks)
    assert rel_most(m.batch.step([(0, toks)], range(260)), want) < REL16
    got = feed(m, 1, toks, [3, 40, 2, 100, 17, 70])          # then 28 single tokens: key splits
    assert rel_most(got, want) < REL16
    sizes_seen = rel(m.ref(toks, cfg=with_window(m.cfg, -size // 2))[size:], want[size:])
    assert sizes_seen > 1e-3                                  # the window's far half matters to the oracle


def test_bf16_window_edge_on_the_matrix_cores(model):
    """Beacon tokens at the window's last key and just beyond it, on the matrix-core kernel (32-key blocks, pages of
    32) in prompts, portions and decoding, for windows around the block and page sizes."""
    for size in (31, 32, 33, 64, 65):
        m = model([attn(heads=4, kv_heads=1, dim=32, vdim=32, size=size, coef=0.0, scale=0.375, mlp=None)], seed=size, width=64,
                  dtype="bfloat16", page_tokens=32, tweak=beacon)
        n = 3 * size + 30
        toks = beacon_tokens(m, n, range(2, n, size + 3))
        want = m.ref(toks)
        wrong = [m.ref(toks, cfg=with_window(m.cfg, d)) for d in (-1, 1)]
        assert_right_window(m.batch.step([(0, toks)], range(n)), want, wrong, REL16)
        assert_right_window(feed(m, 1, toks, [size - 1, 2, size + 1, 5]), want, wrong, REL16)


# ------------------------------------------------------------------ generation, graphs, programs
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
    m = model(MIXED, seed=71)
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
    layers = MIXED if dtype == "float32" else [attn(heads=4, kv_heads=1, dim=32, vdim=32, size=40, mlp=None), gru(mlp=moe())]
    kw = dict(seed=91, dtype=dtype, width=40 if dtype == "float32" else 64, page_tokens=32)
    a = Model(layers, **kw)
    b = Model(layers, use_graph=False, **kw)
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
        assert err_of(a)(np.stack(a.tail), a.ref(toks)[40:60]) < a.tol
    finally:
        a.close()
        b.close()


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
    cfg = O.config(MIXED, vocab=89, width=40)
    T = O.random_weights(cfg, seed=81)
    W64 = {k: np.asarray(v, dtype=np.float64) for k, v in T.items()}
    write_model_dir(tmp_path, cfg, T)
    reqs = {k: [int(t) for t in rng.integers(0, 89, n)] for k, n in (("a", 70), ("b", 9), ("c", 33), ("d", 50), ("e", 64))}
    want = {k: O.forward(cfg, W64, v) for k, v in reqs.items()}
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
        ref = staticmethod(lambda toks: O.forward(cfg, W64, toks))
    assert got["tokens[0]"] == oracle_greedy(M, reqs["b"], 5)
    assert got["tokens[1]"] == oracle_greedy(M, reqs["c"], 5)
