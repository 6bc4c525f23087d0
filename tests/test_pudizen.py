"""Pudizen on the CPU engine (fp32) against the plain reference in
pudizen_oracle.py: each mechanism alone, then the engine's step function,
cache manager and scheduler under many ways of cutting and batching the same
sequences. Configurations are small and deliberately irregular (see
pudizen_util.small_config)."""

import math

import pytest
import torch

import pudizen_oracle as oracle
import pudizen_util as U
from parallax_amd import ops
from parallax_amd.models.config import ModelConfig
from parallax_amd.models.forward_meta import ForwardMeta
from parallax_amd.models.pudizen import PudizenShardModel
from parallax_amd.models.rope import wavelength_scaled_frequencies
from parallax_amd.parallel.layers import PairHashEmbedding
from parallax_amd.server.kv_cache import MLAKVCache
from parallax_amd.server.sampling_params import SamplingParams

D = torch.float64
TOL = 2e-5
EPS = 1e-5
WIDTH = 40


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = U.small_config()
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("pz")), cfg, w)
    return cfg, w, path


# -- mechanisms alone ------------------------------------------------------------


def test_config_reader():
    cfg = U.small_config()
    mc = ModelConfig.from_hf_config(cfg)
    assert mc.architecture == "Pudizen" and mc.num_layers == 6
    assert mc.layer_types == ["sliding_attention", "latent_attention", "attention",
                              "sliding_attention", "attention", "latent_attention"]
    # (key width, value width) over all kv heads; the latent alone
    assert mc.latent_cache_dims(0, 6) == [(16, 8), (24, 0), (24, 40), (24, 36),
                                          (64, 32), (40, 0)]
    assert mc.latent_cache_dims(2, 4) == [(24, 40), (24, 36)]
    assert mc.pooled_cache_blocks(0, 6) == [0] * 6
    assert mc.linear_state_shapes(0, 6) == [] and not mc.has_linear_layers
    assert mc.norm_groups == 5 and mc.embed_scale == 2.5
    assert mc.pair_hash == {"buckets": 61, "mul_prev": 13, "mul_cur": 5}
    with pytest.raises(ValueError):
        ModelConfig.from_hf_config(
            U.small_config([{"type": "gla", "mixer": {"heads": 1, "dim": 8}, "mlp": None}]))
    with pytest.raises(ValueError):
        ModelConfig.from_hf_config(U.small_config(groups=7))     # 40 / 7


@pytest.mark.parametrize("groups", [1, 5, 8, 40])
def test_grouped_norm_over_the_parallel_residual(groups):
    g = torch.Generator().manual_seed(groups)
    T, W = 6, 40
    x = torch.randn(T, W, generator=g) * 2 + 0.5
    x[:, :W // 2] *= 30.0        # groups of very different size: one shared rms would show
    a = torch.randn(T, W, generator=g) * 5
    b = torch.randn(T, W, generator=g) * 0.1
    wn = 1.0 + torch.randn(W, generator=g) * 0.3
    x1 = x.clone()
    h = ops.group_rmsnorm_add(x1, a, b, wn, groups, EPS, torch.float32)
    want_x = x.double() + (a.double() + b.double())
    torch.testing.assert_close(x1.double(), want_x, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(h.double(), oracle.group_norm(want_x, wn.double(), groups, EPS),
                               rtol=1e-5, atol=1e-5)
    if groups not in (1, 40):
        one = oracle.group_norm(want_x, wn.double(), 1, EPS)
        assert (h.double() - one).abs().max() > 0.1
    # the norm alone (the first layer's), one branch alone, and no norm at all
    x2 = x.clone()
    h2 = ops.group_rmsnorm_add(x2, None, None, wn, groups, EPS, torch.float32)
    assert torch.equal(x2, x)
    torch.testing.assert_close(h2.double(), oracle.group_norm(x.double(), wn.double(), groups, EPS),
                               rtol=1e-5, atol=1e-5)
    x3 = x.clone()
    assert ops.group_rmsnorm_add(x3, a, None, None, groups, EPS, torch.float32) is None
    torch.testing.assert_close(x3.double(), x.double() + a.double(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("buckets,mp,mc", [(61, 13, 5), (1, 3, 2), (7, 1, 1), (499, 1000003, 999983)])
def test_pair_hash_embedding(buckets, mp, mc):
    g = torch.Generator().manual_seed(1)
    V, W = 83, 12
    emb = PairHashEmbedding(V, W, buckets, mp, mc, 1.75)
    emb.weight.data.copy_(torch.randn(V, W, generator=g))
    emb.pair.data.copy_(torch.randn(buckets + 1, W, generator=g))
    toks = U.tokens(40, V, 2)
    w = {"embed": emb.weight.double(), "bigram": emb.pair.double()}
    spec = {"scale": 1.75, "bigram": {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}}
    want = oracle.embedding(toks, w, spec)
    ids = torch.tensor(toks)
    prev = torch.tensor([-1] + toks[:-1])
    torch.testing.assert_close(emb(ids, prev).double(), want, rtol=1e-6, atol=1e-6)
    # the first token takes the extra last row, whatever it is
    torch.testing.assert_close(emb(ids[:1], prev[:1])[0].double(),
                               w["embed"][toks[0]] * 1.75 + w["bigram"][buckets])
    # a portion that starts in the middle: its first token has a predecessor
    torch.testing.assert_close(emb(ids[17:], prev[17:]).double(), want[17:], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("spec", [U.rot(8), U.rot(16, 10000.0, None), U.rot(32, 40000.0),
                                  U.rot(64, 60000.0, {"factor": 8.0, "low": 1.0, "high": 3.0,
                                                      "original": 1024}),
                                  U.rot(4, 100.0, {"factor": 2.0, "low": 2.0, "high": 2.0,
                                                   "original": 16})])
def test_rotation_frequencies(spec):
    sc = spec.get("scaling") or {}
    got = wavelength_scaled_frequencies(
        spec["dims"], spec["base"], float(sc.get("factor", 1.0)), float(sc.get("low", 1.0)),
        float(sc.get("high", 4.0)), float(sc.get("original", 0.0)))
    want = oracle.pair_frequencies(spec["dims"], spec["base"], spec.get("scaling"))
    torch.testing.assert_close(got.double(), want, rtol=1e-6, atol=0)
    if sc:
        plain = oracle.pair_frequencies(spec["dims"], spec["base"])
        assert got[0] == plain[0].float()                       # short waves stay
        assert abs(float(got[-1]) * sc["factor"] / float(plain[-1]) - 1) < 1e-6 \
            or 2 * math.pi / float(plain[-1]) <= sc["original"] / sc["low"]


def test_squared_relu():
    x = torch.randn(5, 30, generator=torch.Generator().manual_seed(2))
    want = torch.clamp(x.double(), min=0) ** 2
    torch.testing.assert_close(ops.relu_squared(x[:, 3:24]).double(), want[:, 3:24])


def _one_layer(spec, w, groups=5):
    """The serving path's layer built from a one-layer checkpoint: forward(h,
    meta) gives (mixer result, feed-forward result)."""
    cfg = U.small_config([spec], groups=groups)
    model = PudizenShardModel(ModelConfig.from_hf_config(cfg)).float()
    for name, t in w.items():
        assert model.load_hf_weight(name, t.float()), name
    model.finalize_weights()
    return model.layers[0]


def _meta(pos0, n, table, bs, cache):
    pos = torch.arange(pos0, pos0 + n)
    bt = torch.tensor(table)
    return ForwardMeta(
        is_prefill=n > 1,
        positions=pos.int(),
        slot_mapping=bt[pos // bs] * bs + pos % bs,
        block_tables=bt.int().unsqueeze(0),
        seq_lens=torch.tensor([pos0 + n], dtype=torch.int32),
        query_lens=torch.tensor([n], dtype=torch.int32) if n > 1 else None,
        mla_cache=cache, max_seq_len=pos0 + n,
    )


def _run_cut(layer, h, cuts, bs, table, cache):
    outs, at = [], 0
    for n in cuts:
        outs.append(layer(h[at:at + n], _meta(at, n, table, bs, cache))[0])
        at += n
    assert at == h.shape[0]
    return torch.cat(outs)


def _cache_for(spec, bs, pages):
    dims = ModelConfig.from_hf_config(U.small_config([spec])).latent_cache_dims(0, 1)
    cache = MLAKVCache(1, [dims[0][0]], [dims[0][1]], bs, pages, torch.device("cpu"),
                       torch.float32)
    cache.layer(0).fill_(7.0)      # rows of earlier owners must not be read
    return cache


@pytest.mark.parametrize("li", [0, 1, 2, 3, 4, 5])
def test_each_mixer_alone_portions_and_pages(li):
    spec = dict(U.small_config()["layers"][li], mlp=None)
    w = oracle.random_weights(U.small_config([spec]), seed=7 + li)
    layer = _one_layer(spec, w)
    T, bs = 120, 8
    h = torch.randn(T, WIDTH, generator=torch.Generator().manual_seed(5))
    want = oracle.MIXERS[spec["type"]](h.double(), w, "l0.mix.", spec["mixer"], EPS)
    pages = T // bs
    cache = _cache_for(spec, bs, pages + 5)
    table = torch.randperm(pages + 5, generator=torch.Generator().manual_seed(6))[:pages].tolist()
    got = _run_cut(layer, h, [3, 2, 1, 1, 1, 30, 7, 1, 2, 71, 1], bs, table, cache)
    torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)


def test_a_latent_wider_than_one_share_of_value_columns():
    """The attention kernels sum a bounded number of value columns per head;
    a wider latent is summed in shares of its columns."""
    spec = U.latent_layer(3, 8, 12, 300, 0.3, None)
    w = oracle.random_weights(U.small_config([spec]), seed=33)
    layer = _one_layer(spec, w)
    assert layer.mixer.rank > layer.mixer.VALUE_COLS
    h = torch.randn(40, WIDTH, generator=torch.Generator().manual_seed(8))
    want = oracle.latent_attention(h.double(), w, "l0.mix.", spec["mixer"], EPS)
    got = _run_cut(layer, h, [9, 1, 1, 29], 8, [3, 1, 4, 0, 2], _cache_for(spec, 8, 5))
    torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)


def test_softmax_attention_with_a_window_too():
    """The window is a switch of the mixer class, not of a layer type."""
    spec = U.softmax_layer(4, 2, 8, 12, 0.4, U.rot(4, 50.0, None), None, window=7)
    w = oracle.random_weights(U.small_config([spec]), seed=31)
    layer = _one_layer(spec, w)
    h = torch.randn(50, WIDTH, generator=torch.Generator().manual_seed(8))
    want = oracle.softmax_attention(h.double(), w, "l0.mix.", spec["mixer"], EPS)
    got = _run_cut(layer, h, [9, 1, 1, 20, 19], 8, list(range(8)), _cache_for(spec, 8, 8))
    torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)
    spec["mixer"].pop("mask")
    full = oracle.softmax_attention(h.double(), w, "l0.mix.", spec["mixer"], EPS)
    assert (full[20:] - want[20:]).abs().max() > 1e-2


def _plant(w, p, d, heads, kv_heads, qgain, kgain, q_rows=None):
    """Hidden dimension 0 marks the planted token and alone feeds the LAST key
    dimension (which no rotation touches); hidden dimension 1 is 1 everywhere
    and alone feeds the last dimension of every query head."""
    wq = w[p + "q"] * 0.02
    wq[:, :2] = 0.0
    for hd in range(heads):
        wq[hd * d + d - 1, :] = 0.0
        wq[hd * d + d - 1, 1] = qgain
    key = p + ("k" if p + "k" in w else "dkv")
    wk = w[key].clone()
    wk[:, :2] = 0.0
    rows = [g * d + d - 1 for g in range(kv_heads)] if q_rows is None else q_rows
    for r in rows:
        wk[r, :] = 0.0
        wk[r, 0] = kgain
    w[p + "q"] = wq.to(torch.bfloat16).to(D)
    w[key] = wk.to(torch.bfloat16).to(D)


def _hidden(T, planted, seed=9):
    base = torch.randn(T, WIDTH, generator=torch.Generator().manual_seed(seed))
    base[:, 0] = 0.0
    base[:, 1] = 1.0
    h = base.clone()
    h[planted] = 0.0
    h[planted, 0] = h[planted, 1] = 1.0
    return base, h


@pytest.mark.parametrize("decode", [False, True])
def test_window_edges_of_the_sigmoid_mixer(decode):
    """Score biases of -12 silence every key (weights of about 1e-5) except
    one planted token's, whose score is large: the queries at distance 0 ...
    window - 1 from it carry its value, the query at distance `window` and
    all later ones do not, nobody before it sees it; at page borders and
    inside pages, in prompt portions and in decoding."""
    window = 11
    spec = U.window_layer(2, 1, 8, 12, 3.0, window, U.rot(4, 100.0, None), None)
    mx = spec["mixer"]
    w = oracle.random_weights(U.small_config([spec]), seed=21)
    p = "l0.mix."
    w[p + "pb"] = torch.full((2,), -12.0, dtype=D)
    _plant(w, p, 8, 2, 1, 2.0, 4.0)
    layer = _one_layer(spec, w)
    T, bs = 64, 8
    for planted in (0, 5, 7, 8, 29):
        base, h = _hidden(T, planted)
        want = oracle.sigmoid_attention(h.double(), w, p, mx, EPS)
        without = oracle.sigmoid_attention(base.double(), w, p, mx, EPS)
        table = torch.randperm(12, generator=torch.Generator().manual_seed(3)).tolist()
        cuts = [planted + 1] + [1] * (T - planted - 1) if decode else \
            [planted + window - 1, 2, T - planted - window - 1]
        got = _run_cut(layer, h, cuts, bs, table, _cache_for(spec, bs, 12))
        torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)
        inside, outside = planted + window - 1, planted + window
        assert (got[inside].double() - without[inside]).abs().max() > 0.05, planted
        assert (got[planted + 1].double() - without[planted + 1]).abs().max() > 0.05
        torch.testing.assert_close(got[outside:].double(), without[outside:], rtol=2e-4, atol=2e-4)
        if planted:
            torch.testing.assert_close(got[:planted].double(), without[:planted],
                                       rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("decode", [False, True])
def test_a_far_key_takes_the_softmax(kind, decode):
    """One planted token whose key scores far above all others: every later
    query's softmax puts nearly all its weight there, hundreds of tokens back
    and pages away, so the result is that token's value (turned back by the
    right angle where values rotate); nobody before it sees it."""
    if kind == "attention":
        spec = U.softmax_layer(2, 1, 8, 12, 1.0, U.rot(4, 100.0, None), None)
        d, G = 8, 1
    else:
        spec = U.latent_layer(2, 8, 12, 8, 1.0, None)
        d, G = 8, 1
    mx = spec["mixer"]
    w = oracle.random_weights(U.small_config([spec]), seed=22)
    p = "l0.mix."
    if kind == "attention":
        w[p + "q.norm"] = torch.ones(16, dtype=D)
        w[p + "k.norm"] = torch.ones(8, dtype=D)
        _plant(w, p, d, 2, G, 8.0, 60.0)
    else:
        # latent dimension 7 carries the mark; both heads' last key dimension
        # reads latent dimension 7 alone
        w[p + "dkv.norm"] = torch.ones(8, dtype=D)
        _plant(w, p, d, 2, G, 8.0, 60.0, q_rows=[7])
        uk = w[p + "uk"].clone()
        for hd in range(2):
            uk[hd * 8 + 7, :] = 0.0
            uk[hd * 8 + 7, 7] = 4.0
            uk[hd * 8:hd * 8 + 7, 7] = 0.0
        w[p + "uk"] = uk
    layer = _one_layer(spec, w)
    fn = oracle.MIXERS[kind]
    T, bs = 400, 8
    for planted in (0, 7, 8, 250):
        base, h = _hidden(T, planted)
        want = fn(h.double(), w, p, mx, EPS)
        without = fn(base.double(), w, p, mx, EPS)
        table = torch.randperm(64, generator=torch.Generator().manual_seed(3)).tolist()
        cuts = [planted + 1] + [1] * (T - planted - 1) if decode else [5, 3, 250, 2, 140]
        got = _run_cut(layer, h, cuts, bs, table, _cache_for(spec, bs, 64))
        torch.testing.assert_close(got.double(), want, rtol=3e-4, atol=3e-4)
        for i in (planted + 1, T - 1):
            assert (want[i] - without[i]).abs().max() > 0.05, (planted, i)
        if planted:
            torch.testing.assert_close(got[:planted].double(), without[:planted],
                                       rtol=3e-4, atol=3e-4)


# -- the engine ------------------------------------------------------------------


def test_whole_prompt_and_layers(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path)
    toks = U.tokens(70, cfg["vocab"], 1)
    streams = {}
    eng.model.tap = lambda i, x: streams.__setitem__(i, x.clone())
    got = U.run_schedule(eng, {"a": toks}, [[("a", 70)]])["a"]
    want, layers = oracle.forward(cfg, w, toks, return_layers=True)
    for i in range(len(cfg["layers"])):
        torch.testing.assert_close(streams[i].double(), layers[i], rtol=1e-4, atol=1e-4)
    assert U.rel_err(got, want) < TOL


def test_first_tokens_and_single_token_prompt(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path)
    for n in (1, 2, 3):
        toks = U.tokens(n, cfg["vocab"], 20 + n)
        got = U.run_schedule(eng, {"a": toks}, [[("a", n)]])["a"]
        assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL
    # a request whose first step brings ONE token, then goes on
    toks = U.tokens(12, cfg["vocab"], 25)
    got = U.run_schedule(eng, {"b": toks}, [[("b", 1)], [("b", 1)], [("b", 10)]])["b"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_prefill_equals_token_by_token_decoding(ckpt):
    cfg, w, path = ckpt
    toks = U.tokens(60, cfg["vocab"], 2)
    want = oracle.forward(cfg, w, toks)
    eng = U.make_engine(path)
    whole = U.run_schedule(eng, {"a": toks}, [[("a", 60)]])["a"]
    one = U.run_schedule(eng, {"b": toks}, [[("b", 1)] for _ in toks])["b"]
    assert U.rel_err(whole, want) < TOL and U.rel_err(one, want) < TOL
    assert U.rel_err(one, whole.double()) < TOL


@pytest.mark.parametrize("cuts", [[2] * 40, [3, 2, 7, 1, 1, 1, 33, 2, 5, 25], [79, 1],
                                  [8, 8, 8, 8, 8, 8, 8, 8, 8, 8], [5, 1, 1, 1, 9, 1, 62],
                                  [9, 9, 33, 29]])
def test_portions_of_several_sizes(ckpt, cuts):
    cfg, w, path = ckpt
    assert sum(cuts) == 80
    toks = U.tokens(80, cfg["vocab"], 3)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in cuts])["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_the_pair_row_survives_every_cut(ckpt):
    """Two sequences that differ in ONE token: the logits of the token after
    it differ through the pair row, also when a portion starts right there."""
    cfg, w, path = ckpt
    a = U.tokens(30, cfg["vocab"], 70)
    b = list(a)
    b[13] = (a[13] + 1) % cfg["vocab"]
    eng = U.make_engine(path)
    for cuts in ([14, 16], [13, 1, 16], [14, 1, 15]):
        ga = U.run_schedule(eng, {"a": a}, [[("a", n)] for n in cuts])["a"]
        gb = U.run_schedule(eng, {"b": b}, [[("b", n)] for n in cuts])["b"]
        assert U.rel_err(ga, oracle.forward(cfg, w, a)) < TOL
        assert U.rel_err(gb, oracle.forward(cfg, w, b)) < TOL
        assert torch.equal(ga[:13], gb[:13])


def test_mixed_batches_of_unequal_requests(ckpt):
    cfg, w, path = ckpt
    seqs = {"a": U.tokens(90, cfg["vocab"], 4), "b": U.tokens(7, cfg["vocab"], 5),
            "c": U.tokens(41, cfg["vocab"], 6), "d": U.tokens(1, cfg["vocab"], 7),
            "e": U.tokens(30, cfg["vocab"], 8)}
    schedule = [
        [("a", 16), ("b", 1)],
        [("b", 1), ("a", 31), ("c", 2)],
        [("c", 1), ("b", 1), ("a", 1), ("d", 1)],          # d ends: e takes its place
        [("e", 9), ("a", 1), ("b", 4), ("c", 30)],          # b ends
        [("a", 40), ("c", 1), ("e", 1)],
        [("e", 20), ("a", 1), ("c", 7)],
    ]
    eng = U.make_engine(path, pages=24, block_size=8)  # 192 tokens: pages are tight
    got = U.run_schedule(eng, seqs, schedule)
    for name, toks in seqs.items():
        assert got[name].shape[0] == len(toks)
        assert U.rel_err(got[name], oracle.forward(cfg, w, toks)) < TOL, name
    assert eng.cache_manager.num_free_blocks == 24


def test_pages_freed_and_used_again(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, pages=8, block_size=8, max_requests=2)
    for k in range(5):   # 5 requests through 8 pages
        toks = U.tokens(50 + k, cfg["vocab"], 30 + k)
        cuts = [20, 1, 1] + [len(toks) - 22]
        got = U.run_schedule(eng, {"r%d" % k: toks}, [[("r%d" % k, n)] for n in cuts])
        assert U.rel_err(got["r%d" % k], oracle.forward(cfg, w, toks)) < TOL
        assert eng.cache_manager.num_free_blocks == 8
    with pytest.raises(RuntimeError):
        U.run_schedule(eng, {"x": [1, 2], "y": [3, 4], "z": [5, 6]},
                       [[("x", 1), ("y", 1), ("z", 1)]])


def test_long_decoding_past_every_window(ckpt):
    cfg, w, path = ckpt
    toks = U.tokens(150, cfg["vocab"], 9)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", 12)]] + [[("a", 1)]] * 138)["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


@pytest.mark.parametrize("layers,groups", [
    # one head everywhere, key width = value width = latent width, a window of
    # one token (a token sees itself alone), two rotated dimensions, one group
    ([U.window_layer(1, 1, 8, 8, 1.0, 1, U.rot(2, 10.0, None), U.dense(8)),
      U.latent_layer(1, 8, 8, 8, 1.0, U.dense(8)),
      U.softmax_layer(1, 1, 8, 8, 1.0, U.rot(2, 10.0, None), U.dense(8))], 1),
    # no feed-forward anywhere; no rotation of q and k at all; a window longer
    # than the sequence; groups of two channels; scaling whose ramp is empty
    ([U.window_layer(4, 2, 20, 4, window=500, rotation=None, mlp=None),
      U.softmax_layer(6, 6, 4, 20, rotation={"dims": 0, "base": 77.0}, mlp=None),
      U.latent_layer(5, 4, 6, 3, mlp=None),
      U.softmax_layer(2, 1, 12, 6, rotation=U.rot(12, 50.0, {"factor": 8.0, "low": 2.0,
                                                             "high": 2.0, "original": 32}),
                      mlp=None)], 12),
    # only latent layers; only windows
    ([U.latent_layer(), U.latent_layer(4, 6, 2, 50, 0.5, None)], 2),
    ([U.window_layer(window=2), U.window_layer(6, 3, 4, 4, window=64, rotation=U.rot(4, 20.0), mlp=U.dense(8))], 3),
])
def test_other_sizes(tmp_path, layers, groups):
    cfg = U.small_config(layers, width=24, vocab=53, eps=1e-6, groups=groups, scale=1.0,
                         buckets=1 if groups == 1 else 97, mul_prev=1, mul_cur=1)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    toks = U.tokens(60, 53, 10)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 20]])["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_layer_ranges_hand_the_stream_on(ckpt):
    """Two shards of the stack, run one after the other, give the whole
    stack's result: the fp32 stream is what travels between them."""
    cfg, w, path = ckpt
    mc = ModelConfig.from_pretrained(path)
    from parallax_amd.server.shard_loader import load_shard_weights

    toks = U.tokens(20, cfg["vocab"], 50)
    parts = []
    for lo, hi in ((0, 2), (2, 6)):
        m = PudizenShardModel(mc, lo, hi)
        load_shard_weights(m, path)
        m.finalize_weights()
        parts.append(m.float())
    dims = mc.latent_cache_dims(0, 6)
    hidden = parts[0].embed(torch.tensor(toks), torch.tensor([-1] + toks[:-1])).float()
    at = 0
    for m in parts:
        n = m.num_local_layers
        cache = MLAKVCache(n, [a for a, _ in dims[at:at + n]], [b for _, b in dims[at:at + n]],
                           8, 8, torch.device("cpu"), torch.float32)
        hidden = m(hidden, _meta(0, len(toks), list(range(8)), 8, cache))
        at += n
    got = parts[1].compute_logits(hidden)
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_greedy_generation_through_the_scheduler(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, prefill_chunk_size=16)
    prompts = [U.tokens(37, cfg["vocab"], 11), U.tokens(5, cfg["vocab"], 12),
               U.tokens(18, cfg["vocab"], 13), U.tokens(1, cfg["vocab"], 14)]
    sp = [SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True)
          for n in (12, 20, 7, 9)]
    out = list(eng.generate(prompts, sp).values())
    for p, s, got in zip(prompts, sp, out):
        seq = list(p)
        for _ in range(s.max_new_tokens):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert got == seq[len(p):]
    assert eng.cache_manager.num_free_blocks == 64


def test_two_peer_pipeline_greedy(ckpt):
    """The packet-driven multi-host path: two peers split the stack (the fp32
    residual travels between them; the head peer looks the pair rows up),
    greedy tokens equal the reference's."""
    from parallax_amd.p2p.peer_executor import PeerExecutor
    from parallax_amd.p2p.transport import LoopbackTransport

    cfg, w, path = ckpt
    mc = ModelConfig.from_pretrained(path)
    registry, peers = {}, []
    for pid, (s, e) in zip(["p0", "p1"], [(0, 4), (4, 6)]):
        peers.append(PeerExecutor(mc, s, e, pid, LoopbackTransport(pid, registry),
                                  dtype=torch.float32, num_kv_blocks=64, block_size=8,
                                  model_path=path))
    head = peers[0]
    prompts = [U.tokens(19, cfg["vocab"], 70), U.tokens(4, cfg["vocab"], 71),
               U.tokens(1, cfg["vocab"], 72)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True)
    rids = [head.submit(p, sp, ["p0", "p1"]) for p in prompts]
    outputs, done = {r: [] for r in rids}, set()
    for _ in range(2000):
        for px in peers:
            px.step(recv_timeout=0.001)
        for out in head.drain_outputs():
            outputs[out.rid].append(out.token_id)
            if out.finished:
                done.add(out.rid)
        if len(done) == len(rids):
            break
    for p, rid in zip(prompts, rids):
        seq = list(p)
        for _ in range(6):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert outputs[rid] == seq[len(p):]


def _pp_worker(rank, world, port, path, prompts, out_file):
    import os

    os.environ.update(MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port),
                      RANK=str(rank), WORLD_SIZE=str(world))
    import torch.distributed as dist

    from parallax_amd.parallel.comm import init_distributed
    from parallax_amd.server.engine import Engine, EngineArgs

    comm = init_distributed(pp_size=world, tp_size=1, backend="gloo",
                            device=torch.device("cpu"))
    eng = Engine(ModelConfig.from_pretrained(path),
                 EngineArgs(block_size=8, num_kv_blocks=64, max_batch_size=4,
                            dtype=torch.float32, micro_batches=2,
                            enable_prefix_cache=False, max_model_len=512),
                 comm=comm, model_path=path)
    sp = [SamplingParams(temperature=0.0, max_new_tokens=5, ignore_eos=True)] * len(prompts)
    outs = list(eng.generate(prompts, sp).values())
    if rank == 0:
        torch.save(outs, out_file)
    dist.barrier()
    dist.destroy_process_group()


def test_pipeline_stages_over_gloo(ckpt, tmp_path):
    """Two pipeline stages in two processes (gloo): the fp32 residual crosses
    the stage boundary, greedy tokens equal the reference's."""
    import torch.multiprocessing as mp

    cfg, w, path = ckpt
    prompts = [U.tokens(13, cfg["vocab"], 80), U.tokens(3, cfg["vocab"], 81),
               U.tokens(26, cfg["vocab"], 82)]
    out_file = str(tmp_path / "pp2.pt")
    mp.spawn(_pp_worker, args=(2, 29683, path, prompts, out_file), nprocs=2, join=True)
    got = torch.load(out_file)
    for p, toks in zip(prompts, got):
        seq = list(p)
        for _ in range(5):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert toks == seq[len(p):]


def test_a_config_without_a_pair_table(tmp_path):
    cfg = U.small_config([U.window_layer(), U.latent_layer()])
    del cfg["embedding"]["bigram"]
    w = oracle.random_weights(dict(cfg, embedding={"scale": 2.5, "bigram": {"buckets": 1}}),
                              seed=5)
    w.pop("bigram")
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    toks = U.tokens(20, cfg["vocab"], 3)
    got = U.run_schedule(U.make_engine(path), {"a": toks}, [[("a", 9)], [("a", 11)]])["a"]
    ref_cfg = dict(cfg, embedding={"scale": 2.5, "bigram": {"buckets": 1, "mul_prev": 0,
                                                          "mul_cur": 0}})
    w["bigram"] = torch.zeros(2, cfg["width"], dtype=D)
    assert U.rel_err(got, oracle.forward(ref_cfg, w, toks)) < TOL


def test_trace_replay_program(ckpt, tmp_path):
    """bin/trace_run picks the model class from config.json; ended requests
    give their pages back."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, w, path = ckpt
    a, b = U.tokens(21, cfg["vocab"], 60), U.tokens(9, cfg["vocab"], 61)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:16], "want": [0, 15]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[16:17], "want": []},
                                {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]},
                                {"id": "a", "tokens": a[17:], "want": [3]}], "end": ["a", "b"]},
    ]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "logits"
    p = subprocess.run(
        [sys.executable, os.path.join(repo, "bin", "trace_run"), "--model", path,
         "--dtype", "float32", "--out", str(out), "--max-tokens", "64", "--device", "cpu"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
        text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    V = cfg["vocab"]
    la, lb = oracle.forward(cfg, w, a), oracle.forward(cfg, w, b)
    got = torch.from_numpy(np.concatenate(
        [np.fromfile(out / ("%d.f32" % i), dtype="<f4").reshape(-1, V) for i in range(3)]))
    want = torch.stack([la[0], la[15], lb[7], lb[8], la[20]])
    assert U.rel_err(got, want) < TOL
