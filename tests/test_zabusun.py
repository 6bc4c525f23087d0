"""Zabusun on the CPU engine (fp32) against the plain reference in
zabusun_oracle.py: each mechanism alone, then the engine's step function,
cache manager and scheduler under many ways of cutting and batching the same
sequences. Configurations are small and deliberately irregular (see
zabusun_util.small_config)."""

import math

import pytest
import torch

import zabusun_oracle as oracle
import zabusun_util as U
from parallax_amd import ops
from parallax_amd.models.config import ModelConfig
from parallax_amd.models.forward_meta import ForwardMeta
from parallax_amd.models.linear_attention import MinGRU
from parallax_amd.models.moe import FusedMoE
from parallax_amd.models.rope import yarn_ramp_frequencies
from parallax_amd.models.row_attention import GatedSigmoidAttention
from parallax_amd.models.zabusun import (
    ClampedGluMLP, ZabusunShardModel, _expert_config,
)
from parallax_amd.server.kv_cache import LinearStateCache, MLAKVCache
from parallax_amd.server.sampling_params import SamplingParams

D = torch.float64
TOL = 2e-5
EPS = 1e-5
WIDTH = 40


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = U.small_config()
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("zb")), cfg, w)
    return cfg, w, path


# -- mechanisms alone ------------------------------------------------------------


def test_config_reader():
    cfg = U.small_config()
    mc = ModelConfig.from_hf_config(cfg)
    assert mc.architecture == "Zabusun" and mc.num_layers == 4
    assert mc.layer_types == ["parallel_attention_recurrent"] * 4
    # (key width, value width) over all kv heads, and the recurrent widths
    assert mc.latent_cache_dims(0, 4) == [(24, 40), (64, 32), (24, 24), (8, 12)]
    assert mc.latent_cache_dims(1, 3) == [(64, 32), (24, 24)]
    assert mc.pooled_cache_blocks(0, 4) == [0, 0, 0, 0]
    assert mc.linear_state_shapes(0, 4) == [((0,), (28,)), ((0,), (52,)),
                                            ((0,), (8,)), ((0,), (33,))]
    assert mc.has_linear_layers and mc.logit_scale == 0.7
    with pytest.raises(ValueError):
        ModelConfig.from_hf_config(
            U.small_config([{"type": "serial", "mixer": {"heads": 1, "dim": 8}, "mlp": None}]))


def test_post_norm_residual_step():
    g = torch.Generator().manual_seed(0)
    T, W = 6, 40
    x = torch.randn(T, W, generator=g) * 2 + 0.5
    a = torch.randn(T, W, generator=g) * 5
    b = torch.randn(T, W, generator=g) * 0.1
    wn = 1.0 + torch.randn(W, generator=g) * 0.3
    # two branches with a scale each
    x1 = x.clone()
    got_x, got_h = ops.branch_rmsnorm_add(x1, a, b, 0.6, 1.7, wn, EPS, torch.float32)
    want = x.double() + oracle.rms_norm(0.6 * a.double() + 1.7 * b.double(), wn.double(), EPS)
    assert got_x is x1
    torch.testing.assert_close(x1.double(), want, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(got_h.double(), want, rtol=1e-6, atol=1e-6)
    # a stream that starts as the normed branch (the embedding)
    x0, h0 = ops.branch_rmsnorm_add(None, a, None, 1.0, 0.0, wn, EPS, torch.float32)
    torch.testing.assert_close(x0.double(), oracle.rms_norm(a.double(), wn.double(), EPS),
                               rtol=1e-6, atol=1e-6)
    # the norm alone (the last one): the stream stays as it was
    x2 = x.clone()
    none, h2 = ops.branch_rmsnorm_add(None, x2, None, 1.0, 0.0, wn, EPS,
                                      torch.float32, keep_stream=False)
    assert none is None and torch.equal(x2, x)
    torch.testing.assert_close(h2.double(), oracle.rms_norm(x.double(), wn.double(), EPS),
                               rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("limit", [1.2, 0.3, 50.0])
def test_clamped_feed_forward(limit):
    g = torch.Generator().manual_seed(1)
    w = {"m.gate": torch.randn(24, WIDTH, generator=g) / 3,
         "m.up": torch.randn(24, WIDTH, generator=g) / 3,
         "m.down": torch.randn(WIDTH, 24, generator=g) / 5}
    mlp = ClampedGluMLP(WIDTH, 24, limit)
    mlp.gate_up.load_full_weight_part(0, w["m.gate"])
    mlp.gate_up.load_full_weight_part(1, w["m.up"])
    mlp.down.load_full_weight(w["m.down"])
    h = torch.randn(9, WIDTH, generator=g) * 3
    wd = {k: v.double() for k, v in w.items()}
    torch.testing.assert_close(mlp(h).double(), oracle.clamped_glu(h.double(), wd, "m.", limit),
                               rtol=1e-5, atol=1e-5)
    # the clamps bite: gate from above only, up on both sides
    z = torch.tensor([[-9.0, 0.5, 9.0, -9.0, 0.5, 9.0]])
    got = ops.clamped_glu(z, 2.0)
    want = [min(t, 2.0) / (1 + math.exp(-1.702 * min(t, 2.0))) * (max(-2.0, min(u, 2.0)) + 1)
            for t, u in zip([-9.0, 0.5, 9.0], [-9.0, 0.5, 9.0])]
    torch.testing.assert_close(got[0].double(), torch.tensor(want, dtype=D), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("n,top", [(5, 2), (3, 1), (4, 4), (1, 1)])
def test_experts_weighted_on_their_input(n, top):
    mlp = U.experts(n, top, 16, 0.8)
    cfg = U.small_config([U.layer(mlp=mlp)])
    w = oracle.random_weights(cfg, seed=5)
    moe = FusedMoE(_expert_config(ModelConfig.from_hf_config(cfg), mlp), act_limit=0.8)
    moe.fp32_output = moe.weight_on_input = True
    moe.router.weight.data.copy_(w["l0.mlp.router"])
    for e in range(n):
        moe.load_expert_gate(e, w[f"l0.mlp.e{e}.gate"].float())
        moe.load_expert_up(e, w[f"l0.mlp.e{e}.up"].float())
        moe.load_expert_down(e, w[f"l0.mlp.e{e}.down"].float())
    h = torch.randn(17, WIDTH, generator=torch.Generator().manual_seed(2)) * 2
    want, ids = oracle.routed_experts(h.double(), w, "l0.mlp.", mlp)
    got_ids, got_w = moe.router(h)
    assert torch.equal(got_ids.sort(-1).values, ids.sort(-1).values)
    # the weights are the chosen scores themselves: they do not sum to one
    scores = torch.sigmoid(h.double() @ w["l0.mlp.router"].T)
    torch.testing.assert_close(got_w.double().sum(-1), scores.gather(1, got_ids).sum(-1),
                               rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(moe(h).double(), want, rtol=1e-5, atol=1e-5)
    # weighting the OUTPUT instead is a different function (the clamps)
    moe.weight_on_input = False
    assert (moe(h).double() - want).abs().max() > 1e-3 or n == 0


@pytest.mark.parametrize("spec", [U.rot(8), U.rot(16, 10000.0, None), U.rot(32, 40000.0),
                                  U.rot(4, 100.0, {"factor": 2.0, "original": 16,
                                                   "fast": 4.0, "slow": 1.0})])
def test_rotation_frequencies(spec):
    sc = spec.get("scaling") or {}
    f, mult = yarn_ramp_frequencies(spec["dims"], spec["base"], float(sc.get("factor", 1.0)),
                                    float(sc.get("original", 0.0)), float(sc.get("fast", 32.0)),
                                    float(sc.get("slow", 1.0)))
    want, wmult = oracle.rotary_frequencies(spec)
    torch.testing.assert_close(f.double(), want, rtol=1e-6, atol=0)
    assert abs(mult - wmult) < 1e-12


def _attention_module(w, mx, pre="l0.mix.left."):
    rot = mx.get("rot") or {}
    m = GatedSigmoidAttention(
        WIDTH, mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"],
        mx["scale"], EPS, 0, True, rot_dims=int(rot.get("dims", 0)),
        rot_base=float(rot.get("base", 10000.0)), rot_scaling=rot.get("scaling"))
    for slot, key in enumerate(("q", "k", "v", "g")):
        m.in_proj.load_full_weight_part(slot, w[pre + key].float())
    m.q_norm.data.copy_(w[pre + "q.norm"])
    m.k_norm.data.copy_(w[pre + "k.norm"])
    m.score_bias.data.copy_(w[pre + "pb"])
    m.o_proj.load_full_weight(w[pre + "o"].float())
    return m


def _meta(pos0, n, table, bs, cache=None, linear=None, slot=0):
    pos = torch.arange(pos0, pos0 + n)
    bt = torch.tensor(table)
    return ForwardMeta(
        is_prefill=n > 1,
        positions=pos.int(),
        slot_mapping=bt[pos // bs] * bs + pos % bs,
        block_tables=bt.int().unsqueeze(0),
        seq_lens=torch.tensor([pos0 + n], dtype=torch.int32),
        query_lens=torch.tensor([n], dtype=torch.int32) if n > 1 else None,
        mla_cache=cache, linear_cache=linear,
        linear_slots=torch.tensor([slot], dtype=torch.int64),
        max_seq_len=pos0 + n,
    )


def _run_cut(module, h, cuts, bs=8, table=None, cache=None, linear=None, slot=0):
    outs, at = [], 0
    for n in cuts:
        meta = _meta(at, n, table or list(range(64)), bs, cache, linear, slot)
        outs.append(module(h[at:at + n], meta))
        at += n
    assert at == h.shape[0]
    return torch.cat(outs)


@pytest.mark.parametrize("li", [0, 1, 2, 3])
def test_sigmoid_attention_alone_portions_and_pages(li):
    cfg = U.small_config()
    spec = cfg["layers"][li]
    mx = spec["mixer"]["left"]
    w = oracle.random_weights(U.small_config([spec]), seed=7 + li)
    m = _attention_module(w, mx)
    T, bs = 120, 8
    h = torch.randn(T, WIDTH, generator=torch.Generator().manual_seed(5))
    want = oracle.sigmoid_attention(h.double(), w, "l0.mix.left.", mx, EPS)
    G = mx.get("kv_heads", mx["heads"])
    pages = T // bs
    cache = MLAKVCache(1, [G * mx["dim"]], [G * mx["vdim"]], bs, pages + 5,
                       torch.device("cpu"), torch.float32)
    cache.layer(0).fill_(7.0)      # rows of earlier owners must not be read
    table = torch.randperm(pages + 5, generator=torch.Generator().manual_seed(6))[:pages].tolist()
    got = _run_cut(m, h, [3, 2, 1, 1, 1, 30, 7, 1, 2, 71, 1], bs, table, cache)
    torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("decode", [False, True])
def test_a_far_key_among_hundreds_and_the_causal_edge(decode):
    """Score biases of -12 silence every key (weights of about 1e-5) except
    one planted token's: hidden dimension 0 marks it and is projected onto
    key dimension 3, which no other token's key has, and every query points
    along dimension 3 (from a hidden dimension that is 1 everywhere). Its
    weight is then about 1 for itself and for every LATER position and it is
    not seen by any earlier one, also when it lies hundreds of tokens back
    and pages away, in prompt portions and in decoding."""
    spec = U.layer(2, 1, 8, 12, scale=3.0, rotation=None, mlp=None)
    mx = spec["mixer"]["left"]
    w = oracle.random_weights(U.small_config([spec]), seed=21)
    p = "l0.mix.left."
    w[p + "pb"] = torch.full((2,), -12.0, dtype=D)
    w[p + "q.norm"] = torch.ones(8, dtype=D)
    w[p + "k.norm"] = torch.ones(8, dtype=D)
    wq = w[p + "q"] * 0.02
    wq[:, :2] = 0.0
    wq[3, 1] = wq[8 + 3, 1] = 1.0          # both heads: dimension 3, constant
    wk = w[p + "k"].clone()
    wk[:, :2] = 0.0
    wk[3, :] = 0.0
    wk[3, 0] = 4.0                          # the marker alone feeds dimension 3
    w[p + "q"] = wq.to(torch.bfloat16).to(D)
    w[p + "k"] = wk.to(torch.bfloat16).to(D)
    m = _attention_module(w, mx)
    T, bs = 400, 8
    base = torch.randn(T, WIDTH, generator=torch.Generator().manual_seed(9))
    base[:, 0] = 0.0
    base[:, 1] = 1.0
    for planted in (0, 7, 8, 250):
        h = base.clone()
        h[planted] = 0.0
        h[planted, 0] = h[planted, 1] = 1.0
        want = oracle.sigmoid_attention(h.double(), w, p, mx, EPS)
        cache = MLAKVCache(1, [8], [12], bs, 64, torch.device("cpu"), torch.float32)
        table = torch.randperm(64, generator=torch.Generator().manual_seed(3)).tolist()
        cuts = [planted + 1] + [1] * (T - planted - 1) if decode else [5, 3, 250, 2, 140]
        got = _run_cut(m, h, cuts, bs, table, cache)
        torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)
        # the planted key's weight stands out for every query at or after it
        q = oracle.rms_norm((h.double() @ w[p + "q"].T).view(T, 2, 8), w[p + "q.norm"], EPS)
        k = oracle.rms_norm((h.double() @ w[p + "k"].T).view(T, 1, 8), w[p + "k.norm"], EPS)
        s = torch.sigmoid(q[:, 0] @ k[:, 0].T * 3.0 - 12.0)
        for i in (planted, planted + 1, T - 1):
            others = torch.cat([s[i, :planted], s[i, planted + 1:i + 1]])
            assert s[i, planted] > 0.99 and s[i, planted] > 50 * others.sum(), (planted, i)
        if planted:
            # nobody before it sees it: their outputs equal a run without it
            before = oracle.sigmoid_attention(base.double(), w, p, mx, EPS)[:planted]
            torch.testing.assert_close(got[:planted].double(), before, rtol=2e-4, atol=2e-4)
            # and the first one after it differs from that run
            after = oracle.sigmoid_attention(base.double(), w, p, mx, EPS)[planted + 1]
            assert (got[planted + 1].double() - after).abs().max() > 1e-2


def _gru_module(w, width, pre="l0.mix.right."):
    m = MinGRU(WIDTH, width, 0)
    for slot, key in enumerate(("z", "x", "g")):
        m.in_proj.load_full_weight_part(slot, w[pre + key].float())
    m.z_bias.data.copy_(w[pre + "z.b"])
    m.x_bias.data.copy_(w[pre + "x.b"])
    m.o_proj.load_full_weight(w[pre + "o"].float())
    return m


@pytest.mark.parametrize("width", [28, 1, 300])
def test_min_gru_alone_portions_and_slots(width):
    spec = U.layer(width=width, mlp=None)
    w = oracle.random_weights(U.small_config([spec]), seed=11)
    m = _gru_module(w, width)
    T = 90
    h = torch.randn(T, WIDTH, generator=torch.Generator().manual_seed(4)) * 2
    want, last = oracle.min_gru(h.double(), w, "l0.mix.right.")
    lin = LinearStateCache(1, (0,), (width,), 3, torch.device("cpu"), torch.float32)
    lin.recurrent_states[0].fill_(9.0)     # what an earlier owner left behind
    got = _run_cut(m, h, [4, 1, 1, 2, 40, 1, 41], linear=lin, slot=2)
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(lin.recurrent_states[0][2].double(), last, rtol=1e-5, atol=1e-6)
    assert torch.all(lin.recurrent_states[0][:2] == 9.0)
    # both branches of the candidate occur, and the state is carried: a run
    # from the middle with a zero state differs
    u = h.double() @ w["l0.mix.right.x"].T + w["l0.mix.right.x.b"]
    assert (u >= 0).any() and (u < 0).any()
    if width > 1:
        fresh, _ = oracle.min_gru(h[45:].double(), w, "l0.mix.right.")
        assert (fresh - want[45:]).abs().max() > 1e-3


# -- the engine: step function, cache manager, scheduler ----------------------------


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
                                  [8, 8, 8, 8, 8, 8, 8, 8, 8, 8], [5, 1, 1, 1, 9, 1, 62]])
def test_portions_of_several_sizes(ckpt, cuts):
    cfg, w, path = ckpt
    assert sum(cuts) == 80
    toks = U.tokens(80, cfg["vocab"], 3)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in cuts])["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_mixed_batches_of_unequal_requests(ckpt):
    cfg, w, path = ckpt
    seqs = {"a": U.tokens(90, cfg["vocab"], 4), "b": U.tokens(7, cfg["vocab"], 5),
            "c": U.tokens(41, cfg["vocab"], 6), "d": U.tokens(1, cfg["vocab"], 7),
            "e": U.tokens(30, cfg["vocab"], 8)}
    schedule = [
        [("a", 16), ("b", 1)],
        [("b", 1), ("a", 31), ("c", 2)],
        [("c", 1), ("b", 1), ("a", 1), ("d", 1)],          # d ends: e takes its slot
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


def test_pages_and_slots_freed_and_used_again(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, pages=8, block_size=8, max_requests=2)
    for k in range(5):   # 5 requests through 8 pages and 2 state slots
        toks = U.tokens(50 + k, cfg["vocab"], 30 + k)
        cuts = [20, 1, 1] + [len(toks) - 22]
        got = U.run_schedule(eng, {"r%d" % k: toks}, [[("r%d" % k, n)] for n in cuts])
        assert U.rel_err(got["r%d" % k], oracle.forward(cfg, w, toks)) < TOL
        assert eng.cache_manager.num_free_blocks == 8
        # the state the request leaves behind is not zero: the next owner of
        # the slot must not start from it
        assert any(float(s.abs().max()) > 0 for s in eng.linear_cache.recurrent_states)
    with pytest.raises(RuntimeError):
        U.run_schedule(eng, {"x": [1, 2], "y": [3, 4], "z": [5, 6]},
                       [[("x", 1), ("y", 1), ("z", 1)]])


def test_long_decoding(ckpt):
    cfg, w, path = ckpt
    toks = U.tokens(150, cfg["vocab"], 9)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", 12)]] + [[("a", 1)]] * 138)["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


@pytest.mark.parametrize("layers", [
    # one head everywhere, key width = value width = recurrent width, scales
    # of one, one expert of which one is used, two rotated dimensions
    [U.layer(1, 1, 8, 8, 1.0, U.rot(2, 10.0, None), 8, 1.0, 1.0, U.experts(1, 1, 8, 1.0)),
     U.layer(1, 1, 8, 8, 1.0, None, 8, 1.0, 1.0, U.dense(8, 1.0))],
    # no feed-forward anywhere; every expert used by every token; a recurrent
    # width of one; a frequency ramp that covers no pair (slow = fast)
    [U.layer(4, 2, 20, 4, mlp=None, width=1),
     U.layer(6, 6, 4, 20, rotation=U.rot(4, 50.0, {"factor": 8.0, "original": 32,
                                                  "fast": 2.0, "slow": 2.0}),
             mlp=U.experts(3, 3, 8, 0.5)),
     U.layer(5, 1, 12, 12, rotation=U.rot(12), left_scale=0.0, mlp=None)],
    # the attention half switched off by its scale in one layer and the
    # recurrent half in the next
    [U.layer(left_scale=0.0, right_scale=2.0), U.layer(left_scale=2.0, right_scale=0.0)],
])
def test_other_sizes(tmp_path, layers):
    cfg = U.small_config(layers, width=24, vocab=53, eps=1e-6, logit_scale=1.0)
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
    for lo, hi in ((0, 1), (1, 4)):
        m = ZabusunShardModel(mc, lo, hi)
        load_shard_weights(m, path)
        m.finalize_weights()
        parts.append(m.float())
    dims = mc.latent_cache_dims(0, 4)
    shapes = mc.linear_state_shapes(0, 4)
    hidden = parts[0].embed(torch.tensor(toks)).float()
    at = 0
    for m in parts:
        n = m.num_local_layers
        cache = MLAKVCache(n, [a for a, _ in dims[at:at + n]], [b for _, b in dims[at:at + n]],
                           8, 8, torch.device("cpu"), torch.float32)
        lin = LinearStateCache(n, [c for c, _ in shapes[at:at + n]],
                               [r for _, r in shapes[at:at + n]], 2, torch.device("cpu"),
                               torch.float32)
        hidden = m(hidden, _meta(0, len(toks), list(range(8)), 8, cache, lin, 1))
        at += n
    got = parts[1].compute_logits(hidden)
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


def test_greedy_generation_through_the_scheduler(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, prefill_chunk_size=16)
    prompts = [U.tokens(37, cfg["vocab"], 11), U.tokens(5, cfg["vocab"], 12),
               U.tokens(18, cfg["vocab"], 13)]
    sp = [SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True)
          for n in (12, 20, 7)]
    out = list(eng.generate(prompts, sp).values())
    for p, s, got in zip(prompts, sp, out):
        seq = list(p)
        for _ in range(s.max_new_tokens):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert got == seq[len(p):]
    assert eng.cache_manager.num_free_blocks == 64


def test_trace_replay_program(ckpt, tmp_path):
    """bin/trace_run picks the model class from config.json; ended requests
    give their pages and state slots back."""
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
