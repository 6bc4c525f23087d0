"""Pudizen on the GPU engine (HIP kernels, bf16 and float32) against the plain
reference in pudizen_oracle.py: mixed batches, portions, decoding through
hipGraphs, pages used again, irregular sizes, long contexts, greedy
generation."""

import pytest
import torch

import pudizen_oracle as oracle
import pudizen_util as U
from parallax_amd import ops
from parallax_amd.server.sampling_params import SamplingParams

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 5e-5, torch.bfloat16: 0.06}


def close(got, want, dtype) -> bool:
    """float32: every row within rounding of the float64 reference. bfloat16:
    the projections, cache rows and mixer results are rounded to 8 bits of
    mantissa and a sharp softmax amplifies that for single rows: nine rows in
    ten within 0.06 and the median under 0.03; same_as_whole() is the sharp
    bf16 check."""
    if dtype == torch.bfloat16:
        e = U.row_errs(got, want)
        few = e.numel() < 8
        return bool((e < TOL[dtype]).double().mean() >= 0.9 and (few or e.median() < 0.03))
    return U.rel_err(got, want) < TOL[dtype]


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    # the layer mix of the CPU tests at a width the tuned GEMM path takes:
    # key and value widths on both the vector path (multiples of 8) and the
    # scalar path (12 / 20) of the attention kernel
    layers = [
        U.window_layer(),
        U.latent_layer(),
        U.softmax_layer(),
        U.window_layer(3, 3, 8, 12, 0.35, 33, U.rot(8, 100.0, {"factor": 2.0, "low": 1.0,
                                                               "high": 2.0, "original": 16}),
                       None),
        U.softmax_layer(8, 2, 40, 72, 0.15, U.rot(20), U.dense(64)),
        U.latent_layer(2, 8, 8, 40, 0.2, None),
    ]
    cfg = U.small_config(layers, width=64, vocab=131, groups=8)
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("pzg")), cfg, w)
    return cfg, w, path


SEQS = {"a": (90, 4), "b": (7, 5), "c": (41, 6), "d": (1, 7), "e": (30, 8)}
SCHEDULE = [
    [("a", 16), ("b", 1)],
    [("b", 1), ("a", 31), ("c", 2)],
    [("c", 1), ("b", 1), ("a", 1), ("d", 1)],
    [("e", 9), ("a", 1), ("b", 4), ("c", 30)],
    [("a", 40), ("c", 1), ("e", 1)],
    [("e", 20), ("a", 1), ("c", 7)],
]


@pytest.mark.parametrize("dtype,graphs", [(torch.float32, False), (torch.bfloat16, False),
                                          (torch.bfloat16, True)])
def test_mixed_batches(ckpt, dtype, graphs):
    cfg, w, path = ckpt
    assert ops.has_mix_extension()
    seqs = {k: U.tokens(n, cfg["vocab"], s) for k, (n, s) in SEQS.items()}
    eng = U.make_engine(path, device="cuda", dtype=dtype, pages=24, graphs=graphs)
    assert (eng.graph_runner is not None) == graphs
    got = U.run_schedule(eng, seqs, SCHEDULE)
    alone = U.make_engine(path, device="cuda", dtype=dtype, pages=24)
    for name, toks in seqs.items():
        assert close(got[name], oracle.forward(cfg, w, toks), dtype), \
            (name, U.describe(got[name], oracle.forward(cfg, w, toks), TOL[dtype]))
        whole = U.run_schedule(alone, {name: toks}, [[(name, len(toks))]])[name]
        assert U.same_as_whole(got[name], whole), (name, U.describe(got[name], whole, 0.02))
    assert eng.cache_manager.num_free_blocks == 24


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_portions_decoding_and_reuse(ckpt, dtype):
    cfg, w, path = ckpt
    eng = U.make_engine(path, device="cuda", dtype=dtype, pages=20, max_requests=2,
                        graphs=dtype == torch.bfloat16)
    alone = U.make_engine(path, device="cuda", dtype=dtype, pages=20)
    for k, cuts in enumerate([[150], [2] * 20 + [1] * 60, [3, 2, 7, 1, 1, 1, 33, 2, 5, 45],
                              [12] + [1] * 128]):
        toks = U.tokens(sum(cuts), cfg["vocab"], 40 + k)
        got = U.run_schedule(eng, {"r": toks}, [[("r", n)] for n in cuts])["r"]
        assert close(got, oracle.forward(cfg, w, toks), dtype), \
            (cuts[:3], U.describe(got, oracle.forward(cfg, w, toks), TOL[dtype]))
        whole = U.run_schedule(alone, {"w": toks}, [[("w", len(toks))]])["w"]
        assert U.same_as_whole(got, whole), (cuts[:3], U.describe(got, whole, 0.02))
        assert eng.cache_manager.num_free_blocks == 20


def test_cutting_changes_nothing_beyond_rounding(ckpt):
    cfg, w, path = ckpt
    toks = U.tokens(100, cfg["vocab"], 50)
    eng = U.make_engine(path, device="cuda", dtype=torch.float32)
    whole = U.run_schedule(eng, {"a": toks}, [[("a", 100)]])["a"]
    cut = U.run_schedule(eng, {"b": toks}, [[("b", n)] for n in [37, 1, 1, 2, 59]])["b"]
    assert U.rel_err(cut, whole.double()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sizes_outside_the_tuned_paths(tmp_path, dtype):
    """A width, vocabulary, head, latent and feed-forward sizes that are no
    multiples of 8 and norm groups of 23 channels: the projections go to the
    vendor's plain GEMM, the attention and norm kernels take their scalar
    paths."""
    layers = [U.window_layer(3, 3, 10, 6, window=4, rotation=U.rot(6), mlp=U.dense(20)),
              U.latent_layer(5, 6, 10, 13, mlp=U.dense(7)),
              U.softmax_layer(1, 1, 20, 4, rotation=U.rot(20, 30.0, None), mlp=None)]
    cfg = U.small_config(layers, width=46, vocab=53, groups=2)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, graphs=dtype == torch.bfloat16)
    toks = U.tokens(75, 53, 10)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 5] + [1] * 30])["a"]
    assert close(got, oracle.forward(cfg, w, toks), dtype), \
        U.describe(got, oracle.forward(cfg, w, toks), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_contexts_and_wide_heads(tmp_path, dtype):
    """Key and value widths on the matrix-core tiles and off them, head groups
    of 8, 3 and 5, a latent of 96 under 8 heads and one of 320 (summed in two
    shares of its columns) under 2, contexts of many pages and a
    window of several: long portions take the tiled kernel, single tokens the
    per-token one with split key lists, and both agree with the reference."""
    layers = [U.softmax_layer(8, 2, 96, 80, 0.1, U.rot(32, 40000.0), U.dense(96)),
              U.window_layer(3, 1, 128, 256, 0.08, 200, U.rot(128, 1000.0, None), None),
              U.latent_layer(8, 48, 32, 96, 0.15, U.dense(128)),
              U.softmax_layer(5, 5, 104, 40, 0.1, U.rot(10), U.dense(128)),
              U.latent_layer(2, 16, 24, 320, 0.2, None)]
    cfg = U.small_config(layers, width=128, vocab=211, groups=8)
    w = oracle.random_weights(cfg, seed=23)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, pages=40, block_size=32,
                        graphs=dtype == torch.bfloat16)
    seqs = {"a": U.tokens(700, 211, 31), "b": U.tokens(235, 211, 32)}
    schedule = [[("a", 333)], [("a", 300), ("b", 200)], [("a", 1), ("b", 1)],
                [("a", 36), ("b", 4)]] + [[("a", 1), ("b", 1)]] * 30
    got = U.run_schedule(eng, seqs, schedule)
    for name, toks in seqs.items():
        want = oracle.forward(cfg, w, toks)
        assert close(got[name], want, dtype), (name, U.describe(got[name], want, TOL[dtype]))


def test_greedy_generation_fp32_matches_the_reference(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, device="cuda", dtype=torch.float32, prefill_chunk_size=16)
    prompts = [U.tokens(37, cfg["vocab"], 11), U.tokens(5, cfg["vocab"], 12)]
    sp = [SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True) for n in (10, 16)]
    out = list(eng.generate(prompts, sp).values())
    for p, s, got in zip(prompts, sp, out):
        seq = list(p)
        for _ in range(s.max_new_tokens):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert got == seq[len(p):]


def test_greedy_generation_bf16_through_graphs(ckpt):
    """bf16 + captured decode graphs + pipelined decode (the pair row's first
    half comes from the device then): every generated token is the
    reference's best token or within rounding of it."""
    cfg, w, path = ckpt
    eng = U.make_engine(path, device="cuda", dtype=torch.bfloat16, graphs=True)
    eng.warmup_serving()   # what `serve` does at start: GEMM picks, every decode graph
    assert len(eng.graph_runner._graphs) == \
        len(eng.graph_runner.buckets) * len(eng.graph_runner.ctx_buckets)
    prompts = [U.tokens(29, cfg["vocab"], 21), U.tokens(3, cfg["vocab"], 22),
               U.tokens(64, cfg["vocab"], 23)]
    sp = [SamplingParams(temperature=0.0, max_new_tokens=24, ignore_eos=True)] * 3
    out = list(eng.generate(prompts, sp).values())
    for p, got in zip(prompts, out):
        assert len(got) == 24
        logits = oracle.forward(cfg, w, list(p) + got)
        spread = float(logits.std())
        for i, tok in enumerate(got):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) < 0.25 * spread, (i, tok)
    assert eng.cache_manager.num_free_blocks == 64
