"""Zabusun on the GPU engine (HIP kernels, bf16 and float32) against the plain
reference in zabusun_oracle.py: mixed batches, portions, decoding through
hipGraphs, pages and state slots used again, irregular sizes, greedy
generation."""

import pytest
import torch

import zabusun_oracle as oracle
import zabusun_util as U
from parallax_amd import ops
from parallax_amd.server.sampling_params import SamplingParams

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 5e-5, torch.bfloat16: 0.08}


def close(got, want, dtype) -> bool:
    """float32: every row within rounding of the float64 reference. bfloat16:
    every sublayer's output is normed to unit size before it joins the
    stream, so each branch's bf16 rounding enters at full weight, and a
    router near-tie that rounding flips changes a row (and, through the
    recurrent state, the rows after it) outright: the eager bf16 CPU engine
    sits at a median row error of 0.015 to 0.03 on these weights, with single
    rows near 1. So: 85 rows in 100 within 0.08 and the median under 0.04;
    same_as_whole() is the sharp bf16 check."""
    if dtype == torch.bfloat16:
        e = U.row_errs(got, want)
        few = e.numel() < 8          # a median of a handful of rows says little
        return bool((e < TOL[dtype]).double().mean() >= 0.85
                    and (few or e.median() < 0.04))
    return U.rel_err(got, want) < TOL[dtype]


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    # the layer mix of the CPU tests at a width the tuned GEMM path takes:
    # key and value widths on both the vector path (multiples of 8) and the
    # scalar path (12 / 20) of the attention kernel, expert widths the
    # grouped-GEMM kernels tile (32, 96)
    layers = [
        U.layer(),
        U.layer(4, 4, 16, 8, 0.25, U.rot(16, 10000.0, None), 52, 1.0, 0.5,
                U.experts(5, 2, 32, 2.0)),
        U.layer(3, 1, 24, 24, 0.2, None, 8, 0.4, 1.0, None),
        U.layer(2, 1, 8, 12, 0.35, U.rot(4, 100.0, {"factor": 2.0, "original": 16,
                                                    "fast": 4.0, "slow": 1.0}),
                33, 1.5, 0.8, U.experts(3, 1, 96, 1.0)),
        U.layer(8, 2, 40, 72, 0.15, U.rot(20), 64, mlp=U.dense(64)),
    ]
    cfg = U.small_config(layers, width=64, vocab=131)
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("zbg")), cfg, w)
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
    """A width, vocabulary, head and expert sizes that are no multiples of 8:
    the projections go to the vendor's plain GEMM, the attention kernel takes
    its scalar path, the experts the per-expert loop (decode then runs
    eagerly), the residual kernel its scalar path."""
    layers = [U.layer(3, 3, 10, 6, rotation=U.rot(6), width=7, mlp=U.dense(20)),
              U.layer(5, 1, 12, 12, rotation=None, width=50, mlp=U.experts(3, 2, 20, 0.7)),
              U.layer(1, 1, 20, 4, rotation=U.rot(20, 30.0, None), width=1, mlp=None)]
    cfg = U.small_config(layers, width=46, vocab=53)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, graphs=dtype == torch.bfloat16)
    assert eng.graph_runner is None     # the per-expert loop reads the routing on the host
    toks = U.tokens(75, 53, 10)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 5] + [1] * 30])["a"]
    assert close(got, oracle.forward(cfg, w, toks), dtype), \
        U.describe(got, oracle.forward(cfg, w, toks), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_contexts_and_wide_heads(tmp_path, dtype):
    """Key and value widths on the matrix-core tiles and off them (96, 128 /
    80, 256, 104), head groups of 8, 3 and 5, contexts of many pages: long
    portions take the tiled kernel, single tokens the per-token one with
    split key lists, and both agree with the reference."""
    layers = [U.layer(8, 2, 96, 80, 0.1, U.rot(32, 40000.0), 200, 0.5, 1.2,
                      U.experts(6, 2, 96, 1.3)),
              U.layer(3, 1, 128, 256, 0.08, U.rot(128, 1000.0, None), 96, mlp=None),
              U.layer(5, 5, 104, 40, 0.1, U.rot(10), 40, mlp=U.dense(128, 3.0))]
    cfg = U.small_config(layers, width=128, vocab=211)
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
    """bf16 + captured decode graphs + async decode: every generated token is
    the reference's best token or within rounding of it."""
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
