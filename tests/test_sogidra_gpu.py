"""Sogidra on the GPU engine (HIP kernels, bf16 and float32) against the plain
reference in sogidra_oracle.py: mixed batches, portions, decoding through
hipGraphs, pages used again, irregular sizes, greedy generation."""

import pytest
import torch

import sogidra_oracle as oracle
import sogidra_util as U
from parallax_amd import ops
from parallax_amd.server.sampling_params import SamplingParams

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 5e-5, torch.bfloat16: 0.06}


def close(got, want, dtype) -> bool:
    if dtype == torch.bfloat16:
        return U.close_in_bf16(got, want, TOL[dtype])
    return U.rel_err(got, want) < TOL[dtype]


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    # the layer mix of the CPU tests at a width the tuned GEMM path takes;
    # key and value widths on both the vector path (multiples of 8) and the
    # scalar path (12 / 20) of the attention kernel
    layers = [
        U.window_spec(),
        U.diff_spec(),
        U.window_spec(heads=2, kv_heads=2, dim=24, size=4, pool=5, softcap=3.0, mlp=None),
        U.diff_spec(heads=6, kv_heads=2, kv_from=1, scale=0.5, coef=0.1, every=3,
                    mlp=U.dense(24)),
        U.window_spec(heads=3, kv_heads=1, dim=8, size=30, pool=8),
        U.diff_spec(heads=8, kv_heads=2, dim=16, vdim=24, mlp=U.dense(64)),
    ]
    cfg = U.small_config(layers, width=64, vocab=131)
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("sgg")), cfg, w)
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
def test_sizes_outside_the_tuned_gemm_path(tmp_path, dtype):
    """A width, vocabulary and head sizes that are no multiples of 8: the
    projections go to the vendor's plain GEMM, the attention kernel takes its
    scalar path, decode still runs from graphs."""
    layers = [U.diff_spec(3, 3, 10, 6, mlp=U.dense(20)),
              U.window_spec(5, 1, 12, size=9, pool=20, mlp=None),
              U.window_spec(1, 1, 20, size=1, pool=1)]
    cfg = U.small_config(layers, width=44, vocab=53)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, graphs=dtype == torch.bfloat16)
    toks = U.tokens(75, 53, 10)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 5] + [1] * 30])["a"]
    assert close(got, oracle.forward(cfg, w, toks), dtype), \
        U.describe(got, oracle.forward(cfg, w, toks), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_widths_the_matrix_core_path_pads(tmp_path, dtype):
    """Key and value widths that are multiples of 8 but not of the matrix-core
    tiles (40, 24 / 72, 104), head groups of 3, 5 and 6, a pooled block longer
    than its window, a window of one token: long portions take the tiled
    kernel, single tokens the per-token one, and both agree with the
    reference."""
    layers = [U.window_spec(6, 2, 40, size=10, pool=4, softcap=5.0, mlp=U.dense(48)),
              U.diff_spec(3, 1, 24, 72, scale=0.2, every=5, mlp=None),
              U.window_spec(5, 1, 104, size=3, pool=7, softcap=0.0, scale=0.1),
              U.diff_spec(6, 1, 24, 72, kv_from=1, scale=0.15, diff=0.4, mlp=U.dense(48)),
              U.window_spec(4, 4, 8, size=1, pool=2, mlp=None)]
    cfg = U.small_config(layers, width=56, vocab=61)
    w = oracle.random_weights(cfg, seed=23)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, pages=40)
    seqs = {"a": U.tokens(140, 61, 31), "b": U.tokens(45, 61, 32)}
    schedule = [[("a", 70)], [("a", 33), ("b", 40)], [("a", 1), ("b", 1)],
                [("a", 36), ("b", 4)]]
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
