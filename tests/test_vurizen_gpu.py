"""Vurizen on the GPU engine (HIP kernels, bf16 and float32) against the plain
reference in vurizen_oracle.py: mixed batches, portions, decoding through
hipGraphs, pages and slots used again, irregular sizes, greedy generation."""

import pytest
import torch

import vurizen_oracle as oracle
import vurizen_util as U
from parallax_amd import ops
from parallax_amd.ops import reference as ref
from parallax_amd.server.sampling_params import SamplingParams

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 5e-5, torch.bfloat16: 0.06}


def close(got, want, dtype) -> bool:
    if dtype == torch.bfloat16:
        return U.close_in_bf16(got, want, TOL[dtype])
    return U.rel_err(got, want) < TOL[dtype]


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    # the irregular sizes of the CPU tests, but expert sizes the grouped-GEMM
    # kernel tiles (width % 32 == 0, ff % 64 == 0) so decode graphs are used
    layers = [
        U.latent_spec(mlp=U.moe_spec(6, 2, 64, (3, 2), 1.5)),
        U.gla_spec(mlp=U.moe_spec(6, 2, 64, (3, 2), 1.5)),
        U.latent_spec(kv_from=0, heads=2, dim=16, vdim=24, window=5, mlp=None),
        U.gla_spec(heads=2, dim=40, vdim=24, tau=3.0, mlp=U.moe_spec(4, 1, 128, (1, 1), 1.0)),
        U.latent_spec(rot_dim=24, rot_dims=8, rank=24, window=33, scaling=None,
                      mlp=U.moe_spec(8, 3, 64, (4, 2), 2.0)),
    ]
    cfg = U.small_config(layers, width=64, vocab=131)
    w = oracle.random_weights(cfg, seed=3)
    # corrections spaced wider than a sigmoid's range: which experts are
    # chosen then never hangs on a near-tie that bf16 rounding could flip
    # (data-dependent choices are held to rounding in the float32 runs and on
    # the CPU engine); the weights of the chosen experts still follow the data
    for k in list(w):
        if k.endswith("mlp.correction"):
            n = w[k].numel()
            order = torch.randperm(n, generator=torch.Generator().manual_seed(n))
            w[k] = (order.float() * 1.5).bfloat16().float()
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("vzg")), cfg, w)
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
    assert eng.cache_manager.slot_allocator.num_free_slots == 4


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
def test_sizes_outside_the_expert_kernel_tiling(tmp_path, dtype):
    """width and ff that the grouped-GEMM kernel does not tile: the experts
    run per-expert GEMMs, and decode stays eager (no graph)."""
    cfg = U.small_config(width=48, vocab=53)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    eng = U.make_engine(path, device="cuda", dtype=dtype, graphs=True)
    assert eng.graph_runner is None
    toks = U.tokens(45, 53, 10)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 5]])["a"]
    assert close(got, oracle.forward(cfg, w, toks), dtype), \
        U.describe(got, oracle.forward(cfg, w, toks), TOL[dtype])


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
    assert eng.cache_manager.slot_allocator.num_free_slots == 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_planted_key_at_window_and_page_edges(dtype):
    """One cache row that every query scores far above the rest: the kernel
    must count it exactly while it is inside the window, in portions and in
    decode rows, with the edge on and off a page border, also far away."""
    H, rank, rot_w, bs, nb = 5, 96, 16, 8, 80
    g = torch.Generator().manual_seed(0)
    L = 600
    cache = (torch.randn(nb, bs, rank + rot_w, generator=g) * 0.1).to(dtype)
    table = torch.randperm(nb, generator=g)[: (L + bs - 1) // bs].int()
    u = torch.randn(rank, generator=g)
    u /= u.norm()
    for window, planted in [(24, 500), (24, 505), (64, 7), (550, 3), (1, 100)]:
        c2 = cache.clone()
        row = torch.zeros(rank + rot_w)
        row[:rank] = 6.0 * u
        c2.view(-1, rank + rot_w)[int(table[planted // bs]) * bs + planted % bs] = row.to(dtype)
        qpos = sorted({planted, planted + window - 1, planted + window, planted + 1,
                       min(L - 1, planted + window + 5)} & set(range(L)))
        positions = torch.tensor(qpos, dtype=torch.int32)
        T = len(qpos)
        q_lat = (torch.randn(T, H, rank, generator=g) * 0.1 + 3.0 * u).contiguous()
        q_rot = torch.randn(T, H, rot_w, generator=g) * 0.1
        seq = torch.zeros(T, dtype=torch.int32)
        want = ref.latent_window_attention(q_lat, q_rot, c2, table.unsqueeze(0), seq,
                                           positions, window, 1.0)
        got = ops.latent_window_attention(
            q_lat.cuda(), q_rot.cuda(), c2.cuda(), table.unsqueeze(0).cuda(), seq.cuda(),
            positions.cuda(), window, 1.0)
        torch.testing.assert_close(got.cpu(), want, rtol=1e-3, atol=1e-4)
        for i, p in enumerate(qpos):          # seen exactly inside the window
            weight = float((got[i, 0].cpu() @ u) / 6.0)
            assert (weight > 0.9) == (0 <= p - planted < window), (window, planted, p)
        # decode rows: one query per sequence, all with the same table
        tables = table.unsqueeze(0).repeat(T, 1).contiguous()
        got_d = ops.latent_window_attention(q_lat.cuda(), q_rot.cuda(), c2.cuda(),
                                            tables.cuda(), None, positions.cuda(),
                                            window, 1.0)
        torch.testing.assert_close(got_d.cpu(), got.cpu(), rtol=0, atol=0)
