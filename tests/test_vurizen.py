"""Vurizen on the CPU engine (fp32) against the plain reference in
vurizen_oracle.py: each mechanism alone, then the engine's step function,
cache manager, state slots and scheduler under many ways of cutting and
batching the same sequences. Configurations are small and deliberately
irregular (see vurizen_util.small_config)."""

import math

import pytest
import torch

import vurizen_oracle as oracle
import vurizen_util as U
from parallax_amd import ops
from parallax_amd.models.config import ModelConfig
from parallax_amd.models.forward_meta import ForwardMeta
from parallax_amd.models.latent_attention import LatentWindowAttention
from parallax_amd.models.linear_attention import GatedLinearAttention
from parallax_amd.models.moe import FusedMoE, MoERouter
from parallax_amd.models.rope import yarn_ramp_frequencies
from parallax_amd.models.vurizen import _moe_config
from parallax_amd.server.kv_cache import LinearStateCache, MLAKVCache
from parallax_amd.server.sampling_params import SamplingParams

D = oracle.DT
TOL = 2e-5


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = U.small_config()
    w = oracle.random_weights(cfg, seed=3)
    path = U.write_checkpoint(str(tmp_path_factory.mktemp("vz")), cfg, w)
    return cfg, w, path


# -- mechanisms alone ------------------------------------------------------------


def test_config_reader():
    cfg = U.small_config()
    mc = ModelConfig.from_hf_config(cfg)
    assert mc.architecture == "Vurizen" and mc.num_layers == 5
    assert mc.layer_types == ["latent_attention", "linear_attention",
                              "latent_attention", "linear_attention",
                              "latent_attention"]
    # only layers with a cache of their own appear; kv_from layers do not
    assert mc.latent_cache_dims(0, 5) == [(40, 16), (24, 24)]
    assert [r for _, r in mc.linear_state_shapes(0, 5)] == [(3, 24, 40), (2, 40, 24)]
    assert mc.has_linear_layers and mc.residual_mult == 0.6
    with pytest.raises(ValueError):
        ModelConfig.from_hf_config(U.small_config([{"type": "conv", "mixer": {}, "mlp": None}]))


@pytest.mark.parametrize("dims,base,sc", [
    (48, 30000.0, {"factor": 6.0, "original": 512, "fast": 16.0, "slow": 2.0}),
    # a slow boundary beyond dims/2 - 1: the ramp's top is clipped at dims - 1
    (8, 50.0, {"factor": 3.0, "original": 4000, "fast": 4.0, "slow": 0.5}),
    (16, 10000.0, None),
])
def test_yarn_frequencies(dims, base, sc):
    want_f, want_m = oracle.yarn_frequencies(dims, base, sc)
    sc = sc or {}
    got_f, got_m = yarn_ramp_frequencies(dims, base, sc.get("factor", 1.0),
                                         sc.get("original", 0.0), sc.get("fast", 32.0),
                                         sc.get("slow", 1.0))
    torch.testing.assert_close(got_f.double(), want_f, rtol=1e-6, atol=0)
    assert abs(got_m - want_m) < 1e-12


def test_layer_norm_with_scaled_update():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 48, generator=g) * 3 + 1
    y = torch.randn(5, 48, generator=g)
    ls, w, b = (torch.randn(48, generator=g) for _ in range(3))
    resid = x.clone()
    got = ops.add_layernorm(resid, y, ls, 0.6, w, b, 1e-5, torch.float32)
    x2 = x.double() + 0.6 * (y.double() * ls.double())
    torch.testing.assert_close(resid.double(), x2, rtol=1e-6, atol=1e-6)
    want = oracle.layer_norm(x2, w.double(), b.double(), 1e-5)
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("experts,top,groups", [(6, 2, (3, 2)), (8, 3, (4, 2)),
                                                (4, 1, (1, 1)), (6, 4, (2, 2))])
def test_router(experts, top, groups):
    mlp = U.moe_spec(experts, top, 16, groups, 2.5)
    mc = _moe_config(ModelConfig.from_hf_config(U.small_config()), mlp)
    router = MoERouter(mc)
    g = torch.Generator().manual_seed(1)
    router.weight.data = torch.randn(experts, 48, generator=g)
    # negative corrections: a masked group must count as -inf, not as 0
    router.e_score_correction_bias.data = -1.5 + torch.randn(experts, generator=g)
    h = torch.randn(40, 48, generator=g)
    ids, wts = router(h)
    w = {"r.router": router.weight.data, "r.correction": router.e_score_correction_bias.data}
    want = oracle.route(h.double(), w, "r.", mlp["router"])
    for t in range(40):
        got = sorted(zip(ids[t].tolist(), wts[t].tolist()))
        exp = sorted(want[t])
        assert [e for e, _ in got] == [e for e, _ in exp]
        assert all(abs(a - b) < 1e-5 for (_, a), (_, b) in zip(got, exp))


def test_moe_block():
    mlp = U.moe_spec(6, 2, 24, (3, 2), 1.5)
    cfgd = U.small_config([U.gla_spec(mlp=mlp)])
    w = oracle.random_weights(cfgd, seed=5)
    moe = FusedMoE(_moe_config(ModelConfig.from_hf_config(cfgd), mlp))
    moe.fp32_output = True
    moe.router.weight.data = w["l0.mlp.router"].clone()
    moe.router.e_score_correction_bias.data = w["l0.mlp.correction"].clone()
    for e in range(6):
        moe.load_expert_gate(e, w["l0.mlp.e%d.gate" % e])
        moe.load_expert_up(e, w["l0.mlp.e%d.up" % e])
        moe.load_expert_down(e, w["l0.mlp.e%d.down" % e])
    h = torch.randn(17, 48, generator=torch.Generator().manual_seed(2))
    want = oracle.moe(h.double(), w, "l0.mlp.", mlp)
    torch.testing.assert_close(moe(h).double(), want, rtol=1e-5, atol=1e-5)


def _gla_module(w, spec, width=48):
    mx = spec["mixer"]
    m = GatedLinearAttention(width, mx["heads"], mx["dim"], mx["vdim"], mx["tau"],
                             1e-5, 0)
    for i, k in enumerate("qkvg"):
        m.in_proj.load_full_weight_part(i, w["l0.mix." + k])
    m.o_proj.load_full_weight(w["l0.mix.o"])
    m.norm_weight.data = w["l0.mix.norm"].clone()
    m.load_decay("a1", w["l0.mix.a1"])
    m.load_decay("a2", w["l0.mix.a2"])
    m.decay_bias.data = w["l0.mix.a2.b"].clone()
    return m


def _gla_meta(cache, lens, starts, slots):
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int()
    prefill = not all(n == 1 and s > 0 for s, n in zip(starts, lens))
    return ForwardMeta(
        is_prefill=prefill, positions=pos, slot_mapping=torch.zeros(len(pos), dtype=torch.long),
        block_tables=torch.zeros(len(lens), 1, dtype=torch.int32),
        seq_lens=torch.tensor([s + n for s, n in zip(starts, lens)], dtype=torch.int32),
        query_lens=torch.tensor(lens, dtype=torch.int32) if prefill else None,
        linear_cache=cache, linear_slots=torch.tensor(slots, dtype=torch.long))


@pytest.mark.parametrize("heads,dim,vdim,tau", [(3, 24, 40, 8.0), (1, 40, 8, 1.0)])
def test_gla_mixer_alone_state_carried_across_portions(heads, dim, vdim, tau):
    spec = U.gla_spec(heads, dim, vdim, tau, mlp=None)
    cfgd = U.small_config([spec])
    w = oracle.random_weights(cfgd, seed=7)
    m = _gla_module(w, spec)
    T = 150
    h = torch.randn(T, 48, generator=torch.Generator().manual_seed(3))
    h[4] *= 12.0  # a far token that dominates the state: losing it shows
    want = oracle.gla(h.double(), w, "l0.mix.", spec["mixer"], 1e-5)
    cache = LinearStateCache(1, (0,), (heads, dim, vdim), 3, torch.device("cpu"),
                             torch.float32)
    cache.recurrent_states[0].fill_(7.0)  # leftovers of an earlier request
    outs, at = [], 0
    for n in [2, 5, 1, 1, 64, 3, 1, 40, 2, 31]:
        outs.append(m(h[at : at + n], _gla_meta(cache, [n], [at], [2])))
        at += n
    assert at == T
    torch.testing.assert_close(torch.cat(outs).double(), want, rtol=2e-4, atol=2e-4)
    assert float(cache.recurrent_states[0][0].min()) == 7.0  # other slots untouched


def _latent_module(w, spec, pre="l0.mix.", cache_idx=0, width=48):
    mx = spec["mixer"]
    owns = mx.get("kv_from") is None
    rot = mx["rot"]
    m = LatentWindowAttention(
        width, mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"],
        mx["mask"]["size"], mx["scale"], 1e-5, cache_idx, owns,
        rot_dims=rot["dims"], rot_base=rot["base"], rot_scaling=rot.get("scaling"))
    m.in_proj.load_full_weight_part(0, w[pre + "q"])
    if owns:
        m.in_proj.load_full_weight_part(1, w[pre + "dkv"])
        m.latent_norm.data = w[pre + "dkv.norm"].clone()
    m.w_uk.data = w[pre + "uk"].view(mx["heads"], mx["dim"], mx["kv_rank"]).clone()
    m.w_uv.data = w[pre + "uv"].view(mx["heads"], mx["vdim"], mx["kv_rank"]).clone()
    m.o_proj.load_full_weight(w[pre + "o"])
    return m


def _latent_meta(cache, table, start, n, bs):
    pos = torch.arange(start, start + n)
    bt = torch.tensor(table)
    return ForwardMeta(
        is_prefill=not (n == 1 and start > 0), positions=pos.int(),
        slot_mapping=bt[pos // bs] * bs + pos % bs,
        block_tables=bt.int().unsqueeze(0),
        seq_lens=torch.tensor([start + n], dtype=torch.int32),
        query_lens=torch.tensor([n], dtype=torch.int32), mla_cache=cache)


@pytest.mark.parametrize("window,rot_dims", [(9, 16), (1, 16), (64, 8), (200, 16)])
def test_latent_mixer_alone_portions_and_pages(window, rot_dims):
    spec = U.latent_spec(window=window, rot_dims=rot_dims, mlp=None)
    w = oracle.random_weights(U.small_config([spec]), seed=11)
    m = _latent_module(w, spec)
    T, bs = 90, 4
    h = torch.randn(T, 48, generator=torch.Generator().manual_seed(4))
    c, kr = oracle.latent_kv(h.double(), w, "l0.mix.", spec["mixer"], 1e-5)
    want = oracle.latent_attention(h.double(), w, "l0.mix.", spec["mixer"], c, kr)
    cache = MLAKVCache(1, 40, 16, bs, 40, torch.device("cpu"), torch.float32)
    table = torch.randperm(40, generator=torch.Generator().manual_seed(5))[:23].tolist()
    outs, at = [], 0
    for n in [3, 2, 1, 1, 1, 30, 7, 1, 2, 41, 1]:
        outs.append(m(h[at : at + n], _latent_meta(cache, table, at, n, bs)))
        at += n
    assert at == T
    torch.testing.assert_close(torch.cat(outs).double(), want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("decode", [False, True])
def test_window_edge_with_a_planted_key(decode):
    """One cached key is made to dominate the scores of every later query. It
    must be seen while 0 <= i - j < window and must vanish one token later,
    in a prompt portion and in single decoded tokens, also when the edge
    falls on a page border."""
    window, bs = 6, 4
    spec = U.latent_spec(window=window, kv_from=0, mlp=None, scaling=None)
    own = U.latent_spec(window=window, mlp=None, scaling=None)
    cfgd = U.small_config([own, spec])
    w = oracle.random_weights(cfgd, seed=13)
    m = _latent_module(w, spec, pre="l1.mix.")
    T = 24
    g = torch.Generator().manual_seed(6)
    h = torch.randn(T, 48, generator=g)
    c = torch.randn(T, 40, generator=g).double() * 0.1
    kr = torch.randn(T, 16, generator=g).double() * 0.1
    for planted in (3, 7, 10):      # 7 + window - 1 = 12: the edge sits on a page border
        c2, kr2 = c.clone(), kr.clone()
        # the key every query scores highest: aligned with W_uk^T q of all heads
        q = (h.double() @ w["l1.mix.q"].double().T).view(T, 3, 40)[..., :24]
        uk = w["l1.mix.uk"].double().view(3, 24, 40)
        c2[planted] = torch.einsum("thd,hdr->r", q[planted + 1 : planted + window + 2], uk)
        c2[planted] *= 40.0 / c2[planted].norm()
        want = oracle.latent_attention(h.double(), w, "l1.mix.", spec["mixer"], c2, kr2)
        cache = MLAKVCache(1, 40, 16, bs, 8, torch.device("cpu"), torch.float32)
        table = [5, 2, 7, 0, 3, 6]
        rows = torch.cat([c2, kr2], -1).float()
        pos = torch.arange(T)
        bt = torch.tensor(table)
        cache.layer(0).view(-1, 56)[bt[pos // bs] * bs + pos % bs] = rows
        if decode:
            got = torch.cat([m(h[t : t + 1], _latent_meta(cache, table, t, 1, bs))
                             for t in range(T)])
        else:
            got = torch.cat([m(h[:5], _latent_meta(cache, table, 0, 5, bs)),
                             m(h[5:], _latent_meta(cache, table, 5, T - 5, bs))])
        torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-4)
        # the planted key matters: inside the window the output differs from
        # the unplanted one, right outside it does not
        base = oracle.latent_attention(h.double(), w, "l1.mix.", spec["mixer"], c, kr)
        inside, outside = planted + window - 1, planted + window
        assert (want[inside] - base[inside]).abs().max() > 1e-2
        torch.testing.assert_close(want[outside], base[outside], rtol=0, atol=1e-12)


# -- the engine: step function, cache manager, slots, scheduler -----------------------


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
        [("c", 1), ("b", 1), ("a", 1), ("d", 1)],          # d ends: its slot goes to e
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
    assert eng.cache_manager.slot_allocator.num_free_slots == 4


def test_pages_and_slots_freed_and_used_again(ckpt):
    cfg, w, path = ckpt
    eng = U.make_engine(path, pages=8, block_size=8, max_requests=2)
    for k in range(5):   # 5 requests through 2 slots and 8 pages
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
    toks = U.tokens(140, cfg["vocab"], 9)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", 12)]] + [[("a", 1)]] * 128)["a"]
    assert U.rel_err(got, oracle.forward(cfg, w, toks)) < TOL


@pytest.mark.parametrize("layers", [
    # equal sizes everywhere, one group, one expert per token, window 1
    [U.gla_spec(1, 16, 16, 1.0, mlp=U.moe_spec(2, 1, 16, (1, 1), 1.0)),
     U.latent_spec(1, 16, 16, 16, 16, window=1, scale=1.0,
                   mlp=U.moe_spec(2, 1, 16, (1, 1), 1.0))],
    # no feed-forward at all, wide heads, a window longer than any sequence
    [U.latent_spec(5, 8, 4, 56, 72, window=500, mlp=None),
     U.latent_spec(2, 40, 4, 8, 72, window=3, kv_from=0, mlp=None),
     U.gla_spec(4, 72, 8, 30.0, mlp=None)],
    # only recurrent layers
    [U.gla_spec(2, 24, 24, 2.0), U.gla_spec(3, 8, 48, 16.0)],
])
def test_other_sizes(tmp_path, layers):
    cfg = U.small_config(layers, width=40, vocab=53, mult=1.0)
    w = oracle.random_weights(cfg, seed=17)
    path = U.write_checkpoint(str(tmp_path), cfg, w)
    toks = U.tokens(45, 53, 10)
    eng = U.make_engine(path)
    got = U.run_schedule(eng, {"a": toks}, [[("a", n)] for n in [6, 1, 1, 30, 2, 5]])["a"]
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
    assert eng.cache_manager.slot_allocator.num_free_slots == 4


def test_trace_replay_program(ckpt, tmp_path):
    """bin/trace_run: JSON lines in, 'done <step>' lines and <step>.f32 files
    out; a step without wanted places writes no file; ended requests give
    their pages and slots back."""
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
    got0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    got1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    got2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V)
    assert got0.shape[0] == 2 and got1.shape[0] == 1 and got2.shape[0] == 2
    want = torch.stack([la[0], la[15], lb[7], lb[8], la[20]])
    got = torch.from_numpy(np.concatenate([got0, got1, got2]))
    assert U.rel_err(got, want) < TOL


def test_two_peer_pipeline_greedy(ckpt):
    """The packet-driven multi-host path: two peers split the stack (the fp32
    residual travels between them), greedy tokens equal the reference's."""
    from parallax_amd.p2p.peer_executor import PeerExecutor
    from parallax_amd.p2p.transport import LoopbackTransport

    cfg, w, path = ckpt
    mc = ModelConfig.from_pretrained(path)
    registry, peers = {}, []
    # layer 2 reads layer 0's cache rows, so the cut comes after it
    for pid, (s, e) in zip(["p0", "p1"], [(0, 3), (3, 5)]):
        peers.append(PeerExecutor(mc, s, e, pid, LoopbackTransport(pid, registry),
                                  dtype=torch.float32, num_kv_blocks=64, block_size=8,
                                  model_path=path))
    head = peers[0]
    prompts = [U.tokens(19, cfg["vocab"], 70), U.tokens(4, cfg["vocab"], 71)]
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
    with pytest.raises(ValueError):   # a cut that separates a layer from the cache it reads
        PeerExecutor(mc, 1, 3, "bad", LoopbackTransport("bad", registry),
                     dtype=torch.float32, num_kv_blocks=8, block_size=8)


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
    mp.spawn(_pp_worker, args=(2, 29671, path, prompts, out_file), nprocs=2, join=True)
    got = torch.load(out_file)
    for p, toks in zip(prompts, got):
        seq = list(p)
        for _ in range(5):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert toks == seq[len(p):]
