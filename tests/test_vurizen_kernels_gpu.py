"""GPU numerics of the sequence-mixer kernels (extension _mix): each HIP kernel
against the eager fp32 torch version of the same op (ops/reference.py), for
bf16 and float32 activations, on shapes that are not multiples of the
kernels' tile sizes."""

import math

import pytest
import torch

from parallax_amd import ops
from parallax_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _rand(*shape, dtype, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _tol(dtype):
    return (2e-2, 2e-2) if dtype == torch.bfloat16 else (2e-5, 2e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [48, 256, 1000, 4500])
@pytest.mark.parametrize("y_fp32", [False, True])
def test_add_layernorm(dtype, W, y_fp32):
    T = 7
    resid = _rand(T, W, dtype=torch.float32, seed=1) + 0.5
    y = _rand(T, W, dtype=torch.float32 if y_fp32 else dtype, seed=2)
    scale = _rand(W, dtype=dtype, seed=3)
    w = _rand(W, dtype=dtype, seed=4) + 1
    b = _rand(W, dtype=dtype, seed=5)
    r_ref = resid.clone()
    want = ref.add_layernorm(r_ref, y, scale, 0.55, w, b, 1e-5, torch.float32)
    r_gpu = resid.to(DEV)
    got = ops.add_layernorm(r_gpu, y.to(DEV), scale.to(DEV), 0.55, w.to(DEV),
                            b.to(DEV), 1e-5, dtype)
    assert got.dtype == dtype
    torch.testing.assert_close(r_gpu.cpu(), r_ref, rtol=1e-6, atol=1e-6)
    rt, at = _tol(dtype)
    torch.testing.assert_close(got.float().cpu(), want, rtol=rt, atol=at)
    # no update, norm only; update only, no norm
    got2 = ops.add_layernorm(r_gpu, None, None, 1.0, w.to(DEV), b.to(DEV), 1e-5, dtype)
    torch.testing.assert_close(got2.float().cpu(), want, rtol=rt, atol=at)
    r3 = resid.to(DEV)
    assert ops.add_layernorm(r3, y.to(DEV), scale.to(DEV), 0.55, None, None, 0.0,
                             dtype) is None
    torch.testing.assert_close(r3.cpu(), r_ref, rtol=1e-6, atol=1e-6)


def _freq(dims, base=10000.0):
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)],
                        dtype=torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rank,rot_w,rot_dims", [(96, 16, 16), (40, 24, 16), (200, 8, 8)])
def test_latent_kv_store_and_rope_rows(dtype, rank, rot_w, rot_dims):
    T, bs, nb, H, dn = 9, 4, 6, 3, 20
    dkv = _rand(T, rank + rot_w + 5, dtype=dtype, seed=1)[:, : rank + rot_w]  # strided rows
    norm_w = _rand(rank, dtype=dtype, seed=2) + 1
    freq = _freq(rot_dims)
    positions = torch.tensor([0, 1, 2, 700, 701, 5, 6, 7, 12345], dtype=torch.int32)
    slots = torch.tensor([3, 0, -1, 23, 22, 9, 10, 11, 17], dtype=torch.int64)
    cache_ref = torch.zeros(nb, bs, rank + rot_w, dtype=dtype)
    ref.latent_kv_store(dkv, norm_w, 1e-5, freq, 1.2, rot_dims, positions, slots,
                        cache_ref, rank)
    cache = torch.zeros(nb, bs, rank + rot_w, dtype=dtype, device=DEV)
    ops.latent_kv_store(dkv.to(DEV), norm_w.to(DEV), 1e-5, freq.to(DEV), 1.2,
                        rot_dims, positions.to(DEV), slots.to(DEV), cache, rank)
    rt, at = _tol(dtype)
    torch.testing.assert_close(cache.float().cpu(), cache_ref.float(), rtol=rt, atol=at)
    q = _rand(T, H, dn + rot_w, dtype=dtype, seed=3)
    want = ref.rope_rows(q, dn, rot_w, freq, 1.2, rot_dims, positions)
    got = ops.rope_rows(q.to(DEV), dn, rot_w, freq.to(DEV), 1.2, rot_dims,
                        positions.to(DEV))
    # position 12345 * freq rounds in fp32 on both sides; angles agree to ~1e-3
    torch.testing.assert_close(got.cpu(), want, rtol=2e-3, atol=2e-3)
    torch.testing.assert_close(got.cpu()[:8], want[:8], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,rank,rot_w,window", [(4, 96, 16, 23), (5, 72, 16, 7),
                                                 (2, 520, 64, 300), (3, 32, 8, 1),
                                                 (3, 36, 6, 11)])
def test_latent_window_attention(dtype, H, rank, rot_w, window):
    bs, nb = 8, 64
    E = rank + rot_w
    cache = _rand(nb, bs, E, dtype=dtype, scale=0.5, seed=1)
    # sequence 0: a portion of 11 tokens ending at length 150; sequence 1: a
    # portion that starts at 0; sequence 2: one token (like a decode row)
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(2)).int()
    block_tables = torch.stack([perm[:20], perm[20:40], perm[40:60]])
    positions = torch.tensor(list(range(139, 150)) + list(range(0, 9)) + [77],
                             dtype=torch.int32)
    token_seq = torch.tensor([0] * 11 + [1] * 9 + [2], dtype=torch.int32)
    T = positions.numel()
    q_lat = _rand(T, H, rank, dtype=torch.float32, scale=0.3, seed=3)
    q_rot = _rand(T, H, rot_w, dtype=torch.float32, scale=0.3, seed=4)
    want = ref.latent_window_attention(q_lat, q_rot, cache, block_tables, token_seq,
                                       positions, window, 0.3)
    got = ops.latent_window_attention(q_lat.to(DEV), q_rot.to(DEV), cache.to(DEV),
                                      block_tables.to(DEV), token_seq.to(DEV),
                                      positions.to(DEV), window, 0.3)
    torch.testing.assert_close(got.cpu(), want, rtol=2e-4, atol=2e-5)
    # decode form: token i is sequence i
    pos_d = torch.tensor([149, 8, 77], dtype=torch.int32)
    idx = [10, 19, 20]
    got_d = ops.latent_window_attention(
        q_lat[idx].contiguous().to(DEV), q_rot[idx].contiguous().to(DEV),
        cache.to(DEV), block_tables.to(DEV), None, pos_d.to(DEV), window, 0.3)
    torch.testing.assert_close(got_d.cpu(), want[idx], rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,dk,dv", [(4, 32, 48), (3, 24, 40), (2, 128, 72), (1, 80, 200)])
def test_gla_recurrence_and_gated_norm(dtype, H, dk, dv):
    lens = [37, 1, 5]
    T = sum(lens)
    q = _rand(T, H * dk, dtype=dtype, seed=1)
    k = _rand(T, H * dk, dtype=dtype, scale=0.5, seed=2)
    v = _rand(T, H * dv, dtype=dtype, seed=3)
    z = _rand(T, H * dk, dtype=dtype, scale=2.0, seed=4)
    zb = _rand(H * dk, dtype=dtype, seed=5) + 1
    state0 = _rand(6, H, dk, dv, dtype=torch.float32, seed=6)
    slots = torch.tensor([4, 1, 2], dtype=torch.int64)
    cu = torch.tensor([0, 37, 38, 43], dtype=torch.int32)
    # sequence 0 continues at position 100 (keeps its slot's state), sequence 1
    # is a single later token, sequence 2 starts at 0 (state must be zeroed)
    positions = torch.tensor(list(range(100, 137)) + [9] + list(range(5)),
                             dtype=torch.int32)
    s_ref = state0.clone()
    want = ref.gla_recurrence(q, k, v, z, zb, s_ref, slots, cu, positions,
                              1 / 12.0, dk ** -0.5)
    s_gpu = state0.to(DEV)
    got = ops.gla_recurrence(q.to(DEV), k.to(DEV), v.to(DEV), z.to(DEV), zb.to(DEV),
                             s_gpu, slots.to(DEV), cu.to(DEV), positions.to(DEV),
                             1 / 12.0, dk ** -0.5)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(s_gpu.cpu(), s_ref, rtol=1e-4, atol=1e-4)
    # untouched slots stay as they were
    torch.testing.assert_close(s_gpu.cpu()[[0, 3, 5]], state0[[0, 3, 5]], rtol=0, atol=0)

    # the same tokens one by one (decode form) land on the same state
    s_dec = state0.to(DEV)
    outs = []
    for t in range(37):
        outs.append(ops.gla_recurrence(
            q[t : t + 1].to(DEV), k[t : t + 1].to(DEV), v[t : t + 1].to(DEV),
            z[t : t + 1].to(DEV), zb.to(DEV), s_dec, slots[:1].to(DEV), None,
            positions[t : t + 1].to(DEV), 1 / 12.0, dk ** -0.5))
    torch.testing.assert_close(torch.cat(outs).cpu(), got.cpu()[:37], rtol=0, atol=0)
    torch.testing.assert_close(s_dec[4].cpu(), s_gpu[4].cpu(), rtol=0, atol=0)

    gate = _rand(T, H * dv, dtype=dtype, seed=7)
    w = _rand(dv, dtype=dtype, seed=8) + 1
    want_n = ref.gated_rmsnorm(want, gate, w, 1e-5, torch.float32)
    got_n = ops.gated_rmsnorm(got, gate.to(DEV), w.to(DEV), 1e-5, dtype)
    rt, at = _tol(dtype)
    torch.testing.assert_close(got_n.float().cpu(), want_n, rtol=rt, atol=at)
