"""GPU numerics of the row-cache attention kernels and the sandwich norm
(extension _mix): each HIP kernel against the eager fp32 torch version of the
same op (ops/reference.py), for bf16 and float32 activations, over paged
caches with shuffled pages, on sizes that are not multiples of the kernels'
tiles (and some that are)."""

import pytest
import torch

from parallax_amd import ops
from parallax_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _tol(dtype):
    return (2e-2, 2e-2) if dtype == torch.bfloat16 else (3e-5, 3e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [40, 46, 256, 1000, 4500])
def test_sandwich_rmsnorm(dtype, W):
    T, n_max = 5, 4
    x = _rand(T, W, seed=1) + 0.3
    hist = _rand(n_max, T, W, seed=2)
    y = _rand(T, W, dtype=dtype, seed=3, scale=3.0)
    wb = _rand(W, dtype=dtype, seed=4, scale=0.2)
    wn = _rand(W, dtype=dtype, seed=5, scale=0.2)
    dwa = _rand(3, seed=6)
    table = _rand(9, W, dtype=dtype, seed=7)
    index = torch.tensor([3, 0, 8, 8, 1], dtype=torch.int32)
    rt, at = _tol(dtype)

    def both(args_of):
        xr, hr = x.clone(), hist.clone()
        want = ref.sandwich_rmsnorm(*args_of(xr, hr, lambda t: t))
        xg, hg = x.to(DEV), hist.to(DEV)
        got = ops.sandwich_rmsnorm(
            *args_of(xg, hg, lambda t: t.to(DEV) if t is not None else None))
        torch.testing.assert_close(xg.cpu(), xr, rtol=2e-6, atol=2e-6)
        torch.testing.assert_close(hg.cpu(), hr, rtol=2e-6, atol=2e-6)
        if want is None:
            assert got is None
        else:
            assert got.dtype == want.dtype
            torch.testing.assert_close(got.float().cpu(), want.float(),
                                       rtol=rt, atol=at)

    # embedding step: table row added, stored as X_0, next norm
    both(lambda xx, hh, d: (xx, None, None, hh, 1, None, d(wn), 1e-6, 1.0,
                            dtype, d(table), d(index)))
    # mid-layer step: branch norm + add + next norm, no history
    both(lambda xx, hh, d: (xx, d(y), d(wb), None, 0, None, d(wn), 1e-6, 1.0,
                            dtype))
    # end of a layer: history store, weighted average, next norm
    both(lambda xx, hh, d: (xx, d(y), d(wb), hh, 3, d(dwa), d(wn), 1e-5, 1.0,
                            dtype))
    # weights used as they are (offset 0), no next norm
    both(lambda xx, hh, d: (xx, d(y), d(wb), hh, 2, d(dwa[:2].contiguous()),
                            None, 1e-6, 0.0, dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [5, 2048, 4099])
def test_xielu(dtype, n):
    x = _rand(n, dtype=dtype, seed=8, scale=2.0)
    want = ref.xielu(x, 0.7, 0.3)
    got = ops.xielu(x.to(DEV), 0.7, 0.3)
    rt, at = _tol(dtype)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at)


class _Paged:
    """Sequences of given lengths in a paged row cache with shuffled pages."""

    def __init__(self, lens, width, block, dtype, pool_tokens=0, seed=0):
        g = torch.Generator().manual_seed(seed)
        need = [(n + block - 1) // block for n in lens]
        total = sum(need) + 3
        perm = torch.randperm(total, generator=g).tolist()
        self.block = block
        self.tables, k = [], 0
        for n in need:
            self.tables.append(perm[k:k + n])
            k += n
        mb = max(need)
        self.block_tables = torch.zeros(len(lens), mb, dtype=torch.int32)
        for i, bt in enumerate(self.tables):
            self.block_tables[i, :len(bt)] = torch.tensor(bt, dtype=torch.int32)
        self.cache = torch.zeros(total, block, width, dtype=dtype)
        self.pool = None
        if pool_tokens:
            per = (block + pool_tokens - 1) // pool_tokens
            self.pool = torch.zeros(total, per, width, dtype=torch.float32)

    def slots(self, seq, start, n):
        pos = torch.arange(start, start + n)
        bt = torch.tensor(self.tables[seq])
        return bt[pos // self.block] * self.block + pos % self.block


def _step(paged, chunks):
    """Packed step metadata for chunks [(seq, start, n)]."""
    pos = torch.cat([torch.arange(s, s + n) for _, s, n in chunks]).to(torch.int32)
    seq = torch.cat([torch.full((n,), q, dtype=torch.int32) for q, _, n in chunks])
    slots = torch.cat([paged.slots(q, s, n) for q, s, n in chunks])
    return pos, seq, slots


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("norm,seg,wq,wk,wv", [
    (True, 24, 96, 48, 0), (True, 128, 256, 128, 0), (False, 16, 160, 64, 56),
    (False, 20, 40, 0, 0),
])
def test_qkv_store(dtype, norm, seg, wq, wk, wv):
    lens = [37, 70]
    block = 16
    width = wk + (wv or wk) if wk else 8
    pg = _Paged(lens, width, block, dtype, seed=3)
    chunks = [(0, 5, 32), (1, 64, 6)]
    pos, _, slots = _step(pg, chunks)
    slots[3] = -1
    T = pos.numel()
    q = _rand(T, wq, dtype=dtype, seed=1)
    k = _rand(T, wk, dtype=dtype, seed=2) if wk else None
    v = _rand(T, wv, dtype=dtype, seed=3) if wv else None
    eps = 1e-6 if norm else None
    c_ref = pg.cache.clone()
    want = ref.qkv_store(q, k, v, pos, slots, c_ref, seg, eps, 0.25, 16)
    c_gpu = pg.cache.to(DEV)
    d = lambda t: t.to(DEV) if t is not None else None
    got = ops.qkv_store(d(q), d(k), d(v), d(pos), d(slots), c_gpu, seg, eps,
                        0.25, 16)
    rt, at = (1e-5, 1e-5)
    torch.testing.assert_close(got.cpu(), want, rtol=rt, atol=at)
    rt, at = _tol(dtype)
    torch.testing.assert_close(c_gpu.float().cpu(), c_ref.float(), rtol=rt, atol=at)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("P,block", [(4, 16), (6, 16), (16, 16), (40, 16), (1, 8)])
def test_pool_cache_update(dtype, P, block):
    lens = [3 * P + 2, 5 * P]
    E = 72
    pg = _Paged(lens, E, block, dtype, pool_tokens=P, seed=4)
    pg.cache.copy_(_rand(*pg.cache.shape, dtype=dtype, seed=5))
    # a step that completes blocks in the middle and at the end of a portion
    chunks = [(0, P - 1, 2 * P + 1), (1, 5 * P - 1, 1)]
    pos, seq, slots = _step(pg, chunks)
    p_ref = pg.pool.clone()
    ref.pool_cache_update(pg.cache, p_ref, pg.block_tables, seq, pos, slots, P)
    p_gpu = pg.pool.to(DEV)
    ops.pool_cache_update(pg.cache.to(DEV), p_gpu, pg.block_tables.to(DEV),
                          seq.to(DEV), pos.to(DEV), slots.to(DEV), P)
    assert p_ref.abs().sum() > 0
    torch.testing.assert_close(p_gpu.cpu(), p_ref, rtol=1e-5, atol=1e-5)


CASES = [
    # H, G, M, d, dv, window, P, softcap, norm
    (4, 2, 1, 32, 32, 20, 4, 30.0, False),     # pooled window, vector path
    (6, 2, 1, 24, 24, 33, 5, 0.0, False),      # block does not divide a page
    (3, 3, 1, 20, 20, 7, 1, 10.0, False),      # scalar path, blocks of one token
    (8, 1, 1, 64, 64, 200, 32, 40.0, False),   # eight heads share one kv head
    (4, 2, 2, 16, 40, 0, 0, 0.0, True),        # two maps, full causal, head norm
    (2, 2, 2, 12, 10, 0, 0, 0.0, True),        # scalar path
    (4, 1, 2, 64, 128, 0, 0, 0.0, True),
    (2, 1, 1, 8, 256, 50, 0, 0.0, False),      # window without pooled blocks
    (2, 1, 2, 128, 256, 0, 0, 0.0, True),      # the widest the matrix-core path takes
    (5, 1, 1, 48, 96, 40, 8, 20.0, False),     # widths padded to the tile sizes
    (4, 4, 1, 136, 64, 0, 0, 0.0, False),      # keys wider than the matrix-core path
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("decode", [False, True])
def test_row_attention(dtype, case, decode):
    H, G, M, d, dv, window, P, softcap, norm = case
    E = G * M * d + G * dv
    lens = [300, 77, 1]
    block = 16
    pg = _Paged(lens, E, block, dtype, pool_tokens=P if window else 0, seed=6)
    pg.cache.copy_(_rand(*pg.cache.shape, dtype=dtype, seed=7))
    # pooled rows of every complete block, through the reference op
    if pg.pool is not None:
        for s, n in enumerate(lens):
            pos, seq, slots = _step(pg, [(s, 0, n)])
            ref.pool_cache_update(pg.cache, pg.pool, pg.block_tables, seq, pos,
                                  slots, P)
    bounds = None
    if decode:
        pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
        seq = None
        max_len = max(lens)
    else:
        pos, seq, _ = _step(pg, [(0, 250, 50), (1, 0, 77), (2, 0, 1)])
        bounds = torch.tensor([0, 50, 127, 128], dtype=torch.int32)
        max_len = max(lens)
    T = pos.numel()
    q = _rand(T, H * M * d, seed=8)
    eps = 1e-6 if norm else None
    args = (H, G, M, d, dv, window, P if window else 0, d ** -0.5, softcap,
            0.37, eps, 0.8)
    want = ref.row_attention(q, pg.cache, pg.pool, pg.block_tables, seq, pos,
                             *args, torch.float32)
    dd = lambda t: t.to(DEV) if t is not None else None
    got = ops.row_attention(dd(q), dd(pg.cache), dd(pg.pool),
                            dd(pg.block_tables), dd(seq), dd(pos), *args, dtype,
                            max_seq_len=max_len, query_bounds=dd(bounds))
    assert got.dtype == dtype
    if not decode:
        # the same tokens without their bounds: one workgroup per token
        per_token = ops.row_attention(dd(q), dd(pg.cache), dd(pg.pool),
                                      dd(pg.block_tables), dd(seq), dd(pos),
                                      *args, dtype, max_seq_len=max_len)
        rt, at = _tol(dtype)
        torch.testing.assert_close(per_token.float().cpu(), want, rtol=rt, atol=at)
    rt, at = _tol(dtype)
    torch.testing.assert_close(got.float().cpu(), want, rtol=rt, atol=at)
    if decode:
        # the split of the keys over workgroups follows the host's bound only
        got2 = ops.row_attention(dd(q), dd(pg.cache), dd(pg.pool),
                                 dd(pg.block_tables), None, dd(pos), *args,
                                 dtype, max_seq_len=8192)
        torch.testing.assert_close(got2.float().cpu(), want, rtol=rt, atol=at)


def test_row_attention_far_key_stands_out():
    """One pooled block and one far key carry a planted direction: a kernel
    that drops either gives a visibly different row."""
    H, G, d, window, P = 2, 1, 32, 24, 8
    n, block = 400, 16
    E = 2 * G * d
    pg = _Paged([n], E, block, torch.float32, pool_tokens=P, seed=9)
    pg.cache.copy_(_rand(*pg.cache.shape, seed=10, scale=0.1))
    flat = pg.cache.view(-1, E)
    probe = torch.zeros(d)
    probe[3] = 6.0
    # the keys of block 5 (positions 40..47) but its last point along the
    # probe; position 47 is still inside the window of the last query
    for j in range(40, 47):
        flat[pg.slots(0, j, 1)[0], :d] += probe
        flat[pg.slots(0, j, 1)[0], d:] = 1.0
    pos, seq, slots = _step(pg, [(0, 0, n)])
    ref.pool_cache_update(pg.cache, pg.pool, pg.block_tables, seq, pos, slots, P)
    qpos = torch.tensor([n - 1, 47 + window, 46 + window], dtype=torch.int32)
    q = probe.repeat(3, H)
    args = (H, G, 1, d, d, window, P, 1.0, 0.0, 0.0, None, 1.0)
    want = ref.row_attention(q, pg.cache, pg.pool, pg.block_tables,
                             torch.zeros(3, dtype=torch.int32), qpos, *args,
                             torch.float32)
    got = ops.row_attention(q.to(DEV), pg.cache.to(DEV), pg.pool.to(DEV),
                            pg.block_tables.to(DEV),
                            torch.zeros(3, dtype=torch.int32, device=DEV),
                            qpos.to(DEV), *args, torch.float32, max_seq_len=n)
    # block 5 is seen from 47 + window on, and not one position earlier
    assert want[0, :d].mean() > 0.8 and want[1, :d].mean() > 0.8
    assert want[2, :d].mean() < 0.5
    torch.testing.assert_close(got.cpu(), want, rtol=3e-5, atol=3e-5)
