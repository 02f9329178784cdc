"""Parity of every HIP kernel, called through the C ABI, with the CPU oracle.

Same seeded inputs on both sides; bf16 outputs within rtol 1e-2 / atol 1e-2 of the
oracle's (f32 accumulation, one rounding), exact for the data movers and the draw.
"""

import math

import numpy as np
import pytest
import torch

from iron_amd import kernels as K
from iron_amd.bf16 import from_torch, round_bf16, to_torch
from oracle import ops

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-2


def bf(rng, *shape, scale=1.0):
    return round_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale))


def dev(x, cuda):
    return to_torch(x).to(cuda)


def out_like(shape, cuda, fill=None):
    t = torch.empty(shape, dtype=torch.bfloat16, device=cuda)
    if fill is not None:
        t.fill_(fill)
    return t


def word(v, cuda):
    return torch.tensor([v], dtype=torch.int32, device=cuda)


def close(got, want, rtol=RTOL, atol=ATOL, frac=0.0):
    got = from_torch(got).reshape(np.shape(want)) if isinstance(got, torch.Tensor) else got
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bad = ~(err <= atol + rtol * np.abs(want))
    assert bad.mean() <= frac, (
        f"{bad.sum()}/{bad.size} outside rtol {rtol} atol {atol}; max err {np.nanmax(err):.5f} "
        f"at {np.unravel_index(np.nanargmax(err), err.shape)}"
    )


# ------------------------------------------------------------------------ GEMV
@pytest.mark.parametrize("Kdim,N", [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048), (2048, 128256)])
def test_gemv_decode_sweep(cuda, Kdim, N):
    rng = np.random.default_rng(42)
    W, x = bf(rng, N, Kdim, scale=0.02), bf(rng, Kdim)
    y = out_like((N,), cuda)
    K.gemv(dev(W, cuda), dev(x, cuda), y, M=N, K=Kdim)
    close(y, ops.gemv(W, x))


@pytest.mark.parametrize("rpw,ks", [(1, 1), (1, 2), (1, 4), (2, 1), (2, 2), (2, 4), (4, 1), (4, 2), (4, 4), (8, 1)])
def test_gemv_every_launch_shape_and_ragged_rows(cuda, rpw, ks):
    rng = np.random.default_rng(1)
    M, Kdim = 77, 1096  # rows not a multiple of any block, K not a multiple of 512
    W, x = bf(rng, M, Kdim), bf(rng, Kdim)
    y = out_like((M,), cuda)
    K.gemv(dev(W, cuda), dev(x, cuda), y, M=M, K=Kdim, rows_per_wave=rpw, k_split=ks)
    close(y, ops.gemv(W, x), rtol=1e-2, atol=3e-2)


def test_gemv_batches_repeat_and_bound(cuda):
    rng = np.random.default_rng(2)
    # Llama decode's scores shape: 32 heads over 8 groups (gemv.py:51).
    W, x = bf(rng, 8, 256, 64), bf(rng, 32, 64)
    y = out_like((32, 256), cuda)
    K.gemv(dev(W, cuda), dev(x, cuda), y, M=256, K=64, batches=32, repeat=4)
    close(y, ops.gemv(W, x, repeat=4))
    # A bound on the rows: rows past it are left as they were.
    W, x = bf(rng, 300, 128), bf(rng, 128)
    y = out_like((300,), cuda, fill=7.0)
    K.gemv(dev(W, cuda), dev(x, cuda), y, M=300, K=128, valid=word(123, cuda))
    got = from_torch(y)
    close(got[:123], ops.gemv(W, x)[:123])
    assert np.all(got[123:] == 7.0)


# ------------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("b_col_maj", [False, True])
@pytest.mark.parametrize("c_col_maj", [False, True])
def test_gemm_layouts(cuda, b_col_maj, c_col_maj):
    rng = np.random.default_rng(3)
    M, Kdim, N = 384, 512, 640
    A, B = bf(rng, M, Kdim), bf(rng, (N if b_col_maj else Kdim), (Kdim if b_col_maj else N), scale=0.05)
    C = out_like((N, M) if c_col_maj else (M, N), cuda)
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim, b_col_maj=b_col_maj, c_col_maj=c_col_maj)
    want = ops.gemm(A, B, b_col_maj=b_col_maj, c_col_maj=c_col_maj)
    close(C, want)
    # And by the reference's own bound: 2 units of 2^-8 |A|@|B| (gemm.py:704-735).
    bound = ops.gemm_bound(A, B, b_col_maj=b_col_maj, c_col_maj=c_col_maj)
    assert np.all(np.abs(from_torch(C) - want) <= bound)


@pytest.mark.parametrize("b_col_maj", [True, False])
@pytest.mark.parametrize("n", [4096, 8192])
def test_gemm_large_squares_on_sampled_rows(cuda, n, b_col_maj):
    """The 256 x 256-tile kernel at the benchmark's large squares, B as (N, K) and as (K, N): a sample
    of rows (tile edges and random ones) of the product against float64 dot products, and nothing
    left unwritten."""
    rng = np.random.default_rng(n)
    A, B = bf(rng, n, n, scale=0.02), bf(rng, n, n, scale=0.02)   # B is (N, K) or (K, N) as the flag says
    C = out_like((n, n), cuda, fill=float("nan"))
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=n, N=n, K=n, b_col_maj=b_col_maj)
    got = from_torch(C)
    assert not np.isnan(got).any()
    rows = sorted({0, 1, 127, 128, 255, 256, 257, n // 2 - 1, n // 2, n - 256, n - 1, *rng.integers(0, n, 21).tolist()})
    Bd = B.astype(np.float64)
    want = round_bf16((A[rows].astype(np.float64) @ (Bd.T if b_col_maj else Bd)).astype(np.float32))
    close(got[rows], want, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("M,Kdim,N", [(2048, 192, 6144), (4096, 64, 3072), (3072, 1152, 4096)])
def test_gemm_large_tiles_with_b_as_stored_by_default(cuda, M, Kdim, N):
    """B (K, N) through the 256 x 256 tiles (192 whole tiles or more): one stage, three, and
    eighteen of them, every element against the oracle."""
    rng = np.random.default_rng(M + N + Kdim)
    A, B = bf(rng, M, Kdim), bf(rng, Kdim, N)
    C = out_like((M, N), cuda, fill=float("nan"))
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim)
    close(C, ops.gemm(A, B))


def test_gemm_headline_shape(cuda):
    rng = np.random.default_rng(4)
    A, B = bf(rng, 2048, 2048, scale=0.02), bf(rng, 2048, 2048, scale=0.02)
    C = out_like((2048, 2048), cuda)
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=2048, N=2048, K=2048)
    close(C, ops.gemm(A, B), rtol=1e-2, atol=1e-3)
    Bt = np.ascontiguousarray(B.T)
    K.gemm(dev(A, cuda), dev(Bt, cuda), C, M=2048, N=2048, K=2048, b_col_maj=True)
    close(C, ops.gemm(A, B), rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("M,Kdim,N", [(100, 136, 72), (32, 1152, 2048), (1, 64, 8), (130, 8, 264), (2048, 2048, 512), (192, 8192, 128)])
@pytest.mark.parametrize("b_col_maj", [False, True])
def test_gemm_ragged_shapes(cuda, M, Kdim, N, b_col_maj):
    rng = np.random.default_rng(5)
    A, B = bf(rng, M, Kdim), bf(rng, (N if b_col_maj else Kdim), (Kdim if b_col_maj else N), scale=0.1)
    C = out_like((M, N), cuda)
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim, b_col_maj=b_col_maj)
    close(C, ops.gemm(A, B, b_col_maj=b_col_maj), rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("M,Kdim,N,rows", [(2048, 512, 8192, None), (2048, 64, 6144, None), (4096, 192, 4096, 1000), (4096, 192, 4096, 3000), (2048, 128, 2048, 512), (2048, 128, 2048, 1500), (2048, 192, 512, 700),
                                           (128, 64, 128, None), (256, 128, 192, None)])
def test_gemm_weight_layout_fast_paths(cuda, M, Kdim, N, rows):
    """B (N,K): the 256x256-tile kernel (>= 192 whole tiles) and the 128x128 one, down to a single
    k stage, with a row bound that cuts through a tile."""
    rng = np.random.default_rng(55)
    A, B = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.1)
    want = ops.gemm(A, B, b_col_maj=True)
    if rows is not None:
        A[rows:] = np.nan
    C = out_like((M, N), cuda, fill=5.0)
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim, b_col_maj=True,
           valid=None if rows is None else word(rows, cuda))
    got = from_torch(C)
    lim = M if rows is None else rows
    close(got[:lim], want[:lim], rtol=1e-2, atol=2e-2)
    assert np.all(got[lim:] == 5.0)


@pytest.mark.parametrize("M,Kdim,N", [(130, 128, 264), (200, 192, 136), (1000, 256, 1000), (65, 64, 65), (2047, 320, 2050), (333, 128, 384)])
@pytest.mark.parametrize("b_col_maj", [False, True])
def test_gemm_direct_to_lds_tiles_at_ragged_edges(cuda, M, Kdim, N, b_col_maj):
    """K a multiple of 64 takes the direct-to-LDS tiles whatever M and N are: rows and columns past
    the edge are clamped on the way in and never stored, and nothing beyond C is touched."""
    if not b_col_maj:
        N = (N + 7) // 8 * 8   # B as (K,N) is loaded 16 bytes along N
    rng = np.random.default_rng(M * 7 + N)
    A, B = bf(rng, M, Kdim), bf(rng, (N if b_col_maj else Kdim), (Kdim if b_col_maj else N), scale=0.1)
    guard = 64
    C = out_like((M * N + guard,), cuda, fill=3.0)
    K.gemm(dev(A, cuda), dev(B, cuda), C[: M * N].view(M, N), M=M, N=N, K=Kdim, b_col_maj=b_col_maj)
    got = from_torch(C)
    close(got[: M * N].reshape(M, N), ops.gemm(A, B, b_col_maj=b_col_maj), rtol=1e-2, atol=2e-2)
    assert np.all(got[M * N:] == 3.0)


@pytest.mark.parametrize("M,Kdim,N,rows", [
    # 64 x 64 tiles, eight stages (no more tiles than CUs): fewer k-stages than the pipeline is deep, an odd count, many
    (512, 64, 2048, None), (512, 192, 2048, None), (512, 576, 2048, None), (448, 1024, 1024, None),
    # 64 x 64 tiles, four stages (more tiles than CUs, too few for 128 x 128 ones): one stage, odd, even
    (1024, 64, 1536, None), (1024, 320, 1536, None), (1024, 512, 1536, 1000),
    # a row bound under which the blocks of one launch pick 64 x 64 tiles, short and odd in k
    (2048, 64, 2048, 512), (2048, 192, 2048, 300), (2048, 576, 2048, 896), (2048, 576, 2048, 897)])
@pytest.mark.parametrize("residual", [False, True])
def test_gemm_small_tiles_at_every_depth(cuda, M, Kdim, N, rows, residual):
    """The whole-stage-ahead pipelines of the 64 x 64 tiles where they start and end: K of one stage,
    fewer stages than are in flight, odd and even counts, with and without the residual epilogue."""
    rng = np.random.default_rng(M + Kdim + N)
    A, B, R = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.1), bf(rng, M, N)
    want = ops.gemm(A, B, b_col_maj=True)
    if residual:
        want = round_bf16(np.float32(0.5) * want + R)
    lim = M if rows is None else rows
    if rows is not None:
        A[rows:] = np.nan
    C = out_like((M, N), cuda, fill=5.0)
    bound = None if rows is None else word(rows, cuda)
    if residual:
        K.gemm_residual(dev(A, cuda), dev(B, cuda), dev(R, cuda), C, M=M, N=N, K=Kdim, residual_scale=0.5, valid=bound)
    else:
        K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim, b_col_maj=True, valid=bound)
    got = from_torch(C)
    close(got[:lim], want[:lim], rtol=1e-2, atol=2e-2)
    assert np.all(got[lim:] == 5.0)


@pytest.mark.parametrize("rows,bound,H,G", [(2048, None, 32, 8), (256, 150, 16, 4), (128, None, 2, 2),
                                            # bounds on either side of where the 192-wide tiles take over
                                            (2048, 1280, 32, 8), (2048, 1281, 32, 8), (2048, 1999, 32, 8),
                                            (2048, 2048, 32, 8), (2048, 70, 32, 8),
                                            # heads that do not come in threes keep the 128-wide tiles
                                            (2048, None, 32, 4), (1024, None, 8, 2), (4096, 3000, 16, 4)])
def test_prefill_qkv_equals_three_projections_then_rope(cuda, rows, bound, H, G):
    """The fused launch against the oracle's separate steps: project and round, rotate and round."""
    rng = np.random.default_rng(91)
    E, D = 512, 64
    x = bf(rng, rows, E)
    Wq, Wk, Wv = bf(rng, H * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05)
    table = round_bf16(ops.rope_angles(D, rows + 5, 500000.0))[5:]
    lim = rows if bound is None else bound
    q, k, v = (ops.gemm(x, W, b_col_maj=True) for W in (Wq, Wk, Wv))
    want_q = ops.rope(q.reshape(rows * H, D), table).reshape(rows, H * D)
    want_k = ops.rope(k.reshape(rows * G, D), table).reshape(rows, G * D)
    if bound is not None:
        x[bound:] = np.nan
    outs = [out_like((rows, n), cuda, fill=7.0) for n in (H * D, G * D, G * D)]
    K.prefill_qkv(dev(x, cuda), dev(Wq, cuda), dev(Wk, cuda), dev(Wv, cuda), dev(table, cuda), *outs, rows=rows,
                  hidden=E, heads=H, kv_heads=G, d=D, valid=None if bound is None else word(bound, cuda))
    for got, want in zip(outs, (want_q, want_k, v)):
        got = from_torch(got)
        close(got[:lim], want[:lim], rtol=1e-2, atol=1e-2)
        assert np.all(got[lim:] == 7.0)


@pytest.mark.parametrize("E", [64, 192, 320])
@pytest.mark.parametrize("rows,bound", [(512, None), (2048, 600)])
def test_prefill_qkv_one_head_tiles_at_short_hidden(cuda, E, rows, bound):
    """The one-head tiles a short chunk takes (whole-stage-ahead pipeline, five stages) with fewer
    k-stages than are in flight and an odd count of them."""
    rng = np.random.default_rng(E + rows)
    H, G, D = 32, 8, 64
    x = bf(rng, rows, E)
    Wq, Wk, Wv = bf(rng, H * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05)
    table = round_bf16(ops.rope_angles(D, rows, 500000.0))
    lim = rows if bound is None else bound
    q, k, v = (ops.gemm(x, W, b_col_maj=True) for W in (Wq, Wk, Wv))
    want_q = ops.rope(q.reshape(rows * H, D), table).reshape(rows, H * D)
    want_k = ops.rope(k.reshape(rows * G, D), table).reshape(rows, G * D)
    if bound is not None:
        x[bound:] = np.nan
    outs = [out_like((rows, n), cuda, fill=7.0) for n in (H * D, G * D, G * D)]
    K.prefill_qkv(dev(x, cuda), dev(Wq, cuda), dev(Wk, cuda), dev(Wv, cuda), dev(table, cuda), *outs, rows=rows,
                  hidden=E, heads=H, kv_heads=G, d=D, valid=None if bound is None else word(bound, cuda))
    for got, want in zip(outs, (want_q, want_k, v)):
        got = from_torch(got)
        close(got[:lim], want[:lim], rtol=1e-2, atol=1e-2)
        assert np.all(got[lim:] == 7.0)


@pytest.mark.parametrize("rows,bound,start,L,H,G", [(256, 150, 300, 1024, 16, 4), (2048, 512, 0, 2048, 32, 8),
                                                    (2048, 1500, 548, 2048, 32, 8), (128, None, 128, 256, 2, 2),
                                                    (256, 64, 960, 1024, 6, 2)])
def test_prefill_qkv_writes_k_and_v_into_the_cache_rows(cuda, rows, bound, start, L, H, G):
    """k and v land in rows start .. start + bound of the caches, bit for bit what the launch with
    outputs of its own writes; every other cache row is left as it was."""
    rng = np.random.default_rng(92)
    E, D = 512, 64
    x = bf(rng, rows, E)
    Wq, Wk, Wv = bf(rng, H * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05), bf(rng, G * D, E, scale=0.05)
    table = round_bf16(ops.rope_angles(D, rows, 500000.0))
    lim = rows if bound is None else bound
    if bound is not None:
        x[bound:] = np.nan
    valid = None if bound is None else word(bound, cuda)
    args = [dev(a, cuda) for a in (x, Wq, Wk, Wv, table)]
    outs = [out_like((rows, n), cuda, fill=7.0) for n in (H * D, G * D, G * D)]
    K.prefill_qkv(*args, *outs, rows=rows, hidden=E, heads=H, kv_heads=G, d=D, valid=valid)
    q = out_like((rows, H * D), cuda, fill=7.0)
    keys, values = (out_like((L, G * D), cuda, fill=3.0) for _ in range(2))
    K.prefill_qkv_cache(*args, q, keys, values, rows=rows, hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                        start=word(start, cuda), valid=valid)
    assert torch.equal(q, outs[0])
    for cache, own in ((keys, outs[1]), (values, outs[2])):
        assert torch.equal(cache[start : start + lim], own[:lim])
        assert bool((cache[:start] == 3.0).all()) and bool((cache[start + lim :] == 3.0).all())
    # A first row whose rows would end past the cache is held inside it.
    K.prefill_qkv_cache(*args, q, keys, values, rows=rows, hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                        start=word(L, cuda), valid=valid)
    assert torch.equal(keys[L - lim :], outs[1][:lim])


@pytest.mark.parametrize("M,Kdim,N,rows,scale", [(2048, 512, 2048, None, 1.0), (2048, 256, 2048, 512, 1.0),
                                                 (2048, 256, 2048, 1500, 0.22), (256, 128, 512, 100, 1.0),
                                                 (128, 64, 64, None, -0.5), (4096, 192, 1024, 3000, 1.0)])
def test_gemm_residual_epilogue(cuda, M, Kdim, N, rows, scale):
    """A projection over many rows with its residual in the epilogue: the product rounded as the
    separate step would store it, then one fused multiply-add with the residual (the sum, or AXPY)."""
    rng = np.random.default_rng(M + N)
    A, B, R = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.05), bf(rng, M, N)
    lim = M if rows is None else rows
    want = ops.axpy(scale, ops.gemm(A, B, b_col_maj=True), R)
    if scale == 1.0:
        assert np.array_equal(want, ops.add(ops.gemm(A, B, b_col_maj=True), R))
    if rows is not None:
        A[rows:] = np.nan
    C = out_like((M, N), cuda, fill=7.0)
    K.gemm_residual(dev(A, cuda), dev(B, cuda), dev(R, cuda), C, M=M, N=N, K=Kdim, residual_scale=scale,
                    valid=None if rows is None else word(rows, cuda))
    got = from_torch(C)
    close(got[:lim], want[:lim], rtol=1e-2, atol=1e-2)
    assert np.all(got[lim:] == 7.0)
    # in place: the residual stream is its own output
    Rd = dev(R, cuda)
    K.gemm_residual(dev(np.nan_to_num(A), cuda), dev(B, cuda), Rd, Rd, M=M, N=N, K=Kdim, residual_scale=scale,
                    valid=None if rows is None else word(rows, cuda))
    close(from_torch(Rd)[:lim], want[:lim], rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M,Kdim,N,rows,scale", [
    (2048, 8192, 2048, 512, 1.0),     # a prompt chunk's down projection: K dealt four ways, a slice an XCD pair
    (2048, 4096, 2048, 1024, 1.0),    # two ways
    (2048, 4096, 2048, 1281, 0.22),   # whole K: the first launch is the plain residual product's
    (512, 4096, 2048, None, 1.0),
    (256, 4096, 128, 130, 1.0),       # one tile column, a tile row the bound cuts
    (384, 4096, 384, 300, -0.5),      # pairs that do not fill whole XCD rounds
    (256, 4096, 4096, 77, 1.0),       # two pieces of a row a thread
    (128, 4608, 8192, None, 1.0)])    # four
def test_gemm_residual_then_rmsnorm_with_k_dealt_over_blocks(cuda, M, Kdim, N, rows, scale):
    """A residual product of few rows over a long K and the norm of its rows as two launches: the
    product's K dealt over several blocks a tile (float32 sums through a workspace holding garbage),
    the rows finished and normed by the second.  C against the oracle's product and sum; Y is the
    norm kernel's of that C bit for bit, and within tolerance of the oracle's norm of it; rows past
    the bound are not touched; in place on the residual stream."""
    rng = np.random.default_rng(M + N + Kdim)
    lim = M if rows is None else rows
    A, B, R, gain = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.02), bf(rng, M, N), bf(rng, N)
    product = ops.gemm(A[:lim], B, b_col_maj=True)
    want = ops.axpy(scale, product, R[:lim])
    # The product is rounded before the sum: where the float32 sums differ in their last bits it may
    # round to the neighbouring bf16 (2^-7 of it at most), whatever the sum then cancels to.
    ulp = np.abs(scale * product) * 2.0 ** -7

    def near(got, want):
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        bad = ~(err <= 1e-2 + 1e-2 * np.abs(want) + ulp)
        assert not bad.any(), f"{bad.sum()}/{bad.size} outside the tolerance; max err {err.max():.5f}"

    if rows is not None:
        A[rows:] = np.nan
    valid = None if rows is None else word(rows, cuda)
    need = K.gemm_residual_norm_workspace_bytes(M, N, Kdim)
    assert need > 0
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device=cuda)
    Ad, Bd, Rd, gd = dev(A, cuda), dev(B, cuda), dev(R, cuda), dev(gain, cuda)
    C, Y = out_like((M, N), cuda, fill=7.0), out_like((M, N), cuda, fill=7.0)
    K.gemm_residual_norm(Ad, Bd, Rd, gd, C, Y, ws, M=M, N=N, K=Kdim, eps=1e-6, residual_scale=scale, valid=valid)
    got = from_torch(C)
    near(got[:lim], want)
    assert np.all(got[lim:] == 7.0) and bool((Y[lim:] == 7.0).all())
    normed = out_like((M, N), cuda, fill=7.0)
    K.rmsnorm(C, gd, normed, rows=M, cols=N, eps=1e-6, valid=valid)
    assert torch.equal(Y[:lim], normed[:lim])
    close(from_torch(Y)[:lim], ops.rms_norm(got[:lim], gain, epsilon=1e-6), rtol=1e-2, atol=1e-2)
    # again over the workspace the first call left, in place on the residual stream: the same bits
    Y2 = out_like((M, N), cuda, fill=7.0)
    K.gemm_residual_norm(Ad, Bd, Rd, gd, Rd, Y2, ws, M=M, N=N, K=Kdim, eps=1e-6, residual_scale=scale, valid=valid)
    assert torch.equal(Rd[:lim], C[:lim]) and torch.equal(Y2[:lim], Y[:lim])
    assert np.array_equal(from_torch(Rd)[lim:], R[lim:])


def test_gemm_residual_then_rmsnorm_refuses_other_shapes(cuda):
    """Shapes whose K is too short to deal, or whose rows the second launch cannot hold, report no
    workspace and are refused with a reason before any launch."""
    for M, N, Kdim in ((64, 2048, 8192), (512, 2048, 2048), (512, 2000, 8192), (512, 16384, 8192), (512, 2048, 8192 + 64)):
        assert K.gemm_residual_norm_workspace_bytes(M, N, Kdim) == 0
    t, w = out_like((512 * 2048,), cuda, fill=0.0), out_like((2048 * 2048,), cuda, fill=0.0)
    with pytest.raises(Exception, match="iron_gemm_residual_norm_bf16 refused"):
        K.gemm_residual_norm(t, w, t, t[:2048], t, out_like((512 * 2048,), cuda), torch.empty(16, device=cuda),
                             M=512, N=2048, K=2048, eps=1e-6)


@pytest.mark.parametrize("M,Kdim,N,rows,activation", [
    (2048, 2048, 8192, 512, "silu"), (2048, 256, 8192, None, "silu"), (2048, 256, 2048, 1500, "silu"),
    (256, 128, 512, 100, "silu"), (128, 64, 64, None, "silu"), (4096, 192, 1024, 3000, "silu"), (200, 128, 136, None, "silu"),
    (2048, 256, 8192, 512, "gelu_tanh"), (256, 128, 512, 100, "gelu_tanh"), (200, 128, 136, None, "gelu_tanh")])
def test_gemm_gated_epilogue(cuda, M, Kdim, N, rows, activation):
    """A gated feed-forward's second projection over many rows with the activated gate (SiLU, or
    GELU by its tanh form) in its epilogue.  The chain rounds twice (the product, then the gated
    product), so it is checked link by link: the product of the separate launch against the oracle's
    GEMM, the fused launch against the oracle's activation and ElementwiseMul of that product, and
    bit for bit against this library's own separate launches.  The first case is Llama-3.2-1B's
    prompt chunk."""
    rng = np.random.default_rng(M + N + 1)
    A, B, G = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.05), bf(rng, M, N, scale=2.0)
    lim = M if rows is None else rows
    product = ops.gemm(A[:lim], B, b_col_maj=True)
    if rows is not None:
        A[rows:] = np.nan
    bound = None if rows is None else word(rows, cuda)
    flat_bound = None if rows is None else word(rows * N, cuda)
    # the separate launches: the product, then the activation and the multiplication
    U, Y = out_like((M, N), cuda, fill=7.0), out_like((M, N), cuda, fill=7.0)
    K.gemm(dev(A, cuda), dev(B, cuda), U, M=M, N=N, K=Kdim, b_col_maj=True, valid=bound)
    if activation == "silu":
        K.silu_mul(dev(G, cuda).reshape(-1), U.reshape(-1), Y.reshape(-1), n=M * N, valid=flat_bound)
        activated = ops.silu(G[:lim])
    else:
        act = out_like((M, N), cuda, fill=7.0)
        K.unary(dev(G, cuda).reshape(-1), act.reshape(-1), "gelu_tanh", n=M * N, valid=flat_bound)
        K.mul(act.reshape(-1), U.reshape(-1), Y.reshape(-1), n=M * N, valid=flat_bound)
        activated = ops.gelu(G[:lim], approximate="tanh")
    close(U[:lim], product, rtol=1e-2, atol=1e-2)
    C = out_like((M, N), cuda, fill=7.0)
    K.gemm_gated(dev(A, cuda), dev(B, cuda), dev(G, cuda), C, M=M, N=N, K=Kdim, activation=activation, valid=bound)
    got = from_torch(C)
    close(got[:lim], ops.mul(activated, from_torch(U)[:lim]), rtol=1e-2, atol=1e-2)
    assert np.all(got[lim:] == 7.0)
    assert torch.equal(Y[:lim], C[:lim])
    # in place: the gate's product is its own output
    Gd = dev(G, cuda)
    K.gemm_gated(dev(np.nan_to_num(A), cuda), dev(B, cuda), Gd, Gd, M=M, N=N, K=Kdim, activation=activation, valid=bound)
    assert torch.equal(Gd[:lim], C[:lim])


@pytest.mark.parametrize("M,Kdim,N,rows", [(2048, 2048, 8192, 512), (2048, 2048, 8192, 1281), (2048, 2048, 8192, 100),
                                           (256, 512, 1024, None), (192, 128, 320, 70)])
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_gemm_gated_pair_is_the_two_launches_bit_for_bit(cuda, M, Kdim, N, rows, activation):
    """Both first projections of a gated feed-forward in one launch: the gate's product and the gated
    output against the two launches they replace (the gate's GEMM, then the gated GEMM) bit for bit --
    under row bounds that pick the 128 x 128 tiles, the 64 x 64 ones and neither whole -- and the gate's
    product against the oracle's GEMM; rows past the bound are left as they were.  The first case is
    Llama-3.2-1B's prompt chunk."""
    rng = np.random.default_rng(M + N + 3)
    A, Bg, Bu = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.05), bf(rng, N, Kdim, scale=0.05)
    lim = M if rows is None else rows
    if rows is not None:
        A[rows:] = np.nan
    bound = None if rows is None else word(rows, cuda)
    dA, dBg, dBu = dev(A, cuda), dev(Bg, cuda), dev(Bu, cuda)
    G2, C2 = out_like((M, N), cuda, fill=7.0), out_like((M, N), cuda, fill=7.0)
    K.gemm(dA, dBg, G2, M=M, N=N, K=Kdim, b_col_maj=True, valid=bound)
    K.gemm_gated(dA, dBu, G2, C2, M=M, N=N, K=Kdim, activation=activation, valid=bound)
    G1, C1 = out_like((M, N), cuda, fill=7.0), out_like((M, N), cuda, fill=7.0)
    K.gemm_gated_pair(dA, dBg, dBu, G1, C1, M=M, N=N, K=Kdim, activation=activation, valid=bound)
    close(G1[:lim], ops.gemm(A[:lim], Bg, b_col_maj=True), rtol=1e-2, atol=1e-2)
    assert torch.equal(G1[:lim], G2[:lim]) and torch.equal(C1[:lim], C2[:lim])
    assert np.all(from_torch(C1)[lim:] == 7.0) and np.all(from_torch(G1)[lim:] == 7.0)


@pytest.mark.parametrize("bound", [None, 512, 1281])
@pytest.mark.parametrize("cache", [False, True])
def test_prefill_qkv_at_the_decoder_s_width(cuda, bound, cache):
    """The fused pre-attention launch at Llama-3.2-1B's own sizes: a 2048-row chunk of hidden 2048,
    32 query and 8 KV heads, whole and under the bounds a prompt leaves (512 rows: the one-head
    tiles; 1281: the 192-wide ones), against the oracle's three GEMMs, then RoPE."""
    rng = np.random.default_rng(93)
    rows, E, H, G, D, L, start = 2048, 2048, 32, 8, 64, 4096, 777
    x = bf(rng, rows, E)
    Wq, Wk, Wv = bf(rng, H * D, E, scale=0.02), bf(rng, G * D, E, scale=0.02), bf(rng, G * D, E, scale=0.02)
    table = round_bf16(ops.rope_angles(D, rows, 500000.0))
    lim = rows if bound is None else bound
    q, k, v = (ops.gemm(x[:lim], W, b_col_maj=True) for W in (Wq, Wk, Wv))
    want_q = ops.rope(q.reshape(lim * H, D), table[:lim]).reshape(lim, H * D)
    want_k = ops.rope(k.reshape(lim * G, D), table[:lim]).reshape(lim, G * D)
    if bound is not None:
        x[bound:] = np.nan
    valid = None if bound is None else word(bound, cuda)
    args = [dev(a, cuda) for a in (x, Wq, Wk, Wv, table)]
    q_out = out_like((rows, H * D), cuda, fill=7.0)
    if cache:
        keys, values = (out_like((L, G * D), cuda, fill=3.0) for _ in range(2))
        K.prefill_qkv_cache(*args, q_out, keys, values, rows=rows, hidden=E, heads=H, kv_heads=G, d=D,
                            cache_rows=L, start=word(start, cuda), valid=valid)
        k_got, v_got = from_torch(keys), from_torch(values)
        for got in (k_got, v_got):
            assert np.all(got[:start] == 3.0) and np.all(got[start + lim :] == 3.0)
        k_got, v_got = k_got[start : start + lim], v_got[start : start + lim]
    else:
        k_out, v_out = (out_like((rows, G * D), cuda, fill=7.0) for _ in range(2))
        K.prefill_qkv(*args, q_out, k_out, v_out, rows=rows, hidden=E, heads=H, kv_heads=G, d=D, valid=valid)
        k_got, v_got = from_torch(k_out), from_torch(v_out)
        assert np.all(k_got[lim:] == 7.0) and np.all(v_got[lim:] == 7.0)
        k_got, v_got = k_got[:lim], v_got[:lim]
    q_got = from_torch(q_out)
    assert np.all(q_got[lim:] == 7.0)
    close(q_got[:lim], want_q)
    close(k_got, want_k)
    close(v_got, v)


@pytest.mark.parametrize("M,Kdim,N", [(2048, 2048, 8192), (2048, 8192, 2048), (2048, 2048, 2048), (2048, 2048, 512)])
@pytest.mark.parametrize("rows", [512, 1281])
def test_prompt_chunk_projections_under_a_row_bound(cuda, M, Kdim, N, rows):
    """The launches a bounded prompt chunk takes at Llama-3.2-1B's widths (blocks choosing their tile
    by the bound, the ranges of the bound served by two launches): the plain product and the one
    with its residual, at the full depth of K, poison past the bound, nothing written past it."""
    rng = np.random.default_rng(M + Kdim + N + rows)
    A, B, R = bf(rng, M, Kdim), bf(rng, N, Kdim, scale=0.02), bf(rng, M, N)
    want = ops.gemm(A[:rows], B, b_col_maj=True)
    A[rows:] = np.nan
    C = out_like((M, N), cuda, fill=5.0)
    K.gemm(dev(A, cuda), dev(B, cuda), C, M=M, N=N, K=Kdim, b_col_maj=True, valid=word(rows, cuda))
    got = from_torch(C)
    close(got[:rows], want)
    assert np.all(got[rows:] == 5.0)
    Rd = dev(R, cuda)
    K.gemm_residual(dev(A, cuda), dev(B, cuda), Rd, Rd, M=M, N=N, K=Kdim, residual_scale=1.0, valid=word(rows, cuda))
    got = from_torch(Rd)
    # The product is rounded to bf16 before the sum, as the separate step stores it: where float32
    # sums in another order round it the other way, the sum moves by the PRODUCT's last place,
    # however small the sum itself comes out.
    total = ops.add(want, R[:rows])
    assert np.all(np.abs(got[:rows] - total) <= ATOL + RTOL * np.abs(total) + 2.0**-7 * np.abs(want))
    assert np.array_equal(got[rows:], R[rows:])


@pytest.mark.parametrize("b_col_maj", [False, True])
def test_gemm_bounded_rows_and_k_do_not_read_the_poison(cuda, b_col_maj):
    """NaN past the bounds must not reach the output (test_gemm_bounded_k.py)."""
    rng = np.random.default_rng(6)
    M, Kdim, N, rows, kv = 256, 512, 128, 150, 332
    A, B = bf(rng, M, Kdim), bf(rng, Kdim, N, scale=0.1)
    want = ops.gemm(A, B, valid_k=kv)
    A[:, kv:], B[kv:], A[rows:] = np.nan, np.nan, np.nan
    Bs = np.ascontiguousarray(B.T) if b_col_maj else B
    C = out_like((M, N), cuda, fill=5.0)
    K.gemm(dev(A, cuda), dev(Bs, cuda), C, M=M, N=N, K=Kdim, b_col_maj=b_col_maj,
           valid=word(rows, cuda), valid_k=word(kv, cuda))
    got = from_torch(C)
    close(got[:rows], want[:rows], rtol=1e-2, atol=2e-2)
    assert np.all(got[rows:] == 5.0)


@pytest.mark.parametrize("rows,cols", [(1, 2048), (8, 512), (2048, 512), (64, 5120), (7, 12288)])
@pytest.mark.parametrize("multiply", [False, True])
def test_row_broadcast_exact(cuda, rows, cols, multiply):
    rng = np.random.default_rng(70)
    x, row = bf(rng, rows, cols), bf(rng, cols)
    y = out_like((rows, cols), cuda, fill=3.0)
    bound = max(1, rows - 3)
    K.row_broadcast(dev(x, cuda), dev(row, cuda), y, rows=rows, cols=cols, multiply=multiply, valid=word(bound, cuda))
    want = (ops.mul if multiply else ops.add)(x, np.broadcast_to(row, x.shape))
    got = from_torch(y)
    assert np.array_equal(got[:bound], want[:bound])
    assert np.all(got[bound:] == 3.0)


# --------------------------------------------------------------------- rowwise
@pytest.mark.parametrize("rows,cols", [(1, 2048), (2048, 2048), (7, 64), (3, 8192), (2, 16640)])
@pytest.mark.parametrize("weighted", [False, True])
def test_rmsnorm(cuda, rows, cols, weighted):
    rng = np.random.default_rng(7)
    x = bf(rng, rows, cols)
    w = round_bf16(rng.uniform(0.9, 1.1, cols)) if weighted else None
    y = out_like((rows, cols), cuda)
    K.rmsnorm(dev(x, cuda), None if w is None else dev(w, cuda), y, rows=rows, cols=cols, eps=1e-5)
    close(y, ops.rms_norm(x, w, epsilon=1e-5))


def test_rmsnorm_bound(cuda):
    rng = np.random.default_rng(8)
    x = bf(rng, 16, 256)
    y = out_like((16, 256), cuda, fill=3.0)
    K.rmsnorm(dev(x, cuda), None, y, rows=16, cols=256, eps=1e-5, valid=word(5, cuda))
    got = from_torch(y)
    close(got[:5], ops.rms_norm(x[:5]))
    assert np.all(got[5:] == 3.0)


@pytest.mark.parametrize("rows,row,cols,angle_rows,halves", [(64, 128, 32, 2, True), (32, 64, 32, 1, True), (96, 256, 64, 96, True),
                                                             (40, 80, 16, 5, False), (2048 * 8, 64, 32, 2048, True)])
def test_rope_over_the_first_columns_of_each_row(cuda, rows, row, cols, angle_rows, halves):
    """Partial rotary: the first ``cols`` columns of a ``row``-wide row turn exactly as a row of that
    width would, the rest come through bit for bit; rows past a bound are left alone."""
    rng = np.random.default_rng(rows + row)
    x = bf(rng, rows, row)
    table = round_bf16(ops.rope_angles(cols, angle_rows + 3, 10000.0))[3:]
    bound = rows - rows // 3
    y = out_like((rows, row), cuda, fill=9.0)
    K.rope(dev(x, cuda), dev(table, cuda), y, rows=rows, cols=cols, angle_rows=angle_rows, two_halves=halves,
           valid=word(bound, cuda), row_cols=row)
    got = from_torch(y)
    want = ops.rope(x[:, :cols], table, two_halves=halves)
    close(got[:bound, :cols], want[:bound])
    assert np.array_equal(got[:bound, cols:], x[:bound, cols:]) and np.all(got[bound:] == 9.0)
    # ... and the turned columns are the bits the whole-row launch gives a row of that width
    narrow = out_like((rows, cols), cuda)
    K.rope(dev(np.ascontiguousarray(x[:, :cols]), cuda), dev(table, cuda), narrow, rows=rows, cols=cols,
           angle_rows=angle_rows, two_halves=halves)
    assert np.array_equal(got[:bound, :cols], from_torch(narrow)[:bound])


@pytest.mark.parametrize("rows,cols,weighted,bound", [(1, 2048, True, None), (64, 512, True, 40), (7, 8192, False, None)])
def test_rmsnorm_with_its_residual(cuda, rows, cols, weighted, bound):
    """The normed rows added to a residual in the norm's own pass: bit for bit the norm launch
    followed by the sum (each rounds where the other does), in place too; rows past a bound keep theirs."""
    rng = np.random.default_rng(9)
    x, r = bf(rng, rows, cols), bf(rng, rows, cols)
    w = dev(round_bf16(rng.uniform(0.9, 1.1, cols)), cuda) if weighted else None
    valid = None if bound is None else word(bound, cuda)
    lim = rows if bound is None else bound
    normed, summed = out_like((rows, cols), cuda), out_like((rows, cols), cuda, fill=3.0)
    K.rmsnorm(dev(x, cuda), w, normed, rows=rows, cols=cols, eps=1e-6)
    K.add(dev(r, cuda).reshape(-1), normed.reshape(-1), summed.reshape(-1), n=rows * cols,
          valid=None if bound is None else word(bound * cols, cuda))
    once = out_like((rows, cols), cuda, fill=3.0)
    K.rmsnorm(dev(x, cuda), w, once, rows=rows, cols=cols, eps=1e-6, valid=valid, residual=dev(r, cuda))
    assert torch.equal(once, summed)
    close(from_torch(once)[:lim], ops.add(r, ops.rms_norm(x, None if w is None else from_torch(w), epsilon=1e-6))[:lim])
    stream = dev(r, cuda)
    K.rmsnorm(dev(x, cuda), w, stream, rows=rows, cols=cols, eps=1e-6, valid=valid, residual=stream)
    assert torch.equal(stream[:lim], summed[:lim]) and np.array_equal(from_torch(stream)[lim:], r[lim:])


def angle_table(rng, angle_rows, cols):
    theta = rng.uniform(-np.pi, np.pi, (angle_rows, cols // 2))
    table = np.empty((angle_rows, cols), np.float32)
    table[:, ::2], table[:, 1::2] = np.cos(theta), np.sin(theta)
    return round_bf16(table)


@pytest.mark.parametrize("rows,cols,angle_rows", [(8, 32, 2), (1024, 32, 1), (13, 32, 13), (12, 32, 4),
                                                  (32, 64, 1), (8, 64, 1), (2048 * 32, 64, 2048),
                                                  (32, 512, 8), (64, 128, 16)])
@pytest.mark.parametrize("two_halves", [True, False])
def test_rope(cuda, rows, cols, angle_rows, two_halves):
    rng = np.random.default_rng(0)
    x, ang = bf(rng, rows, cols), angle_table(rng, angle_rows, cols)
    y = out_like((rows, cols), cuda)
    K.rope(dev(x, cuda), dev(ang, cuda), y, rows=rows, cols=cols, angle_rows=angle_rows, two_halves=two_halves)
    want = ops.rope(x, ang, two_halves=two_halves)
    got = from_torch(y)
    close(got, want)
    # Same f32 formula, one rounding: all but fused-multiply-add ties agree bit for bit.
    assert (got != want).mean() < 0.02


def test_rope_bound(cuda):
    rng = np.random.default_rng(1)
    x, ang = bf(rng, 64 * 4, 64), angle_table(rng, 64, 64)
    y = out_like((256, 64), cuda, fill=9.0)
    K.rope(dev(x, cuda), dev(ang, cuda), y, rows=256, cols=64, angle_rows=64, valid=word(40, cuda))
    got = from_torch(y)
    close(got[:40], ops.rope(x, ang)[:40])
    assert np.all(got[40:] == 9.0)


@pytest.mark.parametrize("n", [8192, 2048, 1003, 5, 2048 * 8192])
def test_elementwise(cuda, n):
    rng = np.random.default_rng(9)
    a, b = bf(rng, n, scale=3), bf(rng, n, scale=3)
    da, db = dev(a, cuda), dev(b, cuda)
    y = out_like((n,), cuda)
    K.add(da, db, y)
    assert np.array_equal(from_torch(y), ops.add(a, b))  # bit-exact (test_elementwise.py:125-132)
    K.mul(da, db, y)
    assert np.array_equal(from_torch(y), ops.mul(a, b))
    K.silu(da, y)
    close(y, ops.silu(a))
    K.silu_mul(da, db, y)
    close(y, ops.mul(ops.silu(a), b), atol=2e-2)


def test_elementwise_bound(cuda):
    rng = np.random.default_rng(10)
    a, b = bf(rng, 4096), bf(rng, 4096)
    y = out_like((4096,), cuda, fill=2.0)
    K.add(dev(a, cuda), dev(b, cuda), y, valid=word(1001, cuda))
    got = from_torch(y)
    assert np.array_equal(got[:1001], ops.add(a, b)[:1001]) and np.all(got[1001:] == 2.0)


# ------------------------------------------------------------------- attention
def run_prefill(cuda, Q, Kc, Vc, *, H, G, d, seq, seq_len, kv_len, causal=True, window=None,
                interleaved=True, valid=None, kv_valid=None, scale=None):
    O = out_like(Q.shape, cuda, fill=float("nan"))
    K.mha_prefill(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, seq=seq,
                  seq_len=seq_len, kv_len=kv_len, scale=scale, causal=causal, window=window,
                  q_interleaved=interleaved, kv_interleaved=interleaved,
                  valid=None if valid is None else word(valid, cuda),
                  kv_valid=None if kv_valid is None else word(kv_valid, cuda))
    want = ops.mha(Q, Kc, Vc, num_heads=H, num_KV_heads=G, seq_len=seq_len, kv_len=kv_len, d=d,
                   causal=causal, window=window, scale=scale, heads_interleaved=interleaved,
                   kv_interleaved=interleaved, valid=valid, kv_valid=kv_valid)
    return from_torch(O), want


def test_mha_prefill_longest_shape_on_sampled_queries(cuda):
    """S = 8192 (the longest of the benchmark's shapes): the whole output would take the oracle
    minutes, so every head of a sample of queries -- tile edges, both ends, random rows -- is
    checked against the oracle's attention of that one query over its keys."""
    rng = np.random.default_rng(12)
    S, H, G, d = 8192, 32, 8, 64
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    O = out_like(Q.shape, cuda, fill=float("nan"))
    K.mha_prefill(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, seq=S, seq_len=S,
                  kv_len=S, scale=0.125, causal=True, q_interleaved=True, kv_interleaved=True)
    got = from_torch(O)
    assert not np.isnan(got).any()
    rows = sorted({0, 1, 63, 64, 127, 128, 129, 4095, 4096, 8063, 8064, 8191, *rng.integers(0, S, 12).tolist()})
    for r in rows:
        # The query at position r attends keys 0..r: the one-query form of the same operator.
        want = ops.mha(Q[r : r + 1], Kc[: r + 1], Vc[: r + 1], num_heads=H, num_KV_heads=G, seq_len=1, kv_len=r + 1,
                       d=d, causal=True, scale=0.125, heads_interleaved=True, kv_interleaved=True)
        close(got[r : r + 1], want)


@pytest.mark.parametrize("rows", [512, 1500])
def test_mha_prefill_bounded_chunk_at_the_decoder_s_width(cuda, rows):
    """A 2048-row prompt chunk of 32 heads under row and key bounds read on the device (512 rows
    as the benchmark's prompt leaves, and 1500): every head of a sample of rows against the oracle's
    one-query attention over the keys before it; the rows past the bound are zero, and NaN there
    reaches nothing."""
    rng = np.random.default_rng(rows)
    S, H, G, d = 2048, 32, 8, 64
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    Q[rows:], Kc[rows:], Vc[rows:] = np.nan, np.nan, np.nan
    O = out_like(Q.shape, cuda, fill=float("nan"))
    K.mha_prefill(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, seq=S, seq_len=S,
                  kv_len=S, scale=0.125, causal=True, q_interleaved=True, kv_interleaved=True,
                  valid=word(rows, cuda), kv_valid=word(rows, cuda))
    got = from_torch(O)
    assert np.all(got[rows:] == 0)
    assert not np.isnan(got[:rows]).any()
    for r in sorted({0, 1, 31, 32, 63, 64, 65, 127, 128, 129, rows - 65, rows - 64, rows - 1, *rng.integers(0, rows, 10).tolist()}):
        want = ops.mha(Q[r : r + 1], Kc[: r + 1], Vc[: r + 1], num_heads=H, num_KV_heads=G, seq_len=1, kv_len=r + 1,
                       d=d, causal=True, scale=0.125, heads_interleaved=True, kv_interleaved=True)
        close(got[r : r + 1], want)


@pytest.mark.parametrize("S", [512, 2048])
def test_mha_prefill_llama_shape(cuda, S):
    rng = np.random.default_rng(11)
    H, G, d = 32, 8, 64
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=S, scale=0.125)
    close(got, want)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("shape", ["huge_range", "rising", "falling", "constant", "far_below_zero", "far_above_zero"])
def test_mha_prefill_scores_that_move_the_softmax_reference(cuda, d, shape):
    """The exponentials are taken against a reference that follows the maxima lazily, and a tile is
    first tried without taking its maximum at all: scores spread over hundreds of doublings, scores
    that rise or fall along the keys by far more than float32's exponent range holds, equal scores,
    and scores all far below or far above zero (where a reference of zero would under- or overflow)
    against the oracle's softmax, causal and not, over many tiles."""
    rng = np.random.default_rng(len(shape) + d)
    H, G, S = 4, 2, 1100
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    ramp = np.linspace(0.0, 1.0, S, dtype=np.float32)[:, None, None]
    scale = None
    if shape == "huge_range":
        Q, Kc = round_bf16(Q * 6), round_bf16(Kc * 6)            # scaled scores of a few hundred either way
    elif shape in ("rising", "falling"):
        # one direction of the head carries a score that climbs (or drops) by ~1500 along the keys
        Q[..., 0] = 8.0
        Kc[..., 0] = round_bf16((ramp if shape == "rising" else 1 - ramp) * 190.0)[..., 0]
        scale = 1.0
    elif shape == "constant":
        Q[:], Kc[:] = 0.0, 0.0
    else:
        Q[..., 0] = 16.0
        Kc[..., 0] = -40.0 if shape == "far_below_zero" else 40.0   # every score near -640 / +640 before the scale
        scale = 1.0
    for causal in (True, False):
        got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=S, causal=causal, scale=scale)
        assert not np.isnan(got).any()
        close(got, want)


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("causal,window", [(True, None), (True, 100), (False, 70), (False, None)])
def test_mha_prefill_masks_and_layouts(cuda, causal, window, interleaved):
    rng = np.random.default_rng(12)
    H, G, d, S, L = 8, 2, 64, 192, 448
    qs = (S, H, d) if interleaved else (H, S, d)
    ks = (L, G, d) if interleaved else (G, L, d)
    Q, Kc, Vc = bf(rng, *qs), bf(rng, *ks), bf(rng, *ks)
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=L, causal=causal,
                            window=window, interleaved=interleaved)
    close(got, want)


def test_mha_prefill_chunk_over_cache_bounded(cuda):
    """A prompt chunk: `valid` of 256 rows at the end of `kv_valid` keys of a longer cache; NaN
    past the bounds must not reach the output and padding rows are exactly zero
    (test_mha_bounded_rows.py:98-102,197-225)."""
    rng = np.random.default_rng(13)
    H, G, d, C, L = 8, 2, 64, 256, 1024
    rows, kv = 150, 600
    Q, Kc, Vc = bf(rng, C, H, d), bf(rng, L, G, d), bf(rng, L, G, d)
    Q[rows:], Kc[kv:], Vc[kv:] = np.nan, np.nan, np.nan
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=C, seq_len=C, kv_len=L, valid=rows, kv_valid=kv)
    assert np.all(got[rows:] == 0)
    close(got[:rows], want[:rows])


def test_mha_prefill_d128_and_ragged_seq(cuda):
    rng = np.random.default_rng(14)
    H, G, d, S = 6, 2, 128, 200
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=S)
    close(got, want)


def test_mha_prefill_d256_ragged_windowed_and_bounded(cuda):
    """256-wide heads (a global layer's of a toy Gemma 4): a ragged causal sequence, a window, and a
    prompt chunk bounded by device words at the end of a longer cache, unscaled as Gemma attends."""
    rng = np.random.default_rng(21)
    H, G, d, S = 4, 1, 256, 200
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    for window in (None, 37):
        got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=S, window=window)
        close(got, want)
    C, L, rows, kv = 64, 512, 40, 300
    Q, Kc, Vc = bf(rng, C, H, d) * 0.25, bf(rng, L, G, d) * 0.25, bf(rng, L, G, d)
    Q[rows:], Kc[kv:], Vc[kv:] = np.nan, np.nan, np.nan
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=C, seq_len=C, kv_len=L, valid=rows, kv_valid=kv,
                            scale=1.0)
    assert np.all(got[rows:] == 0)
    close(got[:rows], want[:rows])


@pytest.mark.parametrize("d,H,G,S,window", [(512, 32, 8, 2048, None), (256, 32, 8, 2048, 300), (256, 32, 4, 4096, None),
                                             (512, 16, 16, 1100, None)])
def test_mha_prefill_wide_heads_at_every_block_shape_on_sampled_queries(cuda, d, H, G, S, window):
    """256- and 512-wide heads where the launch has blocks enough for its larger shapes (128-query
    blocks of eight waves; at 256 two query groups a wave from a thousand blocks on): the whole
    output would take the oracle minutes, so every head of a sample of queries -- tile and block
    edges, both ends, random rows -- is checked against the oracle's attention of that one query."""
    rng = np.random.default_rng(d + S)
    Q, Kc, Vc = bf(rng, S, H, d) * 0.25, bf(rng, S, G, d) * 0.25, bf(rng, S, G, d)
    O = out_like(Q.shape, cuda, fill=float("nan"))
    K.mha_prefill(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, seq=S, seq_len=S,
                  kv_len=S, scale=1.0, causal=True, window=window, q_interleaved=True, kv_interleaved=True)
    got = from_torch(O)
    assert not np.isnan(got).any()
    for r in sorted({0, 1, 15, 16, 31, 32, 33, 63, 64, 127, 128, 129, 255, 256, S - 129, S - 128, S - 1,
                     *rng.integers(0, S, 8).tolist()}):
        lo = 0 if window is None else max(0, r - window)
        want = ops.mha(Q[r : r + 1], Kc[lo : r + 1], Vc[lo : r + 1], num_heads=H, num_KV_heads=G, seq_len=1,
                       kv_len=r + 1 - lo, d=d, causal=True, scale=1.0, heads_interleaved=True, kv_interleaved=True)
        close(got[r : r + 1], want)


@pytest.mark.parametrize("interleaved", [True, False])
def test_mha_prefill_512_wide_heads_over_many_tiles(cuda, interleaved):
    """512-wide heads past a block's 64 queries and a tile's 32 keys: several heads a KV head, a ragged
    causal sequence, a window that drops whole tiles, no mask at all, a chunk at the end of a longer
    cache under bounds on both sides, and an unscaled product."""
    rng = np.random.default_rng(24)
    H, G, d, S = 4, 2, 512, 333
    Q, Kc, Vc = bf(rng, S, H, d) * 0.25, bf(rng, S, G, d) * 0.25, bf(rng, S, G, d)
    if not interleaved:
        Q, Kc, Vc = (np.ascontiguousarray(a.transpose(1, 0, 2)) for a in (Q, Kc, Vc))
    for causal, window in ((True, None), (True, 70), (False, 45), (False, None)):
        got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=S, causal=causal,
                                window=window, interleaved=interleaved)
        close(got, want)
    C, L, rows, kv = 192, 700, 130, 611
    Q, Kc, Vc = bf(rng, C, H, d) * 0.25, bf(rng, L, G, d) * 0.25, bf(rng, L, G, d)
    Q[rows:], Kc[kv:], Vc[kv:] = np.nan, np.nan, np.nan
    if not interleaved:
        Q, Kc, Vc = (np.ascontiguousarray(a.transpose(1, 0, 2)) for a in (Q, Kc, Vc))
    got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=C, seq_len=C, kv_len=L, valid=rows, kv_valid=kv,
                            scale=1.0, interleaved=interleaved)
    if interleaved:
        assert np.all(got[rows:] == 0)
        close(got[:rows], want[:rows])
    else:
        assert np.all(got[:, rows:] == 0)
        close(got[:, :rows], want[:, :rows])


@pytest.mark.parametrize("d,H,G", [(64, 8, 2), (128, 4, 1), (256, 4, 1), (512, 4, 1)])
def test_mha_over_a_window_of_a_longer_buffer(cuda, d, H, G):
    """Keys that are a run of rows of a longer buffer, from a row a device word names (a ring cache's
    window): the launch that is handed those rows as tensors of their own, bit for bit; the buffer's
    other rows (NaN here) reach nothing, and a word past the end is held inside the buffer."""
    rng = np.random.default_rng(23)
    rows, L, S = 300, 96, 64
    Kb, Vb = bf(rng, rows, G, d) * 0.25, bf(rng, rows, G, d)
    Q = bf(rng, S, H, d) * 0.25
    ws = K.mha_decode_workspace(H, d, cuda)
    for first, kv_valid in ((0, 96), (37, 80), (204, 96), (1000, 70)):
        held = max(0, min(first, rows - L))
        Kw, Vw = Kb[held : held + L].copy(), Vb[held : held + L].copy()
        Kp, Vp = np.full_like(Kb, np.nan), np.full_like(Vb, np.nan)
        Kp[held : held + kv_valid], Vp[held : held + kv_valid] = Kb[held : held + kv_valid], Vb[held : held + kv_valid]
        for window in (None, 20):
            own = out_like((S, H, d), cuda)
            K.mha_prefill(dev(Q, cuda), dev(Kw, cuda), dev(Vw, cuda), own, heads=H, kv_heads=G, d=d, seq=S, kv_len=L,
                          scale=1.0, window=window, q_interleaved=True, kv_interleaved=True, kv_valid=word(kv_valid, cuda))
            at = out_like((S, H, d), cuda, fill=float("nan"))
            K.mha_prefill(dev(Q, cuda), dev(Kp, cuda), dev(Vp, cuda), at, heads=H, kv_heads=G, d=d, seq=S, kv_len=L,
                          scale=1.0, window=window, q_interleaved=True, kv_interleaved=True, kv_valid=word(kv_valid, cuda),
                          kv_first=word(first, cuda), kv_rows=rows)
            assert torch.equal(own, at), (first, kv_valid, window)
            own1, at1 = out_like((1, H, d), cuda), out_like((1, H, d), cuda, fill=float("nan"))
            K.mha_decode(dev(Q[:1], cuda), dev(Kw, cuda), dev(Vw, cuda), own1, heads=H, kv_heads=G, d=d, kv_len=L, scale=1.0,
                         window=window, kv_interleaved=True, kv_valid=word(kv_valid, cuda), workspace=ws)
            K.mha_decode(dev(Q[:1], cuda), dev(Kp, cuda), dev(Vp, cuda), at1, heads=H, kv_heads=G, d=d, kv_len=L, scale=1.0,
                         window=window, kv_interleaved=True, kv_valid=word(kv_valid, cuda), workspace=ws,
                         kv_first=word(first, cuda), kv_rows=rows)
            assert torch.equal(own1, at1), (first, kv_valid, window)
    # ... and the long-cache kernel (splits and their merge) over a window.
    if d == 64:
        rows, L = 6000, 4096
        Kb, Vb, q = bf(rng, rows, G, d), bf(rng, rows, G, d), bf(rng, 1, H, d)
        own1, at1 = out_like((1, H, d), cuda), out_like((1, H, d), cuda)
        K.mha_decode(q_t := dev(q, cuda), dev(Kb[1500:5596], cuda), dev(Vb[1500:5596], cuda), own1, heads=H, kv_heads=G, d=d,
                     kv_len=L, kv_interleaved=True, kv_valid=word(3000, cuda), workspace=ws)
        K.mha_decode(q_t, dev(Kb, cuda), dev(Vb, cuda), at1, heads=H, kv_heads=G, d=d, kv_len=L, kv_interleaved=True,
                     kv_valid=word(3000, cuda), workspace=ws, kv_first=word(1500, cuda), kv_rows=rows)
        assert torch.equal(own1, at1)
    with pytest.raises(ValueError, match="row by row"):
        K.mha_decode(dev(Q[:1], cuda), dev(Kb, cuda), dev(Vb, cuda), out_like((1, H, d), cuda), heads=H, kv_heads=G, d=d,
                     kv_len=96, kv_interleaved=False, workspace=ws, kv_first=word(0, cuda), kv_rows=300)


def test_mha_512_wide_heads_prefill_and_decode(cuda):
    """512-wide heads (a global layer's of Gemma 4): the prompt kernel under every mask and a bound,
    and the one-query kernel on either side of 2048 keys."""
    rng = np.random.default_rng(22)
    H, G, d, S, L = 4, 1, 512, 70, 200
    Q, Kc, Vc = bf(rng, S, H, d) * 0.25, bf(rng, L, G, d) * 0.25, bf(rng, L, G, d)
    for causal, window in ((True, None), (True, 37), (False, 20), (False, None)):
        got, want = run_prefill(cuda, Q, Kc, Vc, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=L, causal=causal,
                                window=window, scale=1.0)
        close(got, want)
    Qp, Kp, Vp = Q.copy(), Kc.copy(), Vc.copy()
    Qp[40:], Kp[150:], Vp[150:] = np.nan, np.nan, np.nan
    got, want = run_prefill(cuda, Qp, Kp, Vp, H=H, G=G, d=d, seq=S, seq_len=S, kv_len=L, valid=40, kv_valid=150, scale=1.0)
    assert np.all(got[40:] == 0)
    close(got[:40], want[:40])
    for L, kv_valid, window in ((300, 257, None), (4096, 3000, None), (4096, 3000, 99)):
        H, G = 8, 2
        Q, Kc, Vc = bf(rng, 1, H, d) * 0.25, bf(rng, L, G, d) * 0.25, bf(rng, L, G, d)
        Kc[kv_valid:], Vc[kv_valid:] = np.nan, np.nan
        O = out_like((1, H, d), cuda, fill=float("nan"))
        K.mha_decode(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, kv_len=L, scale=1.0,
                     window=window, kv_interleaved=True, kv_valid=word(kv_valid, cuda),
                     workspace=K.mha_decode_workspace(H, d, cuda))
        want = ops.mha(Q, Kc, Vc, num_heads=H, num_KV_heads=G, seq_len=1, kv_len=L, d=d, scale=1.0, window=window,
                       heads_interleaved=True, kv_interleaved=True, kv_valid=kv_valid)
        close(O, want)


@pytest.mark.parametrize("E,H,G,d", [(2048, 32, 8, 64), (1000, 3, 1, 128), (4096, 8, 2, 128)])
def test_decode_qkv_reading_its_row_from_the_embedding_table(cuda, E, H, G, d):
    """A token's first layer: the fused q/k/v launch handed the embedding table and the word that names
    the row, against the same launch handed the row itself -- every output bit for bit, the row left
    in ``x`` for the residual sum, and a word past either end of the table held inside it."""
    rng = np.random.default_rng(E + d)
    vocab, L, pos = 77, 16, 9
    table, g = bf(rng, vocab, E), round_bf16(rng.uniform(0.9, 1.1, E).astype(np.float32))
    Wq, Wk, Wv = bf(rng, H * d, E, scale=0.02), bf(rng, G * d, E, scale=0.02), bf(rng, G * d, E, scale=0.02)
    angles = round_bf16(ops.rope_angles(d, L))
    dt, dg, dq, dk, dv, da = (dev(a, cuda) for a in (table, g, Wq, Wk, Wv, angles))
    position, angle_row = word(pos, cuda), word(pos, cuda)
    for token in (0, 41, vocab - 1, vocab + 5, -3):
        held = min(max(token, 0), vocab - 1)
        want_q, want_k, want_v = out_like((H * d,), cuda), out_like((L, G, d), cuda, fill=2.0), out_like((L, G, d), cuda, fill=2.0)
        K.decode_qkv(dev(table[held], cuda), dg, dq, dk, dv, da, want_q, want_k, want_v, eps=1e-5, hidden=E, heads=H,
                     kv_heads=G, d=d, cache_rows=L, position=position, angle_row=angle_row)
        x = out_like((E,), cuda, fill=float("nan"))
        got_q, got_k, got_v = out_like((H * d,), cuda), out_like((L, G, d), cuda, fill=2.0), out_like((L, G, d), cuda, fill=2.0)
        K.decode_qkv(x, dg, dq, dk, dv, da, got_q, got_k, got_v, eps=1e-5, hidden=E, heads=H, kv_heads=G, d=d,
                     cache_rows=L, position=position, angle_row=angle_row, table=dt, token=word(token, cuda))
        assert torch.equal(got_q, want_q) and torch.equal(got_k, want_k) and torch.equal(got_v, want_v), token
        assert np.array_equal(from_torch(x), table[held]), token


@pytest.mark.parametrize("H,G,d,rotary,ring,own_kv", [(4, 1, 128, 128, True, True), (4, 1, 256, 64, False, True),
                                                       (8, 2, 512, 512, True, True), (4, 1, 128, 128, False, False),
                                                       (16, 8, 64, 64, False, True)])
def test_decode_heads_is_the_separate_launches_bit_for_bit(cuda, H, G, d, rotary, ring, own_kv):
    """What lies between a token's projections and its attention where heads are normed one by one:
    per-head RMSNorm of q and k (gains) and v (none), RoPE on q and k (all of a head's columns, or the
    leading ones), k's and v's rows into their caches (twice for a ring) -- one launch against the
    launches of the separate operators bit for bit, and q's norm against the oracle."""
    rng = np.random.default_rng(H + d)
    rows = 24
    q, k, v = bf(rng, H, d), bf(rng, G, d), bf(rng, G, d)
    gq, gk = bf(rng, d, scale=0.3) + 1, bf(rng, d, scale=0.3) + 1
    angles = bf(rng, 1, rotary)
    dq, dk, dv, dgq, dgk, da = (dev(x, cuda) for x in (q, k, v, round_bf16(gq), round_bf16(gk), angles))
    # the separate launches
    def normed(x, gain, n):
        y = out_like((n, d), cuda)
        K.rmsnorm(x, gain, y, rows=n, cols=d, eps=1e-6)
        return y

    def roped(x, n):
        y = out_like((n, d), cuda)
        K.rope(x, da, y, rows=n, cols=rotary, angle_rows=1, row_cols=d)
        return y

    want_q = roped(normed(dq, dgq, H), H)
    close(normed(dq, dgq, H), ops.rms_norm(q, round_bf16(gq), epsilon=1e-6))
    row0, row1 = word(5, cuda), word(5 + rows // 2, cuda)
    got_q = out_like((H, d), cuda, fill=float("nan"))
    if not own_kv:
        K.decode_heads(dq, got_q, heads=H, kv_heads=G, d=d, eps=1e-6, norms=1, q_gain=dgq, q_angles=da, rotary=rotary)
        assert torch.equal(got_q, want_q)
        return
    want_k, want_v = roped(normed(dk, dgk, G), G), normed(dv, None, G)
    keys, values = out_like((rows, G, d), cuda, fill=3.0), out_like((rows, G, d), cuda, fill=3.0)
    K.decode_heads(dq, got_q, heads=H, kv_heads=G, d=d, eps=1e-6, norms=7, k=dk, v=dv, q_gain=dgq, k_gain=dgk,
                   q_angles=da, k_angles=da, rotary=rotary, keys=keys, values=values, row0=row0,
                   row1=row1 if ring else None, cache_rows=rows)
    assert torch.equal(got_q, want_q)
    held = [5, 5 + rows // 2] if ring else [5]
    for r in range(rows):
        if r in held:
            assert torch.equal(keys[r], want_k) and torch.equal(values[r], want_v), r
        else:
            assert bool((keys[r] == 3.0).all()) and bool((values[r] == 3.0).all()), r


@pytest.mark.parametrize("M,Kdim", [(128, 512), (256, 2048), (3000, 1536), (128, 8192)])
@pytest.mark.parametrize("activation", ["gelu_tanh", "silu"])
def test_gemv_with_an_activation_and_a_row_in_its_epilogue(cuda, M, Kdim, activation):
    """A projection of one row, its activation and the product with a given row (Gemma 4's per-layer
    input gate) in one launch: link by link against the oracle, and bit for bit against this library's
    own separate launches."""
    rng = np.random.default_rng(M + Kdim)
    W, x, row = bf(rng, M, Kdim, scale=0.05), bf(rng, Kdim), bf(rng, M)
    dW, dx, drow = dev(W, cuda), dev(x, cuda), dev(row, cuda)
    y = out_like((M,), cuda)
    K.gemv_fused(dW, dx, y, M=M, K=Kdim, residual=drow, epilogue=4 if activation == "gelu_tanh" else 5)
    u, a, want = out_like((M,), cuda), out_like((M,), cuda), out_like((M,), cuda)
    K.gemv(dW, dx, u, M=M, K=Kdim)
    close(u, ops.gemv(W, x))
    if activation == "gelu_tanh":
        K.unary(u, a, "gelu_tanh", n=M)
        close(a, ops.gelu(from_torch(u), approximate="tanh"))
    else:
        K.silu(u, a, n=M)
        close(a, ops.silu(from_torch(u)))
    K.mul(a, drow, want, n=M)
    assert torch.equal(y, want)


@pytest.mark.parametrize("L", [1024, 4096, 16384])
def test_mha_decode_llama_shape(cuda, L):
    rng = np.random.default_rng(15)
    H, G, d = 32, 8, 64
    Q, Kc, Vc = bf(rng, 1, H, d), bf(rng, L, G, d), bf(rng, L, G, d)
    O = out_like((1, H, d), cuda, fill=float("nan"))
    ws = K.mha_decode_workspace(H, d, cuda)
    K.mha_decode(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, kv_len=L,
                 scale=0.125, kv_interleaved=True, workspace=ws)
    want = ops.mha(Q, Kc, Vc, num_heads=H, num_KV_heads=G, seq_len=1, kv_len=L, d=d, scale=0.125,
                   heads_interleaved=True, kv_interleaved=True)
    close(O, want)


def test_mha_decode_is_as_accurate_deep_in_a_32k_cache_as_near_its_start(cuda):
    """The reference's long-context check (iron/tests/operators/test_mha_long_context.py:45-62): one
    query of Llama-3.2-1B's packed heads over a 32768-row cache of 55 distinct rows tiled over its
    length (every key block weighs alike and the outputs stay far from 0, so a running sum that loses
    a block's share shows), at positions 1023 and 32703, within 4 % of the output's peak -- and,
    float32 sums losing nothing of the kind here, within the stated bf16 tolerance as well."""
    rng = np.random.default_rng(0)
    H, G, d, L, distinct = 32, 8, 64, 32768, 55
    Kc = round_bf16(np.resize(rng.standard_normal((distinct, G, d)) * 2, (L, G, d)).astype(np.float32))
    Vc = round_bf16(np.resize(rng.standard_normal((distinct, G, d)), (L, G, d)).astype(np.float32))
    Q = round_bf16(rng.standard_normal((1, H, d)).astype(np.float32))
    ws = K.mha_decode_workspace(H, d, cuda)
    Kd, Vd, Qd = dev(Kc, cuda), dev(Vc, cuda), dev(Q, cuda)
    for position in (1023, L - 65):
        O = out_like((1, H, d), cuda, fill=float("nan"))
        K.mha_decode(Qd, Kd, Vd, O, heads=H, kv_heads=G, d=d, kv_len=L, kv_interleaved=True,
                     kv_valid=word(position + 1, cuda), workspace=ws)
        want = ops.mha(Q, Kc, Vc, num_heads=H, num_KV_heads=G, seq_len=1, kv_len=L, d=d, heads_interleaved=True,
                       kv_interleaved=True, kv_valid=position + 1)
        got = from_torch(O).reshape(want.shape)
        peak = float(np.abs(want).max())
        assert peak > 0.5 and np.abs(got - want).max() <= 0.04 * peak, (position, np.abs(got - want).max(), peak)
        close(got, want)


@pytest.mark.parametrize("H,G,d", [(32, 8, 64), (8, 8, 64), (24, 8, 128), (40, 8, 64), (4, 1, 256), (16, 8, 64), (12, 2, 64), (3, 1, 64)])
@pytest.mark.parametrize("kv_valid,window", [(1, None), (77, None), (700, None), (700, 99), (2048, 511)])
@pytest.mark.parametrize("L", [2048, 4096])  # the one-launch kernel, and the split one with its merge
def test_mha_decode_bounds_windows_groups(cuda, H, G, d, kv_valid, window, L):
    rng = np.random.default_rng(16)
    for interleaved in (True, False):
        ks = (L, G, d) if interleaved else (G, L, d)
        Q, Kc, Vc = bf(rng, 1, H, d), bf(rng, *ks), bf(rng, *ks)
        if interleaved:
            Kc[kv_valid:], Vc[kv_valid:] = np.nan, np.nan
        else:
            Kc[:, kv_valid:], Vc[:, kv_valid:] = np.nan, np.nan
        O = out_like((1, H, d), cuda, fill=float("nan"))
        ws = K.mha_decode_workspace(H, d, cuda)
        K.mha_decode(dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda), O, heads=H, kv_heads=G, d=d, kv_len=L,
                     window=window, kv_interleaved=interleaved, kv_valid=word(kv_valid, cuda), workspace=ws)
        want = ops.mha(Q, Kc, Vc, num_heads=H, num_KV_heads=G, seq_len=1, kv_len=L, d=d, window=window,
                       heads_interleaved=True, kv_interleaved=interleaved, kv_valid=kv_valid)
        close(O, want)


@pytest.mark.parametrize("H,G,d", [(32, 8, 64), (16, 1, 64), (7, 7, 64), (24, 8, 128), (26, 2, 128)])
@pytest.mark.parametrize("form,short_keys", [(1, 0), (2, 0), (2, 48)])
def test_mha_decode_every_form_at_every_context(cuda, H, G, d, form, short_keys):
    """The lane-per-column scans, and the one-shape launch both as a block a query head (few keys) and
    as runs of keys dealt over the chip with a merge behind (forced onto small contexts by
    ``short_keys``): contexts that end inside a wave's 16-key tile, at a run's edge and at the cache's
    last row; windows; rows past the bound and the whole workspace poisoned."""
    if form == 1 and H // G not in (1, 2, 3, 4, 5, 6, 8):
        pytest.skip("the lane-scan kernels take 1, 2, 3, 4, 5, 6 or 8 query heads a KV head")
    rng = np.random.default_rng(161)
    L = 3000
    Q, Kc, Vc = bf(rng, 1, H, d), bf(rng, L, G, d), bf(rng, L, G, d)
    dQ = dev(Q, cuda)
    ws = K.mha_decode_workspace(H, d, cuda)
    for kv_valid, window in ((1, None), (17, None), (48, None), (49, None), (777, None), (2049, None), (3000, None),
                             (2500, 100), (2500, 1500), (3000, 2999)):
        Kp, Vp = Kc.copy(), Vc.copy()
        Kp[kv_valid:], Vp[kv_valid:] = np.nan, np.nan
        ws.fill_(float("nan"))
        O = out_like((1, H, d), cuda, fill=float("nan"))
        K.mha_decode(dQ, dev(Kp, cuda), dev(Vp, cuda), O, heads=H, kv_heads=G, d=d, kv_len=L, window=window,
                     kv_interleaved=True, kv_valid=word(kv_valid, cuda), workspace=ws, form=form, short_keys=short_keys)
        want = ops.mha(Q, Kp, Vp, num_heads=H, num_KV_heads=G, seq_len=1, kv_len=L, d=d, window=window,
                       heads_interleaved=True, kv_interleaved=True, kv_valid=kv_valid)
        close(O, want)


def test_mha_decode_cost_follows_the_context_not_the_cache(cuda):
    """One compile, any context (AGENTS.md:246-255, iron/operators/mha.py:275-278): over a 131072-row
    cache -- Llama-3.2-1B's own max_seq_len -- a context of 600 keys, one just past what a single block
    takes, and the whole cache, each against the oracle; and the launches of the first are those of a
    2048-row cache's (one block a query head does the work), not the cache's."""
    rng = np.random.default_rng(162)
    H, G, d, L = 32, 8, 64, 131072
    Q = bf(rng, 1, H, d)
    Kc = round_bf16(np.resize(rng.standard_normal((4099, G, d)), (L, G, d)).astype(np.float32))
    Vc = round_bf16(np.resize(rng.standard_normal((4099, G, d)), (L, G, d)).astype(np.float32))
    dQ, dK, dV = dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda)
    ws = K.mha_decode_workspace(H, d, cuda)
    for kv_valid in (600, 2049, 40000, L):
        O = out_like((1, H, d), cuda, fill=float("nan"))
        K.mha_decode(dQ, dK, dV, O, heads=H, kv_heads=G, d=d, kv_len=L, kv_interleaved=True,
                     kv_valid=word(kv_valid, cuda), workspace=ws)
        want = ops.mha(Q, Kc[:kv_valid], Vc[:kv_valid], num_heads=H, num_KV_heads=G, seq_len=1, kv_len=kv_valid, d=d,
                       heads_interleaved=True, kv_interleaved=True)
        close(O, want)


def test_mha_decode_equals_last_row_of_prefill(cuda):
    """A size-independent property: the one-query kernel and the last row of the many-query one agree."""
    rng = np.random.default_rng(17)
    H, G, d, S = 32, 8, 64, 1536
    Q, Kc, Vc = bf(rng, S, H, d), bf(rng, S, G, d), bf(rng, S, G, d)
    dQ, dK, dV = dev(Q, cuda), dev(Kc, cuda), dev(Vc, cuda)
    O = out_like((S, H, d), cuda)
    K.mha_prefill(dQ, dK, dV, O, heads=H, kv_heads=G, d=d, seq=S, kv_len=S, q_interleaved=True, kv_interleaved=True)
    o1 = out_like((1, H, d), cuda)
    K.mha_decode(dQ[S - 1 :].contiguous(), dK, dV, o1, heads=H, kv_heads=G, d=d, kv_len=S, kv_interleaved=True,
                 workspace=K.mha_decode_workspace(H, d, cuda))
    close(from_torch(o1)[0], from_torch(O)[S - 1], rtol=1e-2, atol=1e-2)


# ------------------------------------------------------------------------ glue
def test_gather_rows_exact(cuda):
    rng = np.random.default_rng(18)
    table = bf(rng, 1000, 2048)
    ids = rng.integers(0, 1000, 300).astype(np.int32)
    out = out_like((300, 2048), cuda, fill=1.0)
    K.gather_rows(dev(table, cuda), torch.from_numpy(ids).to(cuda), out, valid=word(256, cuda))
    got = from_torch(out)
    assert np.array_equal(got[:256], ops.gather_rows(table, ids[:256])) and np.all(got[256:] == 1.0)
    # int32 rows, a row width that is not a multiple of 16 bytes.
    t32 = torch.arange(50 * 3, dtype=torch.int32, device=cuda).reshape(50, 3)
    o32 = torch.zeros((4, 3), dtype=torch.int32, device=cuda)
    K.gather_rows(t32, torch.tensor([7, 0, 49, 7], dtype=torch.int32, device=cuda), o32)
    assert torch.equal(o32.cpu(), t32.cpu()[[7, 0, 49, 7]])


def test_copy_rows_cache_write_table_row_and_last_row(cuda):
    rng = np.random.default_rng(19)
    L, G, d = 128, 8, 64
    cache = dev(np.zeros((L, G * d), np.float32), cuda)
    k = bf(rng, 1, G * d)
    K.copy_rows(dev(k, cuda), cache, rows=1, row_elems=G * d, src_rows=1, dst_rows=L, dst_row=word(37, cuda))
    got = from_torch(cache)
    assert np.array_equal(got[37], k[0]) and np.count_nonzero(got) == np.count_nonzero(k)
    # A chunk of rows at a per-call start, bounded.
    x = bf(rng, 32, G * d)
    K.copy_rows(dev(x, cuda), cache, rows=32, row_elems=G * d, src_rows=32, dst_rows=L,
                dst_row=word(64, cuda), valid=word(20, cuda))
    got = from_torch(cache)
    assert np.array_equal(got[64:84], x[:20]) and np.all(got[84:] == 0)
    # The last valid row picked out (src index), and a row past the end skipped.
    last = out_like((1, G * d), cuda, fill=4.0)
    K.copy_rows(dev(x, cuda), last, rows=1, row_elems=G * d, src_rows=32, dst_rows=1, src_row=word(19, cuda))
    assert np.array_equal(from_torch(last)[0], x[19])
    K.copy_rows(dev(x, cuda), last, rows=1, row_elems=G * d, src_rows=32, dst_rows=1, src_row=word(32, cuda))
    assert np.array_equal(from_torch(last)[0], x[19])


def test_argmax_first_of_ties_and_record(cuda):
    rng = np.random.default_rng(11)
    logits = round_bf16(rng.normal(0, 3, 128256))
    top = rng.choice(128256, 8, replace=False)
    logits[top] = logits.max()
    first = int(min(top.min(), np.argmax(logits)))  # nine equal maxima: the first wins
    tok = torch.full((1,), -1, dtype=torch.int32, device=cuda)
    rec = torch.full((16,), -1, dtype=torch.int32, device=cuda)
    K.argmax(dev(logits, cuda), tok, record=rec, at=word(5, cuda))
    assert int(tok.item()) == ops.argmax(logits) == first
    assert rec.cpu().tolist() == [-1] * 5 + [first] + [-1] * 10
    odd = round_bf16(rng.normal(0, 1, 1003))
    K.argmax(dev(odd, cuda), tok)
    assert int(tok.item()) == ops.argmax(odd)


# ---------------------------------------------- the sibling decoders' operators
@pytest.mark.parametrize("kind,ref,exact", [
    ("gelu_tanh", lambda x: ops.gelu(x), False), ("gelu_erf", lambda x: ops.gelu(x, "none"), False),
    ("relu", ops.relu, True), ("sigmoid", ops.sigmoid, False), ("tanh", ops.tanh, False),
    ("clamp", lambda x: ops.clamp(x, -0.75, 1.25), True)])
def test_unary_kinds_and_their_bound(cuda, kind, ref, exact):
    rng = np.random.default_rng(50)
    x = bf(rng, 10007, scale=3.0)   # odd: a tail short of a 16-byte piece
    y = out_like((10007,), cuda, fill=7.0)
    K.unary(dev(x, cuda), y, kind, low=-0.75, high=1.25)
    if exact:
        assert np.array_equal(from_torch(y), ref(x))
    else:
        close(y, ref(x), rtol=2.0**-7, atol=1e-5)
    # A bound read on the device leaves the rest as it was.
    y.fill_(7.0)
    K.unary(dev(x, cuda), y, kind, low=-0.75, high=1.25, valid=word(4001, cuda))
    got = from_torch(y)
    close(got[:4001], ref(x)[:4001], rtol=2.0**-7, atol=1e-5)
    assert np.all(got[4001:] == 7.0)


def test_axpy_and_its_bound(cuda):
    rng = np.random.default_rng(51)
    x, y = bf(rng, 70001, scale=4.0), bf(rng, 70001, scale=4.0)
    out = out_like((70001,), cuda, fill=7.0)
    for a in (3.0, 1.003, -0.5):
        K.axpy(dev(x, cuda), dev(y, cuda), out, a=a)
        assert np.array_equal(from_torch(out), ops.axpy(a, x, y))   # one fma, one rounding: exact
    out.fill_(7.0)
    K.axpy(dev(x, cuda), dev(y, cuda), out, a=3.0, valid=word(13, cuda))
    got = from_torch(out)
    assert np.array_equal(got[:13], ops.axpy(3.0, x, y)[:13]) and np.all(got[13:] == 7.0)


@pytest.mark.parametrize("rows,cols,weighted", [(1, 2048, True), (33, 1024, False), (16, 4096, True), (5, 8192, True),
                                                (3, 12288, True), (64, 768, True)])
def test_layernorm_rows(cuda, rows, cols, weighted):
    rng = np.random.default_rng(cols + rows)
    x = round_bf16(bf(rng, rows, cols, scale=2.0) + np.float32(1.5))
    w = round_bf16(rng.uniform(0.9, 1.1, cols).astype(np.float32)) if weighted else None
    y = out_like((rows, cols), cuda, fill=7.0)
    K.layernorm(dev(x, cuda), None if w is None else dev(w, cuda), y, rows=rows, cols=cols, eps=1e-5)
    close(y, ops.layer_norm(x, w))
    if rows > 2:
        y.fill_(7.0)
        K.layernorm(dev(x, cuda), None if w is None else dev(w, cuda), y, rows=rows, cols=cols, eps=1e-5,
                    valid=word(2, cuda))
        got = from_torch(y)
        close(got[:2], ops.layer_norm(x, w)[:2])
        assert np.all(got[2:] == 7.0)


@pytest.mark.parametrize("rows,cols,f32,addend,cap", [(32, 1024, False, False, None), (16, 4608, False, False, None),
                                                      (4, 32768, False, False, None), (32, 1024, True, False, None),
                                                      (64, 1536, True, True, 50.0), (16, 80, True, True, None)])
def test_softmax_rows_cap_addend_and_length(cuda, rows, cols, f32, addend, cap):
    rng = np.random.default_rng(cols)
    x = rng.normal(0, 4, (rows, cols)).astype(np.float32)
    x = x if f32 else round_bf16(x)
    add = rng.normal(0, 1, (rows, cols)).astype(np.float32) if addend else None
    xd = torch.from_numpy(x).to(cuda) if f32 else dev(x, cuda)
    ad = None if add is None else torch.from_numpy(add).to(cuda)
    y = out_like((rows, cols), cuda, fill=7.0)
    K.softmax(xd, y, rows=rows, cols=cols, addend=ad, soft_cap=cap)
    close(y, ops.softmax(x, add, soft_cap=cap), rtol=1e-2, atol=1e-4)
    assert abs(float(from_torch(y).sum(axis=-1).mean()) - 1.0) < 5e-3
    # A length read on the device: the first columns' softmax, zeros after them.
    n = cols // 3
    K.softmax(xd, y, rows=rows, cols=cols, addend=ad, soft_cap=cap, length=word(n, cuda))
    got = from_torch(y)
    close(got, ops.softmax(x, add, soft_cap=cap, length=n), rtol=1e-2, atol=1e-4)
    assert not got[:, n:].any()


def _draw_rows(rng, count, temperatures=(0.0, 0.05, 0.7, 1.0, 5.0), k_hi=65):
    from iron_amd.operators.sample import draw_row

    return np.stack([draw_row(rng.choice(temperatures), int(rng.integers(1, k_hi)), int(rng.integers(0, 1 << 53)))
                     for _ in range(count)])


def _host_draw(logits, row, k_max=64):
    return ops.sample_ref(logits, *ops.draw_words(row), k_max)


def _sample_rows(cuda, logits, rows, n=None, k_max=64):
    """The device's draw for each of ``rows`` (picked by a device word), recorded one per slot."""
    steps = len(rows)
    tok = torch.full((1,), -1, dtype=torch.int32, device=cuda)
    rec = torch.full((steps,), -1, dtype=torch.int32, device=cuda)
    lg, dr = dev(logits, cuda), torch.from_numpy(np.ascontiguousarray(rows)).to(cuda)
    for i in range(steps):
        K.sample(lg, dr, tok, n=n, row=word(4 * i, cuda), k_max=k_max, record=rec, at=word(i, cuda))
        assert int(tok.item()) == int(rec[i].item())
    return rec.cpu().tolist()


@pytest.mark.parametrize("vocab,drawable", [(4096, 4096), (128256, 128256), (51866, 51866), (151670, 151669),
                                            (1003, 1003), (100, 100)])
def test_sample_draws_the_host_token(cuda, vocab, drawable):
    rng = np.random.default_rng(vocab)
    logits = round_bf16(rng.normal(0, 3, vocab))
    logits[rng.choice(drawable, 8, replace=False)] = logits[:drawable].max()
    logits[drawable:] = logits.max() + 1   # padding no draw may take
    rows = _draw_rows(rng, 48)
    got = _sample_rows(cuda, logits, rows, n=drawable)
    want = [_host_draw(logits[:drawable], r) for r in rows]
    assert got == want
    assert len(set(got)) > 4   # the draws spread over candidates


def test_sample_ties_at_the_cut_go_to_the_lower_index(cuda):
    # Few distinct values: the top-k cut falls inside a run of equal logits, and the k kept are
    # those of the lowest index.
    rng = np.random.default_rng(21)
    logits = round_bf16(rng.integers(-3, 4, 128256).astype(np.float32) * 0.5)
    rows = _draw_rows(rng, 32, temperatures=(0.7, 1.0, 5.0))
    assert _sample_rows(cuda, logits, rows) == [_host_draw(logits, r) for r in rows]
    # All equal: more logits at the floor than the list holds (the slow path), uniform over the first k.
    flat = np.full(40000, 1.5, np.float32)
    got = _sample_rows(cuda, flat, rows)
    assert got == [_host_draw(flat, r) for r in rows] and max(got) < 64
    # The best first in memory, falling: every thread's maximum is its first logit.
    falling = round_bf16(np.linspace(8, -8, 20000, dtype=np.float32))
    assert _sample_rows(cuda, falling, rows) == [_host_draw(falling, r) for r in rows]


def test_sample_special_values_and_row_bounds(cuda):
    from iron_amd.operators.sample import draw_row

    rng = np.random.default_rng(22)
    logits = round_bf16(rng.normal(0, 1, 5000))
    logits[[7, 1200]] = np.nan
    logits[[9, 4000]] = -np.inf
    logits[[100, 101]] = [-0.0, 0.0]
    rows = np.concatenate([_draw_rows(rng, 16), [draw_row(0.7, 50, 0), draw_row(0.7, 50, (1 << 53) - 1),
                                                 draw_row(1e-3, 64, 1 << 52), draw_row(np.nan, 5, 77),
                                                 draw_row(-1.0, 5, 77)]])
    assert _sample_rows(cuda, logits, rows) == [_host_draw(logits, r) for r in rows]
    infinite = logits.copy()
    infinite[3000] = np.inf
    assert _sample_rows(cuda, infinite, rows[:8]) == [3000] * 8
    hollow = np.full(3000, -np.inf, np.float32)
    hollow[[5, 2500]] = [np.nan, 2.0]
    assert _sample_rows(cuda, hollow, rows[16:18]) == [2500, 2500]
    # A k_max under the row's top-k caps it.
    assert _sample_rows(cuda, logits, rows[:16], k_max=3) == [_host_draw(logits, r, 3) for r in rows[:16]]
    # No draw rows, or a row outside them: greedy.
    tok = torch.full((1,), -1, dtype=torch.int32, device=cuda)
    dr = torch.from_numpy(np.ascontiguousarray(rows[:2])).to(cuda)
    for kw in (dict(draws=None), dict(draws=dr, row=word(8, cuda)), dict(draws=dr, row=word(-4, cuda))):
        K.sample(dev(logits, cuda), kw.pop("draws"), tok, **kw)
        assert int(tok.item()) == ops.sample_ref(logits, 0.0, 1, 0)
    with pytest.raises(Exception, match="k_max"):
        K.sample(dev(logits, cuda), dr, tok, k_max=65)


def test_sample_leaves_its_workspace_ready_for_the_next_draw(cuda):
    # The block count in the workspace's first words must be zero when a draw starts; every draw
    # puts it back, so one zeroed workspace serves any number of draws, of changing lengths.
    rng = np.random.default_rng(23)
    logits = round_bf16(rng.normal(0, 3, 128256))
    rows = _draw_rows(rng, 12)
    lg, dr = dev(logits, cuda), torch.from_numpy(np.ascontiguousarray(rows)).to(cuda)
    ws = K.sample_workspace(logits.size, cuda)
    tok = torch.full((1,), -1, dtype=torch.int32, device=cuda)
    for i, n in enumerate([128256, 100, 51866, 128256, 4096, 1003] * 2):
        K.sample(lg, dr, tok, n=n, row=word(4 * i, cuda), workspace=ws)
        assert int(tok.item()) == _host_draw(logits[:n], rows[i]), (i, n)
        assert not ws[:2].any(), (i, n)


def test_eval_words_advances_a_decode_step(cuda):
    words = torch.tensor([11, 40, 0, 0, 0, 0, 0, 0], dtype=torch.int32, device=cuda)
    # position += 1; kv_valid = position + 1; rope_row = min(position, 5); half = position >> 1;
    # ring_row = max(position - 3, 0) % 16; its mirror's = ring_row + 16
    exprs = torch.tensor([[1, 1, 1, 1, 0, -(2**31), 2**31 - 1, -1, 0], [2, 1, 1, 1, 0, -(2**31), 2**31 - 1, -1, 0],
                          [3, 1, 1, 0, 0, 0, 5, -1, 0], [4, 1, 1, 0, 1, -(2**31), 2**31 - 1, -1, 0],
                          [5, 1, 1, -3, 0, 0, 2**31 - 1, 15, 0], [6, 1, 1, -3, 0, 0, 2**31 - 1, 15, 16]],
                         dtype=torch.int32, device=cuda)
    K.eval_words(words, exprs)
    assert words.cpu().tolist() == [11, 41, 42, 5, 20, 6, 22, 0]
