"""Pins the numpy oracle against things it does not compute itself: brute-force
Python loops on tiny inputs, closed forms for special masks, library routines,
invariants the reference's own tests check (test/unit/test_tesa.py:36-43,101-107)
and a finite difference for the softmax gradient."""
import itertools

import numpy as np
import pytest
import scipy.special

from oracle import bcs, ops


# ---------------------------------------------------------------- index build --
def brute_force_index(mask, BH, BW):
    """Independent restatement with explicit loops: scan block rows, then block
    columns, test every byte of every tile."""
    H, W = mask.shape
    R, C = H // BH, W // BW
    live = [[any(mask[r * BH + i, c * BW + j] != 0 for i in range(BH) for j in range(BW))
             for c in range(C)] for r in range(R)]
    row_ptr, bcsr, pos = [0], [], {}
    for r in range(R):
        for c in range(C):
            if live[r][c]:
                pos[(r, c)] = len(bcsr)
                bcsr.append((r << 16) | c)
        row_ptr.append(len(bcsr))
    col_ptr, bcsc32, bcsc64 = [0], [], []
    for c in range(C):
        for r in range(R):
            if live[r][c]:
                bcsc32.append((c << 16) | r)
                bcsc64.append((pos[(r, c)] << 32) | (c << 16) | r)
        col_ptr.append(len(bcsc32))
    return row_ptr, bcsr, col_ptr, bcsc32, bcsc64


@pytest.mark.parametrize('H,W,BH,BW,sparsity,seed', [
    (16, 24, 4, 8, 0.5, 0), (32, 32, 8, 4, 0.9, 1), (8, 64, 4, 16, 0.7, 2), (64, 8, 16, 4, 0.2, 3),
    (12, 12, 4, 4, 0.97, 4),
])
def test_index_matches_brute_force(H, W, BH, BW, sparsity, seed):
    mask = ops.block_mask((H, W), (1, 1), sparsity, seed)
    row_ptr, bcsr, col_ptr, bcsc64, nnz = bcs.build_bcsrc(mask, BH, BW)
    _, bcsc32, _ = bcs.build_bcsc(mask, BH, BW)
    e_row_ptr, e_bcsr, e_col_ptr, e_bcsc32, e_bcsc64 = brute_force_index(mask, BH, BW)
    assert row_ptr.tolist() == e_row_ptr and bcsr.tolist() == e_bcsr
    assert col_ptr.tolist() == e_col_ptr and bcsc32.tolist() == e_bcsc32
    assert bcsc64.tolist() == e_bcsc64 and nnz == len(e_bcsr)
    assert row_ptr.dtype == np.int32 and bcsr.dtype == np.int32 and bcsc64.dtype == np.int64


def test_index_closed_forms():
    ones = np.ones((64, 96), dtype=np.uint8)
    row_ptr, idx, nnz = bcs.build_bcsr(ones, 16, 32)
    R, C = 4, 3
    assert nnz == R * C
    assert idx.tolist() == [((i // C) << 16) | (i % C) for i in range(R * C)]
    assert row_ptr.tolist() == [C * r for r in range(R + 1)]
    col_ptr, cidx, _ = bcs.build_bcsc(ones, 16, 32)
    assert cidx.tolist() == [((i // R) << 16) | (i % R) for i in range(R * C)]
    assert col_ptr.tolist() == [R * c for c in range(C + 1)]
    zeros = np.zeros((64, 96), dtype=np.uint8)
    row_ptr, idx, nnz = bcs.build_bcsr(zeros, 16, 32)
    assert nnz == 0 and idx.size == 0 and not row_ptr.any()
    one = zeros.copy()
    one[63, 95] = 7  # any non-zero byte makes the tile live
    _, idx, nnz = bcs.build_bcsr(one, 16, 32)
    assert nnz == 1 and idx.tolist() == [(3 << 16) | 2]


@pytest.mark.parametrize('BH,BW', [(4, 4), (8, 32), (32, 8), (64, 64)])
def test_index_invariants_of_the_reference_tests(BH, BW):
    """The checks of test/unit/test_tesa.py on a 1024x768 fine-grained mask."""
    mask = ops.block_mask((1024, 768), (1, 1), 0.999, seed=2023)
    row_ptr, bcsr, col_ptr, bcsc, nnz = bcs.build_bcsrc(mask, BH, BW)
    live = bcs.reduce_block_mask(mask, BH, BW)
    assert row_ptr[-1] == nnz == col_ptr[-1] == live.sum()
    assert (np.diff(row_ptr) >= 0).all() and (np.diff(col_ptr) >= 0).all()
    r, c = bcs.block_coords(bcsr, 'bcsr')
    rebuilt = np.zeros_like(live)
    rebuilt[r, c] = True
    assert np.array_equal(rebuilt, live)
    # BCSR <-> BCSC cross-consistency through the block position field
    pos = bcsc >> 32
    assert np.array_equal(r[pos], bcsc & 0xffff)
    assert np.array_equal(c[pos], (bcsc >> 16) & 0xffff)
    # canonical order
    assert (np.diff(bcsr.astype(np.int64)) > 0).all()
    assert (np.diff((bcsc & 0xffffffff)) > 0).all()


def test_convert_inverse_formula_and_round_trip():
    rng = np.random.default_rng(0)
    H, W, BH, BW = 32, 48, 8, 16
    mask = ops.block_mask((H, W), (BH, BW), 0.5, seed=3)
    dense = rng.standard_normal((2, H, W)).astype(np.float32)
    for fmt, build in (('bcsr', bcs.build_bcsr), ('bcsc', bcs.build_bcsc)):
        _, idx, nnz = build(mask, BH, BW)
        sparse = bcs.convert(dense, idx, fmt, BH, BW)
        assert sparse.shape == (2, nnz * BH * BW)
        br, bc = bcs.block_coords(idx, fmt)
        for b, i, r, c in itertools.product(range(2), range(nnz), range(BH), range(BW)):
            assert sparse[b, i * BH * BW + r * BW + c] == dense[b, br[i] * BH + r, bc[i] * BW + c]
        back = bcs.inverse(sparse, idx, fmt, BH, BW, H, W)
        assert np.array_equal(back, dense * mask)  # dead tiles become zero, live ones are untouched


# ------------------------------------------------------------------- matmul --
@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('tA', [False, True])
@pytest.mark.parametrize('tB', [False, True])
def test_matmul_brute_force(mode, tA, tB):
    rng = np.random.default_rng(5)
    Bt, M, K, N = 2, 4, 6, 8
    A = rng.standard_normal((Bt, K, M) if tA else (Bt, M, K))
    B = rng.standard_normal((Bt, N, K) if tB else (Bt, K, N))
    bias = rng.standard_normal((Bt, N))
    shape = {'sdd': A.shape[1:], 'dsd': B.shape[1:], 'dds': (M, N)}[mode]
    mask = ops.block_mask(shape, (2, 2), 0.5, seed=6)
    got = ops.matmul_reference(A, B, bias, mode=mode, transpose_A=tA, transpose_B=tB, mask=mask,
                               block=(2, 2), dtype=np.float64)
    for b, m, n in itertools.product(range(Bt), range(M), range(N)):
        total = 0.0
        for k in range(K):
            a = A[b, k, m] if tA else A[b, m, k]
            w = B[b, n, k] if tB else B[b, k, n]
            if mode == 'sdd':
                a *= mask[k, m] if tA else mask[m, k]
            if mode == 'dsd':
                w *= mask[n, k] if tB else mask[k, n]
            total += a * w
        total += bias[b, n]
        if mode == 'dds':
            total *= mask[m, n]
        assert abs(got[b, m, n] - total) < 1e-12


def test_matmul_special_cases():
    rng = np.random.default_rng(7)
    A = rng.standard_normal((1, 8, 8))
    B = rng.standard_normal((1, 8, 8))
    ones = np.ones((8, 8), dtype=np.uint8)
    full = ops.matmul_reference(A, B, None, mode='dsd', transpose_A=False, transpose_B=False, mask=ones,
                                dtype=np.float64)
    np.testing.assert_allclose(full, A @ B, rtol=1e-12)
    eye = np.eye(8)[None]
    mask = ops.block_mask((8, 8), (2, 2), 0.5, seed=8)
    masked_copy = ops.matmul_reference(A, eye, None, mode='sdd', transpose_A=False, transpose_B=False,
                                       mask=mask, dtype=np.float64)
    np.testing.assert_allclose(masked_copy, A * mask, rtol=1e-12)
    # dds with a finer mask than the block: the whole live block survives
    fine = np.zeros((8, 8), dtype=np.uint8)
    fine[0, 0] = 1
    out = ops.matmul_reference(A, B, None, mode='dds', transpose_A=False, transpose_B=False, mask=fine,
                               block=(4, 4), dtype=np.float64)
    np.testing.assert_allclose(out[0, :4, :4], (A @ B)[0, :4, :4], rtol=1e-12)
    assert not out[0, 4:, :].any() and not out[0, :, 4:].any()


# ------------------------------------------------------------------ softmax --
def test_softmax_special_cases():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 5, 16)) * 3
    ones = np.ones((5, 16), dtype=np.uint8)
    np.testing.assert_allclose(ops.softmax_forward_reference(x, ones, 2.0),
                               scipy.special.softmax(x / 2.0, axis=-1), rtol=1e-9)
    mask = ops.block_mask((5, 16), (1, 1), 0.6, seed=10)
    mask[2] = 0
    y = ops.softmax_forward_reference(x, mask, 1.5)
    assert not y[:, 2].any()                       # fully masked row -> 0
    assert not y[:, mask == 0].any()               # masked entries -> 0
    live_rows = mask.any(axis=1)
    np.testing.assert_allclose(y.sum(-1)[:, live_rows], 1.0, rtol=1e-8)
    np.testing.assert_allclose(ops.softmax_forward_reference(x + 11.0, mask, 1.5), y, rtol=1e-9)
    # equals a softmax over the live entries only
    for r in np.nonzero(live_rows)[0]:
        sel = mask[r] != 0
        np.testing.assert_allclose(y[0, r, sel], scipy.special.softmax(x[0, r, sel] / 1.5), rtol=1e-8)


def test_softmax_backward_finite_difference():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 12))
    g = rng.standard_normal((4, 12))
    mask = ops.block_mask((4, 12), (1, 1), 0.4, seed=12)
    T = 1.7
    y = ops.softmax_forward_reference(x, mask, T)
    gx = ops.softmax_backward_reference(g, y, mask, T)
    eps = 1e-6
    for r, c in itertools.product(range(4), range(12)):
        xp, xm = x.copy(), x.copy()
        xp[r, c] += eps
        xm[r, c] -= eps
        num = ((ops.softmax_forward_reference(xp, mask, T) - ops.softmax_forward_reference(xm, mask, T)) * g).sum() / (2 * eps)
        want = num if mask[r, c] else 0.0   # the reference zeroes the gradient of masked inputs
        assert abs(gx[r, c] - want) < 1e-6


# ---------------------------------------------------------- attention / moe --
def test_attention_all_ones_is_textbook():
    rng = np.random.default_rng(13)
    q, k, v = (rng.standard_normal((2, 6, 4)) for _ in range(3))
    out = ops.attention_reference(q, k, v, np.ones((6, 6), dtype=np.uint8))
    for b, i in itertools.product(range(2), range(6)):
        scores = np.array([q[b, i] @ k[b, j] for j in range(6)]) / 2.0  # sqrt(E) = 2
        p = np.exp(scores - scores.max())
        p /= p.sum()
        np.testing.assert_allclose(out[b, i], sum(p[j] * v[b, j] for j in range(6)), rtol=1e-8)


def test_attention_masked_tiny_brute_force():
    """Pure-Python loops over a random element mask (some rows fully masked, an explicit
    temperature and the default sqrt(E)): live keys only in the sum, the maximum taken
    over all keys as the reference's softmax does (sparta/testing/math.py:24), masked
    rows exactly zero (the 1e-10 in the denominator makes them 0 / 1e-10)."""
    import math
    rng = np.random.default_rng(21)
    B, Nt, Ns, E = 2, 5, 7, 3
    q, k, v = rng.standard_normal((B, Nt, E)), rng.standard_normal((B, Ns, E)), rng.standard_normal((B, Ns, E))
    mask = (rng.random((Nt, Ns)) < 0.5).astype(np.uint8)
    mask[3] = 0
    for temperature in (None, 0.7):
        T = math.sqrt(E) if temperature is None else temperature
        out = ops.attention_reference(q, k, v, mask, temperature=temperature)
        for b in range(B):
            for i in range(Nt):
                s = [sum(q[b, i, e] * k[b, j, e] for e in range(E)) for j in range(Ns)]
                top = max(s)
                w = [math.exp((s[j] - top) / T) if mask[i, j] else 0.0 for j in range(Ns)]
                tot = sum(w)
                for e in range(E):
                    want = sum(w[j] * v[b, j, e] for j in range(Ns)) / (tot + 1e-10)  # math.py:27
                    assert abs(out[b, i, e] - want) < 1e-12
        assert np.all(out[:, 3] == 0.0)


def test_moe_reference_properties():
    rng = np.random.default_rng(14)
    tokens = rng.standard_normal((10, 6))
    weights = rng.standard_normal((3, 6, 5))
    ids = rng.integers(0, 3, 10)
    out = ops.moe_reference(tokens, weights, ids)
    for t in range(10):
        np.testing.assert_allclose(out[t], tokens[t] @ weights[ids[t]], rtol=1e-12)
    perm = rng.permutation(10)
    np.testing.assert_allclose(ops.moe_reference(tokens[perm], weights, ids[perm]), out[perm], rtol=1e-12)
    np.testing.assert_allclose(ops.moe_reference(tokens, weights[:1], np.zeros(10, dtype=int)),
                               tokens @ weights[0], rtol=1e-12)
    count, offset, order = ops.moe_index_reference(ids.astype(np.int32), 3)
    assert count.tolist() == [int((ids == e).sum()) for e in range(3)]
    assert offset.tolist() == [0] + np.cumsum(count).tolist()
    for e in range(3):
        assert order[offset[e]:offset[e + 1]].tolist() == [t for t in range(10) if ids[t] == e]


def test_block_mask_shape_and_density():
    m = ops.block_mask((128, 256), (8, 16), 0.75, seed=1)
    assert m.shape == (128, 256) and m.dtype == np.uint8
    tiles = m.reshape(16, 8, 16, 16).swapaxes(1, 2)
    assert ((tiles.min(axis=(2, 3)) == tiles.max(axis=(2, 3)))).all()  # blocks are uniform
    assert 0.1 < m.mean() < 0.4
