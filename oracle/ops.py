"""Numpy restatement of the reference's masked-dense operator semantics
(the results every HIP kernel must match)."""
import numpy as np

from . import bcs


def block_mask(shape, block=(1, 1), sparsity=0.99, seed=0):
    """uint8 mask, blocks dropped i.i.d. with probability `sparsity`
    (sparta/testing/mask.py:9-60: `(rand(block_grid) > sparsity)` expanded)."""
    H, W = shape
    assert H % block[0] == 0 and W % block[1] == 0
    rng = np.random.default_rng(seed)
    grid = (rng.random((H // block[0], W // block[1])) > sparsity).astype(np.uint8)
    return bcs.expand_block_mask(grid, block[0], block[1])


def matmul_reference(A, B, bias=None, *, mode, transpose_A, transpose_B, mask, block=None,
                     dtype=np.float32):
    """Masked-dense batched matmul (sparta/specializer/kernels/matmul.py:211-227).

    A: [Bt, K, M] if transpose_A else [Bt, M, K]; B: [Bt, N, K] if transpose_B
    else [Bt, K, N]; bias [Bt, N].  'sdd' masks A elementwise, 'dsd' masks B
    elementwise, 'dds' multiplies C by the *block-expanded* mask of `block`
    (the "DDS known issue", matmul.py:222-226) or by `mask` itself if block is
    None.
    """
    A = A.astype(dtype)
    B = B.astype(dtype)
    if mode == 'sdd':
        A = A * mask
    elif mode == 'dsd':
        B = B * mask
    lhs = np.swapaxes(A, -1, -2) if transpose_A else A   # [Bt, M, K]
    rhs = np.swapaxes(B, -1, -2) if transpose_B else B   # [Bt, K, N]
    C = np.matmul(lhs, rhs)
    if bias is not None:
        C = C + bias.astype(dtype)[:, None, :]
    if mode == 'dds':
        if block is not None:
            live = bcs.reduce_block_mask(mask, *block)
            C = C * bcs.expand_block_mask(live, *block)
        else:
            C = C * mask
    return C


def softmax_forward_reference(x, mask, temperature=1.0):
    """sparta/testing/math.py:8-27: max over ALL entries, exp masked, +1e-10."""
    x = x.astype(np.float64)
    c_max = x.max(axis=-1, keepdims=True)
    c_exp = np.exp((x - c_max) / temperature) * mask
    return c_exp / (c_exp.sum(axis=-1, keepdims=True) + 1e-10)


def softmax_backward_reference(grad, output, mask, temperature=1.0):
    """sparta/testing/math.py:30-50."""
    mo = output.astype(np.float64) * mask
    prod = grad.astype(np.float64) * mo
    return (prod - mo * prod.sum(axis=-1, keepdims=True)) / temperature


def attention_reference(q, k, v, mask, temperature=None):
    """sparta/testing/math.py:53-79; temperature defaults to sqrt(E)."""
    if temperature is None:
        temperature = np.sqrt(q.shape[-1])
    q = q.astype(np.float64)
    k = k.astype(np.float64)
    v = v.astype(np.float64)
    qk = np.einsum('...mk,...nk->...mn', q, k)
    sm = softmax_forward_reference(qk, mask, temperature)
    return np.einsum('...mn,...nk->...mk', sm, v)


def moe_reference(tokens, weights, exp_ids):
    """test/unit/test_sparse_moe.py:17-27 with bias-free experts.
    weights: [n_exp, in, out] (sparse_moe.py:19-22 stacks weight.T)."""
    out = np.zeros((tokens.shape[0], weights.shape[2]), dtype=np.float64)
    for e in range(weights.shape[0]):
        sel = exp_ids == e
        out[sel] = tokens[sel].astype(np.float64) @ weights[e].astype(np.float64)
    return out


def moe_index_reference(exp_ids, n_exp):
    """Stable counting sort of tokens by expert: count[e], offset[e] (exclusive
    prefix), perm[offset[e] + j] = j-th token (ascending) routed to e.
    The reference's convert_sparse_index
    (csrc/moe_sparse_forward_kernel.cu.j2:58-71) stores the same sets in
    atomic-arrival order; ascending order is its deterministic representative."""
    count = np.bincount(exp_ids, minlength=n_exp).astype(np.int32)
    offset = np.zeros(n_exp + 1, dtype=np.int32)
    np.cumsum(count, out=offset[1:])
    perm = np.argsort(exp_ids, kind='stable').astype(np.int32)
    return count, offset, perm
