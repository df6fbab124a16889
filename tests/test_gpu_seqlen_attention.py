"""GPU parity of SeqlenDynamicSparseAttention against the numpy oracle.  Base case
from the reference's test/unit/test_seqlen_attention.py:21-56 (B=12, H=20, N=256,
E=64, fp32, lengths in [1, N), temperature 1, both global and per-call lengths,
atol 1e-4), plus the 16-bit types, N not a multiple of 64 and the length edge cases."""
import numpy as np
import pytest
import torch

from oracle import ops
from sparta_amd.nn import SeqlenDynamicSparseAttention
from helpers import assert_close

pytestmark = pytest.mark.gpu


def reference(q, k, v, seqlens):
    """The reference test's target: the attention oracle under the prefix-square mask
    of each batch entry, temperature 1; rows at or past the length are fully masked -> 0."""
    B, H, N, E = q.shape
    out = np.zeros((B, H, N, E))
    for b in range(B):
        L = int(seqlens[b])
        mask = np.zeros((N, N), dtype=np.uint8)
        mask[:L, :L] = 1
        out[b] = ops.attention_reference(q[b], k[b], v[b], mask, temperature=1.0)
    return out


def rand_qkv(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    ts = [torch.rand(shape, generator=g).to(dtype) for _ in range(3)]
    return ts, [t.to(torch.float64).numpy() for t in ts]


@pytest.mark.parametrize('global_mode', [False, True])
def test_seqlen_attention_reference_case(global_mode, gpu, B=12, H=20, N=256, E=64):
    att = SeqlenDynamicSparseAttention(global_mode)
    rng = np.random.default_rng(2022)
    seqlens = rng.integers(1, N, size=B).astype(np.int32)
    if global_mode:
        SeqlenDynamicSparseAttention.set_global_seqlens(torch.from_numpy(seqlens).to(gpu))
    for seed in range(3):  # dynamic lengths: new ones every call unless global
        if not global_mode:
            seqlens = np.random.default_rng(seed).integers(1, N, size=B).astype(np.int32)
        (q, k, v), (qn, kn, vn) = rand_qkv((B, H, N, E), seed, torch.float32)
        if global_mode:
            out = att(q.to(gpu), k.to(gpu), v.to(gpu))
        else:
            out = att(q.to(gpu), k.to(gpu), v.to(gpu), torch.from_numpy(seqlens).to(gpu))
        assert_close(out, reference(qn, kn, vn, seqlens), torch.float32, f'seqlen attention seed {seed}')


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('N,E', [(96, 32), (128, 96), (64, 128), (160, 64)])
def test_seqlen_attention_shapes_and_edges(dtype, N, E, gpu, B=5, H=3):
    """Lengths 0 (all rows zero), 1, a multiple of the tile, N - 1 and N."""
    seqlens = np.array([0, 1, 32, N - 1, N], dtype=np.int32)
    (q, k, v), (qn, kn, vn) = rand_qkv((B, H, N, E), 7, dtype)
    att = SeqlenDynamicSparseAttention(global_mode=False)
    out = att(q.to(gpu), k.to(gpu), v.to(gpu), torch.from_numpy(seqlens).to(gpu))
    want = reference(qn, kn, vn, seqlens)
    assert_close(out, want, dtype, f'seqlen attention {dtype} N={N} E={E}')
    assert float(out[0].abs().max()) == 0.0
    assert float(out[1, :, 1:].abs().max()) == 0.0
    # full length = plain softmax attention without scaling
    full = torch.softmax(torch.from_numpy(qn[4] @ kn[4].transpose(0, 2, 1)), -1).numpy() @ vn[4]
    assert_close(out[4], full, dtype, 'full length')


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('N,E', [(256, 64), (192, 128), (96, 128), (1024, 64)])
def test_seqlen_attention_pipelined_kernel_instantiations(dtype, N, E, gpu, H=2):
    """16-bit types with head dim 64 / 128 run the pipelined fused kernel in its
    sequence-length mode: key tiles of 64 (N % 64 == 0) or 32, each shape with several
    key tiles and with lengths that end inside a tile, on a tile edge and one past it."""
    seqlens = np.array([0, 1, 31, 32, 33, 63, 64, 65, N // 2 + 7, N - 1, N], dtype=np.int32)
    seqlens = np.minimum(seqlens, N)
    B = len(seqlens)
    (q, k, v), (qn, kn, vn) = rand_qkv((B, H, N, E), 11, dtype)
    att = SeqlenDynamicSparseAttention(global_mode=False)
    out = att(q.to(gpu), k.to(gpu), v.to(gpu), torch.from_numpy(seqlens).to(gpu))
    want = reference(qn, kn, vn, seqlens)
    assert_close(out, want, dtype, f'seqlen attention (pipelined kernel) {dtype} N={N} E={E}')
    for b, L in enumerate(seqlens):
        assert float(out[b, :, int(L):].abs().max() if L < N else 0.0) == 0.0


def test_seqlen_attention_rejects_bad_input(gpu):
    att = SeqlenDynamicSparseAttention(global_mode=False)
    q = torch.rand((2, 2, 48, 64), device=gpu)
    with pytest.raises(AssertionError):
        att(q, q, q, torch.tensor([3, 4], dtype=torch.int32, device=gpu))          # N % 32
    q = torch.rand((2, 2, 64, 64), device=gpu)
    with pytest.raises(AssertionError):
        att(q, q, q, torch.tensor([3, 4], dtype=torch.int64, device=gpu))          # int32 only
    with pytest.raises(AssertionError):
        att(q, q, q, torch.tensor([3, 4, 5], dtype=torch.int32, device=gpu))       # one length per batch
