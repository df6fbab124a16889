"""GPU parity of the MoE path against the numpy oracle: the token->expert index
bit-exact (stable order), the gathered GEMM within tolerance.  Base case from the
reference's test/unit/test_sparse_moe.py (4096 tokens, 8 experts, 3072 -> 768,
fp16 and fp32, three routings), plus skewed routing, empty experts and ragged
token counts."""
import os

import numpy as np
import pytest
import torch

from oracle import ops
from sparta_amd.nn import DynamicSparseMoE
from helpers import assert_close

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'vectors.npz'))


def make_moe(n_exp, in_dims, out_dims, dtype, gpu, seed=2022, scale=0.05):
    rng = np.random.default_rng(seed)
    w = torch.from_numpy(rng.standard_normal((n_exp, out_dims, in_dims)).astype(np.float32) * scale).to(dtype)
    mods = []
    for e in range(n_exp):
        lin = torch.nn.Linear(in_dims, out_dims, bias=False, dtype=dtype, device=gpu)
        with torch.no_grad():
            lin.weight.copy_(w[e].to(gpu))
        mods.append(lin)
    weights_np = w.to(torch.float64).numpy().transpose(0, 2, 1)  # [E, in, out]
    return DynamicSparseMoE(mods), weights_np


def check_forward(moe, weights_np, n_tok, ids_np, dtype, gpu, seed):
    rng = np.random.default_rng(seed)
    data = torch.from_numpy(rng.random((n_tok, weights_np.shape[1]), dtype=np.float32)).to(dtype)
    out = moe(data.to(gpu), torch.from_numpy(ids_np).to(gpu))
    count, offset, perm = ops.moe_index_reference(ids_np, weights_np.shape[0])
    assert np.array_equal(moe.expert_count.cpu().numpy(), count)
    assert np.array_equal(moe.expert_offset.cpu().numpy(), offset)
    assert np.array_equal(moe.sparse_index[:n_tok].cpu().numpy(), perm)
    want = ops.moe_reference(data.to(torch.float64).numpy(), weights_np, ids_np)
    assert out.dtype == dtype and tuple(out.shape) == want.shape
    assert_close(out, want, dtype, f'moe {dtype} n_tok={n_tok}')


@pytest.mark.parametrize('dtype', [torch.float16, torch.float32, torch.bfloat16])
def test_moe_reference_case(dtype, gpu):
    moe, w = make_moe(8, 3072, 768, dtype, gpu)
    for seed in range(3):  # dynamic routing: a new assignment every call
        ids = np.random.default_rng(seed).integers(0, 8, 4096).astype(np.int32)
        check_forward(moe, w, 4096, ids, dtype, gpu, seed)


def test_moe_zipf_skew_exceeds_reference_capacity(gpu):
    """Zipf(1.2) routing: the busiest expert gets more than the 4096-token capacity
    the reference hard-codes (sparse_moe.py:23)."""
    n_tok, n_exp = 16384, 8
    p = np.arange(1, n_exp + 1, dtype=np.float64) ** -1.2
    ids = np.random.default_rng(2022).choice(n_exp, size=n_tok, p=p / p.sum()).astype(np.int32)
    assert np.bincount(ids).max() > 4096
    moe, w = make_moe(n_exp, 256, 512, torch.float16, gpu)
    check_forward(moe, w, n_tok, ids, torch.float16, gpu, 1)


@pytest.mark.parametrize('n_tok', [1, 100, 1000, 1025, 3000])
def test_moe_ragged_token_counts_and_empty_experts(n_tok, gpu):
    n_exp = 6
    moe, w = make_moe(n_exp, 128, 136, torch.float16, gpu)
    ids = np.random.default_rng(n_tok).choice([0, 2, 5], size=n_tok).astype(np.int32)  # experts 1,3,4 stay empty
    check_forward(moe, w, n_tok, ids, torch.float16, gpu, 2)


def test_moe_single_expert_is_one_gemm(gpu):
    moe, w = make_moe(1, 256, 256, torch.float32, gpu)
    check_forward(moe, w, 512, np.zeros(512, dtype=np.int32), torch.float32, gpu, 3)


def test_moe_many_experts(gpu):
    n_exp = 200
    moe, w = make_moe(n_exp, 64, 64, torch.float16, gpu, scale=0.1)
    ids = np.random.default_rng(7).integers(0, n_exp, 5000).astype(np.int32)
    check_forward(moe, w, 5000, ids, torch.float16, gpu, 4)


def test_moe_golden_vectors(gpu):
    tokens, weights, ids = GOLD['moe_tokens'], GOLD['moe_weights'], GOLD['moe_ids']
    mods = []
    for e in range(weights.shape[0]):
        lin = torch.nn.Linear(64, 48, bias=False, dtype=torch.float16, device=gpu)
        with torch.no_grad():
            lin.weight.copy_(torch.from_numpy(weights[e].T.copy()).to(gpu))
        mods.append(lin)
    moe = DynamicSparseMoE(mods)
    out = moe(torch.from_numpy(tokens).half().to(gpu), torch.from_numpy(ids).to(gpu))
    assert np.array_equal(moe.sparse_index[:96].cpu().numpy(), GOLD['moe_perm'])
    assert np.array_equal(moe.expert_offset.cpu().numpy(), GOLD['moe_offset'])
    assert_close(out, GOLD['moe_out'], torch.float16, 'moe golden')

@pytest.mark.parametrize('n_tok,n_exp', [
    (700, 3),          # 256-token chunks, count table scanned by the placement workgroups
    (16384, 8),        # 64 chunks x 9 counts
    (50000, 8),        # 512-token chunks
    (100000, 8),       # 1024-token chunks, still within the 1024-entry table
    (4096, 200),       # many experts: 1024-token chunks, 4 x 201 counts
    (200000, 8),       # table too large: separate scan launch
    (30000, 200),      # separate scan launch, many experts
    (257, 1),
])
def test_moe_index_launch_paths(n_tok, n_exp, gpu):
    """spx_moe_index through the C ABI on routings that take every chunk size of the
    two-launch path and the three-launch path, ids outside [0, n_exp) included: counts,
    offsets and the stable permutation are bit-exact against the oracle."""
    from sparta_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(n_tok + n_exp)
    p = np.arange(1, n_exp + 1, dtype=np.float64) ** -1.2
    ids_np = rng.choice(n_exp, size=n_tok, p=p / p.sum()).astype(np.int32)
    bad = rng.random(n_tok) < 0.01
    ids_np[bad] = rng.choice([-3, n_exp, n_exp + 7], size=int(bad.sum()))
    ids = torch.from_numpy(ids_np).to(gpu)
    count = torch.full((n_exp,), -1, dtype=torch.int32, device=gpu)
    offset = torch.full((n_exp + 1,), -1, dtype=torch.int32, device=gpu)
    perm = torch.full((n_tok,), -1, dtype=torch.int32, device=gpu)
    ws = torch.empty(max(lib.spx_moe_index_workspace_bytes(n_tok, n_exp), 256), dtype=torch.uint8, device=gpu)
    for _ in range(2):  # the workspace is reused as it was left
        _lib.check(lib.spx_moe_index(_lib.dev_ptr(ids), n_tok, n_exp, _lib.dev_ptr(count), _lib.dev_ptr(offset),
                                     _lib.dev_ptr(perm), _lib.dev_ptr(ws), ws.numel(), _lib.current_stream(gpu)),
                   'spx_moe_index')
    valid = (ids_np >= 0) & (ids_np < n_exp)
    key = np.where(valid, ids_np, n_exp)                  # out-of-range ids sort behind every expert
    want_count = np.bincount(key, minlength=n_exp + 1)[:n_exp].astype(np.int32)
    want_offset = np.zeros(n_exp + 1, dtype=np.int32)
    np.cumsum(want_count, out=want_offset[1:])
    want_perm = np.argsort(key, kind='stable').astype(np.int32)
    c2, o2, p2 = ops.moe_index_reference(ids_np[valid], n_exp)
    assert np.array_equal(want_count, c2) and np.array_equal(want_offset, o2)   # the oracle on the valid ids
    assert np.array_equal(count.cpu().numpy(), want_count)
    assert np.array_equal(offset.cpu().numpy(), want_offset)
    assert np.array_equal(perm.cpu().numpy(), want_perm)
    assert np.array_equal(np.flatnonzero(valid)[p2], want_perm[:int(valid.sum())])


def test_moe_weight_layouts_agree(gpu):
    """The [E, in, out] layout of the reference's stacked weight (what the operator feeds
    the kernels) gives the same result as an [E, out, in] copy of it."""
    from sparta_amd import _lib
    moe, w = make_moe(4, 128, 256, torch.float16, gpu)
    ids = torch.from_numpy(np.random.default_rng(0).integers(0, 4, 700).astype(np.int32)).to(gpu)
    x = torch.rand((700, 128), dtype=torch.float16, device=gpu)
    want = moe(x, ids)
    out = torch.empty_like(want)
    w_nk = moe.weight.detach().transpose(1, 2).contiguous()
    rc = _lib.load().spx_moe_forward(_lib.F16, _lib.dev_ptr(x), _lib.dev_ptr(w_nk), 1,
                                     _lib.dev_ptr(out), _lib.dev_ptr(moe.expert_offset),
                                     _lib.dev_ptr(moe.sparse_index), 700, 128, 256, 4, 0,
                                     _lib.current_stream(gpu))
    _lib.check(rc, 'spx_moe_forward')
    assert torch.equal(out, want)


def test_moe_follows_in_place_weight_updates(gpu):
    """The operator reads its stacked parameter at every call: writes through `.data`
    (which do not advance the version counter), `.half()` and optimizer-style updates
    all show up in the next forward."""
    moe, w = make_moe(3, 128, 136, torch.float32, gpu)
    ids_np = np.random.default_rng(3).integers(0, 3, 300).astype(np.int32)
    check_forward(moe, w, 300, ids_np, torch.float32, gpu, 5)
    with torch.no_grad():
        moe.weight.data.mul_(-0.5)
        moe.weight.data[1].add_(0.25)
    w2 = w * -0.5
    w2[1] += 0.25
    check_forward(moe, w2, 300, ids_np, torch.float32, gpu, 6)
    moe.half()
    w3 = moe.weight.detach().to(torch.float64).cpu().numpy()
    check_forward(moe, w3, 300, ids_np, torch.float16, gpu, 7)


def test_moe_out_of_range_ids_give_zero_rows(gpu):
    """Tokens whose expert id is negative or >= n_exp (the reference indexes out of bounds
    for them) get zero output rows and are listed, ascending, behind the routed tokens."""
    n_exp, n_tok = 4, 1000
    moe, w = make_moe(n_exp, 128, 256, torch.float16, gpu)
    rng = np.random.default_rng(11)
    ids_np = rng.integers(0, n_exp, n_tok).astype(np.int32)
    bad = rng.choice(n_tok, 77, replace=False)
    ids_np[bad[:40]] = -3
    ids_np[bad[40:]] = n_exp + 2
    data = torch.from_numpy(rng.random((n_tok, 128), dtype=np.float32)).half()
    out = torch.full((n_tok, 256), float('nan'), dtype=torch.float16, device=gpu)
    got = moe(data.to(gpu), torch.from_numpy(ids_np).to(gpu))
    valid = (ids_np >= 0) & (ids_np < n_exp)
    want = np.zeros((n_tok, 256))
    want[valid] = ops.moe_reference(data.to(torch.float64).numpy()[valid], w, ids_np[valid])
    assert_close(got, want, torch.float16, 'moe with out-of-range ids')
    assert float(got[torch.from_numpy(~valid).to(gpu)].abs().max()) == 0.0
    offset = moe.expert_offset.cpu().numpy()
    assert offset[n_exp] == valid.sum()
    assert np.array_equal(moe.sparse_index[offset[n_exp]:n_tok].cpu().numpy(), np.sort(bad))


@pytest.mark.parametrize('layout', [0, 1])
@pytest.mark.parametrize('tile_cfg', [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize('dtype,n_tok,in_dims,out_dims', [
    (torch.float16, 3000, 256, 520), (torch.bfloat16, 1500, 128, 256), (torch.float32, 700, 96, 136),
    (torch.float16, 5, 64, 64), (torch.float16, 2500, 192, 776)])
def test_moe_tile_configs(layout, tile_cfg, dtype, n_tok, in_dims, out_dims, gpu):
    """Every gathered-GEMM variant through the C ABI, in both weight layouts, on the same
    routing (one stage, two stages and more; ragged last tiles in both directions; an
    empty expert)."""
    from sparta_amd import _lib
    if dtype == torch.float32 and layout == 0 and tile_cfg != 1:
        pytest.skip('fp32 weights stored [E, in, out] run through tile config 1')
    if dtype == torch.float32 and tile_cfg == 6:
        pytest.skip('the cross-stage pipelined configuration takes 16-bit types')
    n_exp = 5
    moe, w = make_moe(n_exp, in_dims, out_dims, dtype, gpu)
    ids_np = np.random.default_rng(n_tok).choice([0, 1, 2, 4], size=n_tok, p=[0.6, 0.2, 0.15, 0.05]).astype(np.int32)
    x = torch.from_numpy(np.random.default_rng(1).random((n_tok, in_dims), dtype=np.float32)).to(dtype)
    xg = x.to(gpu)
    moe(xg, torch.from_numpy(ids_np).to(gpu))  # builds the index
    weight = moe.weight.detach() if layout == 0 else moe.weight.detach().transpose(1, 2).contiguous()
    out = torch.full((n_tok, out_dims), float('nan'), dtype=dtype, device=gpu)
    rc = _lib.load().spx_moe_forward(_lib.dtype_code(dtype), _lib.dev_ptr(xg), _lib.dev_ptr(weight), layout,
                                     _lib.dev_ptr(out), _lib.dev_ptr(moe.expert_offset),
                                     _lib.dev_ptr(moe.sparse_index), n_tok, in_dims, out_dims, n_exp, tile_cfg,
                                     _lib.current_stream(gpu))
    _lib.check(rc, 'spx_moe_forward')
    want = ops.moe_reference(x.to(torch.float64).numpy(), w, ids_np)
    assert_close(out, want, dtype, f'moe tile config {tile_cfg} layout {layout} {dtype}')
