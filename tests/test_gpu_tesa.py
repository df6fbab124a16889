"""GPU parity of the index builder and the converters against the numpy oracle
(bit-exact).  Shapes follow the reference's test/unit/test_tesa.py (1024x768
element-granular mask at 99.9% sparsity, every block shape in {4..128}^2) plus
the benchmark configurations."""
import numpy as np
import pytest
import torch

from oracle import bcs, ops
from sparta_amd.tesa import get_bcs_function

pytestmark = pytest.mark.gpu

EDGES = [4, 8, 16, 32, 64, 128]


def _check_launch_order(order, ptr):
    """The scheduling hint that comes out of the index launch: a permutation of the
    segments, longest first (lengths are bucketed at 255)."""
    order = order.cpu().numpy()
    n = len(ptr) - 1
    assert order.dtype == np.int32 and np.array_equal(np.sort(order), np.arange(n))
    lengths = np.minimum(np.diff(ptr)[order], 255)
    assert np.all(lengths[:-1] >= lengths[1:])


def test_launch_order_matches_standalone_schedule(gpu):
    """spx_bcs_index_scheduled and spx_bcs_schedule sort the same way (a grid large
    enough for the general emit kernel and a small one for the fast one)."""
    from sparta_amd import _lib
    for shape, blk in (((4096, 8192), (4, 4)), ((512, 768), (32, 32))):
        mask_np = ops.block_mask(shape, blk, 0.9, seed=5)
        idx = get_bcs_function(blk[0], blk[1], True, True).build_indexes(torch.from_numpy(mask_np).to(gpu))
        for by, ptr in (('row', idx.row_ptr), ('col', idx.col_ptr)):
            n = ptr.numel() - 1
            alone = torch.empty((n,), dtype=torch.int32, device=gpu)
            _lib.check(_lib.load().spx_bcs_schedule(_lib.dev_ptr(ptr), n, _lib.dev_ptr(alone), _lib.current_stream(gpu)),
                       'spx_bcs_schedule')
            ptr_np = ptr.cpu().numpy()
            _check_launch_order(idx.launch_order(by), ptr_np)
            _check_launch_order(alone, ptr_np)
            fused_len = np.minimum(np.diff(ptr_np)[idx.launch_order(by).cpu().numpy()], 255)
            alone_len = np.minimum(np.diff(ptr_np)[alone.cpu().numpy()], 255)
            assert np.array_equal(fused_len, alone_len)


def _check_indexes(mask_np, BH, BW, gpu):
    mask = torch.from_numpy(mask_np).to(gpu)
    H, W = mask_np.shape
    row_ptr, bcsr, col_ptr, bcsc64, nnz = bcs.build_bcsrc(mask_np, BH, BW)
    _, bcsc32, _ = bcs.build_bcsc(mask_np, BH, BW)

    r = get_bcs_function(BH, BW, True, False).build_indexes(mask)
    assert r.block_nnz == nnz
    assert np.array_equal(r.row_ptr.cpu().numpy(), row_ptr)
    assert np.array_equal(r.BCSR_idx.cpu().numpy(), bcsr)
    assert r.row_ptr.dtype == torch.int32 and r.BCSR_idx.dtype == torch.int32

    c = get_bcs_function(BH, BW, False, True).build_indexes(mask)
    assert c.block_nnz == nnz
    assert np.array_equal(c.col_ptr.cpu().numpy(), col_ptr)
    assert np.array_equal(c.BCSC_idx.cpu().numpy(), bcsc32)
    assert c.BCSC_idx.dtype == torch.int32

    _check_launch_order(r.launch_order('row'), row_ptr)
    _check_launch_order(c.launch_order('col'), col_ptr)

    rc = get_bcs_function(BH, BW, True, True).build_indexes(mask)
    _check_launch_order(rc.launch_order('row'), row_ptr)
    _check_launch_order(rc.launch_order('col'), col_ptr)
    assert rc.block_nnz == nnz
    assert np.array_equal(rc.row_ptr.cpu().numpy(), row_ptr)
    assert np.array_equal(rc.col_ptr.cpu().numpy(), col_ptr)
    assert np.array_equal(rc.BCSR_idx.cpu().numpy(), bcsr)
    assert np.array_equal(rc.BCSC_idx.cpu().numpy(), bcsc64)
    assert rc.BCSC_idx.dtype == torch.int64
    live = bcs.reduce_block_mask(mask_np, BH, BW)
    for idx in (r, c, rc):
        assert np.array_equal(idx.get_block_mask().cpu().numpy().astype(bool), live)
    return r, c, rc


def test_index_batch_equals_single_builds(gpu):
    """spx_bcs_index_batch: several masks in one call - different shapes, block sizes and
    formats, more jobs than share one pair of launches, a mask whose width rules out the
    bit-word path (built on its own inside the call), an empty mask and a full one - give
    exactly the indexes of one build_indexes call each, against the oracle as well."""
    from sparta_amd.tesa import build_indexes_batch
    cases = [((3072, 768), (32, 64), True, False, 0.9), ((768, 3072), (32, 64), True, False, 0.9),
             ((1024, 768), (8, 8), True, True, 0.8), ((256, 4096), (64, 16), False, True, 0.5),
             ((512, 520), (8, 8), True, True, 0.7),          # 520 % 16 != 0: general path
             ((4096, 4096), (32, 32), True, True, 0.95), ((64, 64), (32, 32), True, False, 0.0)]
    requests, masks = [], []
    for i, (shape, blk, r, c, sparsity) in enumerate(cases):
        mask_np = ops.block_mask(shape, blk, sparsity, seed=70 + i)
        if i == 2:
            mask_np[:] = 0
        masks.append(mask_np)
        requests.append((get_bcs_function(blk[0], blk[1], r, c), torch.from_numpy(mask_np).to(gpu)))
    batch = build_indexes_batch(requests)
    assert len(batch) == len(cases)
    for (ctx, mask), got, mask_np, (shape, blk, r, c, _) in zip(requests, batch, masks, cases):
        want = ctx.build_indexes(mask)
        assert type(got) is type(want) and got.block_nnz == want.block_nnz
        row_ptr, bcsr, col_ptr, bcsc64, nnz = bcs.build_bcsrc(mask_np, blk[0], blk[1])
        assert got.block_nnz == nnz
        if r:
            assert np.array_equal(got.row_ptr.cpu().numpy(), row_ptr)
            assert np.array_equal(got.BCSR_idx.cpu().numpy()[:nnz], bcsr)
            assert torch.equal(got.BCSR_idx[:nnz], want.BCSR_idx[:nnz])
            _check_launch_order(got.launch_order('row'), row_ptr)
        if c:
            assert np.array_equal(got.col_ptr.cpu().numpy(), col_ptr)
            assert torch.equal(got.BCSC_idx[:nnz], want.BCSC_idx[:nnz])
            _check_launch_order(got.launch_order('col'), col_ptr)
        if r and c:
            assert np.array_equal(got.BCSC_idx.cpu().numpy()[:nnz], bcsc64)
    assert build_indexes_batch([]) == []


@pytest.mark.parametrize('BH', EDGES)
@pytest.mark.parametrize('BW', EDGES)
def test_index_reference_shapes(BH, BW, gpu):
    mask_np = ops.block_mask((1024, 768), (1, 1), 0.999, seed=2023)
    r, c, rc = _check_indexes(mask_np, BH, BW, gpu)
    # convert / inverse / sum against the oracle, fp32, batch 2
    dense_np = (np.random.default_rng(1).random((2, 1024, 768), dtype=np.float32) * mask_np)
    dense = torch.from_numpy(dense_np).to(gpu)
    for idx, fmt, arr in ((r, 'bcsr', r.BCSR_idx), (c, 'bcsc', c.BCSC_idx), (rc, 'bcsr', rc.BCSR_idx)):
        want = bcs.convert(dense_np, arr.cpu().numpy(), fmt, BH, BW)
        got = idx.convert(dense)
        assert np.array_equal(got.cpu().numpy(), want)
        assert np.array_equal(idx.inverse(got).cpu().numpy(), dense_np)
        np.testing.assert_allclose(idx.sum(got, axis=-1).cpu().numpy(), dense_np.sum(-1), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(idx.sum(got, axis=-2).cpu().numpy(), dense_np.sum(-2), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('shape,block,gran,sparsity', [
    ((4096, 4096), (32, 32), (32, 32), 0.95),    # 4096^3 headline mask
    ((1024, 1024), (32, 32), (8, 8), 0.90),      # README case, 8x8 granular
    ((1024, 1024), (16, 16), (8, 8), 0.90),
    ((4096, 4096), (64, 64), (64, 64), 0.90),    # attention layout grid
    ((3072, 768), (32, 64), (32, 64), 0.90),     # FFN weights
    ((768, 3072), (32, 64), (32, 64), 0.90),
    ((64, 96), (4, 4), (1, 1), 0.5),
    ((256, 8), (4, 8), (1, 1), 0.9),             # single block column
    ((8, 20), (4, 4), (1, 1), 0.3),              # row pitch not a multiple of 16
    ((4096, 4096), (8, 8), (8, 8), 0.90),        # 4096 row words: the general path, one wavefront per word
    ((2048, 1032), (8, 8), (1, 1), 0.999),       # the same path with 4-byte loads and a partial last word per row
])
def test_index_bench_shapes(shape, block, gran, sparsity, gpu):
    _check_indexes(ops.block_mask(shape, gran, sparsity, seed=2022), block[0], block[1], gpu)


@pytest.mark.parametrize('fill', [0, 1])
def test_index_all_or_nothing(fill, gpu):
    mask_np = np.full((256, 512), fill, dtype=np.uint8)
    r, c, rc = _check_indexes(mask_np, 16, 32, gpu)
    assert r.block_nnz == (16 * 16 if fill else 0)
    x = torch.rand((1, 256, 512), device=gpu)
    assert r.convert(x).shape == (1, r.block_nnz * 16 * 32)


def test_index_single_element_makes_block_live(gpu):
    mask_np = np.zeros((128, 128), dtype=np.uint8)
    mask_np[77, 3] = 1
    mask_np[127, 127] = 255
    r, _, _ = _check_indexes(mask_np, 32, 32, gpu)
    assert r.BCSR_idx.cpu().tolist() == [(2 << 16) | 0, (3 << 16) | 3]


def test_index_is_deterministic(gpu):
    mask = torch.from_numpy(ops.block_mask((2048, 2048), (1, 1), 0.99, seed=5)).to(gpu)
    fn = get_bcs_function(32, 32, True, True)
    first = fn.build_indexes(mask)
    a, b = first.BCSR_idx.clone(), first.BCSC_idx.clone()
    for _ in range(5):
        again = fn.build_indexes(mask)
        assert torch.equal(again.BCSR_idx, a) and torch.equal(again.BCSC_idx, b)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.uint8, torch.float64])
def test_convert_other_element_sizes(dtype, gpu):
    mask_np = ops.block_mask((512, 256), (16, 32), 0.7, seed=3)
    idx = get_bcs_function(16, 32, True, False).build_indexes(torch.from_numpy(mask_np).to(gpu))
    src = (torch.rand((3, 512, 256)) * 100).to(dtype) * torch.from_numpy(mask_np).to(dtype)
    got = idx.convert(src.to(gpu))
    want = bcs.convert(src.view(torch.uint8 if dtype == torch.uint8 else torch.int16 if src.element_size() == 2
                                else torch.int64).numpy(), idx.BCSR_idx.cpu().numpy(), 'bcsr', 16, 32)
    raw = got.cpu().view(torch.uint8 if dtype == torch.uint8 else torch.int16 if src.element_size() == 2
                         else torch.int64).numpy()
    assert np.array_equal(raw, want)
    assert torch.equal(idx.inverse(got).cpu(), src)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_sum_of_16_bit_values(dtype, gpu):
    """Row and column sums read 16-bit compressed values as they are (fp32 accumulate) for all
    three index flavours."""
    mask_np = ops.block_mask((256, 384), (16, 32), 0.7, seed=91)
    mask = torch.from_numpy(mask_np).to(gpu)
    dense = (torch.randn((3, 256, 384), generator=torch.Generator().manual_seed(92)).to(gpu) * mask).to(dtype)
    for bcsr, bcsc in ((True, False), (False, True), (True, True)):
        idx = get_bcs_function(16, 32, bcsr, bcsc).build_indexes(mask)
        vals = idx.convert(dense)
        for axis in (-1, -2):
            got = idx.sum(vals, axis=axis)
            assert got.dtype == dtype
            want = dense.float().sum(axis)
            torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()))


@pytest.mark.parametrize('at_capacity', [False, True])
def test_sum_over_an_empty_index_is_zero(at_capacity, gpu):
    """No live block: every entry of the result is written as zero, whether the values are an
    empty tensor (static storage) or a buffer kept at index capacity (dynamic masks)."""
    mask = torch.zeros((128, 192), dtype=torch.uint8, device=gpu)
    dense = torch.randn((2, 128, 192), generator=torch.Generator().manual_seed(5)).to(gpu).half()
    for bcsr, bcsc in ((True, False), (False, True), (True, True)):
        idx = get_bcs_function(32, 32, bcsr, bcsc).build_indexes(mask)
        vals = idx.convert(dense, at_capacity=at_capacity)
        assert vals.shape == (2, (idx.capacity if at_capacity else 0) * 32 * 32)
        for axis, n_out in ((-1, 128), (-2, 192)):
            got = idx.sum(vals, axis=axis)
            assert got.shape == (2, n_out)
            assert torch.count_nonzero(got).item() == 0


def test_sum_of_values_kept_at_capacity(gpu):
    """Values stored at index capacity (dynamic masks) have a longer batch stride than the live
    blocks; the sums must follow the stride of the tensor they are given."""
    mask_np = ops.block_mask((128, 192), (32, 32), 0.6, seed=17)
    mask = torch.from_numpy(mask_np).to(gpu)
    dense = (torch.randn((3, 128, 192), generator=torch.Generator().manual_seed(18)).to(gpu) * mask).half()
    idx = get_bcs_function(32, 32, True, True).build_indexes(mask)
    vals = idx.convert(dense, at_capacity=True)
    assert vals.shape[-1] == idx.capacity * 32 * 32 > idx.block_nnz * 32 * 32
    for axis in (-1, -2):
        assert torch.equal(idx.sum(vals, axis=axis), idx.sum(idx.convert(dense), axis=axis))
