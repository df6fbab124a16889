"""CPU tier: the shared library loads and exports the whole C ABI, host-side
argument validation answers before any launch, the Python operator / tuner layer
behaves like the reference's (search-space keys, connections, trial counts), and
the oracle reproduces the committed golden vectors.  Nothing here launches a
kernel."""
import ctypes
import os
import random
import re
import sys

import numpy as np
import pytest
import torch

import sparta_amd as sparta
from sparta_amd import _lib
from sparta_amd.nn import tune, SparseLinear, SparseBatchMatMul, SparseSoftmax, SparseAttention
from oracle import bcs, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, 'tests', 'golden', 'vectors.npz'))


# ---------------------------------------------------------------- C ABI -----------
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, 'include', 'sparta_hip.h')).read()
    header = re.sub(r'/\*.*?\*/', '', header, flags=re.S)
    declared = set(re.findall(r'\b(spx_[a-z_0-9]+)\s*\(', header))
    assert len(declared) >= 15
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f'{name} is declared in sparta_hip.h but not exported'
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    assert lib.spx_version() == 100


def test_host_validation_without_gpu():
    lib = _lib.load()
    assert lib.spx_bcs_index_workspace_bytes(4096, 4096, 32, 32) > 4096 * 4096 // 1024
    assert lib.spx_bcs_index_workspace_bytes(100, 100, 32, 32) == 0
    rc = lib.spx_bcs_index(None, 64, 64, 3, 32, None, None, None, None, 0, None, 0, None, 0, None)
    assert rc == _lib.E_CONFIG and 'power of two' in _lib.last_error()
    rc = lib.spx_bcs_index(None, 64, 60, 32, 32, None, None, None, None, 0, None, 0, None, 0, None)
    assert rc == _lib.E_SHAPE
    rc = lib.spx_bcs_index(None, 64, 64, 32, 32, None, None, None, None, 0, None, 0, None, 0, None)
    assert rc == _lib.E_NULL
    one = ctypes.c_void_p(256)  # never dereferenced: validation fails first
    rc = lib.spx_matmul(7, 0, 0, 1, 1, one, one, None, one, one, one, 0, None, 1, None, 0, 1, 64, 64, 64, 32, 32, 32, 0, None)
    assert rc == _lib.E_CONFIG
    rc = lib.spx_matmul(1, 9, 0, 1, 1, one, one, None, one, one, one, 0, None, 1, None, 0, 1, 64, 64, 64, 32, 32, 32, 0, None)
    assert rc == _lib.E_DTYPE
    rc = lib.spx_matmul(1, 1, 0, 1, 1, one, one, None, one, one, one, 0, None, 1, None, 0, 1, 64, 64, 64, 32, 48, 32, 0, None)
    assert rc == _lib.E_CONFIG
    rc = lib.spx_matmul(1, 1, 0, 1, 1, one, one, None, one, one, one, 0, None, 1, None, 0, 1, 64, 80, 64, 32, 32, 32, 0, None)
    assert rc == _lib.E_SHAPE and 'K=80' in _lib.last_error()
    rc = lib.spx_matmul(1, 1, 0, 1, 1, one, one, None, one, one, one, 1, None, 1, None, 0, 1, 64, 64, 64, 32, 32, 32, 0, None)
    assert rc == _lib.E_CONFIG  # BCSC index handed to a BCSR-mode kernel
    rc = lib.spx_softmax_forward(1, 0, one, one, one, one, one, 1.0, 1, 64, 64, 5, 32, 0, 0, None)
    assert rc == _lib.E_CONFIG
    # attention entry points: dtype, null pointers, shapes and block shapes are checked before any launch
    f16 = _lib.F16
    rc = lib.spx_attention_forward(0, one, one, one, one, one, one, None, 0.125, 1, 256, 256, 64, 64, 64, 0, None)
    assert rc == _lib.E_DTYPE
    rc = lib.spx_attention_forward(f16, one, one, one, one, one, one, None, 0.125, 1, 250, 256, 64, 64, 64, 0, None)
    assert rc == _lib.E_SHAPE
    rc = lib.spx_attention_forward(f16, one, one, None, one, one, one, None, 0.125, 1, 256, 256, 64, 64, 64, 0, None)
    assert rc == _lib.E_NULL
    rc = lib.spx_attention_forward(f16, one, one, one, one, one, one, None, 0.125, 1, 256, 256, 64, 64, 64, 99, None)
    assert rc == _lib.E_CONFIG
    rc = lib.spx_attention_forward_train(f16, one, one, one, one, one, 4096, one, one, None, 0.125, 1, 256, 256, 48, 64, 64, None)
    assert rc == _lib.E_CONFIG and 'head dim' in _lib.last_error()
    rc = lib.spx_attention_forward_train(f16, one, one, one, one, None, 4096, one, one, None, 0.125, 1, 256, 256, 64, 64, 64, None)
    assert rc == _lib.E_NULL
    rc = lib.spx_attention_backward_scores(f16, one, one, one, one, one, None, one, None, 4096, one, one, 0.125, 1, 256, 256, 64, 16, 64, None)
    assert rc == _lib.E_CONFIG
    rc = lib.spx_attention_backward_scores(f16, one, one, one, one, one, one, one, one, 4100, one, one, 0.125, 1, 256, 256, 64, 64, 64, None)
    assert rc == _lib.E_ALIGN
    rc = lib.spx_attention_backward_scores(0, one, one, one, one, one, one, one, one, 4096, one, one, 0.125, 1, 256, 256, 64, 64, 64, None)
    assert rc == _lib.E_DTYPE
    kv = lambda **kw: lib.spx_attention_backward_kv(
        kw.get('dtype', f16), one, one, one, one, kw.get('row_dot', one), one, one, 4096, one, one, kw.get('kind', _lib.IDX_BCSC_I64),
        0.125, 1, 256, 256, kw.get('E', 64), kw.get('BH', 64), kw.get('BW', 64), None)
    assert kv(dtype=0) == _lib.E_DTYPE
    assert kv(row_dot=None) == _lib.E_NULL
    assert kv(kind=_lib.IDX_BCSR_I32) == _lib.E_CONFIG and 'BCSC' in _lib.last_error()
    assert kv(BH=32, BW=128) == _lib.E_CONFIG
    with pytest.raises(AssertionError):
        _lib.check(_lib.E_SHAPE, 'x')
    with pytest.raises(ValueError):
        _lib.check(_lib.E_NULL, 'x')
    with pytest.raises(RuntimeError):
        _lib.check(700, 'x')


def test_host_validation_of_recompute_batch_and_moe_entry_points():
    """Argument checks that come before any launch or device query: they run without a GPU."""
    lib = _lib.load()
    one = ctypes.c_void_p(256)  # never dereferenced
    f16, i64 = _lib.F16, _lib.IDX_BCSC_I64
    lse = lambda dtype=f16, row_lse=one, Nt=256, E=64: lib.spx_attention_forward_lse(
        dtype, one, one, one, one, row_lse, one, one, None, 0.125, 1, Nt, 256, E, 64, 64, None)
    assert lse(dtype=0) == _lib.E_DTYPE
    assert lse(row_lse=None) == _lib.E_NULL and 'row_lse' in _lib.last_error()
    assert lse(Nt=250) == _lib.E_SHAPE
    assert lse(E=48) == _lib.E_CONFIG
    bq = lambda dtype=f16, row_lse=one, BH=64: lib.spx_attention_backward_q(
        dtype, one, one, one, one, one, row_lse, one, one, one, one, 0.125, 1, 256, 256, 64, BH, 64, None)
    assert bq(dtype=0) == _lib.E_DTYPE
    assert bq(row_lse=None) == _lib.E_NULL
    assert bq(BH=16) == _lib.E_CONFIG
    kv = lambda dtype=f16, row_lse=one, kind=i64, BH=64, BW=64: lib.spx_attention_backward_kv_recompute(
        dtype, one, one, one, one, row_lse, one, one, one, one, one, kind, 0.125, 1, 256, 256, 64, BH, BW, None)
    assert kv(dtype=0) == _lib.E_DTYPE
    assert kv(row_lse=None) == _lib.E_NULL
    assert kv(kind=_lib.IDX_BCSR_I32) == _lib.E_CONFIG and 'BCSC' in _lib.last_error()
    assert kv(BH=128, BW=32) == _lib.E_CONFIG and 'BH <= 2 * BW' in _lib.last_error()
    # batched index build: nothing to do, no job array, a job with a bad shape
    assert lib.spx_bcs_index_batch(None, 0, None) == 0
    assert lib.spx_bcs_index_batch(None, 2, None) == _lib.E_NULL
    jobs = (_lib.BcsIndexJob * 2)()
    assert lib.spx_bcs_index_batch(jobs, 2, None) == _lib.E_CONFIG
    jobs[0].H, jobs[0].W, jobs[0].BH, jobs[0].BW = 64, 60, 32, 32
    assert lib.spx_bcs_index_batch(jobs, 1, None) == _lib.E_SHAPE
    # two jobs of one group must not share workspace memory (they run in the same launches)
    jobs[0].workspace, jobs[0].workspace_bytes = 4096, 1024
    jobs[1].workspace, jobs[1].workspace_bytes = 4096 + 512, 1024
    assert lib.spx_bcs_index_batch(jobs, 2, None) == _lib.E_WORKSPACE and 'share workspace' in _lib.last_error()
    # index build on the library's own scratch: limits are checked before the array is looked up
    assert lib.spx_bcs_index_static_max_bytes() == 1 << 20
    rc = lib.spx_bcs_index_static(None, 64, 64, 3, 32, None, None, None, None, 0, None, 0, None)
    assert rc == _lib.E_CONFIG
    rc = lib.spx_bcs_index_static(None, 64, 64, 32, 32, one, one, None, None, 0, one, 4, None)
    assert rc == _lib.E_NULL
    rc = lib.spx_bcs_index_static(one, 65536, 65536, 4, 4, one, one, None, None, 0, one, 1 << 28, None)
    assert rc == _lib.E_WORKSPACE and 'spx_bcs_index' in _lib.last_error()
    # fused activation: sparse-output products have none
    rc = lib.spx_matmul(_lib.DDS, 1, 0, 1, 1, one, one, None, one, one, one, 0, None, 1, None, 0, 1, 64, 64, 64, 32, 32, 32,
                        _lib.EPILOGUE_RELU, None)
    assert rc == _lib.E_CONFIG and 'sdd and dsd' in _lib.last_error()
    # MoE
    moe = lambda dtype=f16, tokens=one, weight=one, layout=1, n_tok=16, in_dim=64, cfg=0: lib.spx_moe_forward(
        dtype, tokens, weight, layout, one, one, one, n_tok, in_dim, 64, 2, cfg, None)
    assert moe(cfg=9) == _lib.E_CONFIG
    assert moe(dtype=7) == _lib.E_DTYPE
    assert moe(in_dim=72) == _lib.E_SHAPE
    assert moe(layout=3) == _lib.E_CONFIG
    assert moe(n_tok=0, tokens=None, weight=None) == 0
    assert moe(weight=None) == _lib.E_NULL
    assert moe(tokens=ctypes.c_void_p(264)) == _lib.E_ALIGN
    assert lib.spx_moe_index_workspace_bytes(1000, 8) >= 9 * 4 and lib.spx_moe_index_workspace_bytes(1000, 0) == 0
    assert lib.spx_moe_index(one, 16, 0, one, one, one, one, 1024, None) == _lib.E_SHAPE
    assert lib.spx_moe_index(one, 1000, 8, one, one, one, one, 16, None) == _lib.E_WORKSPACE
    assert lib.spx_moe_index(one, 1000, 8, None, one, one, one, 1 << 20, None) == _lib.E_NULL


def test_cpu_tensors_are_rejected_loudly():
    with pytest.raises(RuntimeError, match='GPU only'):
        _lib.dev_ptr(torch.zeros(4))


# ------------------------------------------------------- golden vectors / oracle ----
def test_oracle_reproduces_golden_index_vectors():
    for i in range(4):
        H, W, BH, BW, nnz = GOLD[f'idx{i}_meta'].tolist()
        mask = GOLD[f'idx{i}_mask']
        row_ptr, bcsr, col_ptr, bcsc64, n = bcs.build_bcsrc(mask, BH, BW)
        assert n == nnz
        assert np.array_equal(row_ptr, GOLD[f'idx{i}_row_ptr']) and np.array_equal(bcsr, GOLD[f'idx{i}_bcsr'])
        assert np.array_equal(col_ptr, GOLD[f'idx{i}_col_ptr']) and np.array_equal(bcsc64, GOLD[f'idx{i}_bcsc64'])
        assert np.array_equal(bcs.build_bcsc(mask, BH, BW)[1], GOLD[f'idx{i}_bcsc32'])


def test_torch_reference_functions_match_the_oracle():
    """sparta_amd.testing.* (used by the tuner's correctness check) against the
    golden vectors written by the numpy oracle."""
    x, g, mask = (torch.from_numpy(GOLD[k]) for k in ('sm_x', 'sm_g', 'sm_mask'))
    y = sparta.testing.sparse_softmax_forward_reference(x.double(), mask, 8.0)
    np.testing.assert_allclose(y.numpy(), GOLD['sm_y'], rtol=1e-7, atol=1e-9)
    gx = sparta.testing.sparse_softmax_backward_reference(g.double(), y, mask, 8.0)
    np.testing.assert_allclose(gx.numpy(), GOLD['sm_gx'], rtol=1e-7, atol=1e-9)
    q, k, v, amask = (torch.from_numpy(GOLD[n]) for n in ('att_q', 'att_k', 'att_v', 'att_mask'))
    out = sparta.testing.sparse_multi_head_attention_reference(q.double(), k.double(), v.double(), amask)
    np.testing.assert_allclose(out.numpy(), GOLD['att_out'], rtol=1e-7, atol=1e-9)


def test_block_mask_generator():
    torch.manual_seed(0)
    m = sparta.testing.block_mask((64, 128), block=(8, 16), sparsity=0.5, device='cpu')
    assert m.shape == (64, 128) and m.dtype == torch.uint8
    tiles = m.reshape(8, 8, 8, 16).swapaxes(1, 2)
    assert bool((tiles.amin(dim=(2, 3)) == tiles.amax(dim=(2, 3))).all())
    with pytest.raises(AssertionError):
        sparta.testing.block_mask((10, 10), block=(4, 4), device='cpu')
    with pytest.raises(ValueError):
        sparta.testing.block_mask((8, 8), algo='magic', device='cpu')


# ------------------------------------------------------------- operator layer --------
@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('trans_A', [False, True])
@pytest.mark.parametrize('trans_B', [False, True])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('backward', [False, True])
def test_sparse_matmul_search_space(mode, compressed, trans_A, trans_B, backward):
    """Key structure of test/unit/test_search_space.py:31-56."""
    mask = torch.zeros((64, 64))
    port = {'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]
    op = SparseBatchMatMul(**{f'{port}_mask': mask}, transpose_A=trans_A, transpose_B=trans_B,
                           compressed=compressed)
    space = op.get_search_space(backward=backward)
    names = ['forward:C'] + (['backward:A', 'backward:B'] if backward else [])
    assert set(space) == set(names)
    params = {f'BLOCK_SIZE_{d}_VALUE' for d in 'MKN'}
    for kernel_space in space.values():
        assert set(kernel_space) == {'sparta', 'openai'}
        assert set(kernel_space['sparta']) == params and set(kernel_space['openai']) == params
        assert kernel_space['sparta']['BLOCK_SIZE_M_VALUE']._value == [16, 32, 64]
        assert [kernel_space['openai'][f'BLOCK_SIZE_{d}_VALUE']._value for d in 'MKN'] == [[32], [64], [32]]
    connections = op.get_connections(backward=backward)
    assert len(connections) == (2 if compressed and backward else 0)


def test_derived_backward_kernels_of_sparse_linear():
    """SparseLinear(weight_mask) = dsd(tA=F,tB=T); its gradients are
    dsd(tA=F,tB=F) reading a BCSC index and dds(tA=T,tB=F)
    (sparta/specializer/funtional/batch_matmul.py:47-71)."""
    lin = torch.nn.Linear(64, 96)
    op = SparseLinear(lin, weight_mask=torch.ones((96, 64), dtype=torch.uint8))
    ks = op._sparse_ctx._kernels
    k = {n: p.possible_kernels['sparta'] for n, p in ks.items()}
    assert (k['forward:C']._mode, k['forward:C']._transpose_A, k['forward:C']._transpose_B) == ('dsd', False, True)
    assert (k['backward:A']._mode, k['backward:A']._transpose_A, k['backward:A']._transpose_B) == ('dsd', False, False)
    assert (k['backward:B']._mode, k['backward:B']._transpose_A, k['backward:B']._transpose_B) == ('dds', True, False)
    assert k['forward:C']._bcs_mode == 'BCSR' and k['backward:A']._bcs_mode == 'BCSC'
    assert ks['forward:C'].port_map == {'B': 'B'} and ks['backward:A'].port_map == {'B': 'B'}
    assert ks['backward:B'].port_map == {'B': 'C'}
    conn = op.get_connections(backward=True)
    assert conn[0] == {'forward:C': 'BLOCK_SIZE_N_VALUE', 'backward:A': 'BLOCK_SIZE_K_VALUE',
                       'backward:B': 'BLOCK_SIZE_M_VALUE'}
    assert conn[1] == {'forward:C': 'BLOCK_SIZE_K_VALUE', 'backward:A': 'BLOCK_SIZE_N_VALUE',
                       'backward:B': 'BLOCK_SIZE_N_VALUE'}


def _count_trials(module, sample_inputs, sample_grads=None):
    calls = {'n': 0}

    def debug_func(idx, params):
        calls['n'] += 1
        return random.random()

    try:
        tune(module, sample_inputs=sample_inputs, sample_grads=sample_grads, algo='grid',
             max_trials=sys.maxsize, backward_weight=0 if sample_grads is None else 0.5,
             verbose=False, debug_func=debug_func)
    except AssertionError:
        pass
    return calls['n']


@pytest.mark.parametrize('backward', [False, True])
def test_tuner_trial_counts(backward):
    """Trial counts of test/unit/test_tuners.py with a fake measurement."""
    grads = lambda *shape: [torch.zeros(shape)] if backward else None
    lin = SparseLinear(torch.nn.Linear(128, 128), weight_mask=torch.ones((128, 128), dtype=torch.uint8))
    assert _count_trials(lin, [torch.zeros((128, 128))], grads(128, 128)) == (27 + 1) * (3 if backward else 1)
    mm = SparseBatchMatMul(C_mask=torch.ones((128, 128), dtype=torch.uint8), transpose_A=False,
                           transpose_B=True, compressed=True)
    assert _count_trials(mm, [torch.zeros((4, 128, 128)), torch.zeros((4, 128, 128))],
                         grads(4, 128, 128)) == (27 + 1) * (3 if backward else 1)
    sm = SparseSoftmax(mask=torch.ones((128, 128), dtype=torch.uint8), temperature=128, compressed=True)
    assert _count_trials(sm, [torch.zeros((128, 128))], grads(128, 128)) == 100 * (2 if backward else 1)
    att = SparseAttention(mask=torch.ones((128, 128), dtype=torch.uint8))
    qkv = [torch.rand((1, 128, 128)) for _ in range(3)]
    expected = (27 + 1) * (6 if backward else 2) + 45 * (2 if backward else 1)
    assert _count_trials(att, qkv, [torch.rand((1, 128, 128))] if backward else None) == expected


def test_grid_and_random_tuners():
    from sparta_amd.nn.module_tuner import GridSearchTuner, RandomSearchTuner
    from sparta_amd.common.tuning import TunableItemCfg
    space = {'a': TunableItemCfg('choice', [1, 2]), 'b': TunableItemCfg('choice', [10, 20, 30])}
    seen = []
    t = GridSearchTuner(space, lambda i, c: seen.append((i, c['a'], c['b'])) or c['a'] * c['b'])
    t.tune()
    assert [(a, b) for _, a, b in seen] == [(1, 10), (1, 20), (1, 30), (2, 10), (2, 20), (2, 30)]  # last fastest
    assert t.best_config == {'a': 1, 'b': 10} and t.best_result == 10
    seen.clear()
    random.seed(0)
    r = RandomSearchTuner(space, lambda i, c: seen.append(c) or 0.0, max_trials=4)
    r.tune()
    assert len(seen) == 4 and all(c['a'] in (1, 2) and c['b'] in (10, 20, 30) for c in seen)
    empty = GridSearchTuner({}, lambda i, c: 1.0)
    empty.tune()
    assert empty.best_config == {}


def test_operator_argument_errors():
    lin = torch.nn.Linear(32, 64)
    with pytest.raises(ValueError):
        SparseLinear(lin)
    with pytest.raises(ValueError):
        SparseLinear(torch.nn.Conv1d(1, 1, 1), weight_mask=torch.ones((64, 32)))
    with pytest.raises(AssertionError):
        SparseLinear(lin, weight_mask=torch.ones((32, 64)))
    op = SparseLinear(lin, weight_mask=torch.ones((64, 32)))
    with pytest.raises(ValueError):
        op.update_mask(input_mask=torch.ones((4, 32)), weight_mask=torch.ones((64, 32)))
    with pytest.raises(ValueError):
        SparseBatchMatMul()
    with pytest.raises(AssertionError):
        SparseSoftmax(mask=torch.ones((8, 8))).update_mask(torch.ones((4, 8)))
    with pytest.warns(UserWarning, match='not compiled'):
        y = op(torch.zeros((2, 32)))
    assert y.shape == (2, 64)
    from sparta_amd.specializer.kernels import SparTASparseMatMulKernel, OpenAISparseMatMulKernel
    with pytest.raises(ValueError):
        SparTASparseMatMulKernel(mode='ddd')
    with pytest.raises(ValueError, match='not compiled'):
        SparTASparseMatMulKernel(mode='dsd')(None, None)
    with pytest.raises(AssertionError):
        OpenAISparseMatMulKernel(mode='dsd')._check_parameters({'BLOCK_SIZE_K_VALUE': 32})
    with pytest.raises(AssertionError):
        SparTASparseMatMulKernel(mode='dsd')._check_parameters(
            {'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 8, 'BLOCK_SIZE_N_VALUE': 32})


def test_search_space_filtering_by_fixed_params():
    from sparta_amd.specializer.kernels import SparTASparseMatMulKernel, OpenAISparseMatMulKernel
    k = SparTASparseMatMulKernel(mode='dsd')
    space = k.get_search_space({'BLOCK_SIZE_K_VALUE': 64})
    assert space['BLOCK_SIZE_K_VALUE']._value == [64] and space['BLOCK_SIZE_M_VALUE']._value == [16, 32, 64]
    assert k.get_search_space({'BLOCK_SIZE_K_VALUE': 128}) is None
    assert k.get_search_space({'NOT_A_PARAM': 1}) is None
    assert OpenAISparseMatMulKernel(mode='dsd').get_search_space({'BLOCK_SIZE_K_VALUE': 32}) is None
    assert OpenAISparseMatMulKernel(mode='dsd').get_search_space({'BLOCK_SIZE_K_VALUE': 64}) is not None
    k.set_parameters({'_impl': 'sparta', '_name': 'x', 'THREAD_SIZE_M_VALUE': 4})  # tolerated keys


# ---- tuned-config tables (the reference's test/bench/*/params/*.csv format) --------------
def test_config_table_round_trip(tmp_path):
    from sparta_amd.common import config_table as ct
    cfg_a = {'forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32},
             'backward:A': {'_impl': 'openai'}}
    cfg_b = {'forward:C': {'_impl': 'openai', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32,
                           'TILE_CFG': 7}}
    path = tmp_path / 'params' / 'default.csv'
    ct.save_config_table(str(path), ['granularity', 'sparsity'],
                         [({'granularity': 8, 'sparsity': 0.9}, cfg_a), ({'granularity': 32, 'sparsity': 0.95}, cfg_b)])
    header = path.read_text().splitlines()[0].split(',')
    assert header[:2] == ['granularity', 'sparsity'] and 'forward:C;_impl' in header and 'forward:C;TILE_CFG' in header
    table = ct.load_config_table(str(path.parent), device_name='no such device')   # falls back to default.csv
    assert ct.lookup_config(table, granularity=8, sparsity=0.9) == cfg_a             # absent TILE_CFG (0) is dropped
    assert ct.lookup_config(table, granularity=32, sparsity=0.95) == cfg_b
    with pytest.raises(KeyError):
        ct.lookup_config(table, granularity=1, sparsity=0.5)
    # a device-specific file wins over default.csv
    ct.save_config_table(str(path.parent / 'My GPU.csv'), ['granularity', 'sparsity'],
                         [({'granularity': 8, 'sparsity': 0.9}, cfg_b)])
    table = ct.load_config_table(str(path.parent), device_name='My GPU')
    assert ct.lookup_config(table, granularity=8, sparsity=0.9) == cfg_b
    with pytest.raises(FileNotFoundError):
        ct.load_config_table(str(tmp_path / 'nowhere'))


def test_config_table_reads_reference_style_rows():
    """A row laid out like the reference's default.csv: zeros mean 'not set', _impl is text."""
    from sparta_amd.common import config_table as ct
    row = {'granularity': '1', 'sparsity': '0.0', 'forward:C;BLOCK_SIZE_M_VALUE': '0', 'forward:C;BLOCK_SIZE_K_VALUE': '0',
           'backward:A;BLOCK_SIZE_M_VALUE': '64', 'backward:A;BLOCK_SIZE_K_VALUE': '32.0',
           'forward:C;_impl': 'openai', 'backward:A;_impl': 'sparta'}
    assert ct.unflatten_config(row) == {'forward:C': {'_impl': 'openai'},
                                        'backward:A': {'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 32, '_impl': 'sparta'}}


@pytest.mark.parametrize('op,kernels', [('matmul', {'forward:C', 'backward:A', 'backward:B'}),
                                        ('attention', {'qk/forward:C', 'sm/forward:y', 'out/forward:C', 'qk/backward:A',
                                                       'qk/backward:B', 'sm/backward:x', 'out/backward:A', 'out/backward:B'})])
def test_packaged_config_tables_cover_the_sweep(op, kernels):
    """The tables shipped for gfx950 hold one buildable config per (granularity, sparsity)
    point of the reference's sweeps (test/bench/matmul/matmul.py:16-17)."""
    from sparta_amd.common import config_table as ct
    table = ct.load_config_table(ct.packaged_table_dir(op), device_name='some other GPU')
    for g in (1, 8, 32):
        for s in (0, 0.2, 0.4, 0.6, 0.8, 0.9, 0.95, 0.99, 0.995, 0.999, 0.9995, 0.9999):
            config = ct.lookup_config(table, granularity=g, sparsity=s)
            assert set(config) == kernels
            for params in config.values():
                assert params['_impl'] in ('sparta', 'openai')
                assert all(isinstance(v, int) and v > 0 for k, v in params.items() if k != '_impl')


def _listing(body):
    return '_Z6kernelv:\n' + body + '\ts_endpgm\n'


def _asm(*lines):
    return '\t;;#ASMSTART\n' + ''.join(f'\t{line}\n' for line in lines) + '\t;;#ASMEND\n'


def test_build_check_finds_registers_touched_while_loads_are_in_flight():
    """The build scans the device assembly of kernels that prefetch through inline-assembly
    loads: a compiler instruction that touches a destination register before the explicit
    wait that covers it is reported, everything after the wait is not."""
    from sparta_amd.build import check_inflight_registers
    load_a = _asm('global_load_dwordx4 v[2:5], v[10:11], off nt')
    load_b = _asm('global_load_dwordx4 v[6:9], v[12:13], off')
    # a copy right after the load is issued (what the register allocator did once)
    found = check_inflight_registers(_listing(load_a + '\tv_mov_b32_e32 v20, v3\n'))
    assert [(k, t) for k, _, t in found] == [('_Z6kernelv', 'v_mov_b32_e32 v20, v3')]
    # a spill of a pending register
    assert check_inflight_registers(_listing(load_a + '\tscratch_store_dwordx4 off, v[2:5], off offset:16\n'))
    # overwriting a pending register is just as wrong
    assert check_inflight_registers(_listing(load_a + '\tv_accvgpr_read_b32 v4, a0\n'))
    # the wait covers it
    assert check_inflight_registers(_listing(load_a + _asm('s_waitcnt vmcnt(0)') + '\tds_write_b128 v30, v[2:5]\n')) == []
    # vmcnt(1) leaves the newer load pending: the older registers are free, the newer are not
    two = load_a + load_b + _asm('s_waitcnt vmcnt(1)')
    assert check_inflight_registers(_listing(two + '\tds_write_b128 v30, v[2:5]\n')) == []
    assert len(check_inflight_registers(_listing(two + '\tds_write_b128 v30, v[6:9]\n'))) == 1
    # registers that are not pending, and the address registers of the load, may be used
    assert check_inflight_registers(_listing(load_a + '\tv_add_u32_e32 v10, 4, v10\n\tv_mov_b32_e32 v21, v22\n')) == []
    # text after an unconditional branch is another path
    assert check_inflight_registers(_listing(load_a + '\ts_branch .LBB0_2\n.LBB0_1:\n\tv_mov_b32_e32 v2, 0\n')) == []
    # a new kernel starts clean
    assert check_inflight_registers(_listing(load_a) + '_Z6otherv:\n\tv_mov_b32_e32 v2, 0\n\ts_endpgm\n') == []


def test_build_check_follows_the_control_flow_of_kernels_that_ask_for_it():
    """A kernel that carries the marker comment is also walked along its branches.  The case
    the text-order scan cannot see: a loop leaves loads in flight, and the code behind the loop
    (reached through the loop's branch, not by falling through) reuses their registers."""
    from sparta_amd.build import (STRICT_MARKER, check_inflight_registers,
                                  check_inflight_registers_along_control_flow,
                                  check_inflight_registers_in_text_order)
    marker = _asm(f'; {STRICT_MARKER}')
    load = _asm('global_load_dwordx4 v[2:5], v[10:11], off')
    wait1 = _asm('s_waitcnt vmcnt(1)')
    loop = (load +                                   # two stages in flight ahead of the loop
            _asm('global_load_dwordx4 v[6:9], v[12:13], off') +
            '.LBB0_1:\n' +
            wait1 + '\tds_write_b128 v30, v[2:5]\n' + load +
            wait1 + '\tds_write_b128 v30, v[6:9]\n' + _asm('global_load_dwordx4 v[6:9], v[12:13], off') +
            '\ts_cbranch_scc1 .LBB0_3\n'
            '\ts_branch .LBB0_1\n'
            '.LBB0_2:\n'
            '\tv_mov_b32_e32 v40, 0\n'
            '.LBB0_3:\n')
    reuse = '\tv_lshlrev_b32_e32 v6, 4, v39\n'       # the epilogue takes a ring register
    drain = _asm('s_waitcnt vmcnt(0)')
    bad, good = _listing(marker + loop + reuse), _listing(marker + loop + drain + reuse)
    assert check_inflight_registers_in_text_order(bad) == []
    found = check_inflight_registers_along_control_flow(bad)
    assert [t for _, _, t in found] == ['v_lshlrev_b32_e32 v6, 4, v39']
    assert check_inflight_registers(good) == []
    # without the marker the kernel is only scanned in text order
    assert check_inflight_registers(_listing(loop + reuse)) == []
    # a load that lands in LDS writes no register but counts: behind it vmcnt(1) still covers v[2:5]
    lds = _asm('s_mov_b32 m0, s4', 'global_load_lds_dwordx4 v[14:15], off')
    assert check_inflight_registers(_listing(marker + load + lds + wait1 + '\tds_write_b128 v30, v[2:5]\n')) == []
    # two waits on two sides of a branch: the walk takes both sides, also the one that skips the wait
    skipped = _listing(marker + load + '\ts_cbranch_scc1 .LBB0_5\n' + drain + '.LBB0_5:\n\tds_write_b128 v30, v[2:5]\n')
    assert len(check_inflight_registers_along_control_flow(skipped)) == 1
    # the walk ends: a loop without any wait keeps at most the 63 operations the counter holds
    endless = _listing(marker + '.LBB0_1:\n' + load + '\ts_branch .LBB0_1\n')
    assert check_inflight_registers_along_control_flow(endless) == []
