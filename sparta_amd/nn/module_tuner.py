"""tune() / build() for modules that contain sparse operators.

Search semantics of sparta/nn/module_tuner.py:105-381: a two-level search.  The
"upper" space enumerates the block dimensions that connected kernels must share;
for each upper point every kernel slot searches its remaining parameters over
each implementation (grid: odometer order, last parameter fastest; random:
independent uniform draws), is checked against its dense reference and timed.
A configuration whose check fails with AssertionError counts as infinitely slow.
"""
import itertools
import logging
import math
import random
import sys
import warnings
from typing import Any, Callable, Dict, Iterator, List, Optional

import torch

from sparta_amd.common.tuning import TunableItemCfg
from sparta_amd.specializer import OperatorBase

# A logger of the logging module's registry (a bare logging.Logger(...) keeps its cache of
# enabled levels across setLevel, so `verbose` would stick to its first value).
_logger = logging.getLogger(__name__)
_logger.propagate = False
if not _logger.handlers:
    _logger.addHandler(logging.StreamHandler())


class Tuner:
    """Evaluates configurations drawn from a {param: TunableItemCfg} space and
    remembers the best (lowest) result."""

    def __init__(self, search_space: Dict[Any, TunableItemCfg],
                 eval_func: Callable[[int, Dict[Any, Any]], float], max_trials: int = sys.maxsize):
        self._search_space = search_space
        self._eval_func = eval_func
        size = math.prod(len(space._value) for space in search_space.values())
        self._max_trials = min(max_trials, size)
        self.best_result = math.inf
        self.best_config: Optional[Dict[Any, Any]] = None

    def next_config(self) -> Iterator[Dict[Any, Any]]:
        raise NotImplementedError

    def tune(self):
        for i, config in enumerate(itertools.islice(self.next_config(), self._max_trials)):
            result = self._eval_func(i, config)
            if result < self.best_result:
                self.best_result, self.best_config = result, config


class RandomSearchTuner(Tuner):

    def next_config(self):
        while True:
            yield {name: random.choice(space._value) for name, space in self._search_space.items()}


class GridSearchTuner(Tuner):

    def next_config(self):
        names = list(self._search_space)
        for values in itertools.product(*(self._search_space[n]._value for n in names)):
            yield dict(zip(names, values))


def _tuner_class(algo: str):
    if algo.startswith('grid'):
        return GridSearchTuner
    if algo.startswith('rand'):
        return RandomSearchTuner
    raise ValueError(f'unsupported tuner algorithm "{algo}"')


def tune_sparse_module(module: OperatorBase, name: str, sample_inputs: List[torch.Tensor],
                       sample_grads: Optional[List[torch.Tensor]] = None, algo: str = 'grid',
                       max_trials: int = sys.maxsize, backward_weight: float = 0,
                       debug_func: Optional[Callable[[int, Dict[Any, Any]], float]] = None,
                       refine_tiles: bool = False):
    """Tune one sparse operator and build it with the best configuration found.
    Returns that configuration ({kernel: {'_impl': ..., PARAM: ...}}), or None if
    every trial failed or `debug_func` replaced the measurement.  With `refine_tiles`
    every kernel of the best configuration then tries each gfx950 tile configuration
    with its block sizes kept (see refine_tile_configs)."""
    tuner_cls = _tuner_class(algo)
    with_backward = backward_weight > 0
    module.set_sample_inputs(sample_inputs, sample_grads)
    search_space = module.get_search_space(with_backward)
    connections = module.get_connections(with_backward)

    # Upper space: per connection, the values every connected kernel can take with
    # at least one of its implementations.
    upper_space = {}
    for i, connection in enumerate(connections):
        per_kernel = [
            set().union(*(set(impl_space[param]._value) for impl_space in search_space[kernel].values()))
            for kernel, param in connection.items()
        ]
        upper_space[i] = TunableItemCfg('choice', list(set.intersection(*per_kernel)))
    upper_size = math.prod(len(space._value) for space in upper_space.values())
    trials_per_kernel = int(math.ceil(max_trials / upper_size)) if upper_size else 0
    best_lower: Dict[str, Dict[str, Dict[str, Any]]] = {}
    best_lower_latency: Dict[str, float] = {}

    def lower_search(upper_idx: int, upper_params: Dict[int, Any]) -> float:
        _logger.info(f'[{name}][Upper Search Space] #{upper_idx}: {list(upper_params.values())}')
        chosen: Dict[str, Optional[Dict[str, Any]]] = {}
        total_latency = 0.0
        for kernel_name, kernel in module.get_kernel_placeholders(with_backward).items():
            _logger.info(f'[{name}][Kernel: {kernel_name}]')
            weight = backward_weight if kernel_name.startswith('backward') else 1
            fixed = {connections[i][kernel_name]: value for i, value in upper_params.items()}
            best_params, best_latency = None, math.inf
            for impl, impl_space in kernel.get_search_space(fixed).items():
                kernel.select_impl(impl)

                def measure(lower_idx: int, params: Dict[str, Any], impl=impl):
                    try:
                        kernel.build(params)
                        latency = kernel.test()
                    except AssertionError:
                        latency = math.inf
                    _logger.info(f'{impl} #{lower_idx}: {list(params.values())} => {latency} ms')
                    return latency

                tuner = tuner_cls(impl_space, measure if debug_func is None else debug_func, trials_per_kernel)
                tuner.tune()
                if tuner.best_result < best_latency:
                    best_params = dict(_impl=impl, **tuner.best_config)
                    best_latency = tuner.best_result
            chosen[kernel_name] = best_params
            total_latency += best_latency * weight
        # Random search may draw the same upper point twice: keep the better of the two
        # lower results, so that the point the upper tuner remembers and the kernel
        # configs returned for it belong to the same trial.
        key = str(upper_params)
        if key not in best_lower or total_latency < best_lower_latency[key]:
            best_lower[key] = chosen
            best_lower_latency[key] = total_latency
        return total_latency

    upper_tuner = tuner_cls(upper_space, lower_search, upper_size)
    upper_tuner.tune()
    _logger.info(f'[{name}] Tuning completed.')
    if debug_func is not None:
        return None
    if upper_tuner.best_config is None:
        _logger.warning(f'[{name}] All trials failed.')
        return None
    best_config = best_lower[str(upper_tuner.best_config)]
    if refine_tiles:
        best_config = refine_tile_configs(module, name, best_config, with_backward)
    _logger.info(f'[{name}] Best config:\n{best_config}')
    module.build(best_config, sample_inputs)
    return best_config


_TILE_MARGIN = 0.97


def refine_tile_configs(module: OperatorBase, name: str, config: Dict[str, Dict[str, Any]],
                        with_backward: bool = False) -> Dict[str, Dict[str, Any]]:
    """Second stage of a search that keeps the block sizes of `config`: every kernel that has
    a table of gfx950 tile configurations is built and timed with each of its entries (the
    costs add to those of the block-size search instead of multiplying them).  Returns
    `config` with 'TILE_CFG' set where an entry other than the library's own choice (0) was
    the fastest.  Needs the sample inputs of `module` to be set (tune_sparse_module does)."""
    from sparta_amd import _lib
    refined = {kernel_name: dict(params) for kernel_name, params in config.items() if params is not None}
    for kernel_name, placeholder in module.get_kernel_placeholders(with_backward).items():
        params = refined.get(kernel_name)
        if params is None:
            continue
        placeholder.select_impl(params['_impl'])
        op = placeholder.active_kernel()._tile_op()
        if op is None:
            continue
        best_id, best_latency, own_choice = 0, math.inf, math.inf
        for tile in _lib.tile_configs(op):
            trial = {k: v for k, v in params.items() if k != 'TILE_CFG'}
            trial['TILE_CFG'] = tile['id']
            try:
                placeholder.build(trial)
                latency = placeholder.test()
            except AssertionError:
                latency = math.inf
            _logger.info(f'[{name}][Kernel: {kernel_name}] tile config {tile["id"]} ({tile["name"]}) => {latency} ms')
            if tile['id'] == 0:
                own_choice = latency
            if latency < best_latency:
                best_id, best_latency = tile['id'], latency
        params.pop('TILE_CFG', None)
        # A variant is only recorded when it beats the library's own choice by more than the
        # noise of two timings of one kernel (the choice usually IS one of the variants).  The
        # choice is timed once more at the end: it was the first trial after the block sizes
        # changed, which the later trials were not.
        if best_id:
            try:
                placeholder.build({k: v for k, v in params.items()})
                own_choice = min(own_choice, placeholder.test())
            except AssertionError:
                pass
        if best_id and best_latency < _TILE_MARGIN * own_choice:
            params['TILE_CFG'] = best_id
    return refined


def iter_sparse_modules(module: torch.nn.Module, module_name: str,
                        func: Callable[[OperatorBase, str], None]):
    """Apply `func(op, 'root/child/...')` to every sparse operator below `module`
    (a sparse operator is a leaf: its own children are not visited)."""
    if isinstance(module, OperatorBase):
        func(module, module_name)
        return
    for child_name, child in module.named_children():
        iter_sparse_modules(child, f'{module_name}/{child_name}', func)


def iter_tile_modules(module: torch.nn.Module, module_name: str,
                      func: Callable[[torch.nn.Module, str], None]):
    """Apply `func(op, name)` to every module below `module` that chooses a tile configuration
    for a kernel of its own through `tune_tile_config` / `set_tile_config` (the fused
    attention kernel, the gathered MoE product); such a module is a leaf of the walk."""
    if hasattr(module, 'tune_tile_config'):
        func(module, module_name)
        return
    if isinstance(module, OperatorBase):
        return
    for child_name, child in module.named_children():
        iter_tile_modules(child, f'{module_name}/{child_name}', func)


def get_input_hook(input_dict: Dict[str, List], module_name: str):
    """Forward hook that records the positional inputs of a module."""
    def input_hook(module, inputs, output):
        input_dict[module_name] = list(inputs)
    return input_hook


def get_grad_hook(grad_dict: Dict[str, List], module_name: str):
    """Full backward hook that records the gradients of a module's outputs."""
    def grad_hook(module, grad_input, grad_output):
        grad_dict[module_name] = list(grad_output)
    return grad_hook


def _capture_samples(module: torch.nn.Module, sample_inputs, sample_grads, with_backward: bool):
    """Run the (still dense) module once and collect, per sparse operator, the
    inputs it received and - if requested - the gradients of its outputs."""
    inputs = {'root': sample_inputs}
    grads = {'root': sample_grads}
    handles = []

    def register(op: torch.nn.Module, name: str):
        handles.append(op.register_forward_hook(get_input_hook(inputs, name)))
        if with_backward and isinstance(op, OperatorBase):
            handles.append(op.register_full_backward_hook(get_grad_hook(grads, name)))

    iter_sparse_modules(module, 'root', register)
    iter_tile_modules(module, 'root', lambda op, name: None if isinstance(op, OperatorBase) else register(op, name))
    try:
        with warnings.catch_warnings():
            warnings.simplefilter('ignore')
            if with_backward:
                for x in sample_inputs:
                    x.requires_grad = True
            outputs = module.forward(*sample_inputs)
            if with_backward:
                outputs = outputs if isinstance(outputs, tuple) else (outputs,)
                for output, grad in zip(outputs, sample_grads):
                    if isinstance(output, torch.Tensor):
                        output.backward(grad)
                for x in sample_inputs:
                    x.requires_grad = False
    finally:
        for handle in handles:
            handle.remove()
    return inputs, grads


def tune_combined_module(module: torch.nn.Module, sample_inputs: List[torch.Tensor],
                         sample_grads: Optional[List[torch.Tensor]] = None, algo: str = 'grid',
                         max_trials: int = sys.maxsize, backward_weight: float = 0,
                         verbose: bool = False, debug_func: Optional[Callable] = None,
                         tile_configs=False):
    """Find, tune and build every sparse operator inside `module`.

    Args:
        module: a sparse operator, or any torch module containing some.
        sample_inputs: inputs of `module`.
        sample_grads: gradients of its outputs (needed when backward_weight > 0).
        algo: 'grid' or 'rand'.
        max_trials: trial budget per kernel slot (split over the upper space).
        backward_weight: weight of backward latencies; 0 tunes forward kernels only.
        verbose: log every trial.
        debug_func: replaces build + measurement of a trial (for tests).
        tile_configs: also search the gfx950 tile configurations (parameter TILE_CFG of
            the matmul and softmax kernels, and the kernels that SparseAttention and
            DynamicSparseMoE launch themselves).  False (default) leaves exactly the
            reference's search space and trial counts.  True adds TILE_CFG to the lower
            space of every kernel (a joint search: the trial budget is spent on block
            sizes x tile configurations).  'refine' searches the reference's space first
            and then tries every tile configuration with the best block sizes kept.

    Returns:
        {operator name: best config}; names are 'root' or 'root/child/...'.
    """
    inputs, grads = _capture_samples(module, sample_inputs, sample_grads, backward_weight > 0)

    def set_tile_search(op: OperatorBase, name: str):
        for placeholder in op.get_kernel_placeholders(backward=True).values():
            for kernel in placeholder.possible_kernels.values():
                kernel.enable_tile_search(tile_configs is True)

    iter_sparse_modules(module, 'root', set_tile_search)
    _logger.setLevel(logging.DEBUG if verbose else logging.WARNING)
    best_configs = {}

    def tune_one(op: OperatorBase, name: str):
        best_configs[name] = tune_sparse_module(
            module=op, name=name, sample_inputs=inputs[name], sample_grads=grads.get(name),
            algo=algo, max_trials=max_trials, backward_weight=backward_weight, debug_func=debug_func,
            refine_tiles=tile_configs == 'refine')

    iter_sparse_modules(module, 'root', tune_one)

    def tune_own_kernel(op: torch.nn.Module, name: str):
        # kernels that a module launches itself, outside the kernel placeholders
        if isinstance(op, OperatorBase) and best_configs.get(name) is None:
            return
        own = op.tune_tile_config(inputs[name])
        if own:
            best_configs[name] = {**(best_configs.get(name) or {}), **own}
        _logger.info(f'[{name}] tile configuration of its own kernel: {own}')

    if tile_configs and debug_func is None:
        iter_tile_modules(module, 'root', tune_own_kernel)
    return best_configs


def build_combined_module(module: torch.nn.Module, sample_inputs: List[torch.Tensor],
                          configs: Dict[str, Dict[str, Any]]):
    """Build every sparse operator inside `module` with a known configuration
    (as returned by tune)."""
    inputs, _ = _capture_samples(module, sample_inputs, None, False)
    iter_sparse_modules(module, 'root', lambda op, name: op.build(configs[name], sample_inputs=inputs[name]))
    iter_tile_modules(module, 'root', lambda op, name: None if isinstance(op, OperatorBase) or name not in configs
                      else op.set_tile_config(configs[name]))
