"""Tunable kernel objects: parameter registry, sparse ports, search-space
filtering, self-test.

Interface of sparta/specializer/kernels/kernel_base.py:24-220.  There is no
code generation here: `compile()` validates a configuration, fixes the block
sizes (which triggers the index build of the sparse port) and binds a closure
that launches the ahead-of-time compiled HIP kernel through the C ABI.
"""
from __future__ import annotations

import abc
import dataclasses
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from sparta_amd.common.tuning import TunableItemCfg
from sparta_amd.tesa import get_bcs_function, BCSIndexes
from sparta_amd.testing import profile


@dataclasses.dataclass
class _Parameter:
    name: str
    value: Optional[Any] = None
    is_tunable: bool = False
    is_dynamic: bool = False
    search_space: Optional[TunableItemCfg] = None

    def __post_init__(self):
        assert self.search_space is None or self.is_tunable, \
            f'parameter {self.name} has a search space but is not tunable'


@dataclasses.dataclass
class PortConfig:
    """One tensor argument of a kernel.  A sparse port owns the mask and the
    block-compressed indexes built from it; connecting two ports makes kernels
    share one index object (and one compressed value layout)."""
    name: str
    is_input: bool
    is_sparse: bool = False
    BCSR: bool = False
    BCSC: bool = False

    def __post_init__(self):
        self.mask: Optional[torch.Tensor] = None
        self.indexes: Optional[BCSIndexes] = None
        # Dynamic masks: keep compressed values at index capacity and let kernels read
        # the live block count from device memory, so a mask update never waits for
        # the host.
        self.at_capacity = False
        self._block_H = 0
        self._block_W = 0

    def set_sparse(self, BCSR: bool, BCSC: bool):
        self.is_sparse = True
        self.BCSR = BCSR
        self.BCSC = BCSC

    def set_block_size(self, block_H: int, block_W: int):
        if not self.is_sparse:
            return
        if (block_H, block_W) != (self._block_H, self._block_W):
            self._block_H, self._block_W = block_H, block_W
            self._update_indexes()

    def set_mask(self, mask: torch.Tensor):
        if self.is_sparse:
            self.mask = mask
            self._update_indexes()

    def index_builder(self):
        """The function context that builds this port's indexes (None before block sizes are set)."""
        if not self.is_sparse or not self._block_H or not self._block_W or self._block_H <= 0 or self._block_W <= 0:
            return None
        return get_bcs_function(self._block_H, self._block_W, self.BCSR, self.BCSC)

    def _update_indexes(self):
        if self.mask is None:
            return
        builder = self.index_builder()
        if builder is None:
            return
        self.indexes = builder.build_indexes(self.mask)

    def connect(self, kernel: 'KernelBase', port_name: str):
        """Make `kernel.ports[port_name]` an alias of this port."""
        other = kernel.ports[port_name]
        assert self.is_sparse == other.is_sparse, 'cannot connect a sparse port with a dense one'
        formats = (self.BCSR, self.BCSC)
        self.BCSR = self.BCSR or other.BCSR
        self.BCSC = self.BCSC or other.BCSC
        self.at_capacity = self.at_capacity or other.at_capacity
        kernel.ports[port_name] = self
        if self.indexes is not None and formats != (self.BCSR, self.BCSC):
            self._update_indexes()  # the index built so far lacks a format the new consumer reads


class KernelBase(abc.ABC):

    def __init__(self):
        self._parameters: Dict[str, _Parameter] = {}
        self._func: Optional[Callable] = None
        self.ports: Dict[str, PortConfig] = {}
        self.ready = False
        # A TILE_CFG that the library refuses for the shapes of a call (a tuned table entry used
        # on other shapes) gives way to the library's own choice - except inside test(), where
        # the tuner must see the refusal as a failed trial.
        self._tile_strict = False
        self._add_parameters()
        self._set_ports()

    # ---- to be provided by kernel families ------------------------------------------
    @abc.abstractmethod
    def _set_ports(self):
        """Create the input / output ports."""

    @abc.abstractmethod
    def _add_parameters(self):
        """Register the parameters of the kernel."""

    @abc.abstractmethod
    def set_shape(self, *args, **kwargs):
        """Set the problem shape."""

    @abc.abstractmethod
    def blocks_per_grid(self) -> Tuple[int, ...]:
        """Workgroups per launch (informational)."""

    @abc.abstractmethod
    def threads_per_block(self) -> Tuple[int, ...]:
        """Threads per workgroup (informational)."""

    @abc.abstractmethod
    def _check_parameters(self, params: Dict[str, Any]):
        """Raise AssertionError if the configuration is invalid."""

    @abc.abstractmethod
    def update_func(self):
        """(Re)bind the launch closure to the current indexes and shape."""

    @abc.abstractmethod
    def reference(self, *args) -> Any:
        """Masked-dense reference on dense inputs."""

    @abc.abstractmethod
    def _convert_data(self, inputs: List[torch.Tensor], outputs: List[torch.Tensor]):
        """Mask / compress sample inputs and targets in place."""

    # ---- parameter registry -----------------------------------------------------------
    def _add_parameter(self, name: str, value: Any = None, is_tunable: bool = False,
                       is_dynamic: bool = False, search_space: Optional[TunableItemCfg] = None):
        self._parameters[name] = _Parameter(name, value, is_tunable, is_dynamic, search_space)

    def set_search_space(self, search_space: Dict[str, TunableItemCfg]):
        for name, space in search_space.items():
            self._parameters[name].search_space = space

    def get_search_space(self, fixed_params: Optional[Dict[str, Any]] = None):
        """Tunable parameters and their spaces.  With `fixed_params`, pinned
        parameters collapse to one choice; None is returned when a pinned value
        is impossible for this kernel."""
        space = {n: p.search_space for n, p in self._parameters.items() if p.is_tunable}
        for name, value in (fixed_params or {}).items():
            param = self._parameters.get(name)
            if param is None:
                return None
            if param.is_tunable:
                if not param.search_space.includes(value):
                    return None
                space[name] = TunableItemCfg('choice', [value])
            elif param.value is not None and param.value != value:
                return None
        return space

    def set_parameter(self, name: str, value: Any):
        if name not in self._parameters:
            if name in ('_name', '_impl'):
                return
            raise KeyError(f'unknown kernel parameter {name}')
        self._parameters[name].value = value

    def set_parameters(self, params: Dict[str, Any]):
        for name, value in params.items():
            self.set_parameter(name, value)

    def get_parameter(self, name: str):
        return self._parameters[name].value

    def get_parameters(self, names: Optional[List[str]] = None):
        names = list(self._parameters) if names is None else names
        return {n: self._parameters[n].value for n in names}

    # ---- build / run --------------------------------------------------------------------
    def get_kernel_code(self) -> str:
        """Kept for interface compatibility: kernels are precompiled, so this
        returns a one-line description instead of source code."""
        return f'// {type(self).__name__}: precompiled gfx950 kernel in libsparta_hip.so'

    def sparse_block_shape(self) -> Optional[Tuple['PortConfig', Tuple[int, int]]]:
        """(the port whose index this kernel reads, the (block_H, block_W) it assumes for it);
        None for a kernel without a sparse tensor."""
        return None

    # ---- gfx950 tile configurations ----------------------------------------------------
    def _tile_op(self) -> Optional[int]:
        """Which tile-config table of the library (spx_tile_cfg_info's `op`) lists this kernel's
        variants; None for a kernel without a TILE_CFG parameter."""
        return None

    def enable_tile_search(self, enabled: bool = True):
        """Add (or remove) the gfx950 tile configuration to the tunable parameters.
        Off by default so that the search space equals the reference's; tune(...,
        tile_configs=True) switches it on.  A configuration that does not fit the operand
        layout, block shape or dtype is rejected by the library with an AssertionError,
        which the tuner counts as an infinitely slow trial."""
        op = self._tile_op()
        if op is None:
            return
        from sparta_amd import _lib
        param = self._parameters['TILE_CFG']
        if enabled:
            param.is_tunable = True
            param.search_space = TunableItemCfg('choice', [cfg['id'] for cfg in _lib.tile_configs(op)])
        else:
            param.is_tunable = False
            param.search_space = None

    def compile(self, params: Dict[str, Any]):
        self._check_parameters(params)
        if 'TILE_CFG' in self._parameters and 'TILE_CFG' not in params:
            self.set_parameter('TILE_CFG', 0)   # not the choice of an earlier configuration
        self.set_parameters(params)
        self.update_func()
        self.ready = True

    def test(self, inputs: List[torch.Tensor], num_warmups: int = 10, num_iters: int = 10,
             cuda: bool = True):
        """Check the kernel against `reference()` on dense sample inputs and return
        its latency in ms."""
        sample = list(inputs)
        target = self.reference(*sample)
        targets = list(target) if isinstance(target, tuple) else [target]
        self._convert_data(sample, targets)
        self._tile_strict = True
        try:
            return profile(self, sample, targets, num_warmups, num_iters, cuda)
        finally:
            self._tile_strict = False

    def __call__(self, *args) -> torch.Tensor:
        if not self.ready:
            raise ValueError('The kernel is not compiled.')
        return self._func(*args)
