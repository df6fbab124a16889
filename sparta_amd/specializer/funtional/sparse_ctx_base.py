"""A sparse function context groups the kernels of one operator (forward and the
derived backward kernels), lets each kernel slot choose between implementations
and wires the sparse ports of connected kernels to one shared index.

Interface of sparta/specializer/funtional/sparse_ctx_base.py:12-157.
"""
import abc
from typing import Any, Dict, List, Optional, Type

import torch

from sparta_amd.specializer.kernels import KernelBase, PortConfig


class KernelPlaceholder:
    """One kernel slot with its candidate implementations."""

    def __init__(self, name: str, impls: Dict[str, Type[KernelBase]], args: Dict[str, Any],
                 port_map: Dict[str, str], connectable: bool):
        self.name = name
        self.possible_kernels: Dict[str, KernelBase] = {k: cls(**args) for k, cls in impls.items()}
        self.port_map = port_map
        self.connectable = connectable
        self.sample_inputs: List[torch.Tensor] = []
        self.dense_func = next(iter(self.possible_kernels.values())).reference
        self.ready = False
        self._active_impl: Optional[str] = None

    def select_impl(self, impl: str):
        self._active_impl = impl

    def active_kernel(self) -> Optional[KernelBase]:
        return None if self._active_impl is None else self.possible_kernels[self._active_impl]

    def set_shape(self, *args, **kwargs):
        active = self.active_kernel()
        targets = self.possible_kernels.values() if active is None else [active]
        for kernel in targets:
            kernel.set_shape(*args, **kwargs)

    def update_func(self):
        self.active_kernel().update_func()

    def build(self, config: Dict[str, Any]):
        self.active_kernel().compile(config)
        self.ready = True

    def get_search_space(self, fixed_params: Optional[Dict[str, Any]] = None):
        spaces = {}
        for impl, kernel in self.possible_kernels.items():
            space = kernel.get_search_space(fixed_params)
            if space is not None:
                spaces[impl] = space
        return spaces

    def set_sample_inputs(self, sample_inputs: List[Any]):
        self.sample_inputs = [x.detach() if isinstance(x, torch.Tensor) else x for x in sample_inputs]

    def test(self, num_warmups: int = 10, num_iters: int = 10, cuda: bool = True):
        return self.active_kernel().test(self.sample_inputs, num_warmups, num_iters, cuda)


def check_shared_block_shapes(placeholders: Dict[str, KernelPlaceholder], built) -> None:
    """Kernels that share a sparse tensor share one index object, which is rebuilt for the
    block shape of whichever kernel was bound last: a kernel bound earlier with another
    block shape keeps an index (and a compressed layout) that no longer matches the values
    it will be handed.  The kernels named in `built` must therefore agree with their port
    (AssertionError, like any other invalid combination of parameters); a kernel left
    over from an earlier build that no longer agrees is switched off, so that calling it
    raises instead of computing on a stale layout."""
    for name, placeholder in placeholders.items():
        kernel = placeholder.active_kernel()
        if kernel is None or not kernel.ready:
            continue
        sized = kernel.sparse_block_shape()
        if sized is None:
            continue
        port, want = sized
        if (port._block_H, port._block_W) == tuple(want):
            continue
        if name in built:
            raise AssertionError(
                f'kernel {name} takes {want[0]}x{want[1]} blocks of its sparse tensor, the kernels it shares '
                f'that tensor with take {port._block_H}x{port._block_W}')
        kernel.ready = False
        placeholder.ready = False


class SparseCtxBase(abc.ABC):

    def __init__(self):
        self._kernels: Dict[str, KernelPlaceholder] = {}
        self.sparse_ports: Dict[str, List[PortConfig]] = {}

    def _init_sparse_ports(self, port_names: List[str]):
        """Before implementations are selected, every candidate kernel's port
        receives the mask."""
        self.sparse_ports = {
            port_name: [
                kernel.ports[placeholder.port_map[port_name]]
                for placeholder in self._kernels.values()
                for kernel in placeholder.possible_kernels.values()
            ]
            for port_name in port_names
        }

    def select_impls(self, impls: Dict[str, str]):
        """Activate one implementation per kernel slot; connectable slots end up
        sharing a single port (hence one index) per operator-level sparse port."""
        shared: Dict[str, PortConfig] = {}
        self.sparse_ports = {name: [] for name in self.sparse_ports}
        for kernel_name, impl in impls.items():
            placeholder = self._kernels[kernel_name]
            placeholder.select_impl(impl)
            kernel = placeholder.active_kernel()
            for op_port, kernel_port in placeholder.port_map.items():
                if not placeholder.connectable:
                    self.sparse_ports[op_port].append(kernel.ports[kernel_port])
                elif op_port in shared:
                    shared[op_port].connect(kernel, kernel_port)
                else:
                    shared[op_port] = kernel.ports[kernel_port]
        for op_port, port in shared.items():
            self.sparse_ports[op_port].append(port)

    def update_func(self):
        for placeholder in self._kernels.values():
            if placeholder.active_kernel() is not None and placeholder.ready:
                placeholder.update_func()

    def build(self, config: Dict[str, Dict[str, Any]]):
        for kernel_name, kernel_config in config.items():
            self._kernels[kernel_name].build(kernel_config)
        check_shared_block_shapes({name: k for name, k in self._kernels.items()}, config)

    def get_sparse_indexes(self, port_name: str):
        ports = self.sparse_ports.get(port_name)
        return ports[0].indexes if ports else None

    def get_kernel_placeholders(self, backward: bool = False):
        return {name: k for name, k in self._kernels.items() if backward or name.startswith('forward')}

    def get_search_space(self, backward: bool = False):
        return {name: k.get_search_space() for name, k in self.get_kernel_placeholders(backward).items()}

    @abc.abstractmethod
    def set_shape(self, *args, **kwargs):
        ...

    @abc.abstractmethod
    def set_sample_inputs(self, sample_inputs: List[torch.Tensor],
                          sample_grads: Optional[List[torch.Tensor]] = None):
        ...

    @abc.abstractmethod
    def get_connections(self, backward: bool = False) -> List[Dict[str, str]]:
        ...

    @abc.abstractmethod
    def dense_forward(self, *args) -> Any:
        ...
