"""Sparse linear operator y = x W^T + b with a mask on the input, the weight or
the output (interface of sparta/specializer/operators/sparse_linear.py:12-172)."""
from typing import Any, Dict, List, Optional

import torch

from sparta_amd.specializer.operators.operator_base import OperatorBase
from sparta_amd.specializer.funtional import SparseBatchMatMulCtx, SparseBatchMatMulFunc


class SparseLinear(OperatorBase):
    r"""Args:
        raw_module (torch.nn.Linear): dense linear layer providing weight and bias.
        input_mask: mask of the input  [batch, in_features]  -> 'sdd' kernel, dense storage.
        weight_mask: mask of the weight [out_features, in_features] -> 'dsd' kernel;
            after `build` the `weight` parameter holds the BCSR-compressed values.
        output_mask: mask of the output [batch, out_features] -> 'dds' kernel, dense storage.
        Exactly one of the three masks must be given.
        dynamic: the mask changes every few steps.  `update_mask` then enqueues the
            index rebuild without ever waiting for the host (the reference synchronises
            once per rebuild); with a weight mask the weight stays dense and the kernels
            read its live blocks through the index (no re-compression), with an input
            mask the compressed operand is kept at full capacity.
        activation: None or 'relu' (an extension; the reference's operator has none): the
            activation that follows the layer, applied by the matmul kernel's own epilogue
            instead of a separate elementwise kernel.  Input and weight masks only.

    Shape: input (B, in_features) -> output (B, out_features).

    Example::

        dense = torch.nn.Linear(1024, 1024, device='cuda')
        mask = sparta_amd.testing.block_mask((1024, 1024), block=(32, 32), sparsity=0.9)
        sparse = sparta_amd.nn.SparseLinear(dense, weight_mask=mask)
        sparta_amd.nn.tune(sparse, sample_inputs=[torch.rand((1024, 1024), device='cuda')])
    """

    __base_class__ = torch.nn.Linear
    __sparse_func__ = SparseBatchMatMulFunc

    _PORT_OF = {'input': 'A', 'weight': 'B', 'output': 'C'}

    def __init__(self, raw_module: torch.nn.Linear, input_mask: Optional[torch.Tensor] = None,
                 weight_mask: Optional[torch.Tensor] = None, output_mask: Optional[torch.Tensor] = None,
                 dynamic: bool = False, activation: Optional[str] = None):
        super().__init__(raw_module)
        if activation not in (None, 'relu'):
            raise ValueError(f'unsupported fused activation: {activation!r}')
        self._activation = activation
        N, K = raw_module.weight.shape
        biased = raw_module.bias is not None
        self._raw_weight = torch.clone(raw_module.weight)
        self.weight = None
        self.bias = raw_module.bias
        M = None
        if input_mask is not None:
            self._sparse_ctx = SparseBatchMatMulCtx('sdd', False, True, biased, False)
            M = input_mask.shape[0]
        elif weight_mask is not None:
            # dynamic: the kernels read the live blocks out of the dense weight through the
            # index, so a new mask costs an index rebuild and nothing else
            self._sparse_ctx = SparseBatchMatMulCtx('dsd', False, True, biased, not dynamic)
        elif output_mask is not None:
            self._sparse_ctx = SparseBatchMatMulCtx('dds', False, True, biased, False)
            M = output_mask.shape[0]
        else:
            raise ValueError('expected a sparse mask on input / weight / output')
        self._sparse_ctx.set_activation(activation)
        self._shape = {'batch_size': 1, 'M': M, 'K': K, 'N': N}
        self._dynamic = dynamic
        self._set_dynamic(dynamic)
        self.update_mask(input_mask, weight_mask, output_mask)

    def update_mask(self, input_mask: Optional[torch.Tensor] = None,
                    weight_mask: Optional[torch.Tensor] = None,
                    output_mask: Optional[torch.Tensor] = None):
        self._set_mask(self._mask_arguments(input_mask, weight_mask, output_mask))
        self._after_mask_update()

    def _after_mask_update(self):
        if self.ready:
            self._update_parameters()

    def _mask_arguments(self, input_mask: Optional[torch.Tensor] = None,
                        weight_mask: Optional[torch.Tensor] = None,
                        output_mask: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
        """Check the arguments of `update_mask`; returns {sparse port: mask}."""
        given = {k: v for k, v in (('input', input_mask), ('weight', weight_mask), ('output', output_mask))
                 if v is not None}
        if len(given) > 1:
            raise ValueError('linear operators with multiple sparse masks are not supported')
        if not given:
            raise ValueError('expected a sparse mask on input / weight / output')
        (kind, mask), = given.items()
        M, K, N = self._shape['M'], self._shape['K'], self._shape['N']
        want = {'input': (M, K), 'weight': (N, K), 'output': (M, N)}[kind]
        ok = all(w is None or w == got for w, got in zip(want, mask.shape))
        shown = tuple('?' if w is None else w for w in want)
        assert ok and mask.dim() == 2, f'expected {kind} mask shape {shown}, got {tuple(mask.shape)}'
        return {self._PORT_OF[kind]: mask}

    def _read_sample_inputs(self, A: torch.Tensor):
        M, K = self._shape['M'], self._shape['K']
        if M is None:
            assert A.dim() == 2 and A.shape[1] == K, f'expect input shape (?, {K}), got {tuple(A.shape)}'
            self._shape['M'] = A.shape[0]
        else:
            assert tuple(A.shape) == (M, K), f'expect input shape ({M}, {K}), got {tuple(A.shape)}'

    def _update_parameters(self):
        """(Re)compress the weight with the current index.  The weight is taken as
        it is: values inside live blocks are not multiplied by the element mask."""
        weight = self._raw_weight
        indexes = self.get_sparse_indexes('B')
        if indexes is not None and self._dynamic:
            if self.weight is None:
                self.weight = torch.nn.Parameter(weight, requires_grad=True)
            return
        if indexes is not None:
            weight = indexes.convert(weight.detach())
        self.weight = torch.nn.Parameter(weight, requires_grad=True)

    def _compile(self, config: Optional[Dict[str, Dict[str, Any]]] = None):
        super()._compile(config)
        self._update_parameters()

    def _dense_forward(self, *args):
        out = super()._dense_forward(*args)
        return torch.relu(out) if self._activation == 'relu' else out

    def _sparse_forward(self, input_tensor: torch.Tensor):
        args = [self._sparse_ctx, input_tensor, self.weight]
        if self.bias is not None:
            args.append(self.bias)
        return self.__sparse_func__.apply(*args).squeeze(0)

    def set_sample_inputs(self, sample_inputs: List[torch.Tensor],
                          sample_grads: Optional[List[torch.Tensor]] = None):
        self._read_sample_inputs(*sample_inputs)
        self._sparse_ctx.set_shape(**self._shape)
        tensors = [sample_inputs[0], self._raw_weight]
        if self.bias is not None:
            tensors.append(self.bias)
        batched = [t.unsqueeze(0) for t in tensors]
        grads = None if sample_grads is None else [g.unsqueeze(0) for g in sample_grads]
        self._sparse_ctx.set_sample_inputs(batched, grads)
