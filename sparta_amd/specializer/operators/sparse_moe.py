"""Dynamic sparse mixture-of-experts forward: every token is multiplied by the
weight of the expert it is routed to (interface of
sparta/specializer/operators/sparse_moe.py:11-35).

The token -> expert index is rebuilt on the GPU at every call by a stable
counting sort (no per-expert capacity limit, no host synchronisation) and the
per-expert products run as one gathered GEMM over a flattened list of
(expert, row tile) work items, so skewed routing does not leave workgroups idle.
"""
from typing import List

import torch

from sparta_amd import _lib


class DynamicSparseMoE(torch.nn.Module):
    """Args:
        exp_modules: one bias-free torch.nn.Linear per expert, all of one shape.

        tile_cfg: tile configuration of the gathered product (0 = the library's choice from
            the problem size; see spx_tile_cfg_info, table SPX_OP_MOE).

    forward(tokens [n_tok, in], exp_ids int32 [n_tok]) -> [n_tok, out].
    """

    def __init__(self, exp_modules: List[torch.nn.Linear], tile_cfg: int = 0):
        super().__init__()
        _lib.load()
        self.tile_cfg = int(tile_cfg)
        self._tile_strict = False   # True while tune_tile_config times a variant
        self.num_exps = len(exp_modules)
        self.out_hidden, self.in_hidden = exp_modules[0].weight.shape
        self.device = exp_modules[0].weight.device
        with torch.no_grad():
            # [n_exp, in, out]: each expert's weight transposed once, up front
            stacked = torch.stack([m.weight.t() for m in exp_modules]).contiguous()
        self.weight = torch.nn.Parameter(stacked)
        self._workspace = torch.zeros(0, dtype=torch.uint8, device=self.device)
        i32 = dict(dtype=torch.int32, device=self.device)
        self.expert_count = torch.zeros(self.num_exps, **i32)
        self.expert_offset = torch.zeros(self.num_exps + 1, **i32)
        self.sparse_index = torch.zeros(0, **i32)  # token permutation, sized at first call

    def forward(self, tokens: torch.Tensor, exp_ids: torch.Tensor):
        assert tokens.dim() == 2 and tokens.shape[1] == self.in_hidden, \
            f'expected tokens of width {self.in_hidden}, got {tuple(tokens.shape)}'
        n_tok = tokens.shape[0]
        assert exp_ids.numel() == n_tok, 'one expert id per token is required'
        # the kernel walks num_exps matrices of in_hidden x out_hidden behind the weight pointer
        assert self.weight.numel() == self.num_exps * self.in_hidden * self.out_hidden, \
            f'the weight has shape {tuple(self.weight.shape)}, expected ({self.num_exps}, {self.in_hidden}, {self.out_hidden})'
        if exp_ids.dtype != torch.int32:
            exp_ids = exp_ids.to(torch.int32)
        if self.sparse_index.numel() < n_tok:
            self.sparse_index = torch.empty(n_tok, dtype=torch.int32, device=tokens.device)
        lib = _lib.load()
        ws_bytes = lib.spx_moe_index_workspace_bytes(n_tok, self.num_exps)
        if self._workspace.numel() < ws_bytes:
            self._workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=tokens.device)
        stream = _lib.current_stream(tokens.device)
        rc = lib.spx_moe_index(_lib.dev_ptr(exp_ids.contiguous()), n_tok, self.num_exps,
                               _lib.dev_ptr(self.expert_count), _lib.dev_ptr(self.expert_offset),
                               _lib.dev_ptr(self.sparse_index), _lib.dev_ptr(self._workspace),
                               self._workspace.numel(), stream)
        _lib.check(rc, 'spx_moe_index')
        tokens = tokens.contiguous()
        out = torch.empty((n_tok, self.out_hidden), dtype=tokens.dtype, device=tokens.device)
        # the stacked [n_exp, in, out] parameter is what the kernel reads (weight layout 0):
        # there is no second copy that could go stale when the parameter is written to
        weight = self.weight.detach()
        if weight.dtype != tokens.dtype:
            weight = weight.to(tokens.dtype)
        weight = weight.contiguous()
        while True:
            rc = lib.spx_moe_forward(_lib.dtype_code(tokens.dtype), _lib.dev_ptr(tokens),
                                     _lib.dev_ptr(weight), 0, _lib.dev_ptr(out),
                                     _lib.dev_ptr(self.expert_offset), _lib.dev_ptr(self.sparse_index),
                                     n_tok, self.in_hidden, self.out_hidden, self.num_exps, self.tile_cfg, stream)
            if rc == _lib.E_CONFIG and self.tile_cfg and not self._tile_strict:
                self.tile_cfg = 0   # a tuned variant that does not take this dtype: the library's choice
                continue
            break
        _lib.check(rc, 'spx_moe_forward')
        return out

    # ---- tile configuration (sparta.nn.tune(..., tile_configs=...)) ---------------------
    def set_tile_config(self, config):
        """Accepts what tune_tile_config returns: {'forward': {'TILE_CFG': id}}."""
        self.tile_cfg = int((config or {}).get('forward', {}).get('TILE_CFG', 0) or 0)

    def tune_tile_config(self, sample_inputs, num_warmups: int = 5, num_iters: int = 5):
        """Time the forward pass on `sample_inputs` = [tokens, exp_ids] (device time) under
        every tile configuration of the library's MoE table, keep the fastest one whose
        output agrees with the per-expert dense products, and return it as
        {'forward': {'TILE_CFG': id}}."""
        from sparta_amd.testing import profile
        tokens, exp_ids = (t.detach() for t in sample_inputs)
        with torch.no_grad():
            want = torch.zeros((tokens.shape[0], self.out_hidden), dtype=tokens.dtype, device=tokens.device)
            for e in range(self.num_exps):
                rows = exp_ids == e
                want[rows] = torch.matmul(tokens[rows].float(), self.weight[e].float()).to(tokens.dtype)
            best_id, best_latency = 0, float('inf')
            self._tile_strict = True
            try:
                for tile in _lib.tile_configs(_lib.OP_MOE):
                    self.tile_cfg = tile['id']
                    try:
                        latency = profile(self.forward, [tokens, exp_ids], [want], num_warmups, num_iters, cuda=True)
                    except AssertionError:   # the configuration does not take this dtype / layout
                        latency = float('inf')
                    if latency < best_latency:
                        best_id, best_latency = tile['id'], latency
            finally:
                self._tile_strict = False
        self.tile_cfg = best_id
        return {'forward': {'TILE_CFG': best_id}}
