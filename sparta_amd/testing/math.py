"""Masked-dense reference semantics in PyTorch (API of sparta/testing/math.py:8-79).
They run on whatever device their inputs live on; the kernels' `reference()`
methods and the tuner's correctness check call them on the GPU."""
import math
from typing import Optional

import torch


def sparse_softmax_forward_reference(x: torch.Tensor, mask: torch.Tensor, temperature: float = 1.):
    """Softmax over the last axis where masked entries count as -inf; rows with no
    live entry yield 0.  The row maximum is taken over all entries and 1e-10 is
    added to the denominator, as the reference does (math.py:24-27).  16-bit inputs
    are evaluated in float32 (where 1e-10 is representable; in float16 it would flush
    to zero and turn fully masked rows into 0/0) and the result is cast back."""
    if x.dtype in (torch.float16, torch.bfloat16):
        return sparse_softmax_forward_reference(x.float(), mask, temperature).to(x.dtype)
    shifted = (x - x.amax(dim=-1, keepdim=True)) / temperature
    weights = shifted.exp() * mask
    return weights / (weights.sum(dim=-1, keepdim=True) + 1e-10)


def sparse_softmax_backward_reference(grad: torch.Tensor, output: torch.Tensor, mask: torch.Tensor,
                                      temperature: float = 1.):
    """Gradient of the masked softmax w.r.t. its input; 0 on masked entries
    (math.py:30-50); float32 arithmetic for 16-bit inputs."""
    if grad.dtype in (torch.float16, torch.bfloat16):
        return sparse_softmax_backward_reference(grad.float(), output.float(), mask, temperature).to(grad.dtype)
    y = output * mask
    gy = grad * y
    return (gy - y * gy.sum(dim=-1, keepdim=True)) / temperature


def sparse_multi_head_attention_reference(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                          mask: torch.Tensor, temperature: Optional[float] = float('nan')):
    """softmax_masked(Q K^T / temperature) V over the last two axes; the mask
    [N_target, N_source] broadcasts over leading axes; temperature defaults to
    sqrt(E) (math.py:53-79)."""
    if temperature is None or math.isnan(temperature):
        temperature = math.sqrt(query.shape[-1])
    if query.dtype in (torch.float16, torch.bfloat16):
        return sparse_multi_head_attention_reference(query.float(), key.float(), value.float(), mask,
                                                     temperature).to(query.dtype)
    scores = torch.matmul(query, key.transpose(-1, -2))
    probs = sparse_softmax_forward_reference(scores, mask, temperature)
    return torch.matmul(probs, value)
