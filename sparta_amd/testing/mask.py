"""Random block masks (API of sparta/testing/mask.py:9-60)."""
from typing import Any, Tuple

import torch


def random_mask(shape: Tuple[int, int], sparsity: float = 0.99, device: Any = 'cuda'):
    """uint8 mask whose entries are dropped i.i.d. with probability `sparsity`."""
    keep = torch.rand(shape, device=device) > sparsity
    return keep.to(torch.uint8)


def random_block_mask(shape: Tuple[int, int], block: Tuple[int, int], sparsity: float = 0.99,
                      device: Any = 'cuda'):
    """Draw one Bernoulli per block and expand it to element granularity."""
    grid = random_mask((shape[0] // block[0], shape[1] // block[1]), sparsity, device)
    expanded = grid.repeat_interleave(block[0], dim=0).repeat_interleave(block[1], dim=1)
    return expanded.contiguous()


def block_mask(shape: Tuple[int, int], block: Tuple[int, int] = (1, 1), sparsity: float = 0.99,
               algo: str = 'rand', device: Any = 'cuda'):
    """Generate a 2-D uint8 block mask.

    Args:
        shape: mask shape (H, W).
        block: block shape; (1, 1) is a fine-grained mask.
        sparsity: fraction of blocks that are zero.
        algo: only 'rand' is supported.
        device: where to create the mask.
    """
    assert len(shape) == 2 and len(block) == 2, 'only 2D mask is supported'
    for dim, blk in zip(shape, block):
        assert dim % blk == 0, f'invalid block shape {block}'
    if algo != 'rand':
        raise ValueError(f'unsupported mask generator: {algo}')
    return random_block_mask(tuple(shape), tuple(block), sparsity, device)
