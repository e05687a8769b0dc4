"""Seeded synthetic GGUF block tensors and MoE routing for tests and benchmarks.

No checkpoint is needed: every byte of a block is drawn at random (all bit patterns
of the integer fields are legal in the five formats), then the fp16 super-block
scales ``d`` / ``dmin`` are overwritten with positive normal values so that no
NaN/Inf pattern appears.
"""

from __future__ import annotations

import math

import torch

QK_K = 256
Q3_K, Q4_K, Q5_K, Q6_K, IQ2_S = 11, 12, 13, 14, 22
QUANT_TYPES = {"Q3_K": Q3_K, "Q4_K": Q4_K, "Q5_K": Q5_K, "Q6_K": Q6_K, "IQ2_S": IQ2_S}
BLOCK_BYTES = {Q3_K: 110, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ2_S: 82}
# byte offsets of the fp16 scale fields inside one super-block
_SCALE_FIELDS = {Q3_K: (108,), Q4_K: (0, 2), Q5_K: (0, 2), Q6_K: (208,), IQ2_S: (0,)}


def row_bytes(quant_type: int, in_features: int) -> int:
    return (in_features // QK_K) * BLOCK_BYTES[quant_type]


def random_packed_weight(
    quant_type: int,
    leading_shape: tuple[int, ...],
    in_features: int,
    seed: int,
    device: str | torch.device = "cpu",
    scale_range: tuple[float, float] = (1e-4, 1e-2),
) -> torch.Tensor:
    """uint8 tensor ``[*leading_shape, row_bytes]`` of random super-blocks.

    ``leading_shape`` is ``(out_features,)`` for a dense weight and
    ``(experts, out_features)`` for a grouped one.
    """
    block = BLOCK_BYTES[quant_type]
    blocks_per_row = in_features // QK_K
    rows = math.prod(leading_shape)
    generator = torch.Generator(device=device).manual_seed(seed)
    data = torch.randint(
        0, 256, (rows * blocks_per_row, block), dtype=torch.uint8, device=device, generator=generator
    )
    low, high = scale_range
    for offset in _SCALE_FIELDS[quant_type]:
        scale = torch.rand(rows * blocks_per_row, device=device, generator=generator) * (high - low) + low
        as_bytes = scale.to(torch.float16).view(torch.uint8).reshape(-1, 2)
        data[:, offset : offset + 2] = as_bytes
    return data.reshape(*leading_shape, blocks_per_row * block)


def zipf_routing(
    tokens: int,
    experts: int,
    top_k: int,
    seed: int,
    device: str | torch.device = "cpu",
    exponent: float = 1.1,
):
    """Skewed top-k routing: N(0,1) router logits plus a Zipf(exponent) expert bias.

    Returns ``(token_of_row, expert_indices, expert_offsets, routing_weights)``:
    rows sorted by expert (stable), the experts that received rows in ascending
    order (int64), the inclusive cumulative row ends per such expert (int32) and
    the softmax weight of every routed row.
    """
    generator = torch.Generator(device=device).manual_seed(seed)
    logits = torch.randn(tokens, experts, device=device, generator=generator)
    ranks = torch.arange(1, experts + 1, device=device, dtype=torch.float32)
    pmf = ranks.pow(-exponent)
    pmf = pmf / pmf.sum()
    permutation = torch.randperm(experts, device=device, generator=generator)
    bias = torch.empty(experts, device=device)
    bias[permutation] = pmf.log()
    probabilities = torch.softmax(logits + bias, dim=-1)
    weights, chosen = probabilities.topk(top_k, dim=-1)
    flat_expert = chosen.reshape(-1)
    order = torch.sort(flat_expert, stable=True).indices
    token_of_row = (order // top_k).to(torch.int64)
    counts = torch.bincount(flat_expert, minlength=experts)
    active = torch.nonzero(counts > 0).reshape(-1).to(torch.int64)
    offsets = counts[active].cumsum(0).to(torch.int32)
    return token_of_row, active, offsets, weights.reshape(-1)[order]


def uniform_groups(group_sizes, experts=None, device: str | torch.device = "cpu"):
    """Group metadata for explicit per-group row counts (experts default to 0..G-1)."""
    sizes = torch.tensor(list(group_sizes), dtype=torch.int64)
    if experts is None:
        experts = list(range(len(sizes)))
    indices = torch.tensor(list(experts), dtype=torch.int64, device=device)
    offsets = sizes.cumsum(0).to(torch.int32).to(device)
    return indices, offsets
