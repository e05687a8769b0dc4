"""Cross-entropy through a packed LM head, one chunk of rows at a time.

The logits of an LM head are ``rows x vocabulary`` (248 320 columns for the model family the
reference is tuned on); keeping them for the backward pass of the loss costs more memory than
the rest of the step.  The reference's production schedule therefore walks the rows in chunks of
256 (its measured best; 128 and 64 are its lower-memory fallbacks,
docs/mmq_fwd_optimization.md:293) and runs forward and backward of each chunk back to back:
``mmq`` for the chunk's logits, the loss and its gradient with respect to the logits, and
``mmq_grad_input`` for the chunk's share of the hidden-state gradient.  Only one chunk of logits
exists at a time.  That loop lives in the reference's training code, not in its package; this
module is the same schedule on top of this package's operators.
"""

from __future__ import annotations

import torch

DEFAULT_CHUNK_ROWS = 256   # the reference's production chunk


class _ChunkedLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, packed_weight, targets, quant_type, out_features, chunk_rows, ignore_index):
        ops = torch.ops.torch_ggml_ops
        rows, in_features = hidden.shape
        counted = targets != ignore_index
        # (a tensor: no host synchronisation; the loss of a batch without any counted row is 0 / 1)
        count = counted.sum().clamp(min=1).to(torch.float32)
        total = torch.zeros((), dtype=torch.float32, device=hidden.device)
        need_grad = ctx.needs_input_grad[0]
        grad_hidden = torch.empty_like(hidden) if need_grad else None
        for begin in range(0, rows, chunk_rows):
            end = min(rows, begin + chunk_rows)
            # (the operators take tensors at storage offset zero only: a chunk is copied out, a few hundred rows)
            chunk = hidden if begin == 0 and end == rows else hidden[begin:end].clone()
            logits = ops.mmq.default(chunk, packed_weight, quant_type, out_features).float()
            log_probabilities = torch.log_softmax(logits, dim=-1)
            chunk_targets = targets[begin:end]
            chunk_counted = counted[begin:end]
            safe_targets = torch.where(chunk_counted, chunk_targets, torch.zeros_like(chunk_targets))
            picked = log_probabilities.gather(1, safe_targets.unsqueeze(1)).squeeze(1)
            total = total - (picked * chunk_counted).sum()
            if need_grad:
                # d(mean loss)/d(logits) = (softmax - one_hot) / count on counted rows, 0 elsewhere
                grad_logits = torch.exp(log_probabilities)
                grad_logits.scatter_add_(1, safe_targets.unsqueeze(1), -torch.ones_like(picked).unsqueeze(1))
                grad_logits = grad_logits * (chunk_counted.unsqueeze(1) / count)
                grad_hidden[begin:end] = ops.mmq_grad_input.default(
                    grad_logits.to(hidden.dtype), packed_weight, quant_type, in_features
                )
        if need_grad:
            ctx.save_for_backward(grad_hidden)
        return total / count

    @staticmethod
    def backward(ctx, grad_loss):
        grad_hidden = None
        if ctx.needs_input_grad[0]:
            (saved,) = ctx.saved_tensors
            grad_hidden = (saved.float() * grad_loss).to(saved.dtype)
        return grad_hidden, None, None, None, None, None, None


def chunked_lm_head_loss(
    hidden: torch.Tensor,
    packed_weight: torch.Tensor,
    targets: torch.Tensor,
    quant_type: int,
    out_features: int,
    chunk_rows: int = DEFAULT_CHUNK_ROWS,
    ignore_index: int = -100,
) -> torch.Tensor:
    """Mean cross-entropy of ``mmq(hidden, packed_weight)`` against ``targets`` over the rows whose target is
    not ``ignore_index``, computed ``chunk_rows`` rows at a time.

    ``hidden`` bf16 ``[rows, in_features]`` (contiguous), ``targets`` int64 ``[rows]``.  Differentiable with
    respect to ``hidden``: the gradient is computed chunk by chunk during the forward pass (each chunk's logits
    are dropped as soon as its ``mmq_grad_input`` has run) and scaled by the incoming gradient in backward.
    Equals ``cross_entropy(mmq(hidden, ...).float(), targets)`` up to the bf16 rounding of the logit gradients.
    """
    if hidden.dim() != 2:
        raise RuntimeError("hidden must have shape [rows, in_features]")
    if targets.dim() != 1 or targets.shape[0] != hidden.shape[0] or targets.dtype != torch.int64:
        raise RuntimeError("targets must be an int64 tensor with one entry per row of hidden")
    if chunk_rows <= 0:
        raise RuntimeError("chunk_rows must be positive")
    return _ChunkedLoss.apply(
        hidden, packed_weight, targets, int(quant_type), int(out_features), int(chunk_rows), int(ignore_index)
    )


__all__ = ["DEFAULT_CHUNK_ROWS", "chunked_lm_head_loss"]
