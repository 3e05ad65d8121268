"""Python entry points, mirroring
optimized_transducer/python/optimized_transducer/transducer_loss.py.

Differences from the reference that do not change results:

* the ``grad /= N`` pass of ``reduction="mean"`` (transducer_loss.py:150) is
  folded into the gradient kernel as a multiplication by ``1/N``;
* ``-1 * scores`` and the ``.sum()`` / ``.mean()`` that follows
  (transducer_loss.py:145-147) are one launch with a fixed summation order;
* ``backward`` multiplies by ``loss_grad`` with a kernel that reads the factor
  on the device and does nothing when it equals 1 (transducer_loss.py:162 always
  makes a full pass);
* ``backward`` returns a fresh alias of the gradient buffer, so that autograd
  can adopt it as ``logits.grad`` without the (rows, V) copy the reference's
  shared tensor object forces when ``logits`` is a leaf; a further backward
  through the same graph (``retain_graph=True``), which the reference answers
  with ``ctx.grad.mul_(loss_grad)`` once more (transducer_loss.py:160-162), gets
  a copy of the buffer times ``loss_grad``, the copy being made then and not
  before (it raises if the buffer was changed in place in between, e.g. by
  ``logits.grad.zero_()``, which the reference's private copy would survive);
* ``TransducerLoss.__init__`` calls ``super().__init__()`` so the module can
  actually be called (the reference's class omits it, transducer_loss.py:173-188).

Two additions.  ``logits`` may be float16 or bfloat16 (the reference takes
float32 only, transducer-loss.cc:33): the passes over (rows, V) then read and
write 2-byte elements, all arithmetic is float32, the loss is a float32 scalar
and the gradient has the dtype of ``logits``.  And, off unless asked for: ``defer_gradient=True`` (keyword only) leaves
``logits`` untouched in ``forward`` and makes the single pass over (rows, V) in
``backward``, with ``loss_grad`` and ``1/N`` folded into it.  Results are the
same; what changes is *when* ``logits`` is overwritten (in ``backward`` instead
of ``forward``), and that a loss which is scaled or weighted before
``backward()`` (mixed-precision loss scaling, a weighted sum of losses) costs no
second pass over the gradient.
"""
from typing import Optional

import torch

from . import _optimized_transducer


class TransducerLossFunction(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        logits: torch.Tensor,
        targets: torch.Tensor,
        logit_lengths: torch.Tensor,
        target_lengths: torch.Tensor,
        blank: int,
        from_log_softmax: bool,
        one_sym_per_frame: bool,
        reduction: str = "mean",
        defer_gradient: bool = False,
        denominators: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """See :func:`transducer_loss` for the arguments.

        Caution: when ``from_log_softmax`` is False and ``logits`` requires
        grad, ``logits`` is overwritten with its gradient (reference
        transducer_loss.py:45-48).
        """
        assert reduction in ("mean", "sum")

        batch_size = logit_lengths.size(0)
        grad_scale = 1.0 / batch_size if (reduction == "mean" and batch_size > 0) else 1.0

        ctx.deferred = None
        if defer_gradient:
            # loss = -1 * scores, then .mean() or .sum() (reference transducer_loss.py:145-147),
            # computed by the launch that makes the per-row coefficients
            _, coefficients, loss = _optimized_transducer.compute_transducer_loss_deferred_reduced(
                logits=logits,
                targets=targets,
                logit_lengths=logit_lengths,
                target_lengths=target_lengths,
                blank=blank,
                from_log_softmax=from_log_softmax,
                one_sym_per_frame=one_sym_per_frame,
                grad_scale=grad_scale,
                denominators=denominators,
            )
            if coefficients is not None:
                # saved through autograd: an in-place change of logits before
                # backward is then reported instead of giving a wrong gradient
                ctx.save_for_backward(logits)
                ctx.deferred = (coefficients, from_log_softmax, grad_scale)
            return loss

        # loss = -1 * scores, then .mean() or .sum() (reference transducer_loss.py:145-147):
        # part of the launch that makes the per-row coefficients when there is a gradient,
        # a launch of its own otherwise
        _, grad, loss = _optimized_transducer.compute_transducer_loss_reduced(
            logits=logits,
            targets=targets,
            logit_lengths=logit_lengths,
            target_lengths=target_lengths,
            blank=blank,
            from_log_softmax=from_log_softmax,
            one_sym_per_frame=one_sym_per_frame,
            grad_scale=grad_scale,
            denominators=denominators,
        )

        ctx.grad = grad
        return loss

    @staticmethod
    def backward(ctx, loss_grad):
        assert loss_grad.numel() == 1, loss_grad.numel()
        no_grads = (None,) * 9  # targets ... denominators
        if ctx.deferred is not None:
            coefficients, from_log_softmax, grad_scale = ctx.deferred
            assert coefficients is not None, "backward through a deferred transducer loss runs once"
            (logits,) = ctx.saved_tensors
            ctx.deferred = (None, from_log_softmax, grad_scale)
            factor = loss_grad.detach().to(device=logits.device, dtype=torch.float32).contiguous()
            grad = _optimized_transducer.apply_deferred_gradient(
                logits=logits.detach(),
                coefficients=coefficients,
                from_log_softmax=from_log_softmax,
                grad_scale=grad_scale,
                loss_grad=factor,
            )
            return (grad,) + no_grads
        # Hand autograd a fresh alias of the gradient buffer: when `logits` is a leaf,
        # autograd then adopts the buffer as logits.grad instead of cloning (rows, V)
        # floats because this object still holds the tensor.  From then on the buffer is
        # shared with autograd, which may accumulate into it.  A further backward through
        # the same graph (retain_graph=True), which the reference answers with
        # ctx.grad.mul_(loss_grad) once more (transducer_loss.py:160-162), therefore works
        # on a copy, made only then; the version counter, which every alias shares, tells
        # whether the buffer still holds what the previous backward returned.
        if ctx.grad is None:
            return (None,) + no_grads
        if getattr(ctx, "handed_version", None) is not None:
            if ctx.grad._version != ctx.handed_version:
                raise RuntimeError(
                    "transducer_loss: the gradient buffer that an earlier backward handed to "
                    "autograd has been modified in place since (for example by "
                    "logits.grad.zero_()); call transducer_loss again instead of a second "
                    "backward through the same graph")
            ctx.grad = ctx.grad.clone()
        grad = ctx.grad
        if (
            loss_grad.is_cuda
            and loss_grad.device == grad.device
            and loss_grad.dtype == torch.float32
            and grad.dtype in (torch.float32, torch.float16, torch.bfloat16)
            and grad.is_contiguous()
        ):
            _optimized_transducer.scale_by_device_scalar_(grad, loss_grad.detach().contiguous())
        else:
            with torch.no_grad():
                grad.mul_(loss_grad)
        ctx.handed_version = grad._version
        grad = grad.detach()
        return (grad,) + no_grads


class TransducerLoss(torch.nn.Module):
    def __init__(self, blank: int, reduction: str = "mean"):
        """
        Args:
          blank: ID of the blank symbol.
          reduction: "mean" (average over the utterances of the batch) or
            "sum".  "none" is not supported (reference transducer_loss.py:133).

        Set the attribute ``defer_gradient`` to True afterwards for the deferred
        mode described in :func:`transducer_loss`.
        """
        super().__init__()
        self.blank = blank
        self.reduction = reduction
        self.defer_gradient = False

    def forward(
        self,
        logits: torch.Tensor,
        targets: torch.Tensor,
        logit_lengths: torch.Tensor,
        target_lengths: torch.Tensor,
        from_log_softmax: bool,
        one_sym_per_frame: bool = False,
    ) -> torch.Tensor:
        """See :func:`transducer_loss`."""
        return TransducerLossFunction.apply(
            logits,
            targets,
            logit_lengths,
            target_lengths,
            self.blank,
            from_log_softmax,
            one_sym_per_frame,
            self.reduction,
            self.defer_gradient,
        )


def transducer_loss(
    logits: torch.Tensor,
    targets: torch.Tensor,
    logit_lengths: torch.Tensor,
    target_lengths: torch.Tensor,
    blank: int,
    from_log_softmax: bool,
    one_sym_per_frame: bool = False,
    reduction: str = "mean",
    *,
    defer_gradient: bool = False,
    denominators: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Transducer loss of a packed batch.

    Args:
      logits: (sum_i T_i * (U_i + 1), V) float32, contiguous, on a HIP device
        (CPU tensors are accepted like in the reference: they are copied to the
        current HIP device, computed there and copied back):
        utterance i's (T_i, U_i + 1, V) joiner output reshaped to 2-D, all
        utterances concatenated, no padding.  Output of ``nn.Linear`` when
        ``from_log_softmax`` is False (then it is OVERWRITTEN with its gradient
        if it requires grad), output of ``log_softmax`` otherwise.
      targets: (N, max_i U_i) int32, not prepended with blank; every entry
        must be below V (the reference checks the padding too), the entries
        u < U_i must not be negative.
      logit_lengths: (N,) int32, T_i.
      target_lengths: (N,) int32, U_i.
      blank: ID of the blank symbol, 0 <= blank < V.
      from_log_softmax: whether ``logits`` already went through log-softmax.
      one_sym_per_frame: modified transducer - every arc, blank or symbol,
        advances one frame (needs U_i <= T_i - 1).
      reduction: "mean" or "sum" over the N utterances.
      defer_gradient: not in the reference.  False: the gradient is computed
        in the forward call, as in the reference.  True: the forward call
        leaves ``logits`` alone and ``backward`` computes the gradient (into
        the ``logits`` buffer for logits input), already multiplied by the
        upstream gradient.  ``logits`` must not be modified in between.
      denominators: not in the reference.  The per-row log-sum-exp of
        ``logits`` (float32, shape (logits.size(0),)) when the caller already
        has it, as :func:`project_joiner` returns it: the loss then skips its
        own pass over the logits for it.  Logits input only.
    Returns:
      A 0-dim tensor with the reduced negative log-likelihood.
    """
    return TransducerLossFunction.apply(
        logits,
        targets,
        logit_lengths,
        target_lengths,
        blank,
        from_log_softmax,
        one_sym_per_frame,
        reduction,
        defer_gradient,
        denominators,
    )
