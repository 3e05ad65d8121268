"""Packed joiner input for :func:`transducer_loss`.

The loss expects the joiner output for the valid ``(t, u)`` cells only, all
utterances concatenated, and the reference shows how to build the joiner's
input in that layout with Python lists (README.md:166-177)::

    encoder_out_list = [encoder_out[i, :logit_lengths[i], :] for i in range(N)]
    decoder_out_list = [decoder_out[i, :target_lengths[i]+1, :] for i in range(N)]
    x = [e.unsqueeze(1) + d.unsqueeze(0) for e, d in zip(encoder_out_list, decoder_out_list)]
    x = [p.reshape(-1, D) for p in x]
    x = torch.cat(x)
    activation = torch.tanh(x)

:func:`pack_joiner` computes ``x`` (``activation=None``) or ``tanh(x)``
(``activation="tanh"``) with one kernel, and its gradient with one pass over the
incoming gradient.
"""
from typing import Optional, Tuple

import torch

from . import _optimized_transducer


class PackJoinerFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, encoder_out, decoder_out, logit_lengths, target_lengths, activation,
                out_dtype="float32"):
        out, row_splits = _optimized_transducer.joiner_pack(
            encoder_out=encoder_out,
            decoder_out=decoder_out,
            logit_lengths=logit_lengths,
            target_lengths=target_lengths,
            activation=activation,
            out_dtype=out_dtype,
        )
        ctx.activation = activation
        ctx.save_for_backward(encoder_out, decoder_out, logit_lengths, target_lengths, row_splits)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        encoder_out, decoder_out, logit_lengths, target_lengths, row_splits = ctx.saved_tensors
        # float32, float16 or bfloat16: a 16-bit gradient is widened inside the kernel
        if grad_out.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            grad_out = grad_out.float()
        grad_enc, grad_dec = _optimized_transducer.joiner_unpack_grad(
            grad_out=grad_out.contiguous(),
            encoder_out=encoder_out,
            decoder_out=decoder_out,
            logit_lengths=logit_lengths,
            target_lengths=target_lengths,
            row_splits=row_splits,
            activation=ctx.activation,
        )
        return grad_enc, grad_dec, None, None, None, None


def pack_joiner(
    encoder_out: torch.Tensor,
    decoder_out: torch.Tensor,
    logit_lengths: torch.Tensor,
    target_lengths: torch.Tensor,
    activation: Optional[str] = None,
    out_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Joiner input in the packed row order of :func:`transducer_loss`.

    Args:
      encoder_out: (N, T, D) float32, contiguous, on a HIP device; frames at or
        beyond ``logit_lengths[i]`` are padding.
      decoder_out: (N, U + 1, D) float32, output of the prediction network for
        the blank-prepended targets; positions beyond ``target_lengths[i]`` are
        padding.
      logit_lengths: (N,) int32, T_i (1 <= T_i <= T).
      target_lengths: (N,) int32, U_i (0 <= U_i <= U).
      activation: None / "none" for ``enc + dec``, "tanh" for ``tanh(enc + dec)`` (the
        reference's recipe), "relu" for ``relu(enc + dec)``.
      out_dtype: torch.float32, or torch.float16 / torch.bfloat16 (D a multiple of 8)
        for a projection in 16 bits (:func:`project_joiner`): computed in float32 and
        rounded once, without a float32 array and a cast pass in between.
    Returns:
      (sum_i T_i * (U_i + 1), D) of ``out_dtype``: row ``row_splits[i] + t * (U_i + 1) + u``
      holds ``act(encoder_out[i, t] + decoder_out[i, u])``.  Differentiable with
      respect to ``encoder_out`` and ``decoder_out`` (padding gets zero gradient).
    """
    names = {torch.float32: "float32", torch.float16: "float16", torch.bfloat16: "bfloat16"}
    if out_dtype not in names:
        raise ValueError("pack_joiner: out_dtype must be torch.float32, torch.float16 or "
                         "torch.bfloat16, got %r" % (out_dtype,))
    return PackJoinerFunction.apply(
        encoder_out, decoder_out, logit_lengths, target_lengths,
        "none" if activation is None else activation, names[out_dtype],
    )


class ProjectJoinerFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, float32_logits, vocab_multiple):
        V = weight.shape[0]
        ctx.V = V
        ctx.has_bias = bias is not None
        ctx.bias_dtype = bias.dtype if bias is not None else None
        if vocab_multiple and V % vocab_multiple:
            # masked entries up to the next multiple: rows of zeros in W, -inf in the bias,
            # so their logits are -inf whatever x is and they drop out of every sum
            Vp = -(-V // vocab_multiple) * vocab_multiple
            wp = weight.new_zeros((Vp, weight.shape[1]))
            wp[:V] = weight
            bp = torch.full((Vp,), float("-inf"), dtype=torch.float32, device=weight.device)
            bp[:V] = bias.to(torch.float32) if bias is not None else 0.0
            weight, bias = wp, bp
        logits, den = _optimized_transducer.joiner_project(
            x=x, weight=weight, bias=bias, float32_logits=float32_logits)
        ctx.save_for_backward(x, weight)
        ctx.mark_non_differentiable(den)
        return logits, den

    @staticmethod
    def backward(ctx, grad_logits, _grad_den):
        # With a padded vocabulary the saved weight is the padded one and the incoming
        # gradient is zero in the masked columns.
        x, weight = ctx.saved_tensors
        V = ctx.V
        g = grad_logits if grad_logits.dtype == x.dtype else grad_logits.to(x.dtype)
        # grad_x = g W by the library, handed W^T (a copy of the small weight) so that the
        # contraction index runs fastest in both operands: its kernel for that layout is
        # the faster one here (0.53 against 0.64 ms at 752 k rows, V = D = 512)
        grad_x = None
        if ctx.needs_input_grad[0]:
            grad_x = torch.nn.functional.linear(g, weight.t().contiguous())
        want_w = ctx.needs_input_grad[1]
        want_b = ctx.has_bias and ctx.needs_input_grad[2]
        grad_w = grad_b = None
        if (want_w or want_b) and g.shape[1] % 8 == 0 and x.shape[1] % 8 == 0:
            # grad_W = g^T x and grad_b = sum of g's rows from one pass over g and x.  (The
            # bias gradient is the sum of the 16-bit g here; with float32 logits that is g
            # after its rounding to x's dtype, the same values grad_W is made of.)
            g = g.contiguous()
            gw, gb = _optimized_transducer.joiner_weight_grad(grad_logits=g, x=x)
            if want_w:
                grad_w = gw[:V]
            if want_b:
                grad_b = gb[:V].to(ctx.bias_dtype)
        else:
            if want_w:
                grad_w = (g.t() @ x)[:V]
            if want_b:
                grad_b = grad_logits.sum(0, dtype=torch.float32)[:V].to(ctx.bias_dtype)
        return grad_x, grad_w, grad_b, None, None


def project_joiner(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                   float32_logits: bool = True,
                   vocab_multiple: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """The joiner's output projection in front of the loss (``logits = linear(x)`` in
    the reference's README.md:176-177) for a joiner under mixed precision, with
    the loss's denominators as a by-product.

    Args:
      x: (sum_i T_i * (U_i + 1), D) float16 or bfloat16, contiguous, D a multiple
        of 64: the packed joiner activations, e.g. ``pack_joiner(...).to(torch.bfloat16)``.
      weight: (V, D), dtype of ``x`` (``nn.Linear.weight`` layout).
      bias: (V,) or None.
      float32_logits: True: float32 logits (accumulated in float32, never rounded
        to 16 bits); False: logits in the dtype of ``x``.
      vocab_multiple: None: logits are (rows, V).  An integer m (32 makes every row of
        float32 logits a whole number of 128-byte lines): the vocabulary is padded to
        the next multiple Vp of m with masked entries whose logits are -inf, and
        logits are (rows, Vp).  The loss of the padded logits, with the same targets
        and blank, is the same number; its gradient is bit for bit the same in the V
        real columns and exactly zero in the others.  At V = 500 the projection and
        the loss behind it run 14-17 % faster on 512 columns than on 500, whose
        2000-byte rows start and end inside cache lines.
    Returns:
      (logits, denominators): ``logits`` (rows, V) = x @ weight.T + bias, computed on
      the matrix cores with float32 accumulation; ``denominators`` (rows,) float32 =
      ``logits.logsumexp(1)`` of exactly the stored values, taken from the
      accumulators.  Pass both to ``transducer_loss(logits, ..., from_log_softmax=False,
      denominators=denominators)``: the loss then reads the logits once, not twice.
      Differentiable in ``x``, ``weight`` and ``bias``: the gradients of ``weight`` and
      ``bias`` come from this package's own kernel when V is a multiple of 8 (one pass over
      the gradient of the logits and ``x``, float32 accumulation, the same bits on every
      run), the gradient of ``x`` from torch's product; ``denominators`` carries no gradient.
      With float32 logits their gradient is rounded to the dtype of ``x`` first, for all
      three products (as autograd does for a Linear layer under autocast).
    """
    if vocab_multiple is not None and (not isinstance(vocab_multiple, int) or vocab_multiple < 1):
        raise ValueError("project_joiner: vocab_multiple must be a positive integer or None, "
                         "got %r" % (vocab_multiple,))
    return ProjectJoinerFunction.apply(x, weight, bias, float32_logits, vocab_multiple)


def joiner_transducer_loss(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                           targets: torch.Tensor, logit_lengths: torch.Tensor,
                           target_lengths: torch.Tensor, blank: int,
                           one_sym_per_frame: bool = False, reduction: str = "mean",
                           float32_logits: bool = True) -> torch.Tensor:
    """``transducer_loss(linear(x), ...)`` for a joiner under mixed precision, in the
    fastest arrangement this package has: the projection on the matrix cores with
    the loss's denominators as a by-product (:func:`project_joiner`), the vocabulary
    padded to a multiple of 32 with masked entries so that every row of logits is a
    whole number of cache lines, and the loss started from its gather step.  The
    logits never leave this function, so their padded shape concerns nobody.

    Args:
      x, weight, bias, float32_logits: as for :func:`project_joiner`.
      targets, logit_lengths, target_lengths, blank, one_sym_per_frame, reduction:
        as for :func:`transducer_loss` (README.md:179-187 of the reference).
    Returns:
      The loss, differentiable in ``x``, ``weight`` and ``bias``; the same number,
      and the same gradients, as ``transducer_loss(project_joiner(x, weight,
      bias)[0], ..., from_log_softmax=False)``.
    """
    from .transducer_loss import transducer_loss
    logits, den = project_joiner(x, weight, bias, float32_logits=float32_logits, vocab_multiple=32)
    return transducer_loss(logits, targets, logit_lengths, target_lengths, blank, False,
                           one_sym_per_frame, reduction, denominators=den)

