"""The autograd functions of the six convolution families, built from one table.

Every family follows the same protocol: the forward pass calls the family's op and, when a backward pass can follow,
keeps the projection the op built; the backward pass asks the family's gradient op for exactly the gradient groups
autograd needs (plus the no-atomics flag when the module-wide switch is on) and hands each result to the input it
belongs to.  What differs per family - argument list, which inputs are differentiable, the order in which the
gradient op returns its results - is data (``_FAMILIES`` below), not code.  Class names, ``apply`` argument order and
gradient routing are the reference's (pccnn_lib/op_wrappers/compute_{kpconv,kpconvn,pccnn,mcconv,pointconv,sphconv}.py).
"""
import threading

import torch

from .. import pccnn_lib_ops as _ops

_state = threading.local()


class ConvFunction(torch.autograd.Function):
    """Inside ``Function.forward`` autograd has gradient mode switched off and ``ctx.needs_input_grad`` only says
    which inputs are marked as requiring a gradient (parameters always are), so a forward pass under
    ``torch.no_grad()`` cannot tell from there that nothing will ever ask it for gradients.  ``apply`` notes the
    caller's gradient mode on the way in; ``keeps_projection(ctx)`` is then true only if a backward pass can follow.
    A forward pass that keeps nothing lets the library run the gather and the contraction as one kernel."""

    @classmethod
    def apply(cls, *args, **kwargs):
        stack = _state.__dict__.setdefault("grad_mode", [])
        stack.append(torch.is_grad_enabled())
        try:
            return super().apply(*args, **kwargs)
        finally:
            stack.pop()


def keeps_projection(ctx):
    stack = _state.__dict__.get("grad_mode")
    outer = stack[-1] if stack else True
    return outer and any(ctx.needs_input_grad)


def _conv_function(name, doc, op, grads_op, arity, groups, results, options=(), op_order=None, scalars=(),
                   contiguous=()):
    """One convolution family as a torch.autograd.Function.

    ``arity`` reference arguments, then the optional ones named in ``options`` ("mirror": the mirror index of a
    symmetric neighborhood, "contraction": "f32" or "bf16").  ``op_order``: the positions of the ``apply`` arguments in
    the order the op takes them (identity when None).  ``scalars``: positions of plain numbers (kept on the context,
    not among the saved tensors).  ``groups``: (gradient-group flag, the positions whose gradient needs it).
    ``results``: for every tensor the gradient op returns, the position of the input it belongs to."""
    order = tuple(range(arity)) if op_order is None else tuple(op_order)

    def forward(ctx, *call):
        if not arity <= len(call) <= arity + len(options):
            raise TypeError("%s.apply takes %d to %d arguments, got %d" % (name, arity, arity + len(options), len(call)))
        inputs = list(call[:arity])
        for pos in contiguous:
            inputs[pos] = inputs[pos].contiguous()
        ctx.chosen_ = dict(zip(options, call[arity:]))
        ctx.call_length_ = len(call)
        extra = {"contraction": ctx.chosen_.get("contraction", "f32")} if "contraction" in options else {}
        projection = None
        if keeps_projection(ctx):                  # a backward pass can follow: keep what it reuses
            result, projection = getattr(_ops, op)(*[inputs[i] for i in order], return_proj=True, **extra)
        else:
            result = getattr(_ops, op)(*[inputs[i] for i in order], return_proj=False, **extra)
        ctx.numbers_ = {pos: inputs[pos] for pos in scalars}
        ctx.save_for_backward(*[x for pos, x in enumerate(inputs) if pos not in scalars], projection)
        return result

    def backward(ctx, upstream):
        *tensors, projection = ctx.saved_tensors
        tensors = iter(tensors)
        inputs = [ctx.numbers_[pos] if pos in ctx.numbers_ else next(tensors) for pos in range(arity)]
        need = ctx.needs_input_grad
        wanted = _ops.deterministic_flag()
        for flag, positions in groups:
            if any(need[pos] for pos in positions):
                wanted |= getattr(_ops, flag)
        extra = {}
        if "mirror" in options:
            extra["mirror"] = ctx.chosen_.get("mirror")
        if "contraction" in options:
            extra["contraction"] = ctx.chosen_.get("contraction", "f32")
        grads = getattr(_ops, grads_op)(*[inputs[i] for i in order], upstream, proj=projection, grad_mask=wanted,
                                        **extra)
        answer = [None] * ctx.call_length_
        for value, pos in zip(grads, results):
            if need[pos]:
                answer[pos] = value
        return tuple(answer)

    return type(name, (ConvFunction,), {"forward": staticmethod(forward), "backward": staticmethod(backward),
                                        "__doc__": doc, "__module__": __name__})


def _statistic_function(name, doc, op, op_order=None, contiguous=()):
    """The weight-variance statistic of a family (no gradients): ``apply`` takes the family's arguments without the
    weights."""

    def forward(ctx, *call):
        inputs = list(call)
        for pos in contiguous:
            inputs[pos] = inputs[pos].contiguous()
        ctx.call_length_ = len(call)
        picked = inputs if op_order is None else [inputs[i] for i in op_order]
        return getattr(_ops, op)(*picked)

    def backward(ctx, upstream):
        return (None,) * ctx.call_length_

    return type(name, (torch.autograd.Function,), {"forward": staticmethod(forward),
                                                   "backward": staticmethod(backward), "__doc__": doc,
                                                   "__module__": __name__})


_KEPT = ("The projection built by the forward pass is kept for the backward pass, and only the gradients autograd asks "
         "for are computed.  An optional further argument takes the mirror index of a symmetric neighborhood "
         "(pccnn_lib_ops.mirror_pairs), used to sum point gradients without atomics")

ComputeKPConv = _conv_function(
    "ComputeKPConv",
    "apply(pts, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout].  "
    "Gradients are routed to (pts, features, samples, -, -, -, kernel_pts, -, conv_weights) "
    "(pccnn_lib/op_wrappers/compute_kpconv.py:14-73).  " + _KEPT + "; one more names the operand precision of the "
    "contraction (\"f32\", or \"bf16\" with fp32 accumulation).",
    "kp_conv", "kp_conv_grads", 9,
    groups=(("GRAD_PTS", (0, 2)), ("GRAD_FEATS", (1,)), ("GRAD_BASIS_PARAMS", (6,)), ("GRAD_WEIGHTS", (8,))),
    results=(8, 1, 6, 0, 2), options=("mirror", "contraction"), scalars=(7,))

ComputeKPConvWeightVar = _statistic_function(
    "ComputeKPConvWeightVar",
    "apply(pts, features, samples, neighbors, start_ids, radii, kernel_pts, sigma): the statistic behind the "
    "variance-aware initialisation (pccnn_lib/op_wrappers/compute_kpconv.py:76-113).",
    "kp_conv_weight_var")

ComputeKPConvN = _conv_function(
    "ComputeKPConvN",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout]: "
    "KPConv whose correlation is divided by the density of each neighbor.  Gradients go to (pts, -, features, samples, "
    "-, -, -, kernel_pts, -, conv_weights); the density gets none (pccnn_lib/op_wrappers/compute_kpconvn.py:9-74).  "
    + _KEPT + ".",
    "kp_conv_n", "kp_conv_n_grads", 10,
    groups=(("GRAD_PTS", (0, 3)), ("GRAD_FEATS", (2,)), ("GRAD_BASIS_PARAMS", (7,)), ("GRAD_WEIGHTS", (9,))),
    results=(9, 2, 7, 0, 3), options=("mirror",), scalars=(8,))

ComputeKPConvNWeightVar = _statistic_function(
    "ComputeKPConvNWeightVar",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma) "
    "(pccnn_lib/op_wrappers/compute_kpconvn.py:77-115).",
    "kp_conv_n_weight_var")

# the PCCNN ops take the features before the density; apply() takes the density first, like the reference's wrapper
_PCCNN_ORDER = (0, 2, 1, 3, 4, 5, 6, 7, 8, 9)

ComputePCCNN = _conv_function(
    "ComputePCCNN",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma, conv_weights) -> [M, Cout]: "
    "gaussian kernel-point correlation divided by the density of each neighbor.  Gradients go to (pts, pdf, features, "
    "samples, -, -, -, kernel_pts, -, conv_weights) (pccnn_lib/op_wrappers/compute_pccnn.py:5-67).  " + _KEPT + ".",
    "pccnn", "pccnn_grads", 10,
    groups=(("GRAD_PTS", (0, 3)), ("GRAD_PDF", (1,)), ("GRAD_FEATS", (2,)), ("GRAD_BASIS_PARAMS", (7,)),
            ("GRAD_WEIGHTS", (9,))),
    results=(9, 2, 7, 1, 0, 3), options=("mirror",), op_order=_PCCNN_ORDER, scalars=(8,))

ComputePCCNNWeightVar = _statistic_function(
    "ComputePCCNNWeightVar",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, kernel_pts, sigma) "
    "(pccnn_lib/op_wrappers/compute_pccnn.py:70-107).",
    "pccnn_weight_variance", op_order=_PCCNN_ORDER[:9])

ComputeMCConv = _conv_function(
    "ComputeMCConv",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, proj_axis, proj_bias, conv_weights) -> [M, Cout].  "
    "Gradients are routed to (pts, pdf, features, samples, -, -, -, proj_axis, proj_bias, conv_weights) "
    "(pccnn_lib/op_wrappers/compute_mcconv.py:14-75).  " + _KEPT + "; one more names the operand precision of the "
    "contraction (\"f32\", or \"bf16\" with fp32 accumulation).",
    "mc_conv", "mc_conv_grads", 10,
    groups=(("GRAD_PTS", (0, 3)), ("GRAD_PDF", (1,)), ("GRAD_FEATS", (2,)), ("GRAD_BASIS_PARAMS", (7, 8)),
            ("GRAD_WEIGHTS", (9,))),
    results=(9, 2, 7, 8, 1, 0, 3), options=("mirror", "contraction"))

ComputeMCConvWeightVar = _statistic_function(
    "ComputeMCConvWeightVar",
    "apply(pts, pdf, features, samples, neighbors, start_ids, radii, proj_axis, proj_bias): the statistic behind the "
    "variance-aware initialisation (pccnn_lib/op_wrappers/compute_mcconv.py:78-117).",
    "mc_conv_weight_var")

ComputePointConv = _conv_function(
    "ComputePointConv",
    "apply(basis_proj [T, K], features, neighbors, start_ids, conv_weights) -> [M, Cout]; gradients go to "
    "(basis_proj, features, -, -, conv_weights) (pccnn_lib/op_wrappers/compute_pointconv.py:61-107).",
    "point_conv", "point_conv_grads", 5,
    groups=(("GRAD_BASIS_PARAMS", (0,)), ("GRAD_FEATS", (1,)), ("GRAD_WEIGHTS", (4,))),
    results=(4, 1, 0), contiguous=(0,))

ComputePointConvWeightVar = _statistic_function(
    "ComputePointConvWeightVar",
    "apply(basis, features, neighbors, start_ids) (pccnn_lib/op_wrappers/compute_pointconv.py:110-139).",
    "point_conv_weight_var", contiguous=(0,))

ComputeSPHConv = _conv_function(
    "ComputeSPHConv",
    "apply(pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins, conv_weights) "
    "-> [M, Cout]: one-hot spherical-bin correlation divided by the neighbor count.  Only the features and the weights "
    "get gradients (pccnn_lib/op_wrappers/compute_sphconv.py:5-66).",
    "sph_conv", "sph_conv_grads", 10,
    groups=(("GRAD_FEATS", (1,)), ("GRAD_WEIGHTS", (9,))), results=(9, 1))

ComputeSPHConvWeightVar = _statistic_function(
    "ComputeSPHConvWeightVar",
    "apply(pts, features, samples, neighbors, start_ids, radii, radial_bins, azimuz_bins, polar_bins) "
    "(pccnn_lib/op_wrappers/compute_sphconv.py:69-107).",
    "sph_conv_weight_var")


class ComputePointConvBasis(torch.autograd.Function):
    """apply(pts, samples, neighbors, radii, axis_proj, axis_bias) -> [T, K]: the affine map of the normalised
    offsets; gradients go to (pts, samples, -, -, axis_proj, axis_bias)
    (pccnn_lib/op_wrappers/compute_pointconv.py:5-58).  The op takes the radii second."""

    @staticmethod
    def forward(ctx, *call):
        cloud, centres, pairs, radii, axes, offsets = call
        ctx.save_for_backward(*call)
        return _ops.point_conv_basis(cloud, radii, centres, pairs, axes, offsets)

    @staticmethod
    def backward(ctx, upstream):
        cloud, centres, pairs, radii, axes, offsets = ctx.saved_tensors
        d_cloud, d_centres, d_axes, d_offsets = _ops.point_conv_basis_grads(cloud, radii, centres, pairs, axes,
                                                                           offsets, upstream)
        return d_cloud, d_centres, None, None, d_axes, d_offsets.reshape(offsets.shape)
