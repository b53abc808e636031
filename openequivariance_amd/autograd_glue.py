"""The one formula the batch product and both convolution variants share for their second
derivatives."""
from __future__ import annotations


def double_backward_terms(forward, backward_helper, x, y, w, dz, ddx, ddy, ddw, index=()):
    """Gradients of ``backward_helper(x, y, w, dz) -> (dx, dy, dw)`` with respect to ``(x, y, w, dz)``
    for incoming cotangents ``(ddx, ddy, ddw)`` of its three outputs, composed from the operator's own
    forward and backward launches (reference: TensorProductBase.py:281-298,
    convolution/ConvolutionBase.py:618-636 and :691-709).  The product is trilinear in (x, y, w), so
    every second derivative is the first-order operator with one argument replaced by its cotangent.
    ``index`` are the trailing graph arguments of the convolution (rows, cols[, transpose_perm])."""
    a = backward_helper(ddx, ddy, w, dz, *index)       # x and y replaced
    b = backward_helper(x, y, ddw, dz, *index)         # w replaced
    c = backward_helper(ddx, y, w, dz, *index)
    d = backward_helper(x, ddy, w, dz, *index)
    grad_dz = forward(ddx, y, w, *index) + forward(x, ddy, w, *index) + forward(x, y, ddw, *index)
    return a[0] + b[0], a[1] + b[1], c[2] + d[2], grad_dz
