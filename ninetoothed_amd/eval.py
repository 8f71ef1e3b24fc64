"""``ninetoothed.eval`` / ``ninetoothed.subs`` under the module name the reference keeps them in
(src/ninetoothed/eval.py:14-110: ``_eval`` and ``_subs``, exported by the package as ``eval`` and
``subs``).  Both are methods of :class:`ninetoothed_amd.tensor.Tensor` here."""


def _eval(tensor, subs=None):
    """Evaluates a symbolic tensor into a ``numpy.ndarray`` of source offsets (-1 = masked);
    see :meth:`ninetoothed_amd.tensor.Tensor.eval`."""
    return tensor.eval(subs)


def _subs(tensor, substitutions):
    """Substitutes symbols (sizes, strides, block sizes) in a tensor; see
    :meth:`ninetoothed_amd.tensor.Tensor.subs`."""
    return tensor.subs(substitutions)
