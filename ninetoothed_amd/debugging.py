"""``simulate_arrangement``: what every program of a launch would see.

Same contract as the reference (src/ninetoothed/debugging.py:14-75): for every
tensor the arrangement takes, a *source* tensor whose elements are their own
flat indices, and a *target* tensor with one leading dimension enumerating the
programs of the launch grid followed by the dimensions of the levels below
it, holding the source index each position refers to (``-1`` where the
position is masked).  The reference obtains the targets by running a generated
copy kernel; the index maps are known in closed form here
(:meth:`Tensor.eval`), so they are evaluated on the host and moved to
``device``.
"""

import math

import numpy as np

from ninetoothed_amd.tensor import Tensor


def simulate_arrangement(arrangement, tensors, device=None):
    """Simulates the arrangement of the tensors.

    :param arrangement: The arrangement of the tensors.
    :param tensors: The tensors (with concrete shapes).
    :param device: The device on which the result tensors are created.
    :return: A tuple of source tensors and a tuple of target tensors, in
        the parameter order of ``arrangement``.
    """
    import torch

    if device is None:
        device = "cuda"
    arranged = arrangement(*tensors)
    arranged = arranged if isinstance(arranged, tuple) else (arranged,)
    sources, targets = [], []
    for tensor, view in zip(tensors, arranged):
        if not isinstance(tensor, Tensor) or tensor.ndim == 0:
            sources.append(torch.tensor(0, device=device))
            targets.append(torch.tensor(0, device=device))
            continue
        shape = tuple(int(size) for size in tensor.shape)
        sources.append(torch.arange(math.prod(shape), device=device).view(shape))
        table = np.asarray(view.eval())
        target = table.reshape((-1,) + table.shape[view.ndim :])
        targets.append(torch.from_numpy(np.ascontiguousarray(target).astype(np.int64)).to(device))
    return tuple(sources), tuple(targets)
