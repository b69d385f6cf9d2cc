"""``save`` / ``load``: a tensor and its gradient as one ``.npz`` file (reference:
``mygrad/_io.py``).  Host-side only; the file layout is the reference's (``data`` and, when the
tensor has a gradient, ``grad``), so files written by either library load in the other."""

import numpy as np

from .tensor_base import Tensor, tensor

__all__ = ["save", "load"]


def save(file, tensor_to_save):
    """Save a tensor and, if it has one, its gradient with ``numpy.savez``.

    Parameters
    ----------
    file : str | Path | BinaryIO
        Where to write; NumPy appends ``.npz`` to a path that lacks it.
    tensor_to_save : Tensor

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> from tempfile import TemporaryFile
    >>> outfile = TemporaryFile()
    >>> mg.save(outfile, mg.Tensor([0., 1., 2.]))
    >>> _ = outfile.seek(0)
    >>> mg.load(outfile)
    Tensor([0., 1., 2.])
    """
    if not isinstance(tensor_to_save, Tensor):
        raise TypeError(f"mygrad.save requires a Tensor-type object, got type {type(tensor_to_save)}")
    if tensor_to_save.grad is not None:
        np.savez(file, data=tensor_to_save.data, grad=tensor_to_save.grad)
    else:
        np.savez(file, data=tensor_to_save.data)


def load(file):
    """Load a tensor written by ``save`` (its gradient too, if one was saved).

    The archive is read with NumPy's default loader, which executes nothing from the file."""
    loaded = np.load(file)
    out = tensor(loaded["data"])
    if "grad" in loaded:
        out.backward(loaded["grad"])
    return out
