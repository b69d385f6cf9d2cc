"""Exceptions of the autodiff contract (mirrors mygrad/errors.py and
mygrad/_utils/__init__.py:126-128 of the reference)."""

__all__ = ["InvalidGradient", "InvalidBackprop", "SkipGradient"]


class InvalidGradient(Exception):
    """An operation's ``backward_var`` returned something that is not a real
    scalar or a NumPy array."""


class InvalidBackprop(Exception):
    """Back-propagation was asked to pass through a part of the graph that has
    already been cleared."""


class SkipGradient(Exception):
    """Raised by ``backward_var`` to tell ``Operation.backward`` to skip that input."""
