"""Base class of operator descriptors (minit/core/operator.py)."""
from .object import Object


class Operator(Object):
    def type(self):
        return type(self)
