"""Type-pattern matching for the operator multimethod table.

Same rules as the reference's matcher (minit/core/object.py:30-149): a function
signature is read from the annotations of its positional parameters (and of
``*args``); ``Union`` annotations are flattened into alternatives; an argument
type matches an alternative if it is a subclass of it (compared on the generic
origin, then recursively on the generic arguments), and ``Literal[...]``
patterns match by equality.
"""
import inspect
from dataclasses import dataclass
from typing import Literal, Optional, Tuple, Type, Union, get_args, get_origin


class Object:
    def type(self) -> Type:
        raise NotImplementedError()


@dataclass
class FunctionSignature:
    args: Tuple[Tuple[Type, ...], ...]
    vaargs: Optional[Tuple[Type, ...]]


def _alternatives(annotation) -> Tuple[Type, ...]:
    if get_origin(annotation) is Union:
        out = []
        for arg in get_args(annotation):
            out.extend(_alternatives(arg))
        return tuple(out)
    return (annotation,)


def extract_function_signature(fn) -> FunctionSignature:
    args, vaargs = [], None
    for param in inspect.signature(fn).parameters.values():
        if param.kind == param.VAR_POSITIONAL:
            vaargs = _alternatives(param.annotation)
        elif param.kind in (param.POSITIONAL_ONLY, param.POSITIONAL_OR_KEYWORD):
            args.append(_alternatives(param.annotation))
        else:
            raise TypeError(f"{fn.__name__}: keyword-only parameters cannot be dispatched on")
    return FunctionSignature(tuple(args), vaargs)


def _origin(ty):
    return get_origin(ty) or ty


def match_pattern(pattern, arg) -> bool:
    if _origin(pattern) is Literal:
        return _origin(arg) is Literal and get_args(pattern) == get_args(arg)
    if _origin(pattern) is Union:
        return any(match_pattern(p, arg) for p in get_args(pattern))
    if _origin(arg) is Literal:
        return isinstance(get_args(arg)[0], _origin(pattern))
    p_origin, a_origin = _origin(pattern), _origin(arg)
    if not (isinstance(a_origin, type) and isinstance(p_origin, type) and issubclass(a_origin, p_origin)):
        return False
    p_args, a_args = get_args(pattern), get_args(arg)
    if not p_args:
        return True
    if len(a_args) != len(p_args):
        return False
    return all(match_pattern(p, a) for p, a in zip(p_args, a_args))


def match_function_args(signature: FunctionSignature, tys: Tuple[Type, ...]) -> bool:
    n = len(signature.args)
    if len(tys) < n or (len(tys) > n and signature.vaargs is None):
        return False
    for alts, ty in zip(signature.args, tys):
        if not any(match_pattern(p, ty) for p in alts):
            return False
    for ty in tys[n:]:
        if not any(match_pattern(p, ty) for p in signature.vaargs):
            return False
    return True
