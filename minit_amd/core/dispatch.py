"""Global operator multimethod table.

API-compatible with the reference (minit/core/dispatch.py:9-58):
``register_dispatch(*, predicate=None, priority=0)`` appends an implementation
keyed on the annotated types of its positional parameters; ``dispatch(op,
*tensors)`` looks the implementation up by ``tuple(arg.type() for arg in
args)``, memoises per type tuple, keeps the matches of highest priority and
requires exactly one.  Implementations return a tuple of tensors.
"""
from typing import Callable, Dict, List, Optional, Tuple, Type

from .object import FunctionSignature, Object, extract_function_signature, match_function_args

DISPATCH_CACHE: Dict[Tuple[Type, ...], Callable] = {}
DISPATCH_TABLE: List[Tuple[FunctionSignature, Callable, Optional[Callable], int]] = []
DEFAULT_PRIORITY = 0


def lookup_implementation_from_types(tys: Tuple[Type, ...]) -> Callable:
    matching = []
    for signature, func, predicate, priority in DISPATCH_TABLE:
        if match_function_args(signature, tys) and (predicate is None or predicate(*tys)):
            matching.append((priority, func))
    assert len(matching) > 0, f"no matching function for {tys}"
    top = max(priority for priority, _ in matching)
    selected = [func for priority, func in matching if priority == top]
    assert len(selected) == 1, f"more than one function matches for {tys}"
    return selected[0]


def dispatch(*args: Object):
    arg_types = tuple(arg.type() for arg in args)
    try:
        func = DISPATCH_CACHE[arg_types]
    except KeyError:
        func = lookup_implementation_from_types(arg_types)
        DISPATCH_CACHE[arg_types] = func
    return func(*args)


def register_dispatch(*, predicate: Optional[Callable] = None, priority: int = DEFAULT_PRIORITY):
    def decorator(function):
        DISPATCH_TABLE.append((extract_function_signature(function), function, predicate, priority))
        DISPATCH_CACHE.clear()
        return function
    return decorator
