"""(op, device) -> callable table: the plug-in boundary of the kernel backends.

Same contract as dlgrad/dispatch.py:7-57: runtimes decorate their static
methods with `@dispatcher.register(op, device)` at import time and Buffer calls
`dispatcher.dispatch(op, device, **kwargs)`.  An unregistered pair raises
KeyError, as a bare dict lookup does in the reference (dispatch.py:55).
"""
from collections.abc import Callable
from enum import Enum


class Dispatcher:
    def __init__(self) -> None:
        self._dispatch_table: dict[tuple[Enum, Enum], Callable] = {}

    def register(self, op: Enum, device: Enum) -> Callable:
        def decorator(func: Callable) -> Callable:
            self._dispatch_table[(op, device)] = func
            return func  # keep the function usable under its own name
        return decorator

    def dispatch(self, op: Enum, device: Enum, *args, **kwargs):
        return self._dispatch_table[(op, device)](*args, **kwargs)

    def registered(self, device: Enum) -> set:
        return {op for (op, dev) in self._dispatch_table if dev is device}


dispatcher = Dispatcher()
