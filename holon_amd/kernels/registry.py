"""Kernels that parts bring with them.

The built-in operations are methods of the kernel sets (`holon_amd.kernels.api.Kernels`). A part that needs an operation
of its own registers it here, beside its class, as the reference registers kernels beside the unit that uses them
(core/holon/core/plugins.py:31-122): the operation's name, its plain form in torch (which is also what every kernel
set without a HIP form of it runs, the tests' CPU twin included), and its HIP form: an `extern "C"` symbol with its
ctypes argument types, the function that turns the operation's arguments into the symbol's, and the source file the
symbol is built from when it is not part of this package's own library. Every kernel set then answers
`kernels.<name>(...)`; no file of the framework is edited.

    register_kernel(KernelOp(
        name="decay_scan", plain=decay_scan_plain,
        symbol="toy_decay_scan", argtypes=[c_void_p, c_void_p, ...], source="path/to/decay_scan.hip",
        call=lambda launch, x, state, ...: launch(x.data_ptr(), state.data_ptr(), ...)))

`call` gets `launch(*c_args)`, which appends the current HIP stream as the last argument, calls the symbol and raises
`KernelError` when it returns non-zero; the function returns what the operation returns. The source is compiled for
gfx950 with this package's flags into `lib<stem>.so` beside it (or, where that folder cannot be written, into the
per-user build folder) the first time the operation is called and no such library is there;
`holon_amd.kernels.build.build_source` builds it ahead of time.
"""
from __future__ import annotations

import dataclasses
import pathlib
from collections.abc import Callable, Sequence
from typing import Any


@dataclasses.dataclass(frozen=True)
class KernelOp:
    name: str
    plain: Callable[..., Any]
    symbol: str | None = None
    argtypes: Sequence[Any] = ()                  # without the trailing stream (a void pointer), which `launch` adds
    call: Callable[..., Any] | None = None
    source: str | pathlib.Path | None = None      # None: the symbol is in libholon_hip.so


_OPS: dict[str, KernelOp] = {}


def register_kernel(op: KernelOp) -> KernelOp:
    if op.name in _OPS:
        raise KeyError(f"kernel operation {op.name!r} is registered twice")
    if (op.symbol is None) != (op.call is None):
        raise ValueError(f"kernel operation {op.name!r}: a HIP form needs both `symbol` and `call`")
    _OPS[op.name] = op
    return op


def unregister_kernel(name: str) -> None:
    _OPS.pop(name, None)


def kernel_op(name: str) -> KernelOp | None:
    return _OPS.get(name)


def kernel_ops() -> list[str]:
    return sorted(_OPS)
