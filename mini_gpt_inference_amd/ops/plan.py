"""A step's launches, recorded once and made again from C++ (csrc/hip/launch_plan.hip).

The model's forward pass is Python that chooses kernels and computes their arguments; for every
step of the same shape it chooses the same kernels with the same arguments (buffer addresses in
the workspace and the arena, sizes, constants: what Part.graph_safe promises).  A LaunchPlan holds
those launches; run() makes them with one call into the kernel library, a microsecond or two of
host time per kernel instead of Python's ten."""

from __future__ import annotations

import ctypes
import struct
from typing import List, Optional

from . import kernels, library


def _slot(argtype, value) -> int:
    """An argument as a 64-bit slot: pointers and integers as they are, a float's bits."""
    if isinstance(value, ctypes._SimpleCData):
        value = value.value
    if argtype is ctypes.c_float:
        return struct.unpack("<I", struct.pack("<f", float(value)))[0]
    if value is None:
        return 0
    return int(value) & (2 ** 64 - 1)


def signature_of(launches: List[tuple]) -> List[tuple]:
    """(launcher name, its arguments as 64-bit slots) of every recorded launch; the stream, a launcher's
    last argument, is left out."""
    return [(name, tuple(_slot(t, v) for t, v in zip(argtypes[:-1], args[:-1]))) for name, argtypes, args in launches]


class LaunchPlan:
    def __init__(self, launches: List[tuple]) -> None:
        """launches: what library.record() collected."""
        lib = library.kernels()
        self._lib = lib
        self._h = lib.mgpt_plan_create()
        if not self._h:
            raise kernels.KernelError("no memory for a launch plan")
        self.n_kernels = 0
        self.signature = signature_of(launches)      # what was recorded, for difference()
        for name, argtypes, args in launches:
            slots = (ctypes.c_ulonglong * len(args))(*[_slot(t, v) for t, v in zip(argtypes, args)])
            rc = lib.mgpt_plan_add(self._h, name.encode(), slots, len(args))
            if rc != 0:
                raise kernels.KernelError(f"launch plan: {name} with {len(args)} arguments is refused ({rc})")
            self.n_kernels += 1
        self._failed = ctypes.c_int(-1)

    def __del__(self) -> None:
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mgpt_plan_destroy(h)

    def __len__(self) -> int:
        return self.n_kernels

    def difference(self, launches: List[tuple]) -> Optional[str]:
        """None if `launches` (what library.record() collected of another run of the same step shape)
        are this plan's launches, launcher for launcher and argument for argument; else a line that
        names the first difference.  A part that promises plan_safe and still takes a launcher's
        argument from the host's view of the step (a context length, say) shows here."""
        other = signature_of(launches)
        for i, (mine, theirs) in enumerate(zip(self.signature, other)):
            if mine[0] != theirs[0]:
                return f"launch {i}: the plan has {mine[0]}, this run made {theirs[0]}"
            for j, (a, b) in enumerate(zip(mine[1], theirs[1])):
                if a != b:
                    return f"launch {i} ({mine[0]}): argument {j} was {a:#x} when recorded and is {b:#x} now"
        if len(self.signature) != len(other):
            return f"the plan has {len(self.signature)} launches, this run made {len(other)}"
        return None

    def run(self, stream: Optional[int] = None) -> None:
        """Makes the plan's launches on the stream (default: the current one)."""
        s = kernels._stream() if stream is None else ctypes.c_void_p(stream)
        rc = self._lib.mgpt_plan_run(self._h, s, ctypes.byref(self._failed))
        if rc != 0:
            raise kernels.KernelError(f"launch plan: launch {self._failed.value} of {self.n_kernels} failed ({rc})")
        kernels.launches += self.n_kernels
