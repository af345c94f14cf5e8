"""The typed kernel selector the MoE layer's products go through, shaped as the reference's
(src/dew/nn/kernels/selection.py:33-347): an `Op` lists its `Kernel`s, each a tuple of `Requirement`s checked
in order; a call runs the op's preferred kernel where every requirement holds; a kernel named with
`chosen(grouped_matmul='hip')` that does not take the call raises `KernelRefused` with its first refusal
(src/dew/nn/kernels/selection.py:232-248); routes taken are recorded for `routes()`
(src/dew/nn/kernels/generation.py:1450).

This build holds the HIP kernels only. The names the reference gives its other launches ('xla', 'pallas',
'mosaic', 'triton', 'cutlass') are known and refused as unlowerable on this host, never silently replaced.
"""

import contextlib
import contextvars
import dataclasses
from collections.abc import Callable, Iterator

INHERENT = "inherent"


@dataclasses.dataclass(frozen=True)
class Refusal:
    """Why a kernel does not take a call: a stable `code` and the `detail` a log names."""

    code: str
    detail: str
    row: str | None = None
    kind: str = "capability"

    def __str__(self) -> str:
        return self.detail


@dataclasses.dataclass(frozen=True)
class Requirement:
    """One fact a kernel needs of a case: `holds(case)`, else the refusal `code` with `detail` (text or a
    function of the case). `kind` is 'capability' or 'measured' (a forced choice passes over measured)."""

    code: str
    holds: Callable[[object], bool]
    detail: str | Callable[[object], str] = ""
    row: str = INHERENT
    kind: str = "capability"

    def check(self, case) -> Refusal | None:
        if self.holds(case):
            return None
        detail = self.detail(case) if callable(self.detail) else self.detail
        return Refusal(self.code, detail, self.row, self.kind)


@dataclasses.dataclass(frozen=True)
class Kernel:
    name: str
    supports: tuple[Requirement, ...]
    generic: bool = False

    def refusals(self, case, forced: bool = False) -> Iterator[Refusal]:
        for requirement in self.supports:
            if forced and requirement.kind == "measured":
                continue
            if (refusal := requirement.check(case)) is not None:
                yield refusal

    def refused(self, case, forced: bool = False) -> Refusal | None:
        return next(self.refusals(case, forced), None)


class KernelRefused(ValueError):
    """A forced kernel that does not take a call: the op's `choice`, the `kernel`, its `first` refusal."""

    def __init__(self, choice: str, kernel: str, first: Refusal, rest: Iterator[Refusal]) -> None:
        super().__init__(f"{choice} kernel {kernel!r} was chosen and does not take this call: "
                         f"{first.code}: {first.detail}")
        self.choice, self.kernel, self.first = choice, kernel, first
        self._rest, self._refusals = rest, None

    @property
    def refusals(self) -> list[Refusal]:
        if self._refusals is None:
            self._refusals = [self.first, *self._rest]
        return self._refusals


class Unlowerable(RuntimeError):
    """A kernel the reference names that this host cannot run (src/dew/nn/kernels/selection.py:215-229)."""

    def __init__(self, choice: str, kernel: str, why: str) -> None:
        super().__init__(f"{choice} kernel {kernel!r} does not lower on this host: {why}")
        self.choice, self.kernel, self.why = choice, kernel, why


@dataclasses.dataclass(frozen=True)
class Route:
    """What a call ran: the op's `choice`, the `kernel`, the op's `preferred` one, the preferred one's
    `refusal` where it did not take the call, and what `forced` the kernel."""

    choice: str
    kernel: str
    preferred: str
    refusal: Refusal | None = None
    forced: str | None = None


@dataclasses.dataclass(frozen=True)
class Op:
    choice: str
    kernels: tuple[Kernel, ...]
    preferred: Callable[[object], str | None] | None = None
    unlowered: Callable[[str], str | None] = lambda kernel: None
    foreign: tuple[str, ...] = ()
    """Names the reference gives launches this build does not hold."""

    def kernel(self, name: str) -> Kernel:
        for kernel in self.kernels:
            if kernel.name == name:
                return kernel
        if name in self.foreign:
            raise Unlowerable(self.choice, name, "this build holds the gfx950 HIP kernels only")
        raise ValueError(f"{self.choice} has no kernel {name!r}; its kernels are "
                         f"{', '.join(kernel.name for kernel in self.kernels)}")


_CHOICES: contextvars.ContextVar[dict] = contextvars.ContextVar("dew_amd_kernel_choices", default={})
_ROUTES: list[Route] = []


@contextlib.contextmanager
def chosen(**choices: str):
    """Within the block, each named op runs the named kernel or raises (`KernelRefused`, `Unlowerable`):
    `chosen(grouped_matmul='hip')` (src/dew/nn/kernels/generation.py:215-228)."""
    token = _CHOICES.set({**_CHOICES.get(), **choices})
    try:
        yield
    finally:
        _CHOICES.reset(token)


def forced(choice: str) -> str | None:
    return _CHOICES.get().get(choice)


def routes() -> list[Route]:
    """The routes taken since `clear_routes()`, one per distinct (choice, kernel, refusal)."""
    return list(_ROUTES)


def clear_routes() -> None:
    _ROUTES.clear()


def select(op: Op, case, named: str | None = None) -> Route:
    """The kernel `op` runs for `case`: the named one (or `chosen`'s) where it takes the case, raising
    otherwise; else the op's preference, else the first kernel that takes it."""
    insisted = named or forced(op.choice)
    if insisted is not None:
        kernel = op.kernel(insisted)
        if (why := op.unlowered(kernel.name)) is not None:
            raise Unlowerable(op.choice, kernel.name, why)
        refusals = kernel.refusals(case, forced=True)
        if (first := next(refusals, None)) is not None:
            raise KernelRefused(op.choice, kernel.name, first, refusals)
        route = Route(op.choice, kernel.name, kernel.name, None, insisted)
    else:
        preferred = (op.preferred(case) if op.preferred else None) or op.kernels[0].name
        first_kernel = op.kernel(preferred)
        refusal = None
        route = None
        for kernel in (first_kernel, *(k for k in op.kernels if k is not first_kernel)):
            found = kernel.refused(case)
            if found is None and op.unlowered(kernel.name) is None:
                route = Route(op.choice, kernel.name, preferred, refusal, None)
                break
            if kernel is first_kernel:
                refusal = found
        if route is None:
            raise ValueError(f"no {op.choice} kernel takes this call ({refusal})")
    if route not in _ROUTES:
        _ROUTES.append(route)
    return route
