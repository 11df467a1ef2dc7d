"""Which kernel a matrix product takes where more than one can serve it: a setting, resolved in one place and reported.

The reference resolves every kernel choice as pinned, then preferred, then by priority, and a tie is an error
(core/holon/core/engine.py:61-100 `kernels` / `kernel_preferences`, core/holon/core/build.py:89-106). Here the
candidates are forms of one product (this package's kernels, the vendor library's product in several forms), told
apart by what they compute in which order, so the same rule reads: a pin for the (kind, weight shape, row bucket)
wins; otherwise the engine's mode decides:

    own     this package's kernel wherever one serves the shape, the vendor library's plain form elsewhere
    vendor  the vendor library's plain form everywhere (the few-row kernels, which have no vendor counterpart in the
            engine, are not a choice and stay)
    timed   the candidates are timed against each other once, while the engine starts (never inside a request); a
            bucket that start-up did not reach falls back to `own` and is recorded as such

What every (kind, shape, bucket) took is in `taken`, in the form `pins` accepts: a timed run's choices can be read
from `Engine.stats()["products"]` and given back as `EngineConfig.product_pins`, which makes the run repeatable.
"""
from __future__ import annotations

from collections.abc import Callable, Mapping

MODES = ("own", "vendor", "timed")

# kind -> (this package's form or the plain default, every form)
KINDS: dict[str, tuple[str, tuple[str, ...]]] = {
    "rows": ("rows", ("rows", "vendor")),         # 17 to 64 rows over many tiles, rows shared through LDS
    "glu": ("rows", ("rows", "vendor")),          # the same with SiLU-mul inside
    "parts": ("parts", ("parts", "vendor")),      # a narrow weight, K in shares: 17 to 128 rows; to 1,024 where K is well above N
    "vendor": ("bf16", ("bf16", "f32", "f32x2")),  # the vendor product's own forms (result type, K in halves)
}


class ProductError(ValueError):
    pass


def key_of(kind: str, shape: tuple[int, int], bucket: int) -> str:
    """`kind:NxK:rows`, rows being the largest row count of the bucket."""
    return f"{kind}:{shape[0]}x{shape[1]}:{bucket}"


def row_bucket(rows: int) -> int:
    """The row bucket a step of `rows` rows falls in: up to 32, up to 64, then powers of two, and 768 between 512 and
    1,024 (a portion of 512 tokens beside decode rows is served as it would be alone, not as 1,024 rows are)."""
    if rows <= 32:
        return 32
    if 512 < rows <= 768:
        return 768
    return 1 << (rows - 1).bit_length()


def check_pins(pins: Mapping[str, str] | None) -> dict[str, str]:
    out = {}
    for key, form in (pins or {}).items():
        fields = str(key).split(":")
        sizes = fields[1].split("x") if len(fields) == 3 else []
        if len(fields) != 3 or fields[0] not in KINDS or len(sizes) != 2 or not all(s.isdigit() for s in sizes) \
                or not fields[2].isdigit():
            raise ProductError(f"product pin {key!r}: expected kind:NxK:rows with kind one of {sorted(KINDS)}")
        if form not in KINDS[fields[0]][1]:
            raise ProductError(f"product pin {key!r} = {form!r}: the forms of {fields[0]!r} are {KINDS[fields[0]][1]}")
        out[str(key)] = form
    return out


class ProductPlan:
    """The choices of one engine. `choose` is the one place a choice is made."""

    def __init__(self, mode: str = "own", pins: Mapping[str, str] | None = None) -> None:
        if mode not in MODES:
            raise ProductError(f"products must be one of {MODES}, got {mode!r}")
        self.mode = mode
        self.pins = check_pins(pins)
        self.taken: dict[str, str] = {}           # what each (kind, shape, bucket) took, pins' syntax
        self.how: dict[str, str] = {}             # and why: pinned | own | vendor | timed | untimed
        self.resolving = False                    # True only while the engine starts: `timed` may time now
        self.seconds = 0.0                        # what the timings cost

    def choose(self, kind: str, shape: tuple[int, int], bucket: int, time: Callable[[], str] | None = None) -> str:
        """The form the product `kind` over a weight of `shape` takes at `bucket` rows. `time()` runs the candidates
        against each other and names the winner; it is called at most once per key, and only while the engine
        starts."""
        key = key_of(kind, shape, bucket)
        form = self.taken.get(key)
        if form is not None:
            return form
        own, forms = KINDS[kind]
        if key in self.pins:
            form, how = self.pins[key], "pinned"
        elif self.mode == "vendor":
            form, how = forms[-1] if kind != "vendor" else "bf16", "vendor"
        elif self.mode == "timed" and self.resolving and time is not None:
            import time as clock
            t0 = clock.perf_counter()
            form, how = time(), "timed"
            self.seconds += clock.perf_counter() - t0
            if form not in forms:
                raise ProductError(f"timing {key} named {form!r}, not one of {forms}")
        else:
            form, how = own, "own" if self.mode == "own" else "untimed"
        self.taken[key], self.how[key] = form, how
        return form

    def report(self) -> dict[str, str]:
        return dict(sorted(self.taken.items()))
