"""The HIP kernels behind the `Kernels` contract: ctypes bindings to libholon_hip.so (hand-written gfx950 kernels in
`holon_amd/csrc`). Dense matrix products go to the vendor library through torch where the reference uses its vendor
library for them (std/holon_std/ops/units.py:229); everything else is this package's own code. There is no fallback:
a missing library is built, and if that fails, loading raises."""
from __future__ import annotations

import copy
import ctypes
import sys
import weakref

import torch

from . import build as _build
from .api import AttnRows
from .registry import kernel_op
from ..config.products import ProductPlan, row_bucket

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


class HipKernels:
    name = "hip-gfx950"
    _instance: "HipKernels | None" = None

    @classmethod
    def load(cls, build_if_missing: bool = True) -> "HipKernels":
        if cls._instance is None:
            path = _build.find_library()
            if path is None:
                if not build_if_missing:
                    raise KernelError("libholon_hip.so is not built (run `python -m holon_amd.kernels.build`)")
                path = _build.build()
            else:
                stamp = path.parent / (path.name + ".hash")
                if stamp.is_file() and stamp.read_text().strip() != _build.source_hash():
                    print(f"holon_amd: warning: {path} was built from other sources than holon_amd/csrc holds; "
                          "rebuild with `python -m holon_amd.kernels.build`", file=sys.stderr)
            cls._instance = cls(str(path))
        return cls._instance

    def __init__(self, path: str) -> None:
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from e
        self.path = path
        lib = self.lib
        lib.holon_last_error.restype = ctypes.c_char_p
        sig = {
            "holon_embedding": [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P],
            "holon_row_sumsq": [_P, _P, _I, _I, _I, _P],
            "holon_rmsnorm": [_P, _P, _P, _P, _L, _I, _F, _I, _P],
            "holon_silu_mul": [_P, _P, _L, _I, _I, _P],
            "holon_qk_norm_rope_write": [_P, _L, _P, _I, _I, _I, _I, _P, _P, _F, _P, _I, _I, _P, _P, _P, _P, _I, _I,
                                         _I, _P],
            "holon_kv_write": [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
            "holon_attention_generic": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
            "holon_attention_mfma_supported": [_I, _I, _I],
            "holon_attention_prefill_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I,
                                             _P],
            "holon_attention_decode_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P,
                                            _I, _I, _P],
            "holon_attention_prefill_form": [_I],
            "holon_attention_prefill_copies": [_I],
            "holon_attention_decode_waves_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I,
                                                  _P, _P, _I, _I, _I, _I, _P],
            "holon_attention_decode_fused_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I,
                                                  _P, _P, _F, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _P],
            "holon_gemm_skinny_supported": [_I, _I, _I],
            "holon_gemm_skinny_bf16": [_P, _P, _P, _I, _I, _I, _I, _I, _P],
            "holon_tile_weight_bf16": [_P, _P, _I, _I, _P, _P],
            "holon_gemm_rows_supported": [_I, _I, _I, _I],
            "holon_gemm_rows_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
            "holon_gemm_rows_glu_bf16": [_P, _P, _P, _I, _I, _I, _P],
            "holon_gemm_rows_splits": [_I, _I, _I],
            "holon_gemm_rows_parts_supported": [_I, _I, _I, _I],
            "holon_gemm_rows_parts_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
            "holon_gemm_tiles_splits": [_I, _I, _I],
            "holon_gemm_tiles_parts_supported": [_I, _I, _I, _I],
            "holon_gemm_tiles_parts_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
            "holon_sum_parts": [_P, _P, _I, _L, _P],
            "holon_rmsnorm_parts": [_P, _I, _P, _P, _P, _L, _I, _F, _P],
            "holon_gemm_skinny_scaled_bf16": [_P, _P, _P, _I, _I, _I, _I, _P, _I, _F, _P],
            "holon_gemm_f32": [_P, _P, _P, _I, _I, _I, _P],
            "holon_gemm_skinny_add_bf16": [_P, _P, _P, _I, _I, _I, _P, _P],
            "holon_gemm_skinny_glu_bf16": [_P, _P, _P, _I, _I, _I, _I, _P, _I, _F, _P],
            "holon_argmax": [_P, _P, _I, _I, _P, _P],
            "holon_argmax_pieces": [_I],
            "holon_store_tokens": [_P, _P, _P, _I, _I, _P],
            "holon_sample": [_P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P],
            "holon_scatter_rows": [_P, _P, _P, _I, _I, _I, _P],
            "holon_logprobs": [_P, _P, _I, _I, _I, _P, _P, _P, _P],
        }
        for name, args in sig.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, _I
        self.plan = ProductPlan("own")            # which form a product takes where several serve it: see `configured`
        self._tiled_weights: dict[tuple, list] = {}   # weight shape -> weak (weight, tiled copy) pairs, see _alike
        self._f32_result: bool | None = None      # whether torch has a float32 result for a bfloat16 product (probed once)

    def configured(self, products: str = "own", pins=None) -> "HipKernels":
        """The same kernels with product choices of their own: an engine's `products` mode and `product_pins`. The
        library, and the record of tiled weights by shape, are shared; what a product took is per engine
        (`plan.taken`)."""
        other = copy.copy(self)
        other.plan = ProductPlan(products, pins)
        return other

    def product_choice(self, kind: str, weight, rows: int, time=None) -> str:
        """The one place a product's form is resolved: pinned, else by the engine's mode, else (mode `timed`, while
        the engine starts and outside graph capture) by timing the candidates once."""
        if time is not None and (not self.plan.resolving or torch.cuda.is_current_stream_capturing()):
            time = None
        return self.plan.choose(kind, tuple(weight.shape), row_bucket(rows), time)

    # -- operations that parts bring with them ----------------------------------------------------------------------
    _part_libs: dict[str, ctypes.CDLL] = {}       # libraries built from parts' own sources, by source path

    def __getattr__(self, name: str):
        """An operation registered with `holon_amd.kernels.registry.register_kernel`: its HIP form when it has one
        (the symbol from this library, or from the library built from the operation's own source), else its plain
        form."""
        op = kernel_op(name) if not name.startswith("_") else None
        if op is None:
            raise AttributeError(f"{type(self).__name__} has no operation {name!r}")
        if op.symbol is None:
            return op.plain
        lib = self.lib
        if op.source is not None:
            key = str(op.source)
            lib = self._part_libs.get(key)
            if lib is None:
                path = _build.source_library(op.source) or _build.build_source(op.source)
                try:
                    lib = self._part_libs[key] = ctypes.CDLL(str(path))
                except OSError as e:
                    raise KernelError(f"cannot load {path}: {e}") from e
        fn = getattr(lib, op.symbol)
        fn.argtypes, fn.restype = [*op.argtypes, _P], _I

        def launch(*args) -> None:
            rc = fn(*args, self._stream())
            if rc != 0:
                detail = self.lib.holon_last_error().decode() if op.source is None else f"returned {rc}"
                raise KernelError(f"{op.symbol}: {detail}")
        return lambda *args, **kwargs: op.call(launch, *args, **kwargs)

    # -- plumbing -------------------------------------------------------------------------------------------------
    def _call(self, fn, *args) -> None:
        if fn(*args) != 0:
            raise KernelError(self.lib.holon_last_error().decode())

    @staticmethod
    def _stream() -> int:
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())

    @staticmethod
    def _check(t: torch.Tensor, what: str, dtype: torch.dtype | None = None) -> None:
        if not t.is_cuda:
            raise KernelError(f"{what}: the HIP kernels need a GPU tensor, got one on {t.device}")
        if not t.is_contiguous():
            raise KernelError(f"{what}: tensor must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{what}: expected {dtype}, got {t.dtype}")

    def _check_product(self, what: str, x, weight, tiled=None, *others) -> None:
        """Before a product is launched on raw pointers: every operand on the GPU and contiguous, the tiled copy (which
        the kernels index as they index the weight) of the weight's shape and type."""
        self._check(x, f"{what} x")
        self._check(weight, f"{what} weight")
        if tiled is not None:
            self._check(tiled, f"{what} tiled weight", weight.dtype)
            if tiled.shape != weight.shape:
                raise KernelError(f"{what}: a tiled copy of shape {tuple(tiled.shape)} for a weight of {tuple(weight.shape)}")
        for t in others:
            if t is not None:
                self._check(t, f"{what} operand")

    @staticmethod
    def _dt(t: torch.Tensor, what: str) -> int:
        if t.dtype not in _DT:
            raise KernelError(f"{what}: dtype {t.dtype} is not served (float32 and bfloat16 are)")
        return _DT[t.dtype]

    # -- ops ------------------------------------------------------------------------------------------------------
    def embedding(self, ids, table, take=None, want_stats=False):
        self._check(ids, "embedding ids", torch.int32)
        self._check(table, "embedding table")
        take_slot, last_token = take if take is not None else (None, None)
        if take is not None:
            self._check(take_slot, "embedding take_slot", torch.int32)
            self._check(last_token, "embedding last_token", torch.int32)
            if take_slot.shape != ids.shape:
                raise KernelError(f"embedding: {tuple(take_slot.shape)} slots to take from for {tuple(ids.shape)} tokens")
        out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
        stats = None
        if want_stats and ids.shape[0] <= self.skinny_rows and table.dtype == torch.bfloat16:
            stats = torch.empty((1, 16), dtype=torch.float32, device=table.device)
        self._call(self.lib.holon_embedding, ids.data_ptr(), _ptr(take_slot), _ptr(last_token), table.data_ptr(),
                   out.data_ptr(), ids.shape[0], table.shape[1], table.shape[0], self._dt(table, "embedding"),
                   _ptr(stats), self._stream())
        return (out, stats) if want_stats else out

    def row_sumsq(self, x):
        self._check(x, "row_sumsq x")
        rows, dim = x.shape
        if rows > 16:
            raise KernelError(f"row_sumsq: {rows} rows (at most 16)")
        stats = torch.empty((1, 16), dtype=torch.float32, device=x.device)
        self._call(self.lib.holon_row_sumsq, x.data_ptr(), stats.data_ptr(), rows, dim, self._dt(x, "row_sumsq"),
                   self._stream())
        return stats

    def rmsnorm(self, x, weight, eps):
        self._check(x, "rmsnorm x")
        self._check(weight, "rmsnorm weight", x.dtype)
        dim = x.shape[-1]
        if weight.shape != (dim,):
            raise KernelError(f"rmsnorm: weight {tuple(weight.shape)} does not fit rows of {dim}")
        y = torch.empty_like(x)
        self._call(self.lib.holon_rmsnorm, x.data_ptr(), None, weight.data_ptr(), y.data_ptr(), x.numel() // dim, dim,
                   float(eps), self._dt(x, "rmsnorm"), self._stream())
        return y

    def add_rmsnorm(self, x, residual, weight, eps):
        if x.dtype == torch.float32 and residual.dtype == torch.bfloat16:     # a product as sums over shares of K
            self._check(x, "add_rmsnorm parts")
            self._check(residual, "add_rmsnorm residual")
            self._check(weight, "add_rmsnorm weight", torch.bfloat16)
            dim = residual.shape[-1]
            if x.dim() != residual.dim() + 1 or x.shape[1:] != residual.shape or weight.shape != (dim,):
                raise KernelError(f"add_rmsnorm: parts {tuple(x.shape)} for rows {tuple(residual.shape)}, "
                                  f"weight {tuple(weight.shape)}")
            y = torch.empty_like(residual)
            self._call(self.lib.holon_rmsnorm_parts, x.data_ptr(), x.shape[0], residual.data_ptr(), weight.data_ptr(),
                       y.data_ptr(), residual.numel() // dim, dim, float(eps), self._stream())
            return y
        self._check(x, "add_rmsnorm x")
        self._check(residual, "add_rmsnorm residual", x.dtype)
        self._check(weight, "add_rmsnorm weight", x.dtype)
        dim = x.shape[-1]
        if residual.shape != x.shape or weight.shape != (dim,):
            raise KernelError(f"add_rmsnorm: shapes {tuple(x.shape)}, {tuple(residual.shape)}, {tuple(weight.shape)}")
        y = torch.empty_like(x)
        self._call(self.lib.holon_rmsnorm, x.data_ptr(), residual.data_ptr(), weight.data_ptr(), y.data_ptr(),
                   x.numel() // dim, dim, float(eps), self._dt(x, "add_rmsnorm"), self._stream())
        return y

    skinny_rows = 16          # up to this many rows (one tile of tokens) the hand-written weight-streaming product runs
    deep_k = 8192             # from this K on, prompt portions of up to 1,024 rows choose between the vendor's forms too

    def tile_weight(self, weight, scale=None):
        """A copy of `weight` [N, K] in the layout the few-row product streams fastest, or None when its shape or
        dtype has no such layout (then `linear` reads the rows as they are). With `scale` [K] the copy holds
        weight * scale (a norm's weight folded in)."""
        n, k = weight.shape
        if weight.dtype != torch.bfloat16 or not weight.is_cuda or n % 16 or k % 32 or k < 256:
            return None
        self._check(weight, "tile_weight")
        if scale is not None:
            self._check(scale, "tile_weight scale", torch.bfloat16)
            if scale.shape != (k,):
                raise KernelError(f"tile_weight: scale {tuple(scale.shape)} for K = {k}")
        tiled = torch.empty_like(weight)
        self._call(self.lib.holon_tile_weight_bf16, weight.data_ptr(), tiled.data_ptr(), n, k, _ptr(scale),
                   self._stream())
        known = self._tiled_weights.setdefault((n, k), [])
        known[:] = [(w, t) for w, t in known if w() is not None and t() is not None and w() is not weight]
        known.append((weakref.ref(weight), weakref.ref(tiled)))
        return tiled

    def _alike(self, weight, tiled, most: int = 16, most_bytes: int = 1 << 30) -> list[tuple]:
        """(weight, tiled copy) pairs to time a choice on: the given one, then other live weights of its shape that
        were tiled here (the same projection in other layers). A timing that calls one weight over and over reads it
        from the memory-side cache (256 MB), which flatters the vendor library's kernels by a third and decides
        wrongly; a step streams every layer's weights from memory, so the timings rotate over these pairs."""
        pairs = [(weight, tiled)]
        for w, t in self._tiled_weights.get(tuple(weight.shape), []):
            w, t = w(), t()
            if len(pairs) >= most or len(pairs) * weight.numel() * weight.element_size() >= most_bytes:
                break
            if w is not None and t is not None and w is not weight and w.dtype == weight.dtype \
                    and w.device == weight.device:
                pairs.append((w, t if tiled is not None else None))
        return pairs

    @staticmethod
    def _graph_time(calls: list, replays: int = 3) -> float:
        """Milliseconds a call, for calls that are shorter than a launch from here takes: recorded as one graph
        (each call once, in order), replayed. What a call needs at its first use happens before the recording. A
        candidate that there is no memory to try takes forever (and so is not chosen)."""
        try:
            for call in calls:
                call()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                keep = [call() for call in calls]
            graph.replay()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(replays):
                graph.replay()
            end.record()
            end.synchronize()
            del graph, keep
        except RuntimeError as e:                 # no room to try it (out of memory surfaces from the capture's end as
            torch.cuda.synchronize()              # a plain RuntimeError too), or it cannot be recorded: it does not win
            torch.cuda.empty_cache()
            print(f"holon_amd: a product candidate could not be timed and is not chosen: {str(e).splitlines()[0]}",
                  file=sys.stderr)
            return float("inf")
        return start.elapsed_time(end) / (replays * len(calls))

    @staticmethod
    def _in_turn(pairs: list[tuple], call, at_least: int = 8) -> list:
        """`call(weight, tiled)` for each pair in turn, at least `at_least` calls in all."""
        rounds = -(-at_least // len(pairs))
        return [lambda w=w, t=t: call(w, t) for _ in range(rounds) for w, t in pairs]

    def _row_scale(self, x, tiled, row_scale, what):
        """Checks of a product over un-normed rows with the norm folded into `tiled`; returns (stats, parts, eps)."""
        stats, eps = row_scale
        if tiled is None or x.shape[0] > self.skinny_rows or x.dtype != torch.bfloat16:
            raise KernelError(f"{what}: a folded norm needs tiled weights and at most 16 bfloat16 rows")
        self._check(stats, f"{what} stats", torch.float32)
        if stats.dim() != 2 or stats.shape[1] != 16:
            raise KernelError(f"{what}: stats {tuple(stats.shape)}, expected [parts, 16]")
        return stats, stats.shape[0], float(eps)

    def folds_norm(self, rows, weight, tiled):
        """Whether `linear(x, ..., row_scale=...)` serves `rows` rows over this weight."""
        n, k = weight.shape
        return bool(tiled is not None and weight.dtype == torch.bfloat16 and 1 <= rows <= self.skinny_rows
                    and k >= 256 and self.lib.holon_gemm_skinny_supported(rows, n, k))

    def linear(self, x, weight, out_dtype=None, tiled=None, row_scale=None):
        m, k = x.shape
        n = weight.shape[0]
        if weight.shape[1] != k:
            raise KernelError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(weight.shape)}")
        if row_scale is not None:
            stats, parts, eps = self._row_scale(x, tiled, row_scale, "linear")
            self._check_product("linear", x, weight, tiled)
            to_f32 = out_dtype == torch.float32
            y = torch.empty((m, n), dtype=torch.float32 if to_f32 else torch.bfloat16, device=x.device)
            self._call(self.lib.holon_gemm_skinny_scaled_bf16, x.data_ptr(), tiled.data_ptr(), y.data_ptr(), m, n, k,
                       2 if to_f32 else 0, stats.data_ptr(), parts, eps, self._stream())
            return y
        if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 1 <= m <= self.skinny_rows and k >= 256
                and x.is_contiguous() and weight.is_contiguous() and self.lib.holon_gemm_skinny_supported(m, n, k)):
            to_f32 = out_dtype == torch.float32       # then: the bfloat16 product cast up, as for any number of rows
            self._check_product("linear", x, weight, tiled)
            y = torch.empty((m, n), dtype=torch.float32 if to_f32 else torch.bfloat16, device=x.device)
            source = tiled if tiled is not None else weight
            self._call(self.lib.holon_gemm_skinny_bf16, x.data_ptr(), source.data_ptr(), y.data_ptr(), m, n, k,
                       2 if to_f32 else 0, int(tiled is not None), self._stream())
            return y
        if x.dtype == torch.bfloat16 and x.is_contiguous() and self.serves_rows(m, weight, tiled):
            return self._rows_product(x, weight, tiled, False, out_dtype == torch.float32)
        if x.dtype == torch.float32 and weight.dtype == torch.float32 and out_dtype in (None, torch.float32):
            # the 32-bit path's own product: true float32, every sum in an order that K alone decides
            self._check(x, "linear x")
            self._check(weight, "linear weight")
            y = torch.empty((m, n), dtype=torch.float32, device=x.device)
            self._call(self.lib.holon_gemm_f32, x.data_ptr(), weight.data_ptr(), y.data_ptr(), m, n, k, self._stream())
            return y
        # the vendor library's product of bfloat16 operands, float32 accumulation
        y = self._vendor_product(x, weight)
        return y if out_dtype in (None, y.dtype) else y.to(out_dtype)

    def _vendor_product(self, x, weight):
        """x W^T by the vendor library, rounded once to the operands' type. For steps of 17 to 64 bfloat16 rows the
        library's choice of kernel has holes at some shapes (a deep, narrow weight, 5120 x 25600: 145 us, where its
        product of the same operands with a float32 result takes 83, two such products over the halves of K 73, and
        the weights alone would stream in 42); over deep weights (K of 8,192 and more) the same holds for prompt
        portions of up to 1,024 rows. Which form such a step takes is a product choice of kind `vendor` (pinned, or
        timed at start in mode `timed`, else the plain form). All forms accumulate in float32 and round once."""
        m, k = x.shape[0], weight.shape[1]
        if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and (16 < m <= 64 or (64 < m <= 1024 and k >= self.deep_k))):
            return torch.matmul(x, weight.t())
        form = self.product_choice("vendor", weight, m, lambda: self._time_mid_forms(x, weight))
        if form != "bf16" and not self.has_f32_result():
            raise KernelError(f"product form {form!r} needs torch.mm(..., out_dtype=float32), which this torch lacks")
        return self._MID_FORMS[form](x, weight)

    def has_f32_result(self) -> bool:
        """Whether this torch multiplies bfloat16 operands into a float32 result; probed once, eagerly."""
        if self._f32_result is None:
            try:
                a = torch.zeros((32, 64), dtype=torch.bfloat16, device="cuda")
                torch.mm(a, a.t(), out_dtype=torch.float32)
                self._f32_result = True
            except (RuntimeError, TypeError):
                self._f32_result = False
        return self._f32_result

    @staticmethod
    def _two_halves(x, weight):
        half = weight.shape[1] // 2
        low = torch.mm(x[:, :half], weight[:, :half].t(), out_dtype=torch.float32)
        return low.add_(torch.mm(x[:, half:], weight[:, half:].t(), out_dtype=torch.float32)).to(torch.bfloat16)

    _MID_FORMS = {"bf16": lambda x, w: torch.matmul(x, w.t()),
                  "f32": lambda x, w: torch.mm(x, w.t(), out_dtype=torch.float32).to(torch.bfloat16),
                  "f32x2": lambda x, w: HipKernels._two_halves(x, w)}

    def _time_mid_forms(self, x, weight) -> str:
        if not self.has_f32_result():
            return "bf16"
        pairs = self._alike(weight, None)
        took = {}
        for name, fn in self._MID_FORMS.items():
            if name == "f32x2" and weight.shape[1] % 512:
                continue
            took[name] = self._graph_time(self._in_turn(pairs, lambda w, _t, fn=fn: fn(x, w)))
        best = min(took, key=took.get)
        return best if took[best] < 0.92 * took["bf16"] else "bf16"

    def serves_rows(self, rows, weight, tiled, gated=False):
        """Whether steps of `rows` rows (17 to 64) over this weight run the product that shares the rows through LDS
        (`tiled` is then read; a copy with a norm folded in needs rows normed without the norm's weight). The kernel
        must serve the shape and, timed once per weight shape and row bucket against the vendor library's product of
        the same rows (outside graph capture), be the faster of the two."""
        n, k = weight.shape
        if not (tiled is not None and weight.dtype == torch.bfloat16 and 16 < rows <= 64
                and self.lib.holon_gemm_rows_supported(rows, n // 2 if gated else n, k, int(gated))):
            return False
        return self.product_choice("glu" if gated else "rows", weight, rows,
                                   lambda: self._time_rows(rows, weight, tiled, gated)) == "rows"

    def _rows_product(self, x, weight, tiled, gated, to_f32=False):
        m, k = x.shape
        n = weight.shape[0] // 2 if gated else weight.shape[0]
        self._check_product("linear", x, weight, tiled)
        y = torch.empty((m, n), dtype=torch.float32 if to_f32 else torch.bfloat16, device=x.device)
        if gated:
            self._call(self.lib.holon_gemm_rows_glu_bf16, x.data_ptr(), tiled.data_ptr(), y.data_ptr(), m, n, k, self._stream())
        else:
            self._call(self.lib.holon_gemm_rows_bf16, x.data_ptr(), tiled.data_ptr(), y.data_ptr(), m, n, k, int(to_f32),
                       self._stream())
        return y

    parts_rows = 1024         # the products in shares of K serve steps of 17 to this many rows
    parts_rows_short = 128    # of which the kernel for weights of any K serves up to this many

    def linear_parts(self, x, weight, tiled):
        """-> float32 [splits, M, N], the product over each share of K, when a kernel of that kind serves this step
        (17 to 128 bfloat16 rows over a narrow tiled weight; 129 to 1,024 rows where K is well above N) and,
        timed once per weight shape and row bucket against the vendor library's product (each with the add + norm
        that reads it), is the faster; None otherwise (nothing was done)."""
        (m, k), n = x.shape, weight.shape[0]
        if not (tiled is not None and 16 < m <= self.parts_rows and x.dtype == torch.bfloat16
                and weight.dtype == torch.bfloat16 and weight.shape[1] == k and x.is_contiguous()):
            return None
        splits = (self.lib.holon_gemm_rows_splits if m <= self.parts_rows_short else self.lib.holon_gemm_tiles_splits)(m, n, k)
        if not splits:
            return None
        use = self.product_choice("parts", weight, m, lambda: self._time_parts(x, weight, tiled, splits))
        return self._rows_parts(x, weight, tiled, splits) if use == "parts" else None

    def _rows_parts(self, x, weight, tiled, splits):
        (m, k), n = x.shape, weight.shape[0]
        self._check_product("linear in parts", x, weight, tiled)
        if tiled is None or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.shape[1] != k:
            raise KernelError(f"linear in parts: bfloat16 rows {tuple(x.shape)} over a tiled bfloat16 weight "
                              f"{tuple(weight.shape)} expected")
        parts = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
        entry = self.lib.holon_gemm_rows_parts_bf16 if m <= self.parts_rows_short else self.lib.holon_gemm_tiles_parts_bf16
        self._call(entry, x.data_ptr(), tiled.data_ptr(), parts.data_ptr(), m, n, k, splits, self._stream())
        return parts

    def _time_parts(self, x, weight, tiled, splits) -> str:
        """Each way together with the residual add + norm that reads the product (reading parts costs that kernel a
        little, which the product must win back)."""
        n = weight.shape[0]
        residual = torch.zeros((x.shape[0], n), dtype=torch.bfloat16, device=x.device)
        ones = torch.ones(n, dtype=torch.bfloat16, device=x.device)
        pairs = self._alike(weight, tiled)
        rival = self._MID_FORMS[self._time_mid_forms(x, weight)]      # the vendor library's best form (kept only if it wins)
        took = {
            "parts": self._graph_time(self._in_turn(
                pairs, lambda w, t: self.add_rmsnorm(self._rows_parts(x, w, t, splits), residual, ones, 1e-6))),
            "vendor": self._graph_time(self._in_turn(
                pairs, lambda w, _t: self.add_rmsnorm(rival(x, w), residual, ones, 1e-6)))}
        return "parts" if took["parts"] < 0.97 * took["vendor"] else "vendor"

    def sum_parts(self, parts, dtype=torch.bfloat16):
        """[splits, ...] float32 -> bfloat16 [...]: the parts added up in order, rounded once."""
        self._check(parts, "sum_parts", torch.float32)
        if dtype != torch.bfloat16:
            raise KernelError(f"sum_parts: partial sums are of bfloat16 products, not {dtype}")
        y = torch.empty(parts.shape[1:], dtype=torch.bfloat16, device=parts.device)
        if y.numel() % 4:
            raise KernelError(f"sum_parts: {y.numel()} values are no multiple of 4")
        self._call(self.lib.holon_sum_parts, parts.data_ptr(), y.data_ptr(), parts.shape[0], y.numel(), self._stream())
        return y

    def _time_rows(self, rows, weight, tiled, gated) -> str:
        x = torch.randn(rows, weight.shape[1], device=weight.device).to(torch.bfloat16)
        pairs = self._alike(weight, tiled)
        rival = self._MID_FORMS[self._time_mid_forms(x, weight)]      # the vendor library's best form (kept only if it wins)
        vendor = (lambda w, _t: self.silu_mul(rival(x, w))) if gated else (lambda w, _t: rival(x, w))
        took = {"rows": self._graph_time(self._in_turn(pairs, lambda w, t: self._rows_product(x, w, t, gated))),
                "vendor": self._graph_time(self._in_turn(pairs, vendor))}
        return "rows" if took["rows"] < took["vendor"] else "vendor"

    def linear_add(self, x, weight, tiled, residual, want_stats=False):
        """-> False when not fused; otherwise True, or with `want_stats` the partial sums of squares [N / 16, 16] of
        the residual rows as they now are."""
        (m, k), n = x.shape, weight.shape[0]
        if not (tiled is not None and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and residual.dtype == torch.bfloat16 and 1 <= m <= self.skinny_rows and weight.shape[1] == k
                and k >= 256 and x.is_contiguous() and residual.is_contiguous()
                and self.lib.holon_gemm_skinny_supported(m, n, k)):
            return False
        if tuple(residual.shape) != (m, n):
            raise KernelError(f"linear_add: residual {tuple(residual.shape)} for a product of {(m, n)}")
        self._check_product("linear_add", x, weight, tiled, residual)
        stats = torch.empty((n // 16, 16), dtype=torch.float32, device=x.device) if want_stats else None
        self._call(self.lib.holon_gemm_skinny_add_bf16, x.data_ptr(), tiled.data_ptr(), residual.data_ptr(), m, n, k,
                   _ptr(stats), self._stream())
        return stats if want_stats else True

    def linear_silu_mul(self, x, weight, tiled=None, row_scale=None):
        """silu_mul(linear(x, weight)) in one kernel for steps of few rows, with the roundings of the two kernels one
        after the other (the sums over K may be split differently); None when this shape is not fused (the caller then composes the two)."""
        m, k = x.shape
        two_i = weight.shape[0]
        if row_scale is None and weight.shape[1] == k and x.dtype == torch.bfloat16 and x.is_contiguous() \
                and two_i % 2 == 0 and self.serves_rows(m, weight, tiled, gated=True):
            return self._rows_product(x, weight, tiled, True)
        if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 1 <= m <= self.skinny_rows
                and two_i % 32 == 0 and k % 128 == 0 and k >= 256 and weight.shape[1] == k and x.is_contiguous()):
            return None
        self._check_product("linear_silu_mul", x, weight, tiled)
        y = torch.empty((m, two_i // 2), dtype=torch.bfloat16, device=x.device)
        source = tiled if tiled is not None else weight
        stats, parts, eps = self._row_scale(x, tiled, row_scale, "linear_silu_mul") if row_scale is not None \
            else (None, 0, 0.0)
        self._call(self.lib.holon_gemm_skinny_glu_bf16, x.data_ptr(), source.data_ptr(), y.data_ptr(), m, two_i // 2, k,
                   int(tiled is not None), _ptr(stats), parts, eps, self._stream())
        return y

    def silu_mul(self, gate_up):
        self._check(gate_up, "silu_mul")
        t, two_i = gate_up.shape
        if two_i % 2:
            raise KernelError(f"silu_mul: width {two_i} is odd")
        out = torch.empty((t, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
        self._call(self.lib.holon_silu_mul, gate_up.data_ptr(), out.data_ptr(), t, two_i // 2,
                   self._dt(gate_up, "silu_mul"), self._stream())
        return out

    def rope(self, x, positions, table):
        self._check(x, "rope x")
        self._check(positions, "rope positions", torch.int32)
        self._check(table, "rope table", torch.float32)
        t, heads, d = x.shape
        self._call(self.lib.holon_qk_norm_rope_write, x.data_ptr(), heads * d, x.data_ptr(), t, heads, 0, d, None,
                   None, 0.0, table.data_ptr(), table.shape[1], table.shape[0], positions.data_ptr(), None, None,
                   None, 1, 1, self._dt(x, "rope"), self._stream())

    def kv_write(self, k, v, pages, write_page, write_off, page_size):
        for t, what in ((k, "k"), (v, "v"), (pages, "pages")):
            self._check(t, f"kv_write {what}", k.dtype)
        self._check(write_page, "kv_write page", torch.int32)
        self._check(write_off, "kv_write offset", torch.int32)
        t, hkv, d = k.shape
        if pages.shape[1:] != (2, hkv, page_size * d) or v.shape != k.shape:
            raise KernelError(f"kv_write: pages {tuple(pages.shape)} do not fit {hkv} heads of {d} in pages of {page_size}")
        self._call(self.lib.holon_kv_write, k.data_ptr(), v.data_ptr(), pages.data_ptr(), write_page.data_ptr(),
                   write_off.data_ptr(), t, hkv, d, page_size, pages.shape[0], self._dt(k, "kv_write"), self._stream())

    def qk_norm_rope_write(self, qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, table, positions, pages,
                           write_page, write_off, page_size):
        self._check(qkv, "qkv")
        t, width = qkv.shape
        if width != (heads + 2 * kv_heads) * head_dim:
            raise KernelError(f"qkv width {width} is not ({heads} + 2*{kv_heads}) * {head_dim}")
        for w in (q_weight, k_weight):
            if w is not None:
                self._check(w, "q/k norm weight", qkv.dtype)
                if w.shape != (head_dim,):
                    raise KernelError(f"q/k norm weight {tuple(w.shape)} does not fit head_dim {head_dim}")
        if table is not None:
            self._check(table, "rope table", torch.float32)
            self._check(positions, "positions", torch.int32)
        if pages is not None:
            self._check(pages, "pages", qkv.dtype)
            self._check(write_page, "write_page", torch.int32)
            self._check(write_off, "write_off", torch.int32)
            if pages.shape[1:] != (2, kv_heads, page_size * head_dim):
                raise KernelError(f"pages {tuple(pages.shape)} do not fit {kv_heads} heads of {head_dim}, page {page_size}")
        q = torch.empty((t, heads, head_dim), dtype=qkv.dtype, device=qkv.device)
        self._call(self.lib.holon_qk_norm_rope_write, qkv.data_ptr(), width, q.data_ptr(), t, heads, kv_heads,
                   head_dim, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(table),
                   table.shape[1] if table is not None else 0, table.shape[0] if table is not None else 0,
                   _ptr(positions), _ptr(pages), _ptr(write_page), _ptr(write_off), page_size,
                   pages.shape[0] if pages is not None else 0, self._dt(qkv, "qkv"), self._stream())
        return q

    def check_attention(self, head_dim, page_size, dtype):
        if dtype not in _DT:
            raise KernelError(f"attention: dtype {dtype} is not served (float32 and bfloat16 are)")
        if head_dim % 8 or not 8 <= head_dim <= 512 or page_size < 1:
            raise KernelError(f"attention: head_dim {head_dim} is not served (multiples of 8 up to 512, any page size "
                              f">= 1; got page size {page_size})")

    def paged_attention(self, q, pages, table, rows: AttnRows, page_size, scale, window):
        self._check(q, "attention q")
        self._check(pages, "attention pages", q.dtype)
        self._check(table, "block table", torch.int32)
        t, hq, d = q.shape
        hkv = pages.shape[2]
        if pages.shape[1] != 2 or pages.shape[3] != page_size * d:
            raise KernelError(f"attention: pages {tuple(pages.shape)} do not fit head_dim {d}, page {page_size}")
        out = torch.empty_like(q)
        b = rows.slots.shape[0]
        if self.lib.holon_attention_mfma_supported(d, page_size, self._dt(q, "attention")):
            common = (q.data_ptr(), out.data_ptr(), pages.data_ptr(), table.data_ptr(), table.shape[1],
                      rows.slots.data_ptr(), rows.lens.data_ptr(), rows.query_start.data_ptr())
            if rows.n_chunk:
                self._call(self.lib.holon_attention_prefill_bf16, *common, rows.chunk_rows.data_ptr(), rows.n_chunk,
                           rows.max_chunk_query, rows.max_chunk_len, hq, hkv, d, page_size, float(scale), int(window),
                           self._stream())
            if rows.n_decode:
                span = rows.max_decode_len if not window else min(rows.max_decode_len, window + 31)
                splits, per, waves = self.decode_splits(rows.n_decode * hkv * ((hq // hkv + 15) // 16), span, d)
                part_o, part_ml = self._decode_parts(rows.n_decode * hq * (splits // waves), d, q.device)
                self._call(self.lib.holon_attention_decode_waves_bf16, *common, rows.decode_rows.data_ptr(),
                           rows.n_decode, rows.max_decode_len, hq, hkv, d, page_size, float(scale), int(window),
                           _ptr(part_o), _ptr(part_ml), splits, per, waves, int(rows.in_order and rows.n_decode == t),
                           self._stream())
            return out
        self._call(self.lib.holon_attention_generic, q.data_ptr(), out.data_ptr(), pages.data_ptr(), table.data_ptr(),
                   table.shape[1], rows.slots.data_ptr(), rows.lens.data_ptr(), rows.query_start.data_ptr(), b, t, hq,
                   hkv, d, page_size, pages.shape[0], float(scale), int(window), self._dt(q, "attention"),
                   self._stream())
        return out

    def qkv_attention(self, qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, rope_table, positions, pages,
                      table, write_page, write_off, rows: AttnRows, page_size, scale, window, writes=True):
        """`paged_attention(qk_norm_rope_write(qkv, ...), ...)`. A step of decode rows alone over the matrix-core
        kernels runs as one kernel less: the attention kernel takes the raw projection, norms and rotates the queries
        itself and puts each row's new key and value into the cache before it reads them."""
        t = qkv.shape[0]
        if not (qkv.dtype == torch.bfloat16 and writes and rows.n_chunk == 0 and rows.n_decode == t
                and (rope_table is None or rope_table.shape[1] == head_dim)
                and self.lib.holon_attention_mfma_supported(head_dim, page_size, _DT[torch.bfloat16])):
            q = self.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, rope_table, positions,
                                        pages if writes else None, write_page, write_off, page_size)
            return self.paged_attention(q, pages, table, rows, page_size, scale, window)
        self._check(qkv, "qkv", torch.bfloat16)
        self._check(pages, "attention pages", torch.bfloat16)
        self._check(table, "block table", torch.int32)
        if qkv.shape[1] != (heads + 2 * kv_heads) * head_dim:
            raise KernelError(f"qkv width {qkv.shape[1]} is not ({heads} + 2*{kv_heads}) * {head_dim}")
        if pages.shape[1:] != (2, kv_heads, page_size * head_dim):
            raise KernelError(f"pages {tuple(pages.shape)} do not fit {kv_heads} heads of {head_dim}, page {page_size}")
        for w in (q_weight, k_weight):
            if w is not None:
                self._check(w, "q/k norm weight", torch.bfloat16)
                if w.shape != (head_dim,):
                    raise KernelError(f"q/k norm weight {tuple(w.shape)} does not fit head_dim {head_dim}")
        if (q_weight is None) != (k_weight is None):
            raise KernelError("q and k norm weights come together")
        if rope_table is not None:
            self._check(rope_table, "rope table", torch.float32)
        for ix, what in ((write_page, "write_page"), (write_off, "write_off")):
            self._check(ix, what, torch.int32)
            if ix.shape[0] < t:
                raise KernelError(f"{what}: {ix.shape[0]} entries for {t} tokens")
        out = torch.empty((t, heads, head_dim), dtype=qkv.dtype, device=qkv.device)
        span = rows.max_decode_len if not window else min(rows.max_decode_len, window + 31)
        splits, per, waves = self.decode_splits(rows.n_decode * kv_heads * ((heads // kv_heads + 15) // 16), span,
                                                head_dim)
        part_o, part_ml = self._decode_parts(rows.n_decode * heads * (splits // waves), head_dim, qkv.device)
        self._call(self.lib.holon_attention_decode_fused_bf16, qkv.data_ptr(), out.data_ptr(), pages.data_ptr(),
                   table.data_ptr(), table.shape[1], rows.slots.data_ptr(), rows.lens.data_ptr(),
                   rows.query_start.data_ptr(), rows.decode_rows.data_ptr(), rows.n_decode, rows.max_decode_len, heads,
                   kv_heads, head_dim, page_size, float(scale), int(window), _ptr(q_weight), _ptr(k_weight), float(eps),
                   _ptr(rope_table), rope_table.shape[0] if rope_table is not None else 0, write_page.data_ptr(),
                   write_off.data_ptr(), _ptr(part_o), _ptr(part_ml), splits, per, waves, int(rows.in_order),
                   self._stream())
        return out

    @staticmethod
    def _decode_parts(cells: int, head_dim: int, device):
        """The split partials' workspace: (values [cells, head_dim], maxima and sums [cells, 2]); none where every
        block writes its row's result."""
        if cells == 0:
            return None, None
        return (torch.empty((cells * head_dim,), dtype=torch.float32, device=device),
                torch.empty((cells * 2,), dtype=torch.float32, device=device))

    @staticmethod
    def decode_splits(pairs: int, span: int, head_dim: int = 128, target_waves: int = 2048, min_keys: int = 64,
                      blocks: int | None = None) -> tuple[int, int, int]:
        """How a decode row's keys are cut over waves: (splits, keys per split, waves a block). `pairs`: (row, kv head)
        tiles in the launch. Enough waves to fill the GPU but at least `min_keys` keys each (a multiple of 32); the
        waves of a block combine their partials through LDS, so as many of a row's splits share a block as leave
        `blocks` blocks in the launch and fit LDS (at most 8): a (row, head) then leaves splits / waves partials for
        the merge, and with one block a row none (the block writes the result, no merge runs). The last return value
        times the number of partials is the splits. Measured at context 4,096 (attention + merge, us a layer): one row
        18.3 with 256 blocks against 19.6 with 512; eight rows 37.3 with 512 against 38.6 with 256."""
        if blocks is None:
            blocks = 256 if pairs <= 16 else 512
        want = max(1, min(64, target_waves // max(1, pairs)))
        per = max(min_keys, -(-span // want))
        per = -(-per // 32) * 32
        splits = max(1, -(-span // per))
        cap = max(1, min(8, (64 * 1024 // 4) // (16 * head_dim + 32) + 1))
        outer = min(splits, max(1, -(-blocks // max(1, pairs))))
        waves = min(cap, -(-splits // outer))
        outer = -(-splits // waves)
        return outer * waves, per, waves

    def argmax(self, logits):
        self._check(logits, "argmax logits", torch.float32)
        out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
        n = self.lib.holon_argmax_pieces(logits.shape[1])
        pieces = torch.empty((logits.shape[0] * n, 2), dtype=torch.float32, device=logits.device) if n else None
        self._call(self.lib.holon_argmax, logits.data_ptr(), out.data_ptr(), logits.shape[0], logits.shape[1],
                   _ptr(pieces), self._stream())
        return out

    def store_tokens(self, last_token, slots, tokens):
        for t, what in ((last_token, "last_token"), (slots, "slots"), (tokens, "tokens")):
            self._check(t, f"store_tokens {what}", torch.int32)
        if slots.shape != tokens.shape:
            raise KernelError(f"store_tokens: {tuple(slots.shape)} slots for {tuple(tokens.shape)} tokens")
        self._call(self.lib.holon_store_tokens, last_token.data_ptr(), slots.data_ptr(), tokens.data_ptr(),
                   tokens.shape[0], last_token.shape[0], self._stream())

    def logprobs(self, logits, tokens, k):
        self._check(logits, "logprobs logits", torch.float32)
        self._check(tokens, "logprobs tokens", torch.int32)
        r = logits.shape[0]
        if tokens.shape != (r,) or not 0 <= k <= 32:
            raise KernelError(f"logprobs: {tuple(tokens.shape)} tokens for {r} rows, k={k} (at most 32)")
        token_lp = torch.empty((r,), dtype=torch.float32, device=logits.device)
        top_ids = torch.empty((r, k), dtype=torch.int32, device=logits.device)
        top_lp = torch.empty((r, k), dtype=torch.float32, device=logits.device)
        self._call(self.lib.holon_logprobs, logits.data_ptr(), tokens.data_ptr(), r, logits.shape[1], k,
                   token_lp.data_ptr(), top_ids.data_ptr(), top_lp.data_ptr(), self._stream())
        return token_lp, top_ids, top_lp

    def sample(self, logits, temperature, top_k, top_p, min_p, seeds, positions, slots=None):
        self._check(logits, "sample logits", torch.float32)
        r = logits.shape[0]
        n = r
        if slots is not None:                      # the parameters are tables by slot
            self._check(slots, "sample slots", torch.int32)
            if slots.shape != (r,):
                raise KernelError(f"sample slots: shape {tuple(slots.shape)} for {r} rows")
            n = temperature.shape[0]
        for t, dt, what in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                            (top_p, torch.float32, "top_p"), (min_p, torch.float32, "min_p"),
                            (seeds, torch.int64, "seeds")):
            self._check(t, f"sample {what}", dt)
            if t.shape != (n,):
                raise KernelError(f"sample {what}: shape {tuple(t.shape)}, expected ({n},)")
        if positions.dtype not in (torch.int32, torch.int64) or positions.shape != (r,):
            raise KernelError(f"sample positions: {positions.dtype} {tuple(positions.shape)} for {r} rows")
        self._check(positions, "sample positions")
        out = torch.empty((r,), dtype=torch.int32, device=logits.device)
        self._call(self.lib.holon_sample, logits.data_ptr(), out.data_ptr(), r, logits.shape[1],
                   temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), min_p.data_ptr(), seeds.data_ptr(),
                   positions.data_ptr(), _ptr(slots), int(positions.dtype == torch.int32), self._stream())
        return out

    def scatter_rows(self, dst, idx, src):
        for t, what in ((dst, "dst"), (idx, "idx"), (src, "src")):
            self._check(t, f"scatter_rows {what}", torch.int32)
        n, width = idx.shape[0], dst.shape[1]
        if src.numel() != n * width:
            raise KernelError(f"scatter_rows: {src.numel()} values for {n} rows of {width}")
        self._call(self.lib.holon_scatter_rows, dst.data_ptr(), idx.data_ptr(), src.data_ptr(), n, width, dst.shape[0],
                   self._stream())
