"""Launchers of the HIP library: the only way the parts reach the GPU.

Every method checks on the host that shapes, dtypes and strides are what the kernel and its
grid assume, then calls the ``extern "C"`` entry point on the current stream. There is no CPU
path: without a GPU or without the built library, ``get_kernels()`` raises.

Conventions: the residual stream and logits are float32; norm weights, norm biases and linear
biases are float32 vectors; matrices, tables, activations and the cache are in the compute
dtype (bfloat16 or float32). A linear weight is ``[out, in]`` (each output's inputs contiguous).
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import build as _build

ACTIVATIONS = {"none": 0, "gelu_new": 1, "gelu": 2, "relu": 3, "silu": 4, "swish": 4, "quick_gelu": 5, "tanh": 6, "relu_squared": 7}
_DT = {torch.float32: 0, torch.bfloat16: 1}

c_void_p, c_int, c_long, c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float


class KernelError(RuntimeError):
    pass


class PendingSum:
    """A matrix product whose sum over K was split into ranges and not finished: ``out`` (float32 ``[M, N]``, the
    product's residual, updated in place) still lacks ``ranges[0] + .. + ranges[S-1] + bias``. ``HipKernels.norm`` folds
    that into the norm of ``out``; ``HipKernels.finish`` runs it by itself. Nothing else may read ``out`` or launch
    another product (the ranges live in the library's one workspace) before one of the two has happened."""

    __slots__ = ("out", "workspace", "n_ranges", "bias", "ldo")

    def __init__(self, out, workspace, n_ranges, bias, ldo):
        self.out, self.workspace, self.n_ranges, self.bias, self.ldo = out, workspace, n_ranges, bias, ldo


class PendingProduct(PendingSum):
    """A product without a residual that has left the sum over its K ranges undone: ``out`` (float32 ``[M, N]``) holds nothing
    yet; it is ``ranges[0] + .. + ranges[S-1] + bias``. ``HipKernels.streams_step`` reads the ranges in place of the result;
    ``HipKernels.finish`` computes ``out``. The ranges live in the library's one workspace: no other product may be launched
    before one of the two has happened."""

    __slots__ = ()


class PendingAverage:
    """A weighted sum of residual streams that has not been computed yet (``HipKernels.stream_average(..., defer=True)``):
    ``out`` (float32 ``[T, D]``) still holds the layer's own result. ``HipKernels.norm`` computes the sum inside the norm
    that reads it; ``HipKernels.finish`` runs it by itself. Nothing else may read ``out`` before one of the two."""

    __slots__ = ("out", "streams", "weights", "n")

    def __init__(self, out, streams, weights, n):
        self.out, self.streams, self.weights, self.n = out, streams, weights, n


class PendingStreams:
    """A sublayer's result ``y`` that has not been written into the residual streams yet (``HipKernels.streams_step`` with
    ``defer``): ``streams`` float32 ``[n, T, D]`` still lack ``x_t <- sum_s mix[s, t] x_s + out[t] y``. The next read of the
    streams does it in its own pass. ``out`` is the tensor that stands for the residual stream outside the layers (the sum of
    the streams): ``HipKernels.norm`` of it computes write, sum and norm in one kernel; ``HipKernels.finish`` writes the streams
    and stores their sum there."""

    __slots__ = ("out", "streams", "y", "mix", "w_out", "y_pending")

    def __init__(self, out, streams, y, mix, w_out, y_pending=None):
        self.out, self.streams, self.y, self.mix, self.w_out, self.y_pending = out, streams, y, mix, w_out, y_pending


class PendingGatedNorm:
    """A sublayer's result ``y`` (float32 ``[T, D]``) that has not been added to the residual stream ``out`` yet
    (``HipKernels.group_norm_step`` with ``defer``): ``out`` still lacks ``mult * gn(y * sigmoid(gate), post_weight)`` with
    ``gn`` the RMS norm in ``groups`` groups. The next ``group_norm_step`` that reads ``out`` does it in its own pass;
    ``HipKernels.finish`` runs it by itself."""

    __slots__ = ("out", "y", "gate", "post_weight", "mult", "groups", "eps")

    def __init__(self, out, y, gate, post_weight, mult, groups, eps):
        self.out, self.y, self.gate, self.post_weight, self.mult, self.groups, self.eps = out, y, gate, post_weight, mult, groups, eps


def _ptr(t: Optional[torch.Tensor]):
    """A tensor's address as ctypes takes it for a ``c_void_p`` parameter: a plain integer, or None."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current HIP stream as an integer. ``torch.cuda.current_stream()`` builds a Stream object on every call
    (several microseconds, once per kernel launch); the raw getter is a plain C call."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _req(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*ts) -> None:
    for t in ts:
        if t is not None:
            _req(t.is_cuda, "a kernel was given a tensor that is not on the GPU")


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride (in elements) of a 2-D tensor whose rows are contiguous."""
    st = t.stride()
    if len(st) != 2:
        raise KernelError(f"{name} must have 2 dimensions, has {len(st)}")
    n_rows, n_cols = t.shape
    if st[1] != 1 and n_cols != 1:
        raise KernelError(f"{name}: rows must be contiguous")
    return st[0] if n_rows > 1 else max(st[0], n_cols)


class HipKernels:
    """The built libraries, loaded: ``core`` at once, the bfloat16 GEMMs and the attention of a head size when a
    call first needs them (each is compiled then, if a fresh checkout has not built it yet)."""

    def __init__(self, path: str):
        self.path = path
        # RTLD_GLOBAL: the other units take the error functions (lev_fail, lev_last_error) from this library
        self.lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        L = self.lib
        L.lev_last_error.restype = ctypes.c_char_p
        L.lev_abi_version.restype = c_int
        self._set_signatures(L, _build.UNITS["core"].signatures)
        self.use_mfma = os.environ.get("LEVANTER_AMD_NO_MFMA", "0") != "1"
        # the vendor library's GEMM for prompt-sized row counts (see use_library); "0" keeps every product on our kernels
        self.gemm_library = os.environ.get("LEVANTER_AMD_GEMM_LIBRARY", "1") != "0"
        self._library_refused = set()
        self._slow_attention_warned = set()
        # The library's product may be recorded into HIP graphs: replays with changed inputs and eager work between them
        # give the eager results bit for bit (tests/test_gpu_kernels.py records and replays it at four shapes).
        self.library_in_graphs = True
        self._sample_ws = None
        self._units = {}
        self._held_stream = None  # see hold_stream
        self._library_ws_bytes = None
        self._ws, self._ws_outgrown, self._ws_need = {}, [], {}  # GEMM scratch memory per device, see _workspace
        self._ws_last = None
        L.lev_attention_prefill_tile_rows.restype = c_int
        self.prefill_tile_rows = int(L.lev_attention_prefill_tile_rows())

    @staticmethod
    def _set_signatures(lib, sigs) -> None:
        for name, args in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = c_long if name.endswith("_workspace") else c_int

    def _unit(self, unit: str):
        """The library of a registered unit other than ``core``, built and loaded at its first use."""
        lib = self._units.get(unit)
        if lib is None:
            if unit not in _build.UNITS:
                raise KernelError(f"unknown kernel unit {unit!r}; registered: {', '.join(_build.UNITS)}")
            path = _build.ensure_built(unit)
            try:
                lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelError(f"the HIP library {path} cannot be loaded: {e}") from None
            self._set_signatures(lib, _build.UNITS[unit].signatures)
            self._units[unit] = lib
        return lib

    def call(self, unit: str, entry: str, *args) -> None:
        """Call an ``extern "C"`` entry point of a registered unit (``kernels.build.register_unit``): the way a part reaches
        a kernel of its own. Arguments as the unit's signature says (``tensor_ptr(t)`` for a tensor's address,
        ``stream()`` for the current HIP stream); the entry point returns 0, or a negative code with its message in
        ``lev_last_error()`` (``LEV_REQUIRE`` of ``common.h``), which is raised as a ``KernelError``."""
        lib = self.lib if unit == "core" else (self._units.get(unit) or self._unit(unit))
        try:
            fn = getattr(lib, entry)
        except AttributeError:
            raise KernelError(f"kernel unit {unit!r} has no entry point {entry!r}") from None
        self._check(fn(*args))

    tensor_ptr = staticmethod(lambda t: None if t is None else t.data_ptr())

    def stream(self):
        """The HIP stream that launches go to now (the current one, or the one held for a forward pass)."""
        return self._s()

    def hold_stream(self) -> None:
        """Look the current stream up once and use it for every launch until ``release_stream``: a model's forward pass
        launches hundreds of kernels on one stream, and the lookup is a tenth of a launch's cost on the host."""
        self._held_stream = _stream()

    def release_stream(self) -> None:
        self._held_stream = None

    def _s(self):
        held = self._held_stream
        return _stream() if held is None else held

    def loaded_units(self):
        return ["core", *self._units]

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.lev_last_error().decode())

    # ---- embedding ---------------------------------------------------------------------
    def embed(self, tokens, positions, table, pos_table, out, scale: float = 1.0) -> None:
        """out[t] = (table[tokens[t]] + pos_table[positions[t]]) * scale in float32. Ids are trusted (the step checks them)."""
        _dev(tokens, positions, table, pos_table, out)
        T, D = out.shape
        _req(tokens.dtype == torch.int32 and positions.dtype == torch.int32, "embed: ids must be int32")
        _req(tokens.numel() == T and positions.numel() == T, "embed: one token and one position per output row")
        _req(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
        _req(table.is_contiguous() and table.shape[1] == D and table.dtype in _DT, "embed: bad table")
        if pos_table is not None:
            _req(pos_table.is_contiguous() and pos_table.shape[1] == D and pos_table.dtype == table.dtype, "embed: bad position table")
        self._check(self.lib.lev_embed(_ptr(tokens), _ptr(positions), _ptr(table), _ptr(pos_table), _ptr(out), T, D,
                                       _DT[table.dtype], float(scale), self._s()))

    def pair_embed_add(self, tokens, positions, token_slots, last_token, table, x, buckets: int, mul_prev: int, mul_cur: int) -> None:
        """``x[t] += table[row]`` with ``row = (previous * mul_prev + tokens[t] * mul_cur) % buckets``, or row ``buckets`` (the table's
        last) at position 0. The token before is the step's own token t - 1 where it belongs to the same request one position
        earlier, else ``last_token[slot]`` (int32 ``[slots]``), which afterwards holds the last token of each request's run. Tokens
        of nobody (slot < 0) take row ``buckets`` and store nothing."""
        _dev(tokens, positions, token_slots, last_token, table, x)
        T, D = x.shape
        for t in (tokens, positions, token_slots):
            _req(t.dtype == torch.int32 and t.numel() == T, "pair embedding: one int32 token, position and slot per row")
        _req(last_token.dtype == torch.int32 and last_token.is_contiguous(), "pair embedding: the slots' last tokens must be int32")
        _req(x.dtype == torch.float32 and x.is_contiguous(), "pair embedding: x must be contiguous float32")
        _req(table.is_contiguous() and table.dtype in _DT and tuple(table.shape) == (buckets + 1, D), "pair embedding: the table must be [buckets + 1, D]")
        self._check(self.lib.lev_pair_embed_add(_ptr(tokens), _ptr(positions), _ptr(token_slots), _ptr(last_token), _ptr(table), _ptr(x), T, D,
                                                int(buckets), int(mul_prev), int(mul_cur), _DT[table.dtype], self._s()))

    def feed_tokens(self, dst, src, rows, n: int) -> None:
        """dst[i] = src[rows[i]] (``rows`` None: src[i]) for i < n: int32 token ids that never leave the device."""
        _dev(dst, src, rows)
        _req(dst.dtype == src.dtype == torch.int32 and dst.numel() >= n and dst.is_contiguous() and src.is_contiguous(), "feed_tokens: int32 vectors")
        _req(rows is None or (rows.dtype == torch.int32 and rows.numel() >= n), "feed_tokens: rows must be int32, one per token")
        _req(rows is not None or src.numel() >= n, "feed_tokens: too few source tokens")
        self._check(self.lib.lev_feed_tokens(_ptr(dst), _ptr(src), _ptr(rows), int(n), self._s()))

    # ---- norms ---------------------------------------------------------------------------
    def norm(self, x, weight, bias, eps: float, out, rows=None, rms: bool = False, pending: Optional[PendingSum] = None) -> None:
        """LayerNorm (or RMSNorm) of float32 rows into ``out`` (compute dtype). rows: int32 row indices into x.
        ``pending``: an unfinished product into ``x`` (see ``PendingSum``); its ranges are added to the rows that are
        normalised and normalised in one kernel. Without ``rows`` the sums are stored back and ``x`` is finished; with
        ``rows`` (which may name a row twice) only the selection is computed and ``x`` must not be read again: it is
        either left unfinished or finished, depending on whether the width has a fused kernel."""
        _dev(x, weight, bias, out, rows)
        D = x.shape[1]
        n = out.shape[0]
        _req(x.dtype == torch.float32 and x.is_contiguous(), "norm: x must be contiguous float32")
        _req(weight.dtype == torch.float32 and weight.numel() == D and weight.is_contiguous(), "norm: weight must be contiguous float32 [D]")
        _req(bias is None or (bias.dtype == torch.float32 and bias.numel() == D and bias.is_contiguous()), "norm: bias must be contiguous float32 [D]")
        _req(out.is_contiguous() and out.shape[1] == D and out.dtype in _DT, "norm: bad out")
        if rows is None:
            _req(n == x.shape[0], "norm: out must have as many rows as x")
        else:
            _req(rows.dtype == torch.int32 and rows.numel() == n, "norm: rows must be int32, one per output row")
        if isinstance(pending, PendingGatedNorm):  # another kind of norm behind a gated sublayer: finish that first
            self.finish(pending)
            pending = None
        if isinstance(pending, PendingStreams):
            _req(pending.out is x, "norm: the unfinished streams belong to another tensor")
            if rms and bias is None and D * 4 <= 60 * 1024:
                self.streams_step(pending.streams, y=pending.y, mix=pending.mix, w_out=pending.w_out, norm_weight=weight, eps=eps, h_out=out,
                                  x_out=x if rows is None else None, rows=rows, y_pending=pending.y_pending)
                return
            self.finish(pending)
            pending = None
        if isinstance(pending, PendingAverage):
            _req(pending.out is x, "norm: the unfinished sum belongs to another tensor")
            if rms and bias is None and D * 4 <= 65536:
                self._check(self.lib.lev_norm_average(_ptr(pending.streams), _ptr(x), _ptr(pending.weights), pending.n, x.numel(), _ptr(weight),
                                                      _ptr(out), _ptr(rows), n, D, float(eps), _DT[out.dtype], self._s()))
                return
            self.finish(pending)
        elif pending is not None:
            _req(pending.out is x and pending.ldo == D, "norm: the unfinished product belongs to another tensor")
            rc = self.lib.lev_norm_pending(_ptr(x), _ptr(pending.workspace), pending.n_ranges, _ptr(pending.bias), _ptr(weight), _ptr(bias),
                                           _ptr(out), _ptr(rows), n, x.shape[0], D, float(eps), int(rms), _DT[out.dtype], self._s())
            if rc == 0:
                return
            if rc < 0:
                self._check(rc)
            self.finish(pending)  # no fused kernel at this width: finish the product, then the plain norm
        self._check(self.lib.lev_norm(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _ptr(rows), n, D, float(eps), int(rms),
                                      _DT[out.dtype], self._s()))

    # ---- linear ----------------------------------------------------------------------------
    def _workspace(self, need: int, device) -> torch.Tensor:
        """Scratch memory for partial sums: one buffer per device that only grows. Kernels on one stream take turns
        with it. A buffer that is outgrown stays alive, because recorded HIP graphs may point at it; while a graph is
        being recorded a buffer that is too small is not replaced but a fresh one handed out, which stays with the graph."""
        last = self._ws_last
        if last is not None and last[0] == device and last[2] >= need:
            return last[1]
        ws = self._ws.get(device)
        if ws is not None and ws.numel() >= need:
            self._ws_last = (device, ws, ws.numel())
            return ws
        if torch.cuda.is_current_stream_capturing():
            return torch.empty(need, dtype=torch.uint8, device=device)
        if ws is not None:
            self._ws_outgrown.append(ws)
        new = torch.empty(max(need, 2 * (ws.numel() if ws is not None else 0)), dtype=torch.uint8, device=device)
        self._ws[device] = new
        self._ws_last = None
        return new

    def finish(self, pending: PendingSum) -> None:
        """Finish a product that ``linear(..., may_leave_pending=True)`` left unfinished, or a deferred sum of streams."""
        if isinstance(pending, PendingStreams):
            self.streams_step(pending.streams, y=pending.y, mix=pending.mix, w_out=pending.w_out, x_out=pending.out, y_pending=pending.y_pending)
            return
        if isinstance(pending, PendingGatedNorm):
            self.group_norm_step(pending.out, groups=pending.groups, eps=pending.eps, pending=pending)
            return
        if isinstance(pending, PendingProduct):
            x = pending.out
            self._check(self._unit("gemm_mfma").lev_linear_mfma_finish(_ptr(pending.workspace), _ptr(pending.bias), None, 0, _ptr(x), pending.ldo,
                                                                       x.shape[0], x.shape[1], pending.n_ranges, 0, _DT[torch.float32], self._s()))
            return
        if isinstance(pending, PendingAverage):
            self.stream_average(pending.streams, pending.out, pending.weights, pending.n)
            return
        x = pending.out
        self._check(self._unit("gemm_mfma").lev_linear_mfma_finish(_ptr(pending.workspace), _ptr(pending.bias), _ptr(x), pending.ldo, _ptr(x),
                                                                   pending.ldo, x.shape[0], x.shape[1], pending.n_ranges, 0, _DT[torch.float32],
                                                                   self._s()))

    def linear(self, a, w, bias, out, activation: str = "none", residual=None, may_leave_pending: bool = False) -> Optional[PendingSum]:
        """out = act(a @ w.T + bias) (+ residual). a [M, K], w [N, K], out [M, N]; residual float32, may be ``out``.

        ``may_leave_pending`` (only with ``residual is out`` or without a residual into a float32 ``out``, no activation):
        where the kernel splits the sum over K into ranges, it may stop after writing them and return a ``PendingSum``
        (without a residual: a ``PendingProduct``) instead of running the kernel that adds them up: the caller promises that
        the next thing to touch ``out`` is ``norm(out, ..., pending=...)``, ``streams_step(..., y_pending=...)`` or ``finish``."""
        # one kernel launch per call: the checks are written to cost little
        if not (a.is_cuda and w.is_cuda and out.is_cuda and (bias is None or bias.is_cuda) and (residual is None or residual.is_cuda)):
            raise KernelError("a kernel was given a tensor that is not on the GPU")
        M, K = a.shape
        N = w.shape[0]
        adt, odt = a.dtype, out.dtype
        if not (w.dim() == 2 and w.shape[1] == K and w.is_contiguous()):
            raise KernelError(f"linear: weight must be contiguous [N, {K}]")
        if not (adt == w.dtype and adt in _DT):
            raise KernelError("linear: a and w must share a compute dtype")
        if not (out.shape[0] == M and out.shape[1] == N and odt in _DT):
            raise KernelError("linear: bad out")
        if not (adt == torch.bfloat16 or odt == torch.float32):
            raise KernelError("linear: float32 inputs give float32 outputs")
        if bias is not None and not (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()):
            raise KernelError("linear: bias must be float32 [N]")
        lda, ldo = _rows(a, "linear: a"), _rows(out, "linear: out")
        ldr = 0
        if residual is not None:
            if not (residual.dtype == torch.float32 and residual.shape == out.shape and odt == torch.float32):
                raise KernelError("linear: a residual needs a float32 output of its shape")
            ldr = ldo if residual is out else _rows(residual, "linear: residual")
        act = ACTIVATIONS[activation]
        if adt == torch.bfloat16 and self.use_mfma and K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0:
            if self.gemm_library and self.use_library(M, N, K, act):
                key = (M, N, K, act, bias is None, residual is None, odt)
                # never while a HIP graph is being recorded: what the library records besides its kernel is not ours to vouch for
                if key not in self._library_refused and (self.library_in_graphs or not torch.cuda.is_current_stream_capturing()):
                    lib = self._units.get("gemm_library") or self._unit("gemm_library")
                    need = self._library_ws_bytes
                    if need is None:
                        need = self._library_ws_bytes = lib.lev_linear_library_workspace()
                    ws = self._workspace(need, a.device)
                    rc = lib.lev_linear_library(_ptr(a), lda, _ptr(w), _ptr(bias), _ptr(residual), ldr, _ptr(out), ldo, _ptr(ws), need,
                                                M, N, K, act, _DT[odt], self._s())
                    if rc == 0:
                        return None
                    if rc < 0:
                        self._check(rc)
                    self._library_refused.add(key)  # the library has no kernel for it: ours from now on
            gemm = self._units.get("gemm_mfma") or self._unit("gemm_mfma")
            need = self._ws_need.get((M, N, K))
            if need is None:  # partial sums of a K range split over workgroups
                need = self._ws_need[(M, N, K)] = gemm.lev_linear_mfma_workspace(M, N, K)
            ws = self._workspace(need, a.device) if need > 0 else None
            leave = may_leave_pending and need > 0 and (residual is out or (residual is None and odt == torch.float32)) and act == 0 and ldo == N
            self._check(gemm.lev_linear_mfma(_ptr(a), lda, _ptr(w), _ptr(bias), _ptr(residual), ldr, _ptr(out), ldo, _ptr(ws),
                                             M, N, K, act, _DT[odt], int(leave), self._s()))
            if leave:
                return (PendingSum if residual is out else PendingProduct)(out, ws, need // (M * N * 4), bias, ldo)
        else:
            self._check(self.lib.lev_linear_simple(_ptr(a), lda, _ptr(w), _ptr(bias), _ptr(residual), ldr, _ptr(out), ldo,
                                                   M, N, K, act, _DT[adt], _DT[odt], self._s()))
        return None

    LIBRARY_ACTIVATIONS = (ACTIVATIONS["none"], ACTIVATIONS["gelu_new"], ACTIVATIONS["relu"])
    LIBRARY_MIN_ROWS = 25  # up to 24 rows the skinny kernel streams the weights at the rate a plain read reaches

    @classmethod
    def use_library(cls, M: int, N: int, K: int, act: int) -> bool:
        """Which products go to the vendor library: those with an epilogue it has, at the shapes where it was measured
        ahead on MI355X (widths of GPT-2 7B and XL, with epilogues). From 256 rows: all but long sums into narrow outputs
        (K >= 4 N) below 1,024 rows and, below 320 rows, weights of a few MB unless the output is wide (a 1600-wide layer at 264
        rows, ours / library with its kernel timed: qkv 18.3 / 16.7, fc 24.8 / 18.8, proj 11.9 / 14.2, second MLP matrix 22.7 / 20.4 but
        20.1 / 23.5 at 256 and 22.9 / 23.5 at 288). From 25 to 255 rows: wide outputs of large
        weights (N >= 2 K, 32 MB and more: 7B qkv and fc at 64 rows 28.1 / 25.3 and 37.1 / 33.5 us, ours with the kernel that
        adds its K ranges; at 160 rows 49.7 / 37.2 and 55.7 / 41.6); ours keep N = K (17.4 / 16.3 at 64 rows, 22.1 / 24.6 at
        128) and K = 4 N (36.8 / 41.2, 43.5 / 81.1), and below 96 rows the largest weights (more than 256 MB: the fc of a
        6144-wide layer 64.4 / 72.4 at 32 rows, 70.1 / 75.4 at 64, 85.0 / 84.4 at 128; its qkv, 216 MB, 58.9 / 57.6 and 62.3 / 59.7)."""
        if act not in cls.LIBRARY_ACTIVATIONS or M < cls.LIBRARY_MIN_ROWS:
            return False
        if M < 256:
            if N < 2 * K:
                return False
            if N * K < (1 << 24):
                return M >= 128  # a 1600-wide layer: qkv 16.5 / 14.2 at 128 rows, 17.3 / 14.5 at 192, but 12.8 / 14.3 at 64
            return not (M < 96 and N * K > (1 << 27))
        if M < 320 and N * K < (1 << 24):
            return N >= 2 * K
        return not (K >= 4 * N and M < 1024)

    # ---- cache write -----------------------------------------------------------------------
    def kv_write(self, k, v, k_pages, v_pages, dest, n_kv_heads: int, head_dim: int, page_size: int, value_dim: Optional[int] = None) -> None:
        """Scatter the new tokens' keys and values ([T, n_kv_heads*head_dim] views; values [T, n_kv_heads*value_dim] where a
        value head has a size of its own) to ``dest[t] = page*page_size + offset``."""
        if not (k.is_cuda and v.is_cuda and k_pages.is_cuda and v_pages.is_cuda and dest.is_cuda):
            raise KernelError("a kernel was given a tensor that is not on the GPU")
        T, cols = k.shape
        dt = k.dtype
        vd = head_dim if value_dim is None else int(value_dim)
        if not (v.shape == (T, n_kv_heads * vd) and cols == n_kv_heads * head_dim):
            raise KernelError("kv_write: k must be [T, kv_heads*head_dim] and v [T, kv_heads*value_dim]")
        if not (dt == v.dtype == k_pages.dtype == v_pages.dtype and dt in _DT):
            raise KernelError("kv_write: dtypes differ")
        if not (dest.dtype == torch.int32 and dest.numel() == T):
            raise KernelError("kv_write: one int32 destination per token")
        n_elems = k_pages.numel()
        if not (k_pages.is_contiguous() and v_pages.is_contiguous() and n_elems % (cols * page_size) == 0
                and n_elems * vd == v_pages.numel() * head_dim):
            raise KernelError("kv_write: page tensors must be contiguous and fit the sizes")
        self._check(self.lib.lev_kv_write(_ptr(k), _ptr(v), _rows(k, "kv_write: k"), _rows(v, "kv_write: v"), _ptr(k_pages),
                                          _ptr(v_pages), _ptr(dest), T, n_kv_heads, head_dim, vd, page_size, _DT[dt], self._s()))

    # ---- row-wise steps of layers that are not GPT-2's -----------------------------------------
    def head_prepare(self, qk, n_norm: int, head_dim: int, eps: float, v=None, v_first=None, n_blend: int = 0, value_dim: int = 0,
                     blend=None, norm_dim: Optional[int] = None, norm_weight=None) -> None:
        """In place: the ``n_norm`` heads of ``head_dim`` columns at the start of ``qk``'s rows are divided by their root
        mean square (``sqrt(sum(x^2) / norm_dim + eps)``; ``norm_dim`` is ``head_dim`` unless the heads carry zeros behind
        their true size); the ``n_blend`` heads of ``value_dim`` columns of ``v`` become
        ``(1 - blend) v + blend v_first`` (``blend``: a float32 tensor of one element on the GPU). ``norm_weight`` (float32
        ``[head_dim]``): every normalised head is multiplied by it (an RMS norm with a weight). 32-bit arithmetic."""
        T = (qk if qk is not None else v).shape[0]
        dt = (qk if qk is not None else v).dtype
        _dev(qk, v, v_first, blend, norm_weight)
        _req(dt in _DT, "head_prepare: unknown dtype")
        _req(norm_weight is None or (norm_weight.dtype == torch.float32 and norm_weight.numel() == head_dim and norm_weight.is_contiguous()),
             "head_prepare: the norm's weight must be float32 [head_dim]")
        qs = vs = fs = 0
        if n_norm:
            _req(qk is not None and qk.shape[0] == T and qk.shape[1] >= n_norm * head_dim, "head_prepare: too few columns for the heads to normalise")
            qs = _rows(qk, "head_prepare: qk")
        if n_blend:
            _req(v is not None and v_first is not None and blend is not None, "head_prepare: blending needs both value tensors and the weight")
            _req(v.shape == v_first.shape == (T, n_blend * value_dim) and v.dtype == v_first.dtype == dt, "head_prepare: values must be [T, heads*value_dim]")
            _req(blend.dtype == torch.float32 and blend.numel() == 1, "head_prepare: the blending weight must be one float32")
            vs, fs = _rows(v, "head_prepare: v"), _rows(v_first, "head_prepare: v_first")
        self._check(self.lib.lev_head_prepare(_ptr(qk) if n_norm else None, qs, int(n_norm), int(head_dim), int(norm_dim or head_dim), float(eps), _ptr(v) if n_blend else None,
                                              vs, _ptr(v_first) if n_blend else None, fs, int(n_blend), int(value_dim),
                                              _ptr(blend) if n_blend else None, _ptr(norm_weight), T, _DT[dt], self._s()))

    def head_prepare_write(self, q, k, v, k_pages, v_pages, dest, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int,
                           page_size: int, eps: Optional[float], v_first=None, blend=None, norm_dim: Optional[int] = None,
                           rotary_freqs=None, positions=None, q_norm_weight=None, k_norm_weight=None, rotary_magnitude: float = 1.0) -> None:
        """``head_prepare`` and ``kv_write`` in one kernel, for steps of single tokens: queries are normalised in place
        (``eps`` None: not at all), keys are normalised and values blended (``v_first`` None: not) on their way into the pages;
        ``k`` and ``v`` themselves stay as projected. ``rotary_freqs`` (float32, with ``positions``): the rotation of
        ``rotary_pairs`` too (cosine and sine times ``rotary_magnitude``), on the queries in place and on the keys on their way into
        the pages. ``q_norm_weight`` / ``k_norm_weight`` (float32 ``[head_dim]``): the normalised query / key heads are multiplied by
        it, before the rotation."""
        _dev(q, k, v, k_pages, v_pages, dest, v_first, blend, rotary_freqs, positions, q_norm_weight, k_norm_weight)
        for w in (q_norm_weight, k_norm_weight):
            _req(w is None or (eps is not None and w.dtype == torch.float32 and w.numel() == head_dim and w.is_contiguous()),
                 "head_prepare_write: a norm's weight must be float32 [head_dim] and needs the norm")
        n_pairs = 0
        if rotary_freqs is not None:
            _req(rotary_freqs.dtype == torch.float32 and rotary_freqs.is_contiguous() and 2 * rotary_freqs.numel() <= head_dim, "head_prepare_write: float32 frequencies, at most head_dim / 2")
            _req(positions is not None and positions.dtype == torch.int32 and positions.numel() == q.shape[0], "head_prepare_write: one int32 position per token")
            n_pairs = rotary_freqs.numel()
        T, dt = q.shape[0], q.dtype
        _req(dt in _DT and dt == k.dtype == v.dtype == k_pages.dtype == v_pages.dtype, "head_prepare_write: dtypes differ")
        _req(q.shape == (T, n_heads * head_dim) and k.shape == (T, n_kv_heads * head_dim) and v.shape == (T, n_kv_heads * value_dim),
             "head_prepare_write: q, k, v must be [T, heads*size]")
        _req(dest.dtype == torch.int32 and dest.numel() == T, "head_prepare_write: one int32 destination per token")
        n_elems = k_pages.numel()
        _req(k_pages.is_contiguous() and v_pages.is_contiguous() and n_elems % (n_kv_heads * head_dim * page_size) == 0
             and n_elems * value_dim == v_pages.numel() * head_dim, "head_prepare_write: page tensors must be contiguous and fit the sizes")
        fs = 0
        if v_first is not None:
            _req(v_first.shape == v.shape and v_first.dtype == dt and blend is not None and blend.dtype == torch.float32 and blend.numel() == 1,
                 "head_prepare_write: blending needs values of the same shape and one float32 weight")
            fs = _rows(v_first, "head_prepare_write: v_first")
        self._check(self.lib.lev_head_prepare_write(
            _ptr(q), _rows(q, "head_prepare_write: q"), n_heads, _ptr(k), _rows(k, "head_prepare_write: k"), _ptr(v),
            _rows(v, "head_prepare_write: v"), _ptr(v_first), fs, _ptr(blend) if v_first is not None else None, n_kv_heads, head_dim,
            value_dim, float(eps or 0.0), int(norm_dim or head_dim) if eps is not None else 0, _ptr(k_pages), _ptr(v_pages), _ptr(dest), page_size,
            _ptr(rotary_freqs) if n_pairs else None, n_pairs, _ptr(positions) if n_pairs else None, _ptr(q_norm_weight), _ptr(k_norm_weight),
            float(rotary_magnitude), T, _DT[dt], self._s()))

    def head_norm_rotate(self, q, k, n_heads: int, n_kv_heads: int, head_dim: int, eps: Optional[float], norm_dim: Optional[int] = None,
                         q_norm_weight=None, k_norm_weight=None, rotary_freqs=None, positions=None, rotary_magnitude: float = 1.0) -> None:
        """What ``head_prepare_write`` does to queries and keys, without the write and in place on both: every head divided by its root
        mean square (``eps`` None: not), times the norm's weight of its kind, then the rotation of ``rotary_pairs``. For runs of
        several tokens, whose pages ``kv_write`` fills afterwards; the same arithmetic, so a key is the same bits either way."""
        _dev(q, k, q_norm_weight, k_norm_weight, rotary_freqs, positions)
        T, dt = q.shape[0], q.dtype
        _req(dt in _DT and k.dtype == dt and q.shape == (T, n_heads * head_dim) and k.shape == (T, n_kv_heads * head_dim), "head_norm_rotate: q and k must be [T, heads*head_dim] of one compute dtype")
        for w in (q_norm_weight, k_norm_weight):
            _req(w is None or (eps is not None and w.dtype == torch.float32 and w.numel() == head_dim and w.is_contiguous()),
                 "head_norm_rotate: a norm's weight must be float32 [head_dim] and needs the norm")
        n_pairs = 0
        if rotary_freqs is not None:
            _req(rotary_freqs.dtype == torch.float32 and rotary_freqs.is_contiguous() and 2 * rotary_freqs.numel() <= head_dim, "head_norm_rotate: float32 frequencies, at most head_dim / 2")
            _req(positions is not None and positions.dtype == torch.int32 and positions.numel() == T, "head_norm_rotate: one int32 position per token")
            n_pairs = rotary_freqs.numel()
        self._check(self.lib.lev_head_norm_rotate(_ptr(q), _rows(q, "head_norm_rotate: q"), int(n_heads), _ptr(k), _rows(k, "head_norm_rotate: k"), int(n_kv_heads),
                                                  int(head_dim), float(eps or 0.0), int(norm_dim or head_dim) if eps is not None else 0, _ptr(q_norm_weight),
                                                  _ptr(k_norm_weight), _ptr(rotary_freqs) if n_pairs else None, n_pairs, _ptr(positions) if n_pairs else None,
                                                  float(rotary_magnitude), T, _DT[dt], self._s()))

    def norm_write_latent(self, c, weight, eps: float, norm_dim: int, k_pages, v_pages, dest, page_size: int) -> None:
        """``c`` ``[T, R]`` (one key/value head that all query heads share) becomes its RMS norm with ``weight`` (float32 ``[R]``;
        the mean of squares is over ``norm_dim``), in place, and goes into the key and the value pages at ``dest``: what
        ``head_prepare`` with a weight and ``kv_write(c, c)`` do, in one kernel."""
        _dev(c, weight, k_pages, v_pages, dest)
        T, R = c.shape
        _req(c.dtype in _DT and c.dtype == k_pages.dtype == v_pages.dtype, "norm_write_latent: dtypes differ")
        _req(weight.dtype == torch.float32 and weight.numel() == R and weight.is_contiguous(), "norm_write_latent: the weight must be float32 [R]")
        _req(dest.dtype == torch.int32 and dest.numel() == T, "norm_write_latent: one int32 destination per token")
        _req(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.numel() == v_pages.numel() and k_pages.numel() % (R * page_size) == 0,
             "norm_write_latent: page tensors must be contiguous and fit the sizes")
        self._check(self.lib.lev_norm_write_latent(_ptr(c), _rows(c, "norm_write_latent: c"), R, int(norm_dim), float(eps), _ptr(weight), _ptr(k_pages),
                                                   _ptr(v_pages), _ptr(dest), page_size, T, _DT[c.dtype], self._s()))

    def latent_rope_write(self, kv, latent_dim: int, weight, eps: float, norm_dim: int, q, n_heads: int, q_head: int, q_offset: int, freqs, positions,
                          k_pages, v_pages, dest, page_size: int) -> None:
        """For steps of single tokens, in one kernel: ``kv`` ``[T, latent_dim + rotated part]`` has its latent normed (``head_prepare``
        with ``weight``, the mean of squares over ``norm_dim``) and its rotated part turned (``rotary_half`` from column
        ``latent_dim``), in place; the whole row goes into the key pages and the latent into the value pages at ``dest``
        (``kv_write``); the vectors at ``q_offset`` of the ``n_heads`` heads of ``q_head`` elements of ``q`` are turned too (``q`` None:
        no queries). ``freqs`` float32 (may be empty: nothing turns)."""
        _dev(kv, weight, q, freqs, positions, k_pages, v_pages, dest)
        T, KD = kv.shape
        R, DR = int(latent_dim), KD - int(latent_dim)
        dt = kv.dtype
        _req(dt in _DT and dt == k_pages.dtype == v_pages.dtype and (q is None or q.dtype == dt), "latent_rope_write: dtypes differ")
        _req(weight.dtype == torch.float32 and weight.numel() == R and weight.is_contiguous(), "latent_rope_write: the weight must be float32 [latent_dim]")
        _req(freqs is None or (freqs.dtype == torch.float32 and freqs.is_contiguous()), "latent_rope_write: float32 frequencies")
        n_pairs = 0 if freqs is None else freqs.numel()
        _req(positions.dtype == torch.int32 and positions.numel() == T and dest.dtype == torch.int32 and dest.numel() == T, "latent_rope_write: one int32 position and destination per token")
        _req(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.numel() * R == v_pages.numel() * KD and k_pages.numel() % (KD * page_size) == 0,
             "latent_rope_write: page tensors must be contiguous and fit the sizes")
        _req(q is None or (q.dim() == 2 and q.shape[0] == T and q.shape[1] >= n_heads * q_head), "latent_rope_write: q must be [T, heads*q_head]")
        self._check(self.lib.lev_latent_rope_write(_ptr(kv), _rows(kv, "latent_rope_write: kv"), R, DR, int(norm_dim), float(eps), _ptr(weight), _ptr(q),
                                                   _rows(q, "latent_rope_write: q") if q is not None else 0, int(n_heads), int(q_head), int(q_offset), n_pairs,
                                                   _ptr(freqs) if n_pairs else None, _ptr(positions), _ptr(k_pages), _ptr(v_pages), _ptr(dest), page_size, T,
                                                   _DT[dt], self._s()))

    def recurrent_tokens(self, x, y, taps, conv_bias, gate_weight, gate_bias, decay, state, token_slots, out, out_scale: float = 1.0) -> None:
        """``causal_conv``, the block-diagonal product of the gates and ``gated_recurrence`` for a step in which every token is
        a run of its own, in one kernel (the same bits as the three). ``gate_weight`` ``[B, 2*C/B, C/B]``: both gates of a block
        stacked, ``gate_bias`` float32 ``[B * 2*C/B]``."""
        _dev(x, y, taps, conv_bias, gate_weight, gate_bias, decay, state, token_slots, out)
        T, C = x.shape
        dt = x.dtype
        _req(dt in _DT and y.dtype == out.dtype == gate_weight.dtype == dt and y.shape == out.shape == x.shape, "recurrent_tokens: x, y, out must be [T, C] of the weights' dtype")
        _req(gate_weight.dim() == 3 and gate_weight.is_contiguous() and gate_weight.shape[1] == 2 * gate_weight.shape[2]
             and gate_weight.shape[0] * gate_weight.shape[2] == C, "recurrent_tokens: gate weights must be [B, 2*C/B, C/B]")
        K = taps.shape[1]
        _req(taps.dtype == torch.float32 and tuple(taps.shape) == (C, K) and taps.is_contiguous(), "recurrent_tokens: taps must be float32 [C, K]")
        _req(conv_bias is None or (conv_bias.dtype == torch.float32 and conv_bias.numel() == C), "recurrent_tokens: the convolution's bias must be float32 [C]")
        _req(gate_bias is None or (gate_bias.dtype == torch.float32 and gate_bias.numel() == 2 * C and gate_bias.is_contiguous()), "recurrent_tokens: the gates' bias must be float32 [2*C]")
        _req(decay.dtype == torch.float32 and decay.numel() == C and decay.is_contiguous(), "recurrent_tokens: decay must be float32 [C]")
        _req(state.dtype == torch.float32 and state.dim() == 3 and tuple(state.shape[1:]) == (K, C) and state.is_contiguous(), "recurrent_tokens: state must be float32 [slots, K, C]")
        _req(token_slots.dtype == torch.int32 and token_slots.numel() == T, "recurrent_tokens: one int32 slot per token")
        self._check(self.lib.lev_recurrent_tokens(_ptr(x), _rows(x, "recurrent_tokens: x"), _ptr(y), _rows(y, "recurrent_tokens: y"), _ptr(taps), _ptr(conv_bias),
                                                  _ptr(gate_weight), _ptr(gate_bias), _ptr(decay), _ptr(state), _ptr(token_slots), _ptr(out),
                                                  _rows(out, "recurrent_tokens: out"), T, C, K, gate_weight.shape[2], float(out_scale), _DT[dt], self._s()))

    def poly_norm(self, z, coefficients, eps: float, out) -> None:
        """out = c0 z/rms(z) + c1 z^2/rms(z^2) + c2 z^3/rms(z^3) + c3 per row, rms(u) = sqrt(mean(u^2) + eps); powers element
        by element, statistics in 32-bit. ``coefficients``: float32 [4] on the GPU."""
        _dev(z, coefficients, out)
        _req(z.dim() == 2 and out.shape == z.shape and z.dtype == out.dtype and z.dtype in _DT, "poly_norm: z and out must be [T, F] of one compute dtype")
        _req(coefficients.dtype == torch.float32 and coefficients.numel() == 4 and coefficients.is_contiguous(), "poly_norm: four float32 coefficients")
        self._check(self.lib.lev_poly_norm(_ptr(z), _rows(z, "poly_norm: z"), _ptr(out), _rows(out, "poly_norm: out"), _ptr(coefficients),
                                           z.shape[0], z.shape[1], float(eps), _DT[z.dtype], self._s()))

    def head_talk(self, o, talk, gate, out, n_heads: int, n_kv_heads: int, value_dim: int, out_scale: float = 1.0, gate_elements: bool = False) -> None:
        """``o`` float32 [T, heads, NV, value_dim] (``attention_values``) -> ``out`` [T, heads*value_dim] in the compute dtype:
        head h gets ``sum_g talk[h, g] o[t, g, c(h)]`` with c(h) its own value head (``talk`` None: ``o[t, h, 0]``), times
        ``sigmoid(gate[t, h])`` where ``gate`` [T, heads] (compute dtype) is given (``gate_elements``: ``gate`` [T, heads*value_dim],
        a gate per element of the result), times ``out_scale``."""
        _dev(o, talk, gate, out)
        T = out.shape[0]
        nv = n_kv_heads if talk is not None else 1
        _req(o.dtype == torch.float32 and o.is_contiguous() and o.numel() == T * n_heads * nv * value_dim, "head_talk: o must be float32 [T, heads, NV, value_dim]")
        _req(out.dtype in _DT and out.shape[1] == n_heads * value_dim, "head_talk: out must be [T, heads*value_dim]")
        _req(talk is None or (talk.dtype == torch.float32 and talk.shape == (n_heads, n_heads) and talk.is_contiguous()), "head_talk: the mixing matrix must be float32 [heads, heads]")
        gs = 0
        if gate is not None:
            _req(gate.dtype == out.dtype and gate.shape == (T, n_heads * value_dim if gate_elements else n_heads), "head_talk: the gate must be [T, heads] (or [T, heads*value_dim]) of the compute dtype")
            gs = _rows(gate, "head_talk: gate")
        self._check(self.lib.lev_head_talk(_ptr(o), _ptr(talk), _ptr(gate), gs, _ptr(out), _rows(out, "head_talk: out"), T, n_heads, n_kv_heads,
                                           nv, value_dim, float(out_scale), int(bool(gate_elements) and gate is not None), _DT[out.dtype], self._s()))

    def stream_average(self, streams, x, weights, n: int, defer: bool = False) -> Optional[PendingAverage]:
        """``streams`` float32 [slots, T, D] holds earlier results in entries 0 .. n-2. ``x`` (float32 [T, D]) is kept as entry
        n-1 and becomes ``sum_j weights[j] streams[j]``, j = 0 .. n-1 in that order. ``defer``: nothing is launched; the
        ``PendingAverage`` that comes back goes to the norm that reads ``x`` next (or to ``finish``)."""
        _dev(streams, x, weights)
        _req(x.dtype == streams.dtype == weights.dtype == torch.float32 and x.is_contiguous() and streams.is_contiguous(), "stream_average: contiguous float32 tensors")
        _req(streams.dim() == 3 and streams.shape[1:] == x.shape and 1 <= n <= streams.shape[0], "stream_average: streams must be [slots >= n, T, D]")
        _req(weights.numel() >= n and weights.is_contiguous(), "stream_average: one weight per stream")
        if defer:
            return PendingAverage(x, streams, weights, int(n))
        self._check(self.lib.lev_stream_average(_ptr(streams), _ptr(x), _ptr(weights), int(n), x.numel(), self._s()))
        return None

    def attention_values(self, q, out, k_pages, v_pages, meta, *, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int,
                         all_value_heads: bool, page_size: int, scale: float, window: Optional[int], block_tables,
                         softcap: Optional[float] = None, slopes=None, chunk: Optional[int] = None, sinks=None, keep_first: int = 0) -> None:
        """Causal attention over the pages for heads whose keys and values differ in size. ``out`` float32
        [T, heads, NV, value_dim]: the weights of each query head applied to the values of every key/value head
        (``all_value_heads``: NV = kv heads, for weights that are mixed over the heads afterwards, see ``head_talk``) or of its
        own (NV = 1). Score: ``cap(scale q.k) - slopes[h] * distance`` (``slopes`` float32 [heads] or None), ``cap`` the soft
        cap if given. ``chunk``: a query sees only the keys of its own chunk of that many positions, counted from position 0.
        ``keep_first``: the first so many positions of a sequence stay in sight of every later query, whatever window and chunk say.
        ``sinks`` (float32 [heads] or None): the denominator of head h's softmax also holds ``exp(sinks[h])``, once per query.
        The cache must hold the step's own keys and values already."""
        _dev(q, out, k_pages, v_pages, block_tables, meta.positions, meta.token_seq, slopes, sinks)
        T = q.shape[0]
        dt = q.dtype
        nv = n_kv_heads if all_value_heads else 1
        _req(q.shape[1] == n_heads * head_dim and dt in _DT and dt == k_pages.dtype == v_pages.dtype, "attention_values: q must be [T, heads*head_dim] of the cache's dtype")
        _req(out.dtype == torch.float32 and out.is_contiguous() and out.numel() == T * n_heads * nv * value_dim, "attention_values: out must be float32 [T, heads, NV, value_dim]")
        _req(meta.positions.numel() == T and meta.token_seq.numel() == T, "attention_values: one position and request row per token")
        _req(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(), "attention_values: bad block tables")
        _req(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.numel() * value_dim == v_pages.numel() * head_dim
             and k_pages.numel() % (n_kv_heads * head_dim * page_size) == 0, "attention_values: page tensors do not fit the sizes")
        _req(slopes is None or (slopes.dtype == torch.float32 and slopes.numel() == n_heads and slopes.is_contiguous()), "attention_values: one float32 slope per head")
        _req(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == n_heads and sinks.is_contiguous()), "attention_values: one float32 sink per head")
        if dt == torch.bfloat16 and self.use_mfma and self.mfma_attention_values_supports(head_dim, value_dim):
            # matrix cores: runs of several tokens in tiles of 16 query rows, single tokens with the heads of a key/value head as columns
            lib = self._unit(_build.attention_values_unit(head_dim, value_dim))
            # single tokens: the keys of one token are split over several waves where the step's tokens alone leave the chip
            # empty (about 1,024 waves are aimed at, a block of 64 keys at least per wave); the step's description keeps the
            # choice and the scratch memory for all layers with these sizes
            key = ("values", n_heads, n_kv_heads, value_dim, nv, int(window) if window else 0, int(chunk) if chunk else 0, int(keep_first))
            plan = meta.plans.get(key)
            if plan is None:
                splits = 1
                if meta.n_decode:
                    chunks = 1 if nv == 1 else -(-nv * (value_dim // 16) // 16)
                    reach = min(int(window), meta.max_kv_len) if window else meta.max_kv_len
                    if chunk:
                        reach = min(reach, int(chunk))
                    most = max(1, (reach + 63) // 64 + (1 if window or chunk else 0) + ((int(keep_first) + 63) // 64 if window or chunk else 0))
                    splits = int(max(1, min(most, 32, 1024 // max(1, meta.n_decode * n_kv_heads * chunks))))
                need = lib.lev_attention_values_mfma_workspace(meta.n_decode, splits, n_heads, nv) if splits > 1 else 0
                ws = torch.empty(need, dtype=torch.uint8, device=q.device) if need else None
                plan = meta.plans[key] = (splits, ws)
            splits, ws = plan
            self._check(lib.lev_attention_values_mfma(
                _ptr(q), _rows(q, "attention_values: q"), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(meta.positions), _ptr(meta.token_seq),
                _ptr(block_tables), block_tables.shape[1], _ptr(meta.prefill_tiles), meta.n_prefill_tiles, _ptr(meta.decode_tokens),
                meta.n_decode, n_heads, n_kv_heads, head_dim, value_dim, nv, page_size, float(scale), int(window) if window else 0,
                int(chunk) if chunk else 0, int(keep_first), float(softcap) if softcap else 0.0, _ptr(slopes), _ptr(sinks), splits, _ptr(ws), int(meta.max_kv_len), self._s()))
            return
        self._check(self.lib.lev_attention_values(
            _ptr(q), _rows(q, "attention_values: q"), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(meta.positions), _ptr(meta.token_seq),
            _ptr(block_tables), block_tables.shape[1], T, n_heads, n_kv_heads, head_dim, value_dim, nv, page_size, float(scale),
            int(window) if window else 0, int(chunk) if chunk else 0, int(keep_first), float(softcap) if softcap else 0.0, _ptr(slopes), _ptr(sinks), _DT[dt], self._s()))

    @staticmethod
    def mfma_attention_values_supports(head_dim: int, value_dim: int) -> bool:
        return head_dim % 16 == 0 and value_dim % 16 == 0 and 16 <= head_dim <= 256 and 16 <= value_dim <= 256

    # ---- several residual streams --------------------------------------------------------------
    def streams_step(self, streams, *, x_init=None, y=None, mix=None, w_out=None, w_in=None, norm_weight=None, eps: float = 0.0,
                     h_out=None, x_out=None, rows=None, defer_out=None, y_pending: Optional[PendingProduct] = None) -> Optional[PendingStreams]:
        """One pass over the residual streams (float32 ``[n, T, D]``), doing what it is given, in this order: the write of a
        sublayer's result, ``x_t <- sum_s mix[s, t] x_s + w_out[t] y`` (``y`` float32 ``[T, D]``); the read for the next sublayer,
        ``u = sum_s w_in[s] x_s`` (``w_in`` None: the plain sum); its RMS norm ``u / sqrt(mean(u^2) + eps) * norm_weight`` into
        ``h_out`` (compute dtype); ``u`` itself into ``x_out`` (float32). ``x_init`` (float32 ``[T, D]``): the streams do not
        exist yet and all start as this. ``rows``: only these rows, into ``h_out [len(rows), D]``; nothing else is stored.
        ``defer_out``: nothing is launched; the write comes back as a ``PendingStreams`` standing for that tensor, for the
        next ``streams_step`` (pass it as ``y``, ``mix``, ``w_out``), ``norm`` or ``finish``. ``y_pending``: ``y`` is the
        output of a product that has left its K ranges undone (``PendingProduct``); they are read in its place."""
        if defer_out is not None:
            return PendingStreams(defer_out, streams, y, mix, w_out, y_pending)
        _dev(streams, x_init, y, mix, w_out, w_in, norm_weight, h_out, x_out, rows)
        _req(streams.dim() == 3 and streams.dtype == torch.float32 and streams.is_contiguous(), "streams: the streams must be contiguous float32 [n, T, D]")
        n, T, D = streams.shape
        for name, t in (("x_init", x_init), ("y", y), ("x_out", x_out)):
            _req(t is None or (t.dtype == torch.float32 and tuple(t.shape) == (T, D) and t.is_contiguous()), f"streams: {name} must be contiguous float32 [T, D]")
        _req(y is None or (mix is not None and w_out is not None and mix.dtype == w_out.dtype == torch.float32 and tuple(mix.shape) == (n, n)
                           and w_out.numel() == n and mix.is_contiguous() and w_out.is_contiguous()), "streams: a write needs float32 weights [n, n] and [n]")
        _req(w_in is None or (w_in.dtype == torch.float32 and w_in.numel() == n and w_in.is_contiguous()), "streams: the read's weights must be float32 [n]")
        n_rows, odt = 0, torch.float32
        if rows is not None:
            _req(rows.dtype == torch.int32 and rows.is_contiguous(), "streams: rows must be int32")
            n_rows = rows.numel()
        if h_out is not None:
            _req(norm_weight is not None and norm_weight.dtype == torch.float32 and norm_weight.numel() == D and norm_weight.is_contiguous(),
                 "streams: the norm's weight must be float32 [D]")
            _req(h_out.dtype in _DT and h_out.is_contiguous() and tuple(h_out.shape) == ((n_rows if rows is not None else T), D), "streams: bad normalised output")
            odt = h_out.dtype
        part = n_ranges = part_bias = None
        if y_pending is not None:
            _req(y is not None and y_pending.out is y and y_pending.ldo == D, "streams: the unfinished product belongs to another tensor")
            part, n_ranges, part_bias = y_pending.workspace, y_pending.n_ranges, y_pending.bias
        self._check(self.lib.lev_streams_step(_ptr(streams), n, T, D, _ptr(x_init), None if part is not None else _ptr(y), _ptr(mix), _ptr(w_out), _ptr(w_in),
                                              _ptr(norm_weight), float(eps), _ptr(h_out), _ptr(x_out), _ptr(rows), n_rows, _DT[odt],
                                              _ptr(part), int(n_ranges or 0), _ptr(part_bias), self._s()))
        return None

    # ---- rotation of pairs ---------------------------------------------------------------------
    def rotary_pairs(self, q, k, head_dim: int, freqs, positions, magnitude: float = 1.0) -> None:
        """In place on ``q`` ``[T, heads*head_dim]`` and ``k`` (either may be None): dimensions (2i, 2i+1) of every head turn by
        ``positions[t] * freqs[i]``, i < len(freqs), cosine and sine both times ``magnitude``; the other dimensions stay. 32-bit angles."""
        _dev(q, k, freqs, positions)
        ref = q if q is not None else k
        T, dt = ref.shape[0], ref.dtype
        _req(dt in _DT and (q is None or k is None or q.dtype == k.dtype), "rotary: q and k must share a compute dtype")
        _req(freqs.dtype == torch.float32 and freqs.is_contiguous() and 2 * freqs.numel() <= head_dim, "rotary: float32 frequencies, at most head_dim / 2")
        _req(positions.dtype == torch.int32 and positions.numel() == T, "rotary: one int32 position per token")
        hq = hk = 0
        if q is not None:
            _req(q.shape[0] == T and q.shape[1] % head_dim == 0, "rotary: q must be [T, heads*head_dim]")
            hq = q.shape[1] // head_dim
        if k is not None:
            _req(k.shape[0] == T and k.shape[1] % head_dim == 0, "rotary: k must be [T, heads*head_dim]")
            hk = k.shape[1] // head_dim
        self._check(self.lib.lev_rotary_pairs(_ptr(q), _rows(q, "rotary: q") if q is not None else 0, hq, _ptr(k), _rows(k, "rotary: k") if k is not None else 0,
                                              hk, int(head_dim), freqs.numel(), _ptr(freqs), _ptr(positions), float(magnitude), T, _DT[dt], self._s()))

    # ---- block-diagonal products ---------------------------------------------------------------
    BLOCK_LINEAR_MAX_ROWS = 128  # plain arithmetic: more rows than this go block by block to the matrix products (a launch per block)

    def block_linear(self, a, w, bias, out) -> None:
        """``out[:, b*n_out:(b+1)*n_out] = a[:, b*n_in:(b+1)*n_in] @ w[b].T + bias[b*n_out:(b+1)*n_out]`` for every block b of
        ``w`` ``[B, n_out, n_in]`` (compute dtype). ``a`` is of the weights' dtype or float32; ``out`` of it or float32. bfloat16
        weights whose blocks take a multiple of 8 inputs run on the matrix cores (float32 inputs are rounded to bfloat16 there);
        everything else in plain 32-bit arithmetic."""
        _dev(a, w, bias, out)
        _req(w.dim() == 3 and w.is_contiguous() and w.dtype in _DT, "block_linear: the weights must be contiguous [blocks, out, in]")
        B, n_out, n_in = w.shape
        T = a.shape[0]
        _req(a.dim() == 2 and a.shape[1] == B * n_in and a.dtype in _DT, "block_linear: a must be [T, blocks*in]")
        _req(out.shape == (T, B * n_out) and out.dtype in _DT, "block_linear: out must be [T, blocks*out]")
        _req(a.dtype == w.dtype or a.dtype == torch.float32, "block_linear: a must have the weights' dtype or be float32")
        _req(out.dtype == w.dtype or out.dtype == torch.float32, "block_linear: out must have the weights' dtype or be float32")
        _req(bias is None or (bias.dtype == torch.float32 and bias.numel() == B * n_out and bias.is_contiguous()), "block_linear: bias must be float32 [blocks*out]")
        lda = _rows(a, "block_linear: a")
        if (w.dtype == torch.bfloat16 and self.use_mfma and n_in % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0):
            # matrix cores: one launch for all blocks and any number of rows
            self._check(self.lib.lev_block_linear_mfma(_ptr(a), lda, _ptr(w), _ptr(bias), _ptr(out), _rows(out, "block_linear: out"), T, B, n_in, n_out,
                                                       _DT[a.dtype], _DT[out.dtype], self._s()))
            return
        if T > self.BLOCK_LINEAR_MAX_ROWS and a.dtype == w.dtype:
            for b in range(B):
                self.linear(a[:, b * n_in:(b + 1) * n_in], w[b], None if bias is None else bias[b * n_out:(b + 1) * n_out],
                            out[:, b * n_out:(b + 1) * n_out])
            return
        self._check(self.lib.lev_block_linear(_ptr(a), _rows(a, "block_linear: a"), _ptr(w), _ptr(bias), _ptr(out), _rows(out, "block_linear: out"),
                                              T, B, n_in, n_out, _DT[a.dtype], _DT[w.dtype], _DT[out.dtype], self._s()))

    # ---- the recurrent branch ------------------------------------------------------------------
    def causal_conv(self, x, taps, bias, state, token_slots, u) -> None:
        """``u[t, c] = bias[c] + sum_k taps[c, K-1-k] x[t-k, c]`` over the tokens of each request, reaching back into the last
        ``K - 1`` inputs that the request's slot keeps in ``state`` (float32 ``[slots, K, C]``, rows 0 .. K-2). The state is
        not changed here (``gated_recurrence`` shifts it)."""
        _dev(x, taps, bias, state, token_slots, u)
        T, C = x.shape
        _req(x.dtype in _DT and u.dtype == x.dtype and u.shape == x.shape and u.data_ptr() != x.data_ptr(), "causal_conv: x and u must be two [T, C] tensors of one dtype")
        _req(taps.dtype == torch.float32 and taps.dim() == 2 and taps.shape[0] == C and taps.is_contiguous(), "causal_conv: taps must be float32 [C, K]")
        K = taps.shape[1]
        _req(bias is None or (bias.dtype == torch.float32 and bias.numel() == C and bias.is_contiguous()), "causal_conv: bias must be float32 [C]")
        _req(state.dtype == torch.float32 and state.dim() == 3 and tuple(state.shape[1:]) == (K, C) and state.is_contiguous(), "causal_conv: state must be float32 [slots, K, C]")
        _req(token_slots.dtype == torch.int32 and token_slots.numel() == T, "causal_conv: one int32 slot per token")
        self._check(self.lib.lev_causal_conv(_ptr(x), _rows(x, "causal_conv: x"), _ptr(taps), _ptr(bias), _ptr(state), _ptr(token_slots), _ptr(u),
                                             _rows(u, "causal_conv: u"), T, C, K, _DT[x.dtype], self._s()))

    RECURRENCE_SCAN_MIN_ROWS = 48  # steps of more tokens than this run the recurrence as a scan in segments

    def gated_recurrence(self, u, gates, y, x, decay, state, token_slots, out, n_blocks: int, out_scale: float = 1.0) -> None:
        """Per channel, in 32-bit, along each request's tokens: ``a = exp(decay * sigmoid(gates_r))``,
        ``S <- a S + sqrt(1 - a^2) sigmoid(gates_i) u``, ``out = S * gelu_tanh(y) * out_scale``. ``gates`` float32
        ``[T, blocks, 2, C/blocks]``; ``state`` float32 ``[slots, K, C]``: row K-1 is S (read and stored), rows 0 .. K-2 the
        convolution's history, which is shifted by this step's inputs ``x``."""
        _dev(u, gates, y, x, decay, state, token_slots, out)
        T, C = u.shape
        dt = u.dtype
        _req(dt in _DT and y.dtype == x.dtype == out.dtype == dt and y.shape == x.shape == out.shape == u.shape, "gated_recurrence: u, y, x, out must be [T, C] of one dtype")
        _req(n_blocks > 0 and C % n_blocks == 0, "gated_recurrence: the channels must split into equal blocks")
        _req(gates.dtype == torch.float32 and gates.shape == (T, 2 * C), "gated_recurrence: gates must be float32 [T, 2*C]")
        _req(decay.dtype == torch.float32 and decay.numel() == C and decay.is_contiguous(), "gated_recurrence: decay must be float32 [C]")
        _req(state.dtype == torch.float32 and state.dim() == 3 and state.shape[2] == C and state.is_contiguous(), "gated_recurrence: state must be float32 [slots, K, C]")
        _req(token_slots.dtype == torch.int32 and token_slots.numel() == T, "gated_recurrence: one int32 slot per token")
        if T > self.RECURRENCE_SCAN_MIN_ROWS:
            # many tokens: the recurrence as a scan in segments (the same sums in another order, 32-bit)
            ws = torch.empty(self.lib.lev_gated_recurrence_scan_workspace(T, C), dtype=torch.uint8, device=u.device)
            self._check(self.lib.lev_gated_recurrence_scan(
                _ptr(u), _rows(u, "gated_recurrence: u"), _ptr(gates), _rows(gates, "gated_recurrence: gates"), _ptr(y), _rows(y, "gated_recurrence: y"),
                _ptr(x), _rows(x, "gated_recurrence: x"), _ptr(decay), _ptr(state), _ptr(token_slots), _ptr(out), _rows(out, "gated_recurrence: out"),
                _ptr(ws), T, C, state.shape[1], C // n_blocks, float(out_scale), _DT[dt], self._s()))
            return
        self._check(self.lib.lev_gated_recurrence(
            _ptr(u), _rows(u, "gated_recurrence: u"), _ptr(gates), _rows(gates, "gated_recurrence: gates"), _ptr(y), _rows(y, "gated_recurrence: y"),
            _ptr(x), _rows(x, "gated_recurrence: x"), _ptr(decay), _ptr(state), _ptr(token_slots), _ptr(out), _rows(out, "gated_recurrence: out"),
            T, C, state.shape[1], C // n_blocks, float(out_scale), _DT[dt], self._s()))

    # ---- norms in groups around gated sublayers ------------------------------------------------
    def group_norm_step(self, x, *, groups: int, eps: float, y=None, gate=None, post_weight=None, mult: float = 1.0, weight=None, h_out=None,
                        rows=None, defer: bool = False, pending: Optional[PendingGatedNorm] = None, plain_read: bool = False) -> Optional[PendingGatedNorm]:
        """One pass over the rows of the residual stream ``x`` (float32 ``[T, D]``) with ``gn(v, w)`` = ``v`` split into ``groups``
        equal consecutive parts, each divided by its own ``sqrt(mean(part^2) + eps)``, times ``w``. In this order, whatever is
        given: the write of a sublayer's result, ``x <- x + mult * gn(y * sigmoid(gate), post_weight)`` (``y`` float32 ``[T, D]``;
        ``gate`` ``[T, D]`` float32 or compute dtype, rows may be strided, None: no gate); the read ``h_out = gn(x, weight)``
        (compute dtype or float32; ``plain_read``: ``h_out = x`` as it is, only rounded to ``h_out``'s type, for a sublayer that reads the
        stream itself). ``rows``: only these rows, into ``h_out [len(rows), D]``; ``x`` is not stored then.
        ``defer``: nothing is launched; the write comes back as a ``PendingGatedNorm`` for the next call (``pending=``) or
        ``finish``. ``pending``: the write of an earlier call, done in this pass."""
        if pending is not None:
            _req(pending.out is x and y is None and pending.groups == groups and pending.eps == eps, "group norm: the unfinished sublayer belongs to another tensor or norm")
            y, gate, post_weight, mult = pending.y, pending.gate, pending.post_weight, pending.mult
        if defer:
            return PendingGatedNorm(x, y, gate, post_weight, float(mult), int(groups), float(eps))
        _dev(x, y, gate, post_weight, weight, h_out, rows)
        _req(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "group norm: x must be contiguous float32 [T, D]")
        T, D = x.shape
        _req(y is None or (y.dtype == torch.float32 and tuple(y.shape) == (T, D) and y.is_contiguous() and post_weight is not None),
             "group norm: a sublayer's result must be contiguous float32 [T, D] and have a norm weight")
        for name, w in (("post_weight", post_weight), ("weight", weight)):
            _req(w is None or (w.dtype == torch.float32 and w.numel() == D and w.is_contiguous()), f"group norm: {name} must be float32 [D]")
        gs, gdt = 0, torch.float32
        if gate is not None:
            _req(y is not None and gate.dtype in _DT and tuple(gate.shape) == (T, D), "group norm: the gate must be [T, D]")
            gs, gdt = _rows(gate, "group norm: gate"), gate.dtype
        n, odt = T, torch.float32
        if rows is not None:
            _req(rows.dtype == torch.int32 and rows.is_contiguous() and h_out is not None, "group norm: rows must be int32 and need an output")
            n = rows.numel()
        if h_out is not None:
            _req((weight is not None) != bool(plain_read) and h_out.dtype in _DT and h_out.is_contiguous() and tuple(h_out.shape) == (n, D), "group norm: bad normalised output")
            odt = h_out.dtype
        self._check(self.lib.lev_group_norm_step(_ptr(x), _ptr(y), _ptr(gate), gs, _DT[gdt], _ptr(post_weight), float(mult), _ptr(weight), _ptr(h_out),
                                                 _DT[odt], _ptr(rows), n, D, int(groups), float(eps), self._s()))
        return None

    # ---- rotation, "rotate half" layout --------------------------------------------------------
    def rotary_half(self, x, n_heads: int, head_stride: int, offset: int, freqs, positions) -> None:
        """In place on ``x`` ``[T, >= n_heads*head_stride]``: within each head of ``head_stride`` columns, the vector that starts at
        column ``offset`` has its dimension i < len(freqs) paired with dimension i + len(freqs), and the pair turns by
        ``positions[t] * freqs[i]``; every other column stays. 32-bit angles."""
        _dev(x, freqs, positions)
        T = x.shape[0]
        _req(x.dim() == 2 and x.dtype in _DT and x.shape[1] >= n_heads * head_stride, "rotary: x must be [T, heads*head_stride]")
        _req(freqs.dtype == torch.float32 and freqs.is_contiguous() and offset >= 0 and offset + 2 * freqs.numel() <= head_stride,
             "rotary: float32 frequencies, and the rotated vector must fit the head")
        _req(positions.dtype == torch.int32 and positions.numel() == T, "rotary: one int32 position per token")
        if freqs.numel() == 0:
            return
        self._check(self.lib.lev_rotary_half(_ptr(x), _rows(x, "rotary: x"), int(n_heads), int(head_stride), int(offset), freqs.numel(), _ptr(freqs),
                                             _ptr(positions), T, _DT[x.dtype], self._s()))

    # ---- a matrix state per head with decay and removal (generalized delta rule) ----------------
    def delta_rule(self, r, k, v, a_pre, g, w_pre, norm_weight, state, token_slots, out, n_heads: int, head_dim: int, norm_eps: float,
                   key_eps: float, sharpness: float, max_runs: Optional[int] = None) -> None:
        """Per head, along each request's tokens, in 32-bit: ``u = k / sqrt(sum(k^2) + key_eps)``, ``w = exp(-sharpness *
        sigmoid(w_pre))``, ``a = sigmoid(a_pre)``, ``S <- diag(w) S - (a * u)(u^T S) + k v^T`` (both terms read the old ``S``),
        ``o = S^T r``, ``out = o / sqrt(mean(o^2) + norm_eps) * norm_weight * sigmoid(g)``. ``r, k, v, a_pre, g``: ``[T, H*d]``
        views of one row stride in the compute dtype; ``w_pre`` float32 ``[T, H*d]``; ``state`` float32 ``[slots, H, d, d]``
        (key channel, value channel), read and stored; ``token_slots`` int32 ``[T]`` (-1: a token of nobody, zeros). ``max_runs``: the
        step has at most this many runs of consecutive tokens of one slot; given, and smaller than T, the step takes the path for
        prompts (the vectors of all tokens in parallel, then the walk along each run, then norm and gate in parallel)."""
        _dev(r, k, v, a_pre, g, w_pre, norm_weight, state, token_slots, out)
        T, C = r.shape
        dt = r.dtype
        _req(C == n_heads * head_dim and dt in _DT, "delta_rule: r must be [T, heads*head_dim] of a compute dtype")
        stride = _rows(r, "delta_rule: r")
        for name, t in (("k", k), ("v", v), ("a_pre", a_pre), ("g", g)):
            _req(t.dtype == dt and tuple(t.shape) == (T, C) and _rows(t, f"delta_rule: {name}") == stride, f"delta_rule: {name} must be [T, heads*head_dim] with r's dtype and row stride")
        _req(w_pre.dtype == torch.float32 and tuple(w_pre.shape) == (T, C), "delta_rule: w_pre must be float32 [T, heads*head_dim]")
        _req(norm_weight.dtype == torch.float32 and norm_weight.numel() == C and norm_weight.is_contiguous(), "delta_rule: the norm's weight must be float32 [heads*head_dim]")
        _req(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (n_heads, head_dim, head_dim), "delta_rule: state must be float32 [slots, heads, d, d]")
        _req(token_slots.dtype == torch.int32 and token_slots.numel() == T, "delta_rule: one int32 slot per token")
        _req(out.dtype == dt and tuple(out.shape) == (T, C), "delta_rule: out must be [T, heads*head_dim] of the compute dtype")
        if max_runs is not None and max_runs < T:
            ws = torch.empty(self.lib.lev_delta_rule_scan_workspace(T, n_heads, head_dim) // 4, dtype=torch.float32, device=r.device)
            self._check(self.lib.lev_delta_rule_scan(_ptr(r), _ptr(k), _ptr(v), _ptr(a_pre), _ptr(g), stride, _ptr(w_pre), _rows(w_pre, "delta_rule: w_pre"),
                                                     _ptr(norm_weight), _ptr(state), _ptr(token_slots), _ptr(out), _rows(out, "delta_rule: out"), _ptr(ws), T,
                                                     int(max_runs), n_heads, head_dim, float(norm_eps), float(key_eps), float(sharpness), _DT[dt], self._s()))
            return
        self._check(self.lib.lev_delta_rule(_ptr(r), _ptr(k), _ptr(v), _ptr(a_pre), _ptr(g), stride, _ptr(w_pre), _rows(w_pre, "delta_rule: w_pre"),
                                            _ptr(norm_weight), _ptr(state), _ptr(token_slots), _ptr(out), _rows(out, "delta_rule: out"), T, n_heads,
                                            head_dim, float(norm_eps), float(key_eps), float(sharpness), _DT[dt], self._s()))

    # ---- a matrix state per head that decays by key channel (gated linear attention) ------------
    GLA_GATES = {"sigmoid": 0, "silu": 1}

    def gated_linear_attention(self, q, k, v, g, z, norm_weight, state, token_slots, out, n_heads: int, key_dim: int, value_dim: int, tau: float,
                               q_scale: float, norm_eps: float, gate: str = "silu", max_runs: Optional[int] = None) -> None:
        """Per head, along each request's tokens, in 32-bit: ``a = sigmoid(z)^(1 / tau)``, ``S <- diag(a) S + k v^T``, ``o = S^T (q_scale q)``,
        ``out = o / sqrt(mean(o^2) + norm_eps) * norm_weight * gate(g)`` (``gate``: "sigmoid", or "silu" = g sigmoid(g)). ``q, k``: ``[T, H*dk]``
        views of one row stride, ``v, g``: ``[T, H*dv]`` views of one row stride, compute dtype; ``z`` float32 ``[T, H*dk]``; ``norm_weight``
        float32 ``[H*dv]``; ``state`` float32 ``[slots, H, dk, dv]``, read and stored; ``token_slots`` int32 ``[T]`` (-1: a token of nobody,
        zeros). ``max_runs``: the step has at most this many runs of consecutive tokens of one slot; given, and smaller than T, the step
        takes the path for prompts."""
        _dev(q, k, v, g, z, norm_weight, state, token_slots, out)
        T = q.shape[0]
        dt = q.dtype
        H, dk, dv = int(n_heads), int(key_dim), int(value_dim)
        _req(dt in _DT and tuple(q.shape) == tuple(k.shape) == (T, H * dk) and k.dtype == dt, "linear attention: q and k must be [T, heads*key_dim] of a compute dtype")
        _req(tuple(v.shape) == tuple(g.shape) == (T, H * dv) and v.dtype == g.dtype == dt, "linear attention: v and g must be [T, heads*value_dim] of the same dtype")
        qs, vs = _rows(q, "linear attention: q"), _rows(v, "linear attention: v")
        _req(_rows(k, "linear attention: k") == qs and _rows(g, "linear attention: g") == vs, "linear attention: q and k, and v and g, must share a row stride")
        _req(z.dtype == torch.float32 and tuple(z.shape) == (T, H * dk), "linear attention: z must be float32 [T, heads*key_dim]")
        _req(norm_weight.dtype == torch.float32 and norm_weight.numel() == H * dv and norm_weight.is_contiguous(), "linear attention: the norm's weight must be float32 [heads*value_dim]")
        _req(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, dk, dv), "linear attention: state must be float32 [slots, heads, dk, dv]")
        _req(token_slots.dtype == torch.int32 and token_slots.numel() == T, "linear attention: one int32 slot per token")
        _req(out.dtype == dt and tuple(out.shape) == (T, H * dv), "linear attention: out must be [T, heads*value_dim] of the compute dtype")
        _req(gate in self.GLA_GATES, f"linear attention: unknown gate {gate!r}")
        head = (_ptr(q), _ptr(k), qs, _ptr(v), _ptr(g), vs, _ptr(z), _rows(z, "linear attention: z"), _ptr(norm_weight), _ptr(state), _ptr(token_slots),
                _ptr(out), _rows(out, "linear attention: out"))
        tail = (H, dk, dv, float(tau), float(q_scale), float(norm_eps), self.GLA_GATES[gate], _DT[dt], self._s())
        if max_runs is not None and max_runs < T:
            ws = torch.empty(self.lib.lev_gla_scan_workspace(T, H, dk, dv) // 4, dtype=torch.float32, device=q.device)
            self._check(self.lib.lev_gla_scan(*head, _ptr(ws), T, int(max_runs), *tail))
            return
        self._check(self.lib.lev_gla_tokens(*head, T, *tail))

    # ---- row kernels of gated feed-forwards and of branches with norms of their own ---------------
    def glu_activate(self, z, out, activation: str, limit: float = 0.0, up_shift: float = 0.0) -> None:
        """``z`` ``[T, 2F]`` (gate sums, then up sums; rows may be strided) -> ``out`` ``[T, F]`` (may be ``z[:, :F]``):
        ``act(g) * (u + up_shift)``, with ``limit`` > 0 after ``g = min(g, limit)``, ``u = clamp(u, -limit, limit)``. 32-bit arithmetic."""
        _dev(z, out)
        T, F2 = z.shape
        _req(F2 % 2 == 0 and z.dtype in _DT and out.dtype == z.dtype and tuple(out.shape) == (T, F2 // 2), "glu_activate: z [T, 2F] and out [T, F] of one compute dtype")
        _req(activation in ACTIVATIONS, f"glu_activate: unknown activation {activation!r}")
        self._check(self.lib.lev_glu_activate(_ptr(z), _rows(z, "glu_activate: z"), _ptr(out), _rows(out, "glu_activate: out"), T, F2 // 2,
                                              ACTIVATIONS[activation], float(limit), float(up_shift), _DT[z.dtype], self._s()))

    def norm_sum2(self, a, b, weight_a, weight_b, scale_a: float, scale_b: float, eps: float, y) -> None:
        """``y = scale_a * a / rms(a) * weight_a + scale_b * b / rms(b) * weight_b`` over rows, ``rms(v) = sqrt(mean(v^2) + eps)``; all
        float32, ``y`` may be ``a`` or ``b``."""
        _dev(a, b, weight_a, weight_b, y)
        T, D = a.shape
        for t in (a, b, y):
            _req(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (T, D), "norm_sum2: contiguous float32 [T, D] tensors")
        for w in (weight_a, weight_b):
            _req(w.dtype == torch.float32 and w.is_contiguous() and w.numel() == D, "norm_sum2: the weights must be float32 [D]")
        self._check(self.lib.lev_norm_sum2(_ptr(a), _ptr(b), _ptr(weight_a), _ptr(weight_b), float(scale_a), float(scale_b), float(eps), _ptr(y), T, D, self._s()))

    # ---- mixture of experts --------------------------------------------------------------------
    def moe_route(self, z, correction, chosen, weights, *, n_groups: int = 1, keep: int = 1, group_top: int = 2, renormalize: bool = False,
                  softmax: bool = False) -> None:
        """Per token: ``s = sigmoid(z)`` (``z`` float32 ``[T, E]``), or with ``softmax`` the softmax of ``z`` over all E; the choice goes by ``s + correction``; only experts of the
        ``keep`` groups (of ``n_groups`` equal groups of neighbours) whose ``group_top`` largest choice scores sum highest can be
        chosen; ``chosen`` int32 ``[T, top]`` the winners in the order of falling choice score (ties: lower index first),
        ``weights`` float32 ``[T, top]`` their ``s`` (divided by their sum with ``renormalize``)."""
        _dev(z, correction, chosen, weights)
        T, E = z.shape
        top = chosen.shape[1]
        _req(z.dtype == torch.float32 and chosen.dtype == torch.int32 and weights.dtype == torch.float32, "experts: logits and weights float32, choices int32")
        _req(tuple(chosen.shape) == tuple(weights.shape) == (T, top) and chosen.is_contiguous() and weights.is_contiguous(), "experts: choices and weights must be [T, top]")
        _req(correction is None or (correction.dtype == torch.float32 and correction.numel() == E and correction.is_contiguous()), "experts: the correction must be float32 [E]")
        self._check(self.lib.lev_moe_route(_ptr(z), _rows(z, "experts: z"), _ptr(correction), T, E, int(n_groups), int(keep), int(group_top), top,
                                           int(renormalize), int(bool(softmax)), _ptr(chosen), _ptr(weights), self._s()))

    @staticmethod
    def moe_tile_rows(pairs: int, n_experts: int) -> int:
        """Rows of a tile of the experts' products: 64 where an expert has 32 rows or more on average, else 16."""
        return 64 if pairs >= 32 * n_experts else 16

    def moe_max_tiles(self, pairs: int, n_experts: int, tile_rows: int = 16) -> int:
        return int(self.lib.lev_moe_max_tiles(int(pairs), int(n_experts), int(tile_rows)))

    def moe_sort(self, chosen, n_experts: int, sorted_pairs, pos_of, tiles, meta, tile_rows: int = 16, n_real: Optional[int] = None) -> None:
        """The (token, choice) pairs of ``chosen`` ordered by expert: ``sorted_pairs[pos]`` the pair at place ``pos``, ``pos_of`` its
        inverse, ``tiles`` int32 ``[max_tiles, 3]`` (expert, first place, rows <= ``tile_rows``) covering every expert's stretch,
        ``meta[0]`` their number. Everything stays on the device. ``n_real``: only the experts below it have weights; the pairs of the others
        get places and no tiles (``moe_combine`` gives them the token's own input)."""
        _dev(chosen, sorted_pairs, pos_of, tiles, meta)
        P = chosen.numel()
        for t in (chosen, sorted_pairs, pos_of, tiles, meta):
            _req(t.dtype == torch.int32 and t.is_contiguous(), "experts: int32 tables")
        _req(sorted_pairs.numel() >= P and pos_of.numel() >= P and tiles.numel() >= 3 * self.moe_max_tiles(P, n_experts, tile_rows) and meta.numel() >= 1, "experts: tables too small")
        self._check(self.lib.lev_moe_sort(_ptr(chosen), P, int(n_experts), int(n_experts if n_real is None else n_real), int(tile_rows), _ptr(sorted_pairs), _ptr(pos_of), _ptr(tiles), _ptr(meta), self._s()))

    def moe_linear(self, a, w, out, tiles, meta, sorted_pairs, *, top: int, gather: bool, glu: bool = False, activation: str = "none",
                   tile_rows: int = 16, limit: float = 0.0, up_shift: float = 0.0) -> None:
        """For every tile of ``moe_sort``: ``out[pos] = w[expert] a[row(pos)]``, ``row(pos)`` the pair's token (``gather``) or
        ``pos`` itself. ``w`` ``[E, N, K]``; with ``glu`` N = 2F, gate rows then up rows, and ``out[pos][f] = act(gate_f) * (up_f + up_shift)``;
        with ``limit`` > 0 the gate sum is capped at it and the up sum clamped to +-limit first."""
        _dev(a, w, out, tiles, meta, sorted_pairs)
        _req(w.dim() == 3 and w.is_contiguous() and w.dtype in _DT and a.dtype == w.dtype and a.dim() == 2 and a.shape[1] == w.shape[2], "experts: a [rows, K], w [E, N, K] of one dtype")
        E, N, K = w.shape
        F_ = N // 2 if glu else N
        _req(out.dim() == 2 and out.shape[1] == F_ and out.dtype in _DT and (a.dtype == torch.bfloat16 or out.dtype == torch.float32), "experts: bad output")
        max_tiles = tiles.numel() // 3
        self._check(self.lib.lev_moe_linear(_ptr(a), _rows(a, "experts: a"), _ptr(w), _ptr(out), _rows(out, "experts: out"), _ptr(tiles), _ptr(meta),
                                            _ptr(sorted_pairs), max_tiles, int(tile_rows), int(top), int(gather), K, N, int(glu), ACTIVATIONS[activation], float(limit), float(up_shift), _DT[a.dtype],
                                            _DT[out.dtype], int(self.use_mfma), self._s()))

    def moe_combine(self, expert_out, pos_of, weights, y, accumulate: bool = False, chosen=None, n_real: int = 0, identity_in=None) -> None:
        """``y[t] = sum_c weights[t, c] * expert_out[pos_of[t, c]]``, c in order, float32; ``accumulate``: added to what ``y`` holds.
        ``identity_in`` (``[T, D]``, with ``chosen`` int32 ``[T, top]`` and ``n_real``): a choice of an expert from ``n_real`` on takes
        ``identity_in[t]`` in place of an expert's output."""
        _dev(expert_out, pos_of, weights, y, chosen, identity_in)
        ids, idt = 0, torch.float32
        if identity_in is not None:
            _req(chosen is not None and chosen.dtype == torch.int32 and chosen.is_contiguous() and tuple(chosen.shape) == tuple(weights.shape)
                 and identity_in.dtype in _DT and tuple(identity_in.shape) == tuple(y.shape), "experts: experts that return their input need the choices and the input")
            ids, idt = _rows(identity_in, "experts: identity_in"), identity_in.dtype
        T, D = y.shape
        top = weights.shape[1]
        _req(expert_out.dtype == y.dtype == weights.dtype == torch.float32 and expert_out.is_contiguous() and y.is_contiguous() and weights.is_contiguous()
             and expert_out.shape[1] == D and expert_out.shape[0] >= T * top and pos_of.dtype == torch.int32 and pos_of.numel() >= T * top, "experts: bad arguments of the weighted sum")
        self._check(self.lib.lev_moe_combine(_ptr(expert_out), _ptr(pos_of), _ptr(weights), _ptr(y), T, D, top, int(accumulate),
                                             _ptr(chosen) if identity_in is not None else None, int(n_real), _ptr(identity_in), ids, _DT[idt], self._s()))

    # ---- attention -------------------------------------------------------------------------
    def paged_attention(self, q, out, k_pages, v_pages, meta, *, n_heads: int, n_kv_heads: int, head_dim: int,
                        page_size: int, scale: float, window: Optional[int], block_tables, k_new=None, v_new=None,
                        dest=None, softcap: Optional[float] = None, score_bias=None) -> bool:
        """Causal attention of the step's query tokens over the pages. ``meta`` is the step's
        ``AttentionMeta`` (positions, token_seq and the work lists), block_tables int32 [S, B].

        ``score_bias`` (float32 ``[n_heads, L]``): entry ``[h, min(d, L - 1)]`` is added to the scaled score of head ``h``
        for a key ``d`` positions behind its query; ``softcap``: scores become ``softcap * tanh(score / softcap)`` (after
        the bias, before the mask). Both off by default.

        ``k_new``/``v_new``/``dest``: the step's new keys and values, not yet written. Returns True if this
        call has written them to their pages (a step of single tokens on the matrix-core path does it inside
        the attention kernel); False means the caller must call ``kv_write`` first and call again without them."""
        if not (q.is_cuda and out.is_cuda and k_pages.is_cuda and v_pages.is_cuda):
            raise KernelError("a kernel was given a tensor that is not on the GPU")
        T, cols = q.shape
        dt = q.dtype
        if not (cols == n_heads * head_dim and out.shape == q.shape):
            raise KernelError("attention: q and out must be [T, heads*head_dim]")
        if not (dt == out.dtype == k_pages.dtype == v_pages.dtype and dt in _DT):
            raise KernelError("attention: dtypes differ")
        # what depends on the step and the cache group only (tables, work lists, the split of the key range, scratch memory) is
        # checked and decided at the step's first layer and kept with the step's description
        key = (n_heads, n_kv_heads, head_dim, page_size, id(block_tables), dt)
        plan = meta.plans.get(key)
        if plan is None:
            _dev(block_tables, meta.positions, meta.token_seq)
            _req(meta.positions.numel() == T and meta.token_seq.numel() == T, "attention: one position and request row per token")
            _req(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(), "attention: bad block tables")
            _req(n_heads % n_kv_heads == 0, "attention: heads must be a multiple of kv heads")
            mfma = (dt == torch.bfloat16 and self.use_mfma and self.mfma_attention_supports(head_dim, n_heads // n_kv_heads)
                    and page_size & (page_size - 1) == 0)  # the matrix-core kernels index pages with shifts
            if dt == torch.bfloat16 and self.use_mfma and not mfma:
                self._warn_slow_attention(head_dim, n_heads // n_kv_heads, page_size)
            splits, ws, lib = 1, None, None
            if mfma:
                splits = self.decode_splits(meta, n_heads, n_kv_heads)
                need = self.lib.lev_attention_mfma_workspace(meta.n_decode, splits, n_heads, n_kv_heads, head_dim) if splits > 1 else 0
                ws = meta.workspace(need, q.device)
                lib = self._unit(_build.attention_unit(head_dim))
            plan = meta.plans[key] = (mfma, splits, ws, _ptr(ws), lib, _ptr(block_tables), block_tables.shape[1], _ptr(meta.positions),
                                      _ptr(meta.token_seq), _ptr(meta.prefill_tiles), _ptr(meta.decode_tokens), block_tables)
        mfma, splits, _ws, ws_ptr, lib, bt_ptr, bt_width, pos_ptr, seq_ptr, tiles_ptr, decode_ptr, _bt = plan
        w = int(window) if window else 0
        cap = float(softcap) if softcap else 0.0
        bias_len = 0
        if score_bias is not None:
            if not (score_bias.is_cuda and score_bias.dtype == torch.float32 and score_bias.dim() == 2 and score_bias.shape[0] == n_heads
                    and score_bias.is_contiguous() and score_bias.shape[1] >= 1):
                raise KernelError("attention: the score bias must be a contiguous float32 table [heads, distances] on the GPU")
            bias_len = score_bias.shape[1]
        qs, os_ = _rows(q, "attention: q"), _rows(out, "attention: out")
        kvs = 0
        if k_new is not None:
            fusable = mfma and meta.n_prefill_tiles == 0 and meta.n_decode == T
            if not fusable:
                return False
            _dev(k_new, v_new, dest)
            _req(k_new.shape == v_new.shape == (T, n_kv_heads * head_dim) and k_new.dtype == v_new.dtype == dt,
                 "attention: new keys and values must be [T, kv_heads*head_dim] of the compute dtype")
            _req(dest is not None and dest.dtype == torch.int32 and dest.numel() == T, "attention: one int32 destination per token")
            kvs = _rows(k_new, "attention: k_new")
            _req(kvs == _rows(v_new, "attention: v_new"), "attention: new keys and values must share a row stride")
        if mfma:
            self._check(lib.lev_attention_mfma(
                _ptr(q), qs, _ptr(out), os_, _ptr(k_pages), _ptr(v_pages), pos_ptr, seq_ptr, bt_ptr, bt_width, tiles_ptr,
                meta.n_prefill_tiles, decode_ptr, meta.n_decode, _ptr(k_new), _ptr(v_new), kvs,
                _ptr(dest) if k_new is not None else None, ws_ptr, n_heads, n_kv_heads, head_dim, page_size,
                splits, float(scale), w, cap, _ptr(score_bias), bias_len, self._s()))
            return k_new is not None
        self._check(self.lib.lev_attention_simple(
            _ptr(q), qs, _ptr(out), os_, _ptr(k_pages), _ptr(v_pages), pos_ptr, seq_ptr, bt_ptr, bt_width, T, n_heads, n_kv_heads,
            head_dim, page_size, float(scale), w, _DT[dt], cap, _ptr(score_bias), bias_len, self._s()))
        return False

    @staticmethod
    def decode_splits(meta, n_heads: int, n_kv_heads: int) -> int:
        """Into how many key ranges a single-token query is split so that the chip is filled."""
        if meta.n_decode == 0:
            return 1
        want = max(1, 2048 // max(1, meta.n_decode * n_kv_heads))
        most = max(1, (meta.max_kv_len + 63) // 64)  # at least 64 keys per split
        splits = int(min(want, most, 64))
        if splits > 8 and most <= 16 and meta.n_decode * n_kv_heads >= 128:
            # Up to 8 splits are merged inside one workgroup (no second kernel). That is worth two blocks of keys per
            # wave where the workgroups alone give the chip a few hundred waves; with fewer (one or two requests) a
            # wave per block and the combine kernel are faster at every context length (measured at 32 heads of 128:
            # batch 1, 1,850 keys: 3.73 -> 3.26 ms a step; batch 4, 580 keys: 3.39 ms with the clamp, 3.43 without).
            splits = 8
        return splits

    def _warn_slow_attention(self, head_dim: int, group: int, page_size: int) -> None:
        key = (head_dim, group, page_size)
        if key not in self._slow_attention_warned:
            self._slow_attention_warned.add(key)
            import warnings

            warnings.warn(f"attention with head_dim={head_dim}, {group} query heads per kv head and page_size={page_size} has no matrix-core "
                          f"kernel (head sizes 16..128 in steps of 16, at most 16 query heads per kv head, page sizes that are powers of "
                          f"two): it runs on the plain-arithmetic kernel, which is correct and slow", RuntimeWarning, stacklevel=3)

    @staticmethod
    def mfma_attention_supports(head_dim: int, group: int) -> bool:
        return head_dim % 16 == 0 and 16 <= head_dim <= 128 and group <= 16

    # ---- sampling ----------------------------------------------------------------------------
    def sample(self, logits, temperatures, keys, positions, out_tokens, out_logprobs) -> None:
        """Greedy (temperature 0) or temperature sampling of float32 logits [R, V]; keys int32/uint32 [R, 2]."""
        _dev(logits, temperatures, keys, positions, out_tokens, out_logprobs)
        R, V = logits.shape
        _req(logits.dtype == torch.float32, "sample: logits must be float32")
        _req(temperatures.dtype == torch.float32 and temperatures.numel() == R, "sample: one float32 temperature per row")
        _req(keys.dtype == torch.int32 and keys.numel() == 2 * R and keys.is_contiguous(), "sample: keys must be int32 [R, 2]")
        _req(positions.dtype == torch.int32 and positions.numel() == R, "sample: one int32 position per row")
        _req(out_tokens.dtype == torch.int32 and out_tokens.numel() == R, "sample: tokens out must be int32 [R]")
        _req(out_logprobs.dtype == torch.float32 and out_logprobs.numel() == R, "sample: logprobs out must be float32 [R]")
        need = self.lib.lev_sample_workspace(R)
        if self._sample_ws is None or self._sample_ws.numel() < need or self._sample_ws.device != logits.device:
            self._sample_ws = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=logits.device)
        self._check(self.lib.lev_sample(_ptr(logits), _rows(logits, "sample: logits"), _ptr(temperatures), _ptr(keys),
                                        _ptr(positions), _ptr(out_tokens), _ptr(out_logprobs), _ptr(self._sample_ws), R, V,
                                        self._s()))


_KERNELS = None


def set_kernels(k) -> None:
    """Install a kernel library object (tests install a stand-in to run host logic without a GPU)."""
    global _KERNELS
    _KERNELS = k


def get_kernels():
    """The loaded HIP library. Raises when there is no GPU or the library cannot be built or loaded."""
    global _KERNELS
    if _KERNELS is None:
        if not torch.cuda.is_available():
            raise KernelError("levanter_amd runs on an AMD GPU only (torch.cuda.is_available() is False); there is no CPU path")
        path = _build.ensure_built("core")
        try:
            _KERNELS = HipKernels(path)
        except OSError as e:
            raise KernelError(f"the HIP library {path} cannot be loaded: {e}") from None
    return _KERNELS
