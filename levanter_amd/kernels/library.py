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

ACTIVATIONS = {"none": 0, "gelu_new": 1, "gelu": 2, "relu": 3, "silu": 4, "swish": 4, "quick_gelu": 5, "tanh": 6}
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
    def embed(self, tokens, positions, table, pos_table, out) -> None:
        """out[t] = table[tokens[t]] + pos_table[positions[t]] in float32. Ids are trusted (the step checks them)."""
        _dev(tokens, positions, table, pos_table, out)
        T, D = out.shape
        _req(tokens.dtype == torch.int32 and positions.dtype == torch.int32, "embed: ids must be int32")
        _req(tokens.numel() == T and positions.numel() == T, "embed: one token and one position per output row")
        _req(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
        _req(table.is_contiguous() and table.shape[1] == D and table.dtype in _DT, "embed: bad table")
        if pos_table is not None:
            _req(pos_table.is_contiguous() and pos_table.shape[1] == D and pos_table.dtype == table.dtype, "embed: bad position table")
        self._check(self.lib.lev_embed(_ptr(tokens), _ptr(positions), _ptr(table), _ptr(pos_table), _ptr(out), T, D,
                                       _DT[table.dtype], self._s()))

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
        if pending is not None:
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
        """Finish a product that ``linear(..., may_leave_pending=True)`` left unfinished."""
        x = pending.out
        self._check(self._unit("gemm_mfma").lev_linear_mfma_finish(_ptr(pending.workspace), _ptr(pending.bias), _ptr(x), pending.ldo, _ptr(x),
                                                                   pending.ldo, x.shape[0], x.shape[1], pending.n_ranges, 0, _DT[torch.float32],
                                                                   self._s()))

    def linear(self, a, w, bias, out, activation: str = "none", residual=None, may_leave_pending: bool = False) -> Optional[PendingSum]:
        """out = act(a @ w.T + bias) (+ residual). a [M, K], w [N, K], out [M, N]; residual float32, may be ``out``.

        ``may_leave_pending`` (only with ``residual is out``, no activation): where the kernel splits the sum over K into
        ranges, it may stop after writing them and return a ``PendingSum`` instead of running the kernel that adds them
        up: the caller promises that the next thing to touch ``out`` is ``norm(out, ..., pending=...)`` or ``finish``."""
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
            leave = may_leave_pending and need > 0 and residual is out and act == 0 and ldo == N
            self._check(gemm.lev_linear_mfma(_ptr(a), lda, _ptr(w), _ptr(bias), _ptr(residual), ldr, _ptr(out), ldo, _ptr(ws),
                                             M, N, K, act, _DT[odt], int(leave), self._s()))
            if leave:
                return PendingSum(out, ws, need // (M * N * 4), bias, ldo)
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
    def kv_write(self, k, v, k_pages, v_pages, dest, n_kv_heads: int, head_dim: int, page_size: int) -> None:
        """Scatter the new tokens' keys and values ([T, n_kv_heads*head_dim] views) to ``dest[t] = page*page_size + offset``."""
        if not (k.is_cuda and v.is_cuda and k_pages.is_cuda and v_pages.is_cuda and dest.is_cuda):
            raise KernelError("a kernel was given a tensor that is not on the GPU")
        T, cols = k.shape
        dt = k.dtype
        if not (v.shape == k.shape and cols == n_kv_heads * head_dim):
            raise KernelError("kv_write: k and v must be [T, kv_heads*head_dim]")
        if not (dt == v.dtype == k_pages.dtype == v_pages.dtype and dt in _DT):
            raise KernelError("kv_write: dtypes differ")
        if not (dest.dtype == torch.int32 and dest.numel() == T):
            raise KernelError("kv_write: one int32 destination per token")
        n_elems = k_pages.numel()
        if not (k_pages.is_contiguous() and v_pages.is_contiguous() and n_elems % (cols * page_size) == 0 and n_elems == v_pages.numel()):
            raise KernelError("kv_write: page tensors must be contiguous and fit the sizes")
        self._check(self.lib.lev_kv_write(_ptr(k), _ptr(v), _rows(k, "kv_write: k"), _rows(v, "kv_write: v"), _ptr(k_pages),
                                          _ptr(v_pages), _ptr(dest), T, n_kv_heads, head_dim, page_size, _DT[dt], self._s()))

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
