"""Python face of the HIP kernels: shape checks on the host, then the launch.

Every wrapper verifies what the kernel and its grid assume (device, dtype,
contiguity of rows, matching sizes) before it launches, because a kernel that
reads out of bounds can take the whole GPU down.  Launches go to torch's
current stream, so they order with torch's own copies and can be captured in
a HIP graph.  There is no fallback path: if the library cannot be loaded the
constructor raises.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from . import build as _build

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
STORE, STORE_F32, ADD_F32, SWIGLU = 0, 1, 2, 3


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of ``gate`` and ``up`` (``[I, K]`` each) interleaved in tiles of 16 rows:
    gate rows 0..15, up rows 0..15, gate rows 16..31, ...; the last tile of each is
    padded with zero rows.  This is the weight layout of the SwiGLU epilogue."""
    inter, k = gate.shape
    tiles = -(-inter // 16)
    out = torch.zeros((tiles, 2, 16, k), dtype=gate.dtype)
    pad = tiles * 16 - inter
    g = torch.cat([gate, gate.new_zeros((pad, k))]) if pad else gate
    u = torch.cat([up, up.new_zeros((pad, k))]) if pad else up
    out[:, 0] = g.view(tiles, 16, k)
    out[:, 1] = u.view(tiles, 16, k)
    return out.view(tiles * 32, k)
MAX_HEAD_DIM = 256


class KernelError(RuntimeError):
    pass


def _ptr(t) -> c_void_p:
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> c_void_p:
    """The current stream of the current device (asked through the raw call where torch has it:
    a kernel launch asks for it every time, and the Python stream object costs ten times as much)."""
    if _raw_stream is not None:
        return c_void_p(_raw_stream(_raw_device() if _raw_device is not None else torch.cuda.current_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


# The checks in front of a launch are plain conditionals whose message is made only when a check
# fails: a step runs some two thousand of them.
def _rows_ok(t: torch.Tensor, name: str) -> None:
    if not (t.is_cuda and t.dim() == 2 and t.stride(1) == 1):
        raise KernelError(f"{name} must be 2-D with contiguous rows on the GPU, got shape {tuple(t.shape)} "
                          f"strides {t.stride()} on {t.device}")


class Kernels:
    """The loaded libraries.  One instance per process (see ``kernels()``)."""

    def __init__(self, mutants: bool = False):
        """``mutants``: load the control libraries instead (built with their deliberately wrong
        variants compiled in, all switched off until ``set_mutants``); the tests' positive
        controls use them, the engine never does."""
        self.mutants = mutants
        self.core_path = _build.build_core_mutants() if mutants else _build.build_core()
        self.core = ctypes.CDLL(str(self.core_path))
        self.core.ls_last_error.restype = ctypes.c_char_p
        self.core.ls_sample_scratch_bytes.restype = ctypes.c_long
        self._attention: dict[int, ctypes.CDLL] = {}
        self.attention_paths: dict[int, str] = {}
        self._mixers = None
        self.mixers_path = None
        self._talking: dict[tuple, ctypes.CDLL] = {}
        self.talking_paths: dict[tuple, str] = {}
        self._sink: dict[tuple, ctypes.CDLL] = {}
        self.sink_paths: dict[tuple, str] = {}
        self._experts = None
        self.experts_path = None
        self._argmax_scratch: dict = {}
        self._sample_scratch: dict = {}
        self._sample_scratch_kept: list = []
        self._capabilities: dict = {}
        #: while this is a list, every launch is noted on it as (library, entry point, arguments):
        #: the engine repeats the launches of one layer for the next layers that are alike
        self.tape: list | None = None
        self._listed: dict = {}

    # -- helpers ------------------------------------------------------------
    @staticmethod
    def _check(lib, code: int) -> None:
        if code != 0:
            raise KernelError(lib.ls_last_error().decode())

    def _launch(self, lib, entry, args: tuple) -> None:
        if entry(*args) != 0:
            raise KernelError(lib.ls_last_error().decode())
        if self.tape is not None:
            self.tape.append((lib, entry, args))

    # -- launches handed over as one list ----------------------------------------
    def listed(self, lib, entry):
        """(address of the library's ``ls_call_listed``, the entry point's index there) for an entry point
        that ``run_list`` may name, or None."""
        key = (id(lib), entry.__name__)
        found = self._listed.get(key, False)
        if found is False:
            found = None
            if hasattr(lib, "ls_listed_index"):
                index = lib.ls_listed_index(entry.__name__.encode())
                if index >= 0:
                    found = (ctypes.cast(lib.ls_call_listed, c_void_p).value, index, lib)
            self._listed[key] = found
        return found

    def run_list(self, words, libs=(), period: int = 0) -> None:
        """Make the calls that ``words`` (a contiguous int64 array of records, see ``ls_run_list`` in
        csrc/core_api.h) lists, in order.  ``libs``: (word offset of a record, its library) pairs, for the
        message of a call that fails; with ``period`` the offsets repeat with that many words."""
        failed_at = ctypes.c_long(-1)
        code = self.core.ls_run_list(c_void_p(words.ctypes.data), c_long(words.size), ctypes.byref(failed_at))
        if code != 0:
            at = failed_at.value % period if period else failed_at.value
            lib = dict(libs).get(at, self.core)
            raise KernelError(lib.ls_last_error().decode())

    def attention_lib(self, head_dim: int):
        lib = self._attention.get(head_dim)
        if lib is None:
            path = _build.build_attention_mutants(head_dim) if self.mutants else _build.build_attention(head_dim)
            lib = ctypes.CDLL(str(path))
            lib.ls_last_error.restype = ctypes.c_char_p
            if not (lib.ls_attn_head_dim() == head_dim):
                raise KernelError(f"{path} was built for another head size")
            if self.mutants and getattr(self, "_attention_mask", 0):
                self._check(lib, lib.ls_set_mutants(c_int(self._attention_mask)))
            self._attention[head_dim] = lib
            self.attention_paths[head_dim] = str(path)
        return lib

    #: bits of ``set_mutants`` (csrc/common.h)
    MUTANT_KSLICE_BY_ROWS, MUTANT_NORM_BY_ROWS, MUTANT_SAMPLE_CHUNKS_BY_ROWS = 1, 2, 4      # core library
    MUTANT_REVERSED_FOLD_IN_PRODUCT = 8
    MUTANT_REVERSED_FOLD = 1                               # attention libraries

    def set_mutants(self, core: int = 0, attention: int = 0) -> None:
        """Switch wrong variants of the control libraries on (bit masks) or off (0)."""
        if not self.mutants:
            raise KernelError("these are the product libraries: they hold no mutants")
        self._check(self.core, self.core.ls_set_mutants(c_int(core)))
        for lib in self._attention.values():
            self._check(lib, lib.ls_set_mutants(c_int(attention)))
        self._attention_mask = attention

    def _memo(self, key, compute):
        """Capability queries do not change while the process runs: ask the library once."""
        have = self._capabilities.get(key)
        if have is None:
            have = self._capabilities[key] = compute()
        return have

    def coop_supported(self, head_dim: int, dtype: torch.dtype, page_size: int = 16) -> bool:
        """Whether the cooperative attention kernel can run (its tiles must fit into LDS)."""
        return self._memo(("coop", head_dim, dtype, page_size), lambda: page_size >= 8 and bool(
            self.attention_lib(head_dim).ls_attn_coop_supported(c_int(DTYPE_CODE[dtype]))))

    def decode_fused_supported(self, head_dim: int, dtype: torch.dtype, page_size: int) -> bool:
        """Whether ``attention_decode`` (norm, rotation and cache write inside the attention kernel) can run."""
        return self._memo(("decode_fused", head_dim, dtype, page_size), lambda: page_size >= 8 and bool(
            self.attention_lib(head_dim).ls_attn_decode_fused_supported(c_int(DTYPE_CODE[dtype]))))

    def compute_units(self) -> int:
        """Compute units of the current device."""
        return self._memo(("compute_units",), lambda: int(
            torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count))

    def wide_supported(self, head_dim: int, dtype: torch.dtype, page_size: int) -> bool:
        """Whether the wide attention kernel (variant 4, for prompt portions) can run."""
        return self._memo(("wide", head_dim, dtype, page_size), lambda: page_size >= 8 and bool(
            self.attention_lib(head_dim).ls_attn_wide_supported(c_int(DTYPE_CODE[dtype]))))

    def attention_block_rows(self, head_dim: int, variant: int) -> int:
        """Rows of the row blocks that work items of this variant count in."""
        return self._memo(("block_rows", head_dim, variant),
                          lambda: int(self.attention_lib(head_dim).ls_attn_block_rows(c_int(variant))))

    def attention_geometry(self, head_dim: int) -> tuple[int, int]:
        """(keys per tile, keys per split) of the attention kernels."""
        return self._memo(("geometry", head_dim), lambda: (self.attention_lib(head_dim).ls_attn_tile_keys(),
                                                           self.attention_lib(head_dim).ls_attn_split_keys()))

    # -- matrix product -------------------------------------------------------
    def gemm(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, epilogue: int = STORE,
             norm_weight: torch.Tensor | None = None, eps: float = 0.0) -> None:
        """``out (+)= x @ w.T``; ``x [M,K]``, ``w [N,K]`` contiguous, ``out [M,N]``.

        ``epilogue=SWIGLU``: ``w`` holds gate and up rows interleaved in tiles of
        16 (see ``interleave_gate_up``) and ``out [M, I]`` gets ``silu(gate) * up``.
        ``norm_weight`` (float32 ``[K]``): ``x`` is the float32 residual stream and is
        RMS-normalised on the fly with this weight and ``eps`` (at most 16 rows)."""
        _rows_ok(x, "gemm x"); _rows_ok(w, "gemm w"); _rows_ok(out, "gemm out")
        if not (w.dtype in DTYPE_CODE):
            raise KernelError(f"gemm weights must be float32 or bfloat16, got {w.dtype}")
        if norm_weight is None:
            if not (x.dtype == w.dtype):
                raise KernelError(f"gemm operands must share a dtype, got {x.dtype} and {w.dtype}")
        else:
            if not (x.dtype == torch.float32 and x.shape[0] <= 16):
                raise KernelError("the fused norm reads at most 16 float32 rows")
            if not (norm_weight.is_cuda and norm_weight.dtype == torch.float32 and norm_weight.is_contiguous()
                  and norm_weight.shape == (x.shape[1],)):
                raise KernelError(f"norm weight must be float32 [{x.shape[1]}]")
        m, k = x.shape
        n = w.shape[0]
        if not (w.shape[1] == k and w.is_contiguous()):
            raise KernelError(f"gemm w must be contiguous [N,{k}], got {tuple(w.shape)}")
        if epilogue == SWIGLU:
            cols = out.shape[1]
            if not (n % 32 == 0 and n // 2 - 16 < cols <= n // 2 and out.shape[0] == m):
                raise KernelError(f"SwiGLU output [{m},{cols}] does not fit {n} interleaved weight rows")
        else:
            cols = n
            if not (tuple(out.shape) == (m, n)):
                raise KernelError(f"gemm out must be [{m},{n}], got {tuple(out.shape)}")
        want = w.dtype if epilogue in (STORE, SWIGLU) else torch.float32
        if not (out.dtype == want):
            raise KernelError(f"gemm out dtype {out.dtype} does not fit epilogue {epilogue}")
        if m == 0:
            return
        self._launch(self.core, self.core.ls_gemm, (
            c_int(DTYPE_CODE[w.dtype]), c_int(epilogue), _ptr(x), _ptr(w), _ptr(out), c_int(m), c_int(n), c_int(k),
            c_long(x.stride(0)), c_long(out.stride(0)), _ptr(norm_weight), c_float(eps), c_int(cols), _stream()))

    def gemm_slices_count(self, k: int) -> int:
        """K slices of a product over ``k`` (first dimension of ``gemm_slices``'s output)."""
        return self._memo(("slices", k), lambda: int(self.core.ls_gemm_slices_count(c_int(k))))

    def gemm_slices_max_rows(self, k: int, dtype: torch.dtype) -> int:
        """Most rows ``gemm_slices`` takes for a product over ``k``: 64, or 256 where the kernel that walks
        the column blocks with its rows in registers has an instance for the slice length."""
        return self._memo(("slices_rows", k, dtype),
                          lambda: int(self.core.ls_gemm_slices_max_rows(c_int(DTYPE_CODE[dtype]), c_int(k))))

    def gemm_slices(self, x: torch.Tensor, w: torch.Tensor, partials: torch.Tensor) -> None:
        """Slice sums of ``x @ w.T`` for at most ``gemm_slices_max_rows`` rows: ``partials [slices, M, N]``
        float32, to be added in ascending order by the consumer (``add_rmsnorm``).  The work is cut over K
        as well as over N."""
        _rows_ok(x, "gemm_slices x")
        m, k = x.shape
        n = w.shape[0]
        if not (w.is_cuda and w.dim() == 2 and w.is_contiguous() and w.shape[1] == k and w.dtype == x.dtype
              and w.dtype in DTYPE_CODE):
            raise KernelError("gemm_slices w must be [N, K] contiguous in the dtype of x")
        if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous()
              and partials.shape == (self.gemm_slices_count(k), m, n)):
            raise KernelError(f"gemm_slices partials must be float32 [{self.gemm_slices_count(k)}, {m}, {n}]")
        self._launch(self.core, self.core.ls_gemm_slices, (
            c_int(DTYPE_CODE[w.dtype]), _ptr(x), _ptr(w), _ptr(partials), c_int(m), c_int(n), c_int(k),
            c_long(x.stride(0)), _stream()))

    def gemm_slices_folded_ok(self, dtype: torch.dtype, m: int, n: int, k: int, head_dim: int, splits: int) -> bool:
        """Whether ``gemm_slices_folded`` takes a product of these sizes."""
        return self._memo(("slices_folded", dtype, m, n, k, head_dim, splits), lambda: bool(
            self.core.ls_gemm_slices_folded_ok(c_int(DTYPE_CODE[dtype]), c_int(m), c_int(n), c_int(k), c_int(head_dim),
                                               c_int(splits))))

    def gemm_slices_folded(self, part_acc: torch.Tensor, part_ml: torch.Tensor, splits: int, head_dim: int,
                           w: torch.Tensor, partials: torch.Tensor) -> None:
        """``gemm_slices`` for an operand that still lies as the per-split sums of an attention launch over
        single decoded tokens: row ``(m * heads + h) * splits + s`` of ``part_acc [., head_dim]`` and
        ``part_ml [., 2]`` holds split ``s`` of token ``m``, head ``h``.  The kernel folds them (ascending,
        from the empty state, then sum / weight rounded to the compute dtype: what the combine launch
        would write) on its way; ``partials [slices, M, N]`` gets the bits ``gemm_slices`` would leave."""
        slices, m, n = partials.shape
        k = w.shape[1]
        if not (w.is_cuda and w.dim() == 2 and w.is_contiguous() and w.dtype in DTYPE_CODE and w.shape[0] == n):
            raise KernelError("gemm_slices_folded w must be [N, K] contiguous")
        if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous()
                and slices == self.gemm_slices_count(k)):
            raise KernelError(f"gemm_slices_folded partials must be float32 [{self.gemm_slices_count(k)}, M, N]")
        if not self.gemm_slices_folded_ok(w.dtype, m, n, k, head_dim, splits):
            raise KernelError(f"gemm_slices_folded does not take M={m} N={n} K={k} head_dim={head_dim} splits={splits}")
        rows = m * (k // head_dim) * splits
        for name, t, width in (("part_acc", part_acc, head_dim), ("part_ml", part_ml, 2)):
            if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 2
                    and t.shape[1] == width and t.shape[0] >= rows):
                raise KernelError(f"gemm_slices_folded {name} must be float32 [>= {rows}, {width}]")
        self._launch(self.core, self.core.ls_gemm_slices_folded, (
            c_int(DTYPE_CODE[w.dtype]), _ptr(part_acc), _ptr(part_ml), c_int(splits), c_int(head_dim), _ptr(w),
            _ptr(partials), c_int(m), c_int(n), c_int(k), _stream()))

    def add_rmsnorm(self, h: torch.Tensor, partials: torch.Tensor, weight, out, eps: float = 0.0,
                    rows: torch.Tensor | None = None) -> None:
        """``h[row] += partials[0][row] + partials[1][row] + ...``; then, unless ``out`` is None,
        ``out = rmsnorm(h[row]) * weight`` as ``rmsnorm`` computes it.  ``rows`` selects rows of ``h``."""
        _rows_ok(h, "add_rmsnorm h")
        if not (h.dtype == torch.float32):
            raise KernelError("add_rmsnorm works on the float32 residual stream")
        if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous()
              and partials.dim() == 3 and partials.shape[2] == h.shape[1]):
            raise KernelError("add_rmsnorm partials [slices, rows, width]")
        n_rows = h.shape[0] if rows is None else rows.shape[0]
        if rows is not None:
            if not (rows.is_cuda and rows.dtype == torch.int32 and rows.is_contiguous()):
                raise KernelError("add_rmsnorm rows: int32 on the GPU")
        dtype = torch.float32
        ld_out = 0
        if out is not None:
            _rows_ok(out, "add_rmsnorm out")
            if not (out.dtype in DTYPE_CODE and out.shape == (n_rows, h.shape[1])):
                raise KernelError("add_rmsnorm out shape or dtype")
            if not (weight is not None and weight.dtype == torch.float32 and weight.is_contiguous()
                  and weight.numel() == h.shape[1]):
                raise KernelError("add_rmsnorm weight must be float32 [width]")
            dtype, ld_out = out.dtype, out.stride(0)
        if n_rows == 0:
            return
        self._launch(self.core, self.core.ls_add_rmsnorm, (
            c_int(DTYPE_CODE[dtype]), _ptr(h), _ptr(partials), c_int(partials.shape[0]), c_int(partials.shape[1]),
            _ptr(weight), _ptr(out), _ptr(rows), c_int(n_rows), c_int(h.shape[1]), c_long(h.stride(0)),
            c_long(ld_out), c_float(eps), _stream()))

    # -- rows -------------------------------------------------------------------
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0, copies: int = 1) -> None:
        """``out[t] = table[tokens[t]] * scale`` as float32 rows, ``copies`` times side by side."""
        if not (tokens.is_cuda and tokens.dtype == torch.int32 and tokens.dim() == 1 and tokens.is_contiguous()):
            raise KernelError("embed tokens must be a contiguous int32 vector on the GPU")
        _rows_ok(table, "embed table"); _rows_ok(out, "embed out")
        if not (table.is_contiguous() and table.dtype in DTYPE_CODE):
            raise KernelError("embed table must be contiguous float32/bfloat16")
        if not (copies >= 1 and out.dtype == torch.float32 and out.shape == (tokens.shape[0], copies * table.shape[1])):
            raise KernelError(f"embed out must be float32 [{tokens.shape[0]},{copies * table.shape[1]}]")
        if tokens.shape[0] == 0:
            return
        self._launch(self.core, self.core.ls_embed, (
            c_int(DTYPE_CODE[table.dtype]), _ptr(tokens), _ptr(table), _ptr(out), c_int(tokens.shape[0]),
            c_int(table.shape[0]), c_int(table.shape[1]), c_long(out.stride(0)), c_float(scale), c_int(copies), _stream()))

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, eps: float,
                rows: torch.Tensor | None = None) -> None:
        """Rows of float ``x`` (all, or those listed in ``rows``) normalised into ``out``."""
        _rows_ok(x, "rmsnorm x"); _rows_ok(out, "rmsnorm out")
        if not (x.dtype == torch.float32):
            raise KernelError("rmsnorm reads the float32 residual stream")
        if not (weight.is_cuda and weight.dtype == torch.float32 and weight.is_contiguous()
              and weight.shape == (x.shape[1],)):
            raise KernelError(f"rmsnorm weight must be float32 [{x.shape[1]}]")
        if not (out.dtype in DTYPE_CODE and out.shape[1] == x.shape[1]):
            raise KernelError("rmsnorm out has the wrong width or dtype")
        n = out.shape[0]
        if rows is not None:
            if not (rows.is_cuda and rows.dtype == torch.int32 and rows.is_contiguous() and rows.shape == (n,)):
                raise KernelError(f"rmsnorm rows must be int32 [{n}]")
        else:
            if not (x.shape[0] == n):
                raise KernelError("rmsnorm out must have as many rows as x")
        if n == 0:
            return
        self._launch(self.core, self.core.ls_rmsnorm, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(x), _ptr(weight), _ptr(out), _ptr(rows), c_int(n), c_int(x.shape[1]),
            c_long(x.stride(0)), c_long(out.stride(0)), c_float(eps), _stream()))

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> None:
        _rows_ok(gate_up, "swiglu input"); _rows_ok(out, "swiglu out")
        rows, inter = out.shape
        if not (gate_up.shape == (rows, 2 * inter) and gate_up.dtype == out.dtype and out.dtype in DTYPE_CODE):
            raise KernelError(f"swiglu input must be [{rows},{2 * inter}] of the output's dtype")
        if rows == 0:
            return
        self._launch(self.core, self.core.ls_swiglu, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(gate_up), _ptr(out), c_int(rows), c_int(inter),
            c_long(gate_up.stride(0)), c_long(out.stride(0)), _stream()))

    ACTIVATIONS = {"none": 0, "silu": 1, "gelu_tanh": 2, "gelu": 3, "relu": 4}

    def bias_act(self, x: torch.Tensor, bias, out: torch.Tensor, activation: str = "none", gated: bool = False) -> None:
        """``out = act(x + bias)`` on float32 rows ``x``; gated: ``x`` holds gates then ups and
        ``out = act(gate + bias_gate) * (up + bias_up)``.  ``bias`` float32 or None; ``out`` float32
        or bfloat16, and may be ``x`` itself when not gated."""
        _rows_ok(x, "bias_act x"); _rows_ok(out, "bias_act out")
        if activation not in self.ACTIVATIONS:
            raise KernelError(f"activation {activation!r} is not built; known: {', '.join(self.ACTIVATIONS)}")
        rows, width = out.shape
        if not (x.dtype == torch.float32 and x.shape == (rows, 2 * width if gated else width) and out.dtype in DTYPE_CODE):
            raise KernelError(f"bias_act reads float32 [{rows},{2 * width if gated else width}], got {tuple(x.shape)} {x.dtype}")
        if bias is not None:
            if not (bias.is_cuda and bias.dtype == torch.float32 and bias.is_contiguous() and bias.shape == (x.shape[1],)):
                raise KernelError(f"bias_act bias must be float32 [{x.shape[1]}]")
        if gated and x.data_ptr() == out.data_ptr():
            raise KernelError("a gated bias_act cannot work in place")
        if rows == 0:
            return
        self._launch(self.core, self.core.ls_bias_act, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(x), c_long(x.stride(0)), _ptr(bias), _ptr(out), c_long(out.stride(0)),
            c_int(rows), c_int(width), c_int(self.ACTIVATIONS[activation]), c_int(1 if gated else 0), _stream()))

    #: (row, chunk) pairs the library's static arg-max scratch holds (LS_ARGMAX_STATIC_PAIRS)
    ARGMAX_STATIC_PAIRS = 16384

    def argmax(self, logits: torch.Tensor, out: torch.Tensor) -> None:
        """Lowest index among the maxima of every float32 row.  Calls that fit the library's static
        scratch array go through the entry point that allocates nothing: that array never moves, so
        a captured graph that contains the launch stays valid whatever runs in between.  Larger
        calls bring a scratch buffer; a buffer that was outgrown is kept until the process ends,
        because a captured graph may still write into it.

        The static array is one per GPU and process: calls that overlap on one GPU (two streams, two
        engines in one process that do not order their work) race on it.  This engine launches
        everything on one stream, which orders them."""
        _rows_ok(logits, "argmax logits")
        if not (logits.dtype == torch.float32):
            raise KernelError("argmax reads float32 logits")
        if not (out.is_cuda and out.dtype == torch.int32 and out.is_contiguous() and out.shape == (logits.shape[0],)):
            raise KernelError(f"argmax out must be int32 [{logits.shape[0]}]")
        if logits.shape[0] == 0:
            return
        pairs = logits.shape[0] * self.core.ls_argmax_chunks(c_int(logits.shape[1]))
        if pairs <= self.ARGMAX_STATIC_PAIRS:
            self._launch(self.core, self.core.ls_argmax_static, (
                _ptr(logits), _ptr(out), c_int(logits.shape[0]), c_int(logits.shape[1]), c_long(logits.stride(0)),
                _stream()))
            return
        held = self._argmax_scratch.setdefault(logits.device, [])
        if not held or held[-1].numel() < 2 * pairs:
            held.append(torch.empty(max(2 * pairs, 2 * held[-1].numel() if held else 0), dtype=torch.int32,
                                    device=logits.device))
        scratch = held[-1]
        self._launch(self.core, self.core.ls_argmax, (
            _ptr(logits), _ptr(out), c_int(logits.shape[0]), c_int(logits.shape[1]), c_long(logits.stride(0)),
            _ptr(scratch), c_long(scratch.numel()), _stream()))

    #: one row's request as ``sample_top_p`` takes it (eight 4-byte words; csrc/sample.hip: SampleRow)
    SAMPLE_ROW = [("row", "<i4"), ("temperature", "<f4"), ("top_p", "<f8"), ("key0", "<u4"), ("key1", "<u4"),
                  ("pos_lo", "<u4"), ("pos_hi", "<u4")]
    SAMPLE_ROW_INTS = 8
    SAMPLE_POSITION_AT = 6          # the word of a record that holds the low half of the position

    @classmethod
    def pack_sample_requests(cls, requests, rows: int):
        """``requests``: (row of the logits, temperature > 0, top_p, seed XOR k(uid) as an int of 64 bits,
        position) each; the records as int32 words, eight a request."""
        import numpy as np

        packed = np.zeros(len(requests), dtype=cls.SAMPLE_ROW)
        for i, (row, temperature, top_p, mixed, position) in enumerate(requests):
            if not (0 <= row < rows and temperature > 0):
                raise KernelError(f"sample: row {row} of {rows} at temperature {temperature}")
            packed[i] = (row, temperature, top_p, mixed & 0xFFFFFFFF, (mixed >> 32) & 0xFFFFFFFF,
                         position & 0xFFFFFFFF, (position >> 32) & 0xFFFFFFFF)
        return packed.view(np.int32)

    def sample_top_p(self, logits: torch.Tensor, requests, out: torch.Tensor, records: torch.Tensor | None = None,
                     any_nucleus: bool | None = None, scatter: bool = False) -> None:
        """One token for each request: ``requests`` is a sequence of (row of the float32 ``logits``,
        temperature > 0, top_p, seed XOR k(uid) as an int of 64 bits, position); ``out`` int32 on the GPU
        gets request i's token at ``out[i]`` (with ``scatter`` at ``out[row]``).  Or ``records``: the same
        packed by ``pack_sample_requests`` and already on the GPU (int32, eight words a request), with
        ``any_nucleus`` saying whether any top_p is below one.  The host sampler's procedure in float64
        (sampling/sampler.py) without its sort, the draw included (Philox-4x32-10 keyed as
        sampling/philox.py keys it)."""
        _rows_ok(logits, "sample logits")
        if not (logits.dtype == torch.float32):
            raise KernelError("sample reads float32 logits")
        if records is None:
            n = len(requests)
            if n == 0:
                return
            records = torch.from_numpy(self.pack_sample_requests(requests, logits.shape[0])).to(logits.device)
            any_nucleus = any(top_p < 1.0 for _, _, top_p, _, _ in requests)
        else:
            if not (records.is_cuda and records.dtype == torch.int32 and records.is_contiguous()
                    and records.numel() % self.SAMPLE_ROW_INTS == 0 and any_nucleus is not None):
                raise KernelError("sample records: contiguous int32 on the GPU, eight words a request, and any_nucleus")
            n = records.numel() // self.SAMPLE_ROW_INTS
            if n == 0:
                return
        if not (out.is_cuda and out.dtype == torch.int32 and out.is_contiguous()
                and out.numel() >= (logits.shape[0] if scatter else n)):
            raise KernelError("sample out must be int32 on the GPU, one for every request (with scatter: every row)")
        vocab = logits.shape[1]
        need = int(self.core.ls_sample_scratch_bytes(c_int(n), c_int(vocab)))
        scratch = self._sample_scratch.get(logits.device)
        if scratch is None or scratch.numel() < need:
            # (a buffer that was outgrown is kept: a captured graph may still write into it)
            scratch = torch.empty(need, dtype=torch.uint8, device=logits.device)
            self._sample_scratch_kept.append(self._sample_scratch.get(logits.device))
            self._sample_scratch[logits.device] = scratch
        self._launch(self.core, self.core.ls_sample_top_p, (
            _ptr(logits), c_long(logits.stride(0)), _ptr(records), _ptr(out), _ptr(scratch), c_long(scratch.numel()),
            c_int(n), c_int(vocab), c_int(1 if any_nucleus else 0), c_int(1 if scatter else 0), _stream()))

    def advance_decode(self, meta: torch.Tensor, n_seqs: int, off_tokens: int, picked: torch.Tensor,
                       ring: torch.Tensor, counter: torch.Tensor, off_runs: int, n_runs: int) -> None:
        """Between two decode steps that run without the host: the picked tokens become the next
        inputs inside the uploaded metadata ``meta``, every value named by the ``n_runs`` runs
        (first, stride, count) of the table at ``meta[off_runs]`` moves on by one, and the tokens
        are appended to ``ring[counter]``.  The step's upload builds the table and checks it."""
        for t in (meta, picked, ring, counter):
            if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()):
                raise KernelError("advance_decode works on int32 GPU tensors")
        if not (picked.numel() >= n_seqs):
            raise KernelError("advance_decode: picked is too short")
        self._launch(self.core, self.core.ls_advance_decode, (
            _ptr(meta), c_long(meta.numel()), c_int(n_seqs), c_int(off_tokens), _ptr(picked), _ptr(ring),
            _ptr(counter), c_int(off_runs), c_int(n_runs), _stream()))

    # -- attention ----------------------------------------------------------------
    def qk_rope_kv(self, qkv: torch.Tensor, n_tokens: int, nq: int, nkv: int, d: int, q_weight, k_weight,
                   eps: float, cos, sin, rot: int, tok_seq, tok_pos, seqs, max_pos: int, table, k_pages,
                   v_pages, page_size: int, write_kv: bool) -> None:
        """Per-head norm, rotation and cache write on the fused projection ``qkv``.

        ``max_pos`` is the largest position in the step (checked against the
        tables); ``table`` is the group's block table ``[rows, stride]``.
        """
        _rows_ok(qkv, "qkv")
        if not (qkv.dtype in DTYPE_CODE and qkv.shape[0] >= n_tokens):
            raise KernelError("qkv has too few rows or a wrong dtype")
        heads = nq + 2 * nkv if write_kv else nq
        if not (qkv.shape[1] >= heads * d):
            raise KernelError(f"qkv rows hold {qkv.shape[1]} values, {heads} heads of {d} are needed")
        if not (d <= MAX_HEAD_DIM):
            raise KernelError(f"head size {d} exceeds the supported maximum {MAX_HEAD_DIM}")
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                if not (w.is_cuda and w.dtype == torch.float32 and w.is_contiguous() and w.shape == (d,)):
                    raise KernelError(f"{name} must be float32 [{d}]")
        positions = 0
        if cos is not None:
            if not (sin is not None and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == rot
                  and cos.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous() and cos.is_cuda):
                raise KernelError("rotation tables must be float32 [positions, rotary_dim/2]")
            positions = cos.shape[0]
            if not (max_pos < positions):
                raise KernelError(f"position {max_pos} is beyond the rotation tables ({positions})")
        for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n_tokens):
                raise KernelError(f"{name} must be int32 with at least {n_tokens} entries")
        if write_kv:
            if not (table is not None and table.is_cuda and table.dtype == torch.int32 and table.dim() == 2
                  and table.is_contiguous()):
                raise KernelError("block table must be a contiguous int32 matrix")
            if not (max_pos // page_size < table.shape[1]):
                raise KernelError(f"position {max_pos} needs page {max_pos // page_size}, the block table has {table.shape[1]} columns")
            for name, pages in (("key pages", k_pages), ("value pages", v_pages)):
                if not (pages.is_cuda and pages.dtype == qkv.dtype and pages.is_contiguous() and pages.dim() == 4):
                    raise KernelError(f"{name} must be contiguous 4-D of the compute dtype")
            if not (k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape[1:] == (nkv, d, page_size)
                  and k_pages.shape[0] == v_pages.shape[0]):
                raise KernelError(f"cache pages do not have the layout [pages,{nkv},{page_size},{d}] / [pages,{nkv},{d},{page_size}]")
        if n_tokens == 0:
            return
        self._launch(self.core, self.core.ls_qk_rope_kv, (
            c_int(DTYPE_CODE[qkv.dtype]), _ptr(qkv), c_long(qkv.stride(0)), c_int(n_tokens), c_int(nq), c_int(nkv),
            c_int(d), _ptr(q_weight), _ptr(k_weight), c_float(eps), _ptr(cos), _ptr(sin), c_int(rot),
            c_int(positions), _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs), _ptr(table), c_int(table.shape[1] if table
            is not None else 0), _ptr(k_pages), _ptr(v_pages), c_int(page_size), c_int(1 if write_kv else 0),
            _stream()))

    def attention(self, q: torch.Tensor, nq: int, nkv: int, d: int, k_pages, v_pages, page_size: int, table,
                  seqs, items, n_items: int, out: torch.Tensor, part_acc, part_ml, scale: float,
                  window: int, variant: int = 0, max_rows: int = 0, spans: bool = False,
                  single_tile: bool = False) -> None:
        """Launch the attention kernel over ``n_items`` work items (see attention.hip).
        ``variant``: 0 staged through LDS where it fits, 1 direct from global memory, 2 staged or
        error, 3 cooperative (every item has at most 16 rows; ``max_rows`` states the largest),
        4 wide (prompt portions; items count row blocks of ``attention_block_rows``), 5 the same
        with half the rows a block (for steps with few rows).  ``spans`` (cooperative only): items
        that leave partial results may hold several splits each.  ``single_tile`` (cooperative only): every
        item holds one key tile (a hint: such a launch needs one tile buffer a workgroup, not two)."""
        lib = self.attention_lib(d)
        _rows_ok(q, "attention q"); _rows_ok(out, "attention out")
        if not (q.dtype in DTYPE_CODE and out.dtype == q.dtype):
            raise KernelError("attention q/out dtype")
        if not (nq % nkv == 0):
            raise KernelError(f"{nq} query heads are not a multiple of {nkv} kv heads")
        if not (q.shape[1] >= nq * d and out.shape[1] >= nq * d):
            raise KernelError("attention q/out rows are too short")
        if not (k_pages.dtype == q.dtype and v_pages.dtype == q.dtype and k_pages.is_contiguous()
              and v_pages.is_contiguous() and k_pages.shape[1:] == (nkv, page_size, d)
              and v_pages.shape[1:] == (nkv, d, page_size)):
            raise KernelError("attention cache pages have the wrong layout or dtype")
        if not (table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous()):
            raise KernelError("attention block table")
        if not (items.dtype == torch.int32 and items.is_contiguous() and items.numel() >= ATTENTION_ITEM_INTS * n_items):
            raise KernelError("attention items must hold 32 int32 each (see pack_attention_items)")
        if n_items == 0:
            return
        self._launch(lib, lib.ls_attention, (
            c_int(DTYPE_CODE[q.dtype]), _ptr(q), c_long(q.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(nkv),
            c_int(page_size), _ptr(table), c_int(table.shape[1]), _ptr(seqs), _ptr(items), c_int(n_items),
            _ptr(out), c_long(out.stride(0)), _ptr(part_acc), _ptr(part_ml), c_int(nq // nkv), c_float(scale),
            c_int(window), c_int(variant), c_int(max_rows), c_int((1 if spans else 0) | (2 if single_tile else 0)),
            _stream()))

    def attention_decode(self, qkv: torch.Tensor, nq: int, nkv: int, d: int, k_pages, v_pages, page_size: int,
                         table, seqs, items, n_items: int, out: torch.Tensor, part_acc, part_ml, scale: float,
                         window: int, q_weight, k_weight, eps: float, cos, sin, rot: int, max_pos: int,
                         write_kv: bool, spans: bool = False, single_tile: bool = False) -> None:
        """A step of single decoded tokens: what ``qk_rope_kv`` and ``attention`` (cooperative items) do,
        in one launch.  ``qkv`` is the raw fused projection; every request brings exactly one token."""
        lib = self.attention_lib(d)
        _rows_ok(qkv, "attention_decode qkv"); _rows_ok(out, "attention_decode out")
        if not (qkv.dtype in DTYPE_CODE and out.dtype == qkv.dtype):
            raise KernelError("attention_decode qkv/out dtype")
        if not (nq % nkv == 0):
            raise KernelError(f"{nq} query heads are not a multiple of {nkv} kv heads")
        heads = nq + 2 * nkv if write_kv else nq
        if not (qkv.shape[1] >= heads * d and out.shape[1] >= nq * d):
            raise KernelError("attention_decode rows are too short")
        if not (k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype and k_pages.is_contiguous()
              and v_pages.is_contiguous() and k_pages.shape[1:] == (nkv, page_size, d)
              and v_pages.shape[1:] == (nkv, d, page_size)):
            raise KernelError("attention cache pages have the wrong layout or dtype")
        if not (table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous()):
            raise KernelError("attention block table")
        if not (items.dtype == torch.int32 and items.is_contiguous() and items.numel() >= ATTENTION_ITEM_INTS * n_items):
            raise KernelError("attention items must hold 32 int32 each (see pack_attention_items)")
        for w in (q_weight, k_weight):
            if not (w is None or (w.dtype == torch.float32 and w.is_contiguous() and w.numel() == d)):
                raise KernelError("per-head norm weights must be float32 [head_dim]")
        positions = 0
        if cos is not None:
            if not (sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
                  and cos.is_contiguous() and sin.is_contiguous() and cos.shape == sin.shape
                  and cos.shape[1] == rot // 2):
                raise KernelError("rotation tables must be float32 [positions, rot/2]")
            positions = cos.shape[0]
        if n_items == 0:
            return
        self._launch(lib, lib.ls_attention_decode, (
            c_int(DTYPE_CODE[qkv.dtype]), _ptr(qkv), c_long(qkv.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(nq),
            c_int(nkv), c_int(page_size), _ptr(table), c_int(table.shape[1]), _ptr(seqs), _ptr(items),
            c_int(n_items), _ptr(out), c_long(out.stride(0)), _ptr(part_acc), _ptr(part_ml), c_float(scale),
            c_int(window), _ptr(q_weight), _ptr(k_weight), c_float(eps), _ptr(cos), _ptr(sin), c_int(rot),
            c_int(positions), c_int(max_pos), c_int(1 if write_kv else 0),
            c_int((1 if spans else 0) | (2 if single_tile else 0)), _stream()))

    def attention_combine(self, d: int, seqs, items, n_items: int, nq: int, nkv: int, part_acc, part_ml,
                          out: torch.Tensor, max_rows: int = 0) -> None:
        """Fold the splits' partial results of the requests in ``items`` into ``out``.  ``max_rows``: the
        most rows (tokens times query heads a kv head) a request of an item brings, 0 if unknown; with
        at most 16 the fold that asks for many splits at a time is taken (same bits)."""
        lib = self.attention_lib(d)
        _rows_ok(out, "combine out")
        if not (out.dtype in DTYPE_CODE and out.shape[1] >= nq * d):
            raise KernelError("combine out rows are too short")
        if not (items.dtype == torch.int32 and items.is_contiguous() and items.numel() >= COMBINE_ITEM_INTS * n_items):
            raise KernelError("combine items must hold 8 int32 each (see pack_combine_items)")
        if n_items == 0:
            return
        self._launch(lib, lib.ls_attention_combine, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(seqs), _ptr(items), c_int(n_items), c_int(nkv), _ptr(part_acc),
            _ptr(part_ml), _ptr(out), c_long(out.stride(0)), c_int(nq // nkv), c_int(max_rows), _stream()))

    # -- mixers beyond softmax attention: norms, gated units, recurrences ----------------
    def mixers_lib(self):
        """The library of csrc/mixers.hip, built and loaded when a part first asks for it."""
        if self._mixers is None:
            self.mixers_path = _build.build_mixers()
            lib = ctypes.CDLL(str(self.mixers_path))
            lib.ls_last_error.restype = ctypes.c_char_p
            self._mixers = lib
        return self._mixers

    def talking_lib(self, heads: int, kv_heads: int, dim: int, vdim: int):
        """The talking-heads attention library of one shape."""
        shape = (heads, kv_heads, dim, vdim)
        lib = self._talking.get(shape)
        if lib is None:
            path = _build.build_talking(*shape)
            lib = ctypes.CDLL(str(path))
            lib.ls_last_error.restype = ctypes.c_char_p
            if (lib.ls_talk_heads(), lib.ls_talk_kv_heads(), lib.ls_talk_dim(), lib.ls_talk_vdim()) != shape:
                raise KernelError(f"{path} was built for another shape")
            self._talking[shape] = lib
            self.talking_paths[shape] = str(path)
        return lib

    @staticmethod
    def _f32_vector(t, n: int, name: str) -> None:
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n):
            raise KernelError(f"{name} must be float32 with {n} elements on the GPU")

    def dyt(self, h: torch.Tensor, weight, bias, alpha, out, rows: torch.Tensor | None = None,
            partials: torch.Tensor | None = None) -> None:
        """Dynamic Tanh norm: ``out = tanh(alpha * h[row]) * weight + bias`` on rows of the float32 stream
        ``h`` (all, or those listed in ``rows``); with ``partials [slices, rows, width]`` these are added
        to ``h`` first, in ascending order.  ``out`` None: the addition only."""
        _rows_ok(h, "dyt h")
        if not (h.dtype == torch.float32):
            raise KernelError("dyt reads the float32 residual stream")
        width = h.shape[1]
        n_rows = h.shape[0] if rows is None else rows.shape[0]
        if rows is not None and not (rows.is_cuda and rows.dtype == torch.int32 and rows.is_contiguous()):
            raise KernelError("dyt rows: int32 on the GPU")
        slices = p_rows = 0
        if partials is not None:
            if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous()
                    and partials.dim() == 3 and partials.shape[2] == width and partials.shape[1] >= (h.shape[0] if rows is None else 1)):
                raise KernelError("dyt partials [slices, rows, width] float32")
            slices, p_rows = partials.shape[0], partials.shape[1]
        dtype, ld_out = torch.float32, 0
        if out is not None:
            _rows_ok(out, "dyt out")
            if not (out.dtype in DTYPE_CODE and out.shape == (n_rows, width)):
                raise KernelError(f"dyt out must be [{n_rows},{width}]")
            self._f32_vector(weight, width, "dyt weight"); self._f32_vector(bias, width, "dyt bias")
            self._f32_vector(alpha, 1, "dyt alpha")
            dtype, ld_out = out.dtype, out.stride(0)
        if n_rows == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_dyt, (
            c_int(DTYPE_CODE[dtype]), _ptr(h), _ptr(partials), c_int(slices), c_int(p_rows), _ptr(weight), _ptr(bias),
            _ptr(alpha), _ptr(out), _ptr(rows), c_int(n_rows), c_int(width), c_long(h.stride(0)), c_long(ld_out),
            _stream()))

    def glu_clamped(self, x: torch.Tensor, out: torch.Tensor, limit: float, alpha: float) -> None:
        """``out = g * sigmoid(alpha * g) * (u + 1)`` with ``g = min(gate, limit)``, ``u = clamp(up, -limit,
        limit)``; ``x`` float32 ``[rows, 2 * width]`` holds the gates, then the ups."""
        _rows_ok(x, "glu_clamped x"); _rows_ok(out, "glu_clamped out")
        rows, width = out.shape
        if not (x.dtype == torch.float32 and x.shape == (rows, 2 * width) and out.dtype in DTYPE_CODE):
            raise KernelError(f"glu_clamped reads float32 [{rows},{2 * width}]")
        if rows == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_glu_clamped, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(x), c_long(x.stride(0)), _ptr(out), c_long(out.stride(0)), c_int(rows),
            c_int(width), c_float(limit), c_float(alpha), _stream()))

    def softcap(self, x: torch.Tensor, cap: float) -> None:
        """``x = cap * tanh(x / cap)`` in place on float32 rows."""
        _rows_ok(x, "softcap x")
        if not (x.dtype == torch.float32 and cap > 0):
            raise KernelError("softcap works on float32 rows with a positive cap")
        if x.shape[0] == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_softcap, (_ptr(x), c_long(x.stride(0)), c_int(x.shape[0]), c_int(x.shape[1]),
                                           c_float(cap), _stream()))

    @staticmethod
    def _rotation_tables(cos, sin, rot: int, max_pos: int) -> int:
        if rot == 0:
            return 0
        if not (cos is not None and sin is not None and cos.shape == sin.shape and cos.dim() == 2
                and cos.shape[1] * 2 == rot and cos.dtype == torch.float32 and sin.dtype == torch.float32
                and cos.is_contiguous() and sin.is_contiguous() and cos.is_cuda):
            raise KernelError("rotation tables must be float32 [positions, rotary_dim/2]")
        if not (max_pos < cos.shape[0]):
            raise KernelError(f"position {max_pos} is beyond the rotation tables ({cos.shape[0]})")
        return cos.shape[0]

    def _paged_ok(self, k_pages, v_pages, table, dtype, kv_heads: int, page_size: int, dim: int, vdim: int) -> None:
        if not (k_pages.dtype == dtype and v_pages.dtype == dtype and k_pages.is_contiguous() and v_pages.is_contiguous()
                and k_pages.dim() == 4 and k_pages.shape[1:] == (kv_heads, page_size, dim)
                and v_pages.shape[1:] == (kv_heads, vdim, page_size) and k_pages.shape[0] == v_pages.shape[0]):
            raise KernelError(f"cache pages do not have the layout [pages,{kv_heads},{page_size},{dim}] / "
                              f"[pages,{kv_heads},{vdim},{page_size}] of the compute dtype")
        if not (table.is_cuda and table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous()):
            raise KernelError("block table must be a contiguous int32 matrix")

    def talk_qkv(self, raw: torch.Tensor, n_tokens: int, heads: int, kv_heads: int, dim: int, vdim: int, bias, cos, sin,
                 rot: int, max_pos: int, tok_seq, tok_pos, seqs, table, q_out: torch.Tensor, k_pages, v_pages,
                 page_size: int, vmix_mode: int = 0, vmix=None, v_first=None) -> None:
        """Post pass of the fused projection ``raw`` (float32 ``[T, heads*dim + kv_heads*dim + kv_heads*vdim]``):
        biases, rotation of queries and keys, value mixing (1: keep the values in ``v_first``; 2: mix
        ``v_first`` in with the weight ``vmix``), queries to ``q_out``, keys and values to their pages."""
        _rows_ok(raw, "talk_qkv raw"); _rows_ok(q_out, "talk_qkv q_out")
        width = heads * dim + kv_heads * (dim + vdim)
        if not (raw.dtype == torch.float32 and raw.shape[0] >= n_tokens and raw.shape[1] == width):
            raise KernelError(f"talk_qkv raw must be float32 [>= {n_tokens}, {width}]")
        if not (q_out.dtype in DTYPE_CODE and q_out.shape[0] >= n_tokens and q_out.shape[1] == heads * dim):
            raise KernelError("talk_qkv q_out has the wrong shape or dtype")
        if bias is not None:
            self._f32_vector(bias, width, "talk_qkv bias")
        positions = self._rotation_tables(cos, sin, rot, max_pos)
        self._paged_ok(k_pages, v_pages, table, q_out.dtype, kv_heads, page_size, dim, vdim)
        if not (max_pos // page_size < table.shape[1]):
            raise KernelError(f"position {max_pos} needs page {max_pos // page_size}, the block table has {table.shape[1]} columns")
        for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n_tokens):
                raise KernelError(f"{name} must be int32 with at least {n_tokens} entries")
        ldv = 0
        if vmix_mode:
            if not (v_first is not None and v_first.is_cuda and v_first.dtype == torch.float32 and v_first.dim() == 2
                    and v_first.stride(1) == 1 and v_first.shape[0] >= n_tokens and v_first.shape[1] == kv_heads * vdim):
                raise KernelError(f"talk_qkv v_first must be float32 [>= {n_tokens}, {kv_heads * vdim}]")
            ldv = v_first.stride(0)
            if vmix_mode == 2:
                self._f32_vector(vmix, 1, "talk_qkv vmix")
        if n_tokens == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_talk_qkv, (
            c_int(DTYPE_CODE[q_out.dtype]), _ptr(raw), c_long(raw.stride(0)), c_int(n_tokens), c_int(heads),
            c_int(kv_heads), c_int(dim), c_int(vdim), _ptr(bias), _ptr(cos), _ptr(sin), c_int(rot), c_int(positions),
            c_int(max_pos), _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs), _ptr(table), c_int(table.shape[1]), _ptr(q_out),
            c_long(q_out.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(page_size), c_int(vmix_mode), _ptr(vmix),
            _ptr(v_first), c_long(ldv), _stream()))

    def talk_attention(self, q: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, k_pages, v_pages,
                       page_size: int, table, seqs, blocks: torch.Tensor, n_blocks: int, talk: torch.Tensor,
                       scale: float, window: int, keep_first: int, out: torch.Tensor, folds: torch.Tensor | None = None,
                       n_folds: int = 0, part: torch.Tensor | None = None, part_rows: int = 16,
                       mix_weights: bool = False, sink=None, stats: torch.Tensor | None = None, gate=None) -> None:
        """Talking-heads attention of the step's queries ``q [T, heads*dim]`` over the paged cache; ``blocks``
        lists ``n_blocks`` work items of four ints (request of the step, block of 16 of its rows, run, runs);
        ``talk [heads, heads]``.  A row block whose visible keys are dealt to several work items (runs > 1) has a
        fold item of four ints in ``folds`` (first work item, runs, first packed row, rows); their results wait in
        ``part`` (float32, ``n_blocks * part_rows * heads * (vdim + 2)`` elements; ``part_rows`` 16, or 1 for a step
        of single decoded tokens) until a second launch has folded them.  ``mix_weights``: the heads' weights are
        mixed after each head's own softmax instead of their scores before it (``stats``: float32 scratch of
        ``n_blocks * 16 * heads * 2`` elements), with ``sink [heads]`` (float32 or None) in every head's denominator
        and ``gate`` (float32 rows of ``heads*vdim`` logits or None) whose sigmoid multiplies the output."""
        lib = self.talking_lib(heads, kv_heads, dim, vdim)
        _rows_ok(q, "talk_attention q"); _rows_ok(out, "talk_attention out")
        if not (q.dtype in DTYPE_CODE and out.dtype == q.dtype and q.shape[1] == heads * dim
                and out.shape[1] == heads * vdim and out.shape[0] == q.shape[0]):
            raise KernelError("talk_attention q / out have the wrong shape or dtype")
        self._paged_ok(k_pages, v_pages, table, q.dtype, kv_heads, page_size, dim, vdim)
        if not (blocks.is_cuda and blocks.dtype == torch.int32 and blocks.is_contiguous() and blocks.numel() >= 4 * n_blocks):
            raise KernelError("talk_attention work items must hold four int32 each")
        if n_folds:
            if not (folds is not None and folds.is_cuda and folds.dtype == torch.int32 and folds.is_contiguous()
                    and folds.numel() >= 4 * n_folds and part_rows in (1, 16)
                    and part is not None and part.is_cuda and part.dtype == torch.float32 and part.is_contiguous()
                    and part.numel() >= n_blocks * part_rows * heads * (vdim + 2)):
                raise KernelError("talk_attention folds: four int32 each, and room for every work item's partial result")
        self._f32_vector(talk, heads * heads, "talk_attention talk")
        if not (window > 0 and keep_first >= 0):
            raise KernelError(f"talk_attention window {window} / kept first tokens {keep_first}")
        ldg = 0
        if mix_weights:
            if not (stats is not None and stats.is_cuda and stats.dtype == torch.float32 and stats.is_contiguous()
                    and stats.numel() >= n_blocks * 16 * heads * 2):
                raise KernelError("talk_attention stats: float32 with 32 * heads elements a work item")
            if sink is not None:
                self._f32_vector(sink, heads, "talk_attention sink")
            if gate is not None:
                _rows_ok(gate, "talk_attention gate")
                if not (gate.dtype == torch.float32 and gate.shape[0] >= q.shape[0] and gate.shape[1] == heads * vdim):
                    raise KernelError(f"talk_attention gate must be float32 [>= {q.shape[0]}, {heads * vdim}]")
                ldg = gate.stride(0)
        elif sink is not None or gate is not None:
            raise KernelError("talk_attention: a sink and a gate come with mixed weights only")
        if n_blocks == 0:
            return
        self._launch(lib, lib.ls_talk_attention, (
            c_int(DTYPE_CODE[q.dtype]), _ptr(q), c_long(q.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(page_size),
            _ptr(table), c_int(table.shape[1]), _ptr(seqs), _ptr(blocks), c_int(n_blocks), _ptr(talk), c_float(scale),
            c_int(window), c_int(keep_first), _ptr(out), c_long(out.stride(0)), _ptr(folds), c_int(n_folds), _ptr(part),
            c_int(part_rows), c_int(int(bool(mix_weights))), _ptr(sink), _ptr(stats), _ptr(gate), c_long(ldg), _stream()))

    LINREC_HGRN2, LINREC_RETENTION = 0, 1

    def linrec_max_dim(self) -> int:
        return self._memo(("linrec_max_dim",), lambda: int(self.mixers_lib().ls_linrec_max_dim()))

    def linrec_gate_floats(self, n_tokens: int, heads: int, dim: int) -> int:
        """Floats of the scratch buffer ``linrec`` needs for a step of ``n_tokens`` tokens."""
        lib = self.mixers_lib()
        lib.ls_linrec_gate_floats.restype = ctypes.c_long
        return int(lib.ls_linrec_gate_floats(c_int(n_tokens), c_int(heads), c_int(dim)))

    def linrec(self, mode: int, raw: torch.Tensor, q_at: int, ab_at: int, v_at: int, heads: int, dim: int, vdim: int,
               p0, p1, cos, sin, rot: int, max_pos: int, tok_pos, seqs, n_seqs: int, state: torch.Tensor,
               gates: torch.Tensor, out: torch.Tensor) -> None:
        """The linear recurrence ``S_t = diag(a_t) S_(t-1) + b_t v_t^T``, ``o_t = S_t^T q_t`` over the tokens of
        every request of the step; ``raw`` float32 holds the projections (q at column ``q_at``, the gate or key
        projection at ``ab_at``, v at ``v_at``), ``state`` float32 ``[slots, heads, dim, vdim]`` is read and
        left for the next step, ``out`` float32 ``[T, heads*vdim]`` gets ``o_t``.  Mode ``LINREC_HGRN2``:
        ``p0`` lower bounds ``[heads*dim]``, ``p1`` the gate's bias or None; ``LINREC_RETENTION``: ``p0`` the
        heads' decays, rotation tables for q and k at the positions ``tok_pos``.  ``gates``: float32 scratch of
        ``linrec_gate_floats`` elements (q, decay and write gate of every token, computed once a step)."""
        _rows_ok(raw, "linrec raw"); _rows_ok(out, "linrec out")
        if not (raw.dtype == torch.float32 and out.dtype == torch.float32 and out.shape[1] == heads * vdim
                and out.shape[0] == raw.shape[0]):
            raise KernelError("linrec reads and writes float32 rows, out [T, heads*vdim]")
        if not (0 <= q_at and q_at + heads * dim <= raw.shape[1] and 0 <= ab_at and ab_at + heads * dim <= raw.shape[1]
                and 0 <= v_at and v_at + heads * vdim <= raw.shape[1]):
            raise KernelError("linrec: the projections do not fit the rows of raw")
        if not (dim <= self.linrec_max_dim()):
            raise KernelError(f"linrec takes states of at most {self.linrec_max_dim()} rows, got {dim}")
        if not (state.is_cuda and state.dtype == torch.float32 and state.is_contiguous()
                and tuple(state.shape[1:]) == (heads, dim, vdim)):
            raise KernelError(f"linrec state must be float32 [slots,{heads},{dim},{vdim}]")
        positions = 0
        if mode == self.LINREC_HGRN2:
            self._f32_vector(p0, heads * dim, "linrec lower bounds")
            if p1 is not None:
                self._f32_vector(p1, heads * dim, "linrec gate bias")
        else:
            self._f32_vector(p0, heads, "linrec decays")
            positions = self._rotation_tables(cos, sin, rot, max_pos)
        if not (gates.is_cuda and gates.dtype == torch.float32 and gates.is_contiguous()
                and gates.numel() >= self.linrec_gate_floats(raw.shape[0], heads, dim)):
            raise KernelError("linrec gates: float32 scratch of linrec_gate_floats elements")
        if not (tok_pos.is_cuda and tok_pos.dtype == torch.int32 and tok_pos.is_contiguous() and tok_pos.numel() >= raw.shape[0]):
            raise KernelError("linrec tok_pos: int32, one position a token")
        if n_seqs == 0 or raw.shape[0] == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_linrec, (
            c_int(mode), _ptr(raw), c_long(raw.stride(0)), c_int(q_at), c_int(ab_at), c_int(v_at), c_int(raw.shape[0]),
            c_int(heads), c_int(dim), c_int(vdim), _ptr(p0), _ptr(p1), _ptr(cos), _ptr(sin), c_int(rot),
            c_int(positions), c_int(max_pos), _ptr(tok_pos), _ptr(seqs), c_int(n_seqs), _ptr(state), _ptr(gates),
            _ptr(out), c_long(out.stride(0)), _stream()))

    def head_norm_gate(self, x: torch.Tensor, heads: int, vdim: int, weight, gate, eps: float, out: torch.Tensor,
                       gate_act: str = "silu") -> None:
        """Per (token, head): ``x / sqrt(mean(x^2) + eps)`` over the head's ``vdim`` values, times ``weight
        [vdim]`` and ``silu(gate)`` or, with ``gate_act = "sigmoid"``, ``sigmoid(gate)`` (float32 rows like ``x``)
        where given; ``x`` float32 ``[T, heads*vdim]``."""
        if gate_act not in ("silu", "sigmoid"):
            raise KernelError(f"head_norm_gate: the gate's activation is silu or sigmoid, got {gate_act!r}")
        _rows_ok(x, "head_norm_gate x"); _rows_ok(out, "head_norm_gate out")
        if not (x.dtype == torch.float32 and x.shape[1] == heads * vdim and out.shape == x.shape and out.dtype in DTYPE_CODE):
            raise KernelError("head_norm_gate reads float32 [T, heads*vdim] and writes the same shape")
        if weight is not None:
            self._f32_vector(weight, vdim, "head_norm_gate weight")
        ldg = 0
        if gate is not None:
            if not (gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and gate.stride(1) == 1
                    and gate.shape == x.shape):
                raise KernelError("head_norm_gate gate must be float32 rows of the shape of x")
            ldg = gate.stride(0)
        if x.shape[0] == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_head_norm_gate, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(x), c_long(x.stride(0)), c_int(x.shape[0]), c_int(heads), c_int(vdim),
            _ptr(weight), _ptr(gate), c_long(ldg), c_int(int(gate_act == "sigmoid")), c_float(eps), _ptr(out),
            c_long(out.stride(0)), _stream()))


    # -- attention with a sink, and what comes before it --------------------------------------
    def sink_lib(self, dim: int, vdim: int):
        """The sink attention library of one key size and one value size."""
        shape = (dim, vdim)
        lib = self._sink.get(shape)
        if lib is None:
            path = _build.build_sink(*shape)
            lib = ctypes.CDLL(str(path))
            lib.ls_last_error.restype = ctypes.c_char_p
            if (lib.ls_sink_dim(), lib.ls_sink_vdim()) != shape:
                raise KernelError(f"{path} was built for another shape")
            self._sink[shape] = lib
            self.sink_paths[shape] = str(path)
        return lib

    #: the value of ``row_tiles`` that asks ``sink_attention`` for its kernel with tiles staged in LDS
    SINK_STAGED = 8

    def sink_staged_keys(self, dim: int, vdim: int, dtype: torch.dtype) -> int:
        """Keys of a tile of the staged kernel for prompt portions; 0 where the sizes do not fit it."""
        return self._memo(("sink_staged_keys", dim, vdim, dtype),
                          lambda: int(self.sink_lib(dim, vdim).ls_sink_staged_keys(c_int(DTYPE_CODE[dtype]))))

    def sink_staged_rows(self, heads: int, kv_heads: int) -> int:
        """Rows of a work item's block in the staged kernel: four waves are min(group, 4) heads times groups of 32 rows."""
        group = heads // kv_heads
        return 32 * (4 // min(group, 4))

    def qkv_post(self, raw: torch.Tensor, n_tokens: int, heads: int, kv_heads: int, dim: int, vdim: int, bias, q_norm,
                 k_norm, eps: float, cos, sin, rot: int, neighbours: bool, max_pos: int, tok_seq, tok_pos, seqs, table,
                 q_out: torch.Tensor, k_pages, v_pages, page_size: int, keys_are_values: bool = False,
                 key_pad: int | None = None, per_head: bool = False, head_weights: bool = False) -> None:
        """Post pass of the fused projection ``raw`` (float32, ``q | k | v | ...``; no ``v`` with
        ``keys_are_values``, where the biased, unnormalised keys are stored as the values): biases, a
        root-mean-square norm over the whole of q and of k with the weights ``q_norm`` / ``k_norm``, rotation of
        the first ``rot`` dimensions of each head in pairs ``(i, i + rot/2)`` or of ``neighbours``, queries to
        ``q_out``, keys and values to their pages.  ``key_pad``: the size of a head in ``q_out`` and in the key
        pages where it exceeds ``dim`` (zeros beyond ``dim``).  ``per_head``: every head of q and of k is divided
        by its own root mean square over ``dim`` (``eps`` inside the root, no weights) instead; with
        ``head_weights`` as well, then multiplied by ``q_norm`` / ``k_norm`` of ``dim`` elements, which all heads share."""
        _rows_ok(raw, "qkv_post raw"); _rows_ok(q_out, "qkv_post q_out")
        key_pad = dim if key_pad is None else key_pad
        width = heads * dim + kv_heads * dim + (0 if keys_are_values else kv_heads * vdim)
        if not (raw.dtype == torch.float32 and raw.shape[0] >= n_tokens and raw.shape[1] >= width):
            raise KernelError(f"qkv_post raw must be float32 [>= {n_tokens}, >= {width}]")
        if not (key_pad >= dim and q_out.dtype in DTYPE_CODE and q_out.shape[0] >= n_tokens and q_out.shape[1] == heads * key_pad):
            raise KernelError("qkv_post q_out has the wrong shape or dtype")
        if keys_are_values and dim != vdim:
            raise KernelError(f"keys of {dim} elements cannot be values of {vdim}")
        if bias is not None:
            self._f32_vector(bias, width, "qkv_post bias")
        if (q_norm is None) != (k_norm is None):
            raise KernelError("qkv_post normalises both q and k or neither")
        if head_weights and not (per_head and q_norm is not None):
            raise KernelError("qkv_post: weights that the heads share belong to a norm a head, and both are needed")
        if q_norm is not None:
            self._f32_vector(q_norm, dim if head_weights else heads * dim, "qkv_post q_norm")
            self._f32_vector(k_norm, dim if head_weights else kv_heads * dim, "qkv_post k_norm")
        if per_head and ((q_norm is not None and not head_weights) or not eps > 0):
            raise KernelError("qkv_post: a norm a head takes no weights, or one vector for all heads, and needs a positive eps")
        positions = self._rotation_tables(cos, sin, rot, max_pos)
        self._paged_ok(k_pages, v_pages, table, q_out.dtype, kv_heads, page_size, key_pad, vdim)
        if not (max_pos // page_size < table.shape[1]):
            raise KernelError(f"position {max_pos} needs page {max_pos // page_size}, the block table has {table.shape[1]} columns")
        for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n_tokens):
                raise KernelError(f"{name} must be int32 with at least {n_tokens} entries")
        if n_tokens == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_qkv_post, (
            c_int(DTYPE_CODE[q_out.dtype]), _ptr(raw), c_long(raw.stride(0)), c_int(n_tokens), c_int(heads),
            c_int(kv_heads), c_int(dim), c_int(key_pad), c_int(vdim), c_int(int(keys_are_values)), c_int(2 if head_weights else int(per_head)), _ptr(bias), _ptr(q_norm), _ptr(k_norm),
            c_float(eps), _ptr(cos), _ptr(sin), c_int(rot), c_int(int(neighbours)), c_int(positions), c_int(max_pos),
            _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs), _ptr(table), c_int(table.shape[1]), _ptr(q_out),
            c_long(q_out.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(page_size), _stream()))

    def sink_attention(self, q: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, k_pages, v_pages,
                       page_size: int, table, seqs, items: torch.Tensor, n_items: int, row_tiles: int, scale: float,
                       window: int, chunk: int, sink, dist_bias, gate, out: torch.Tensor,
                       folds: torch.Tensor | None = None, n_folds: int = 0, part: torch.Tensor | None = None,
                       keep_first: int = 0) -> None:
        """Attention of the step's queries ``q [T, heads*dim]`` over the paged cache with a sink in the softmax.
        ``items``: ``n_items`` work items of four ints (request of the step, block of ``16 * row_tiles`` of its
        rows, run, runs); ``row_tiles`` 1, 2 or 4, or 0 for a step of single decoded tokens, or ``SINK_STAGED`` for
        the kernel that stages key tiles in LDS (blocks of ``sink_staged_rows`` rows).  ``window`` /
        ``chunk``: 0 for none; ``keep_first``: with a window, the first that many tokens stay visible.  ``sink [heads]`` float32 or None; ``dist_bias [heads, distances]`` float32 or
        None (its last column serves every larger distance); ``gate``: float32 rows of ``heads*vdim`` logits
        whose sigmoid multiplies the output, or None.  Row blocks whose keys are dealt to several work items
        have a fold item in ``folds`` (first work item, runs, first packed row, rows) and their results wait in
        ``part`` (float32) until a second launch has folded them."""
        lib = self.sink_lib(dim, vdim)
        _rows_ok(q, "sink_attention q"); _rows_ok(out, "sink_attention out")
        if not (q.dtype in DTYPE_CODE and out.dtype == q.dtype and q.shape[1] == heads * dim
                and out.shape[1] == heads * vdim and out.shape[0] == q.shape[0]):
            raise KernelError("sink_attention q / out have the wrong shape or dtype")
        self._paged_ok(k_pages, v_pages, table, q.dtype, kv_heads, page_size, dim, vdim)
        if not (items.is_cuda and items.dtype == torch.int32 and items.is_contiguous() and items.numel() >= 4 * n_items):
            raise KernelError("sink_attention work items must hold four int32 each")
        if row_tiles not in (0, 1, 2, 4, self.SINK_STAGED):
            raise KernelError(f"sink_attention takes 0, 1, 2 or 4 row tiles or {self.SINK_STAGED} for its staged kernel, got {row_tiles}")
        if row_tiles == self.SINK_STAGED:
            if not (self.sink_staged_keys(dim, vdim, q.dtype) and page_size % (16 // q.element_size()) == 0):
                raise KernelError(f"the staged kernel does not take keys of {dim}, values of {vdim} on pages of {page_size}")
            part_rows = self.sink_staged_rows(heads, kv_heads)
        else:
            part_rows = 16 * row_tiles if row_tiles else 1
        if n_folds:
            if not (folds is not None and folds.is_cuda and folds.dtype == torch.int32 and folds.is_contiguous()
                    and folds.numel() >= 4 * n_folds and part is not None and part.is_cuda
                    and part.dtype == torch.float32 and part.is_contiguous()
                    and part.numel() >= n_items * part_rows * heads * (vdim + 2)):
                raise KernelError("sink_attention folds: four int32 each, and room for every work item's partial result")
        if sink is not None:
            self._f32_vector(sink, heads, "sink_attention sink")
        n_dist = 0
        if dist_bias is not None:
            if not (dist_bias.is_cuda and dist_bias.dtype == torch.float32 and dist_bias.is_contiguous()
                    and dist_bias.dim() == 2 and dist_bias.shape[0] == heads and dist_bias.shape[1] > 0):
                raise KernelError(f"sink_attention dist_bias must be float32 [{heads}, distances]")
            n_dist = dist_bias.shape[1]
        ldg = 0
        if gate is not None:
            _rows_ok(gate, "sink_attention gate")
            if not (gate.dtype == torch.float32 and gate.shape[0] >= q.shape[0] and gate.shape[1] == heads * vdim):
                raise KernelError(f"sink_attention gate must be float32 [>= {q.shape[0]}, {heads * vdim}]")
            ldg = gate.stride(0)
        if not (window >= 0 and chunk >= 0):
            raise KernelError(f"sink_attention window {window} / chunk {chunk}")
        if not (keep_first >= 0 and (keep_first == 0 or (window > 0 and chunk == 0))):
            raise KernelError(f"sink_attention: {keep_first} kept first tokens need a window and no chunks")
        if n_items == 0:
            return
        self._launch(lib, lib.ls_sink_attention, (
            c_int(DTYPE_CODE[q.dtype]), _ptr(q), c_long(q.stride(0)), _ptr(k_pages), _ptr(v_pages), c_int(page_size),
            _ptr(table), c_int(table.shape[1]), _ptr(seqs), _ptr(items), c_int(n_items), c_int(row_tiles), c_int(heads),
            c_int(kv_heads), c_float(scale), c_int(window), c_int(chunk), c_int(keep_first), _ptr(sink), _ptr(dist_bias), c_int(n_dist),
            _ptr(gate), c_long(ldg), _ptr(out), c_long(out.stride(0)), _ptr(folds), c_int(n_folds), _ptr(part),
            c_int(part_rows), _stream()))

    # -- many small experts --------------------------------------------------------------------
    def experts_lib(self):
        """The library of csrc/experts.hip, built and loaded when a part first asks for it."""
        if self._experts is None:
            self.experts_path = _build.build_experts()
            lib = ctypes.CDLL(str(self.experts_path))
            lib.ls_last_error.restype = ctypes.c_char_p
            self._experts = lib
        return self._experts

    def experts_max_top(self) -> int:
        return self._memo(("experts_max_top",), lambda: int(self.experts_lib().ls_experts_max_top()))

    def experts_tile_capacity(self, n_tokens: int, experts: int, top: int, rows_a_tile: int) -> int:
        """Tiles of ``rows_a_tile`` rows that the (token, choice) pairs of a step can need at most."""
        pairs = n_tokens * top
        return pairs // rows_a_tile + min(pairs, experts)

    @staticmethod
    def _i32(t, n: int, name: str) -> None:
        if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name} must be int32 with at least {n} elements on the GPU")

    def experts_route(self, logits: torch.Tensor, bias, top: int, rows_a_tile: int, expert: torch.Tensor,
                      weight: torch.Tensor, order: torch.Tensor, tiles: torch.Tensor, counts: torch.Tensor,
                      scoring: str = "softmax") -> None:
        """From router ``logits [T, E]`` (float32) and ``bias [E]``: every token's ``top`` experts (largest logit
        first, the lower index wins a tie) into ``expert [T, top]``, the softmax over the chosen logits into
        ``weight [T, top]``; the pairs ``token * top + choice`` sorted by expert into ``order``, and every
        expert's pairs cut into ``tiles [capacity, 4]`` (expert or -1, first place in ``order``, rows, 0).
        ``scoring = "sigmoid"``: every chosen expert weighs the sigmoid of its own logit instead (the weights of a token need not add up to one)."""
        _rows_ok(logits, "experts_route logits")
        if scoring not in ("softmax", "sigmoid"):
            raise KernelError(f"experts_route: scoring is softmax or sigmoid, got {scoring!r}")
        t, e = logits.shape
        if not (logits.dtype == torch.float32 and 0 < top <= min(e, self.experts_max_top())):
            raise KernelError(f"experts_route: float32 logits and 1 <= top <= {min(e, self.experts_max_top())}, got {top}")
        if bias is not None:
            self._f32_vector(bias, e, "experts_route bias")
        cap = self.experts_tile_capacity(t, e, top, rows_a_tile)
        self._i32(expert, t * top, "experts_route expert"); self._i32(order, t * top, "experts_route order")
        self._i32(tiles, 4 * cap, "experts_route tiles"); self._i32(counts, e, "experts_route counts")
        if not (weight.is_cuda and weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() >= t * top):
            raise KernelError("experts_route weight must be float32 [T, top]")
        if t == 0:
            return
        lib = self.experts_lib()
        self._launch(lib, lib.ls_experts_route, (
            _ptr(logits), c_long(logits.stride(0)), _ptr(bias), c_int(t), c_int(e), c_int(top), c_int(rows_a_tile),
            _ptr(expert), _ptr(weight), _ptr(order), _ptr(tiles), c_int(cap), _ptr(counts), c_int(int(scoring == "sigmoid")),
            _stream()))

    def experts_apply(self, x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, top: int,
                      rows_a_tile: int, order: torch.Tensor, tiles: torch.Tensor, weight: torch.Tensor, limit: float,
                      alpha: float, act: torch.Tensor, partials: torch.Tensor, shift: float = 1.0,
                      weigh_input: bool = False) -> None:
        """``partials[k][t] = weight[t, k] * down_e(act(gate_e x[t], up_e x[t]))`` for every token's ``k``-th
        expert ``e``, with the clamped gated unit of ``glu_clamped`` as activation (``min(g, limit) sigmoid(alpha
        min(g, limit)) (clamp(u, -limit, limit) + shift)``; an infinite ``limit``, ``alpha`` 1 and ``shift`` 0 are the
        plain unit ``silu(g) u``).  ``w_gate``, ``w_up``
        ``[E, F, K]``, ``w_down [E, N, F]`` in the compute dtype; ``act``: scratch ``[T * top, F]`` of the
        compute dtype; ``partials [top, T, N]`` float32; the routing as ``experts_route`` left it.
        ``weigh_input``: the weight multiplies the expert's input instead, ``partials[k][t] = down_e(act(w gate_e
        x[t], w up_e x[t]))``."""
        _rows_ok(x, "experts_apply x"); _rows_ok(act, "experts_apply act")
        t, k = x.shape
        if not (w_gate.dim() == 3 and w_gate.shape == w_up.shape and w_gate.shape[2] == k and w_down.dim() == 3
                and w_down.shape[0] == w_gate.shape[0] and w_down.shape[2] == w_gate.shape[1]
                and w_gate.is_contiguous() and w_up.is_contiguous() and w_down.is_contiguous()
                and w_gate.dtype == x.dtype == w_up.dtype == w_down.dtype == act.dtype and x.dtype in DTYPE_CODE):
            raise KernelError("experts_apply weights must be [E, F, K], [E, F, K], [E, N, F] of the compute dtype")
        e, f, n = w_gate.shape[0], w_gate.shape[1], w_down.shape[1]
        cap = self.experts_tile_capacity(t, e, top, rows_a_tile)
        if not (act.shape[0] >= t * top and act.shape[1] == f):
            raise KernelError(f"experts_apply act must be [>= {t * top}, {f}]")
        if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous()
                and tuple(partials.shape) == (top, t, n)):
            raise KernelError(f"experts_apply partials must be float32 [{top}, {t}, {n}]")
        self._i32(order, t * top, "experts_apply order"); self._i32(tiles, 4 * cap, "experts_apply tiles")
        if not (weight.is_cuda and weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() >= t * top):
            raise KernelError("experts_apply weight must be float32 [T, top]")
        if t == 0:
            return
        lib = self.experts_lib()
        self._launch(lib, lib.ls_experts_apply, (
            c_int(DTYPE_CODE[x.dtype]), _ptr(x), c_long(x.stride(0)), _ptr(w_gate), _ptr(w_up), _ptr(w_down), c_int(t),
            c_int(e), c_int(top), c_int(k), c_int(f), c_int(n), c_int(rows_a_tile), _ptr(order), _ptr(tiles), c_int(cap),
            _ptr(weight), c_float(limit), c_float(alpha), c_float(shift), _ptr(act), c_long(act.stride(0)), _ptr(partials),
            c_int(int(bool(weigh_input))), _stream()))

    def experts_route_table(self, token_ids: torch.Tensor, table: torch.Tensor, experts: int, rows_a_tile: int,
                            expert: torch.Tensor, weight: torch.Tensor, order: torch.Tensor, tiles: torch.Tensor,
                            counts: torch.Tensor) -> None:
        """Routing without a router: token ``t`` uses the experts in row ``token_ids[t]`` of ``table [vocab, top]``
        (int32, entries in ``[0, experts)``, those of a row differ), each with the weight ``1 / top``.  The
        outputs are those of ``experts_route``."""
        if not (table.is_cuda and table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous()):
            raise KernelError("experts_route_table table must be int32 [vocab, top] on the GPU")
        t, top = token_ids.shape[0], table.shape[1]
        if not (0 < top <= experts):
            raise KernelError(f"experts_route_table: {top} experts a token of {experts}")
        self._i32(token_ids, t, "experts_route_table token_ids")
        cap = self.experts_tile_capacity(t, experts, top, rows_a_tile)
        self._i32(expert, t * top, "experts_route_table expert"); self._i32(order, t * top, "experts_route_table order")
        self._i32(tiles, 4 * cap, "experts_route_table tiles"); self._i32(counts, experts, "experts_route_table counts")
        if not (weight.is_cuda and weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() >= t * top):
            raise KernelError("experts_route_table weight must be float32 [T, top]")
        if t == 0:
            return
        lib = self.experts_lib()
        self._launch(lib, lib.ls_experts_route_table, (
            _ptr(token_ids), _ptr(table), c_int(t), c_int(experts), c_int(top), c_int(rows_a_tile), _ptr(expert),
            _ptr(weight), _ptr(order), _ptr(tiles), c_int(cap), _ptr(counts), _stream()))

    # -- a residual stream of several copies ------------------------------------------------------
    def streams_max(self) -> tuple[int, int]:
        """(the most copies, the widest row) that ``streams_step`` takes."""
        return self._memo(("streams_max",), lambda: (int(self.mixers_lib().ls_streams_max()),
                                                     int(self.mixers_lib().ls_streams_max_width())))

    def streams_step(self, x: torch.Tensor, copies: int, partials, mix, gain, take, weight, eps: float, out,
                     rows: torch.Tensor | None = None) -> None:
        """One step of a residual stream of ``copies`` copies, ``x`` float32 ``[T, copies * width]``.  With
        ``partials [slices, T, width]`` (a sublayer's output as slice sums) the copies are rewritten:
        ``x'_t = sum_s mix[s, t] x_s + gain[t] y``, ``y`` the sum of the slices in ascending order.  With ``out
        [rows, width]`` the copies are then read: ``u = sum_t take[t] x'_t`` (``take`` None: their plain sum) and
        ``out = u / sqrt(mean(u^2) + eps) * weight``.  ``rows`` selects rows of ``x`` (all without it)."""
        _rows_ok(x, "streams_step x")
        if not (x.dtype == torch.float32 and copies > 0 and x.shape[1] % copies == 0):
            raise KernelError("streams_step works on float32 rows of whole copies")
        width = x.shape[1] // copies
        most, widest = self.streams_max()
        if not (copies <= most and width <= widest):
            raise KernelError(f"streams_step takes up to {most} copies of up to {widest} elements, got {copies} of {width}")
        n_rows = x.shape[0] if rows is None else rows.shape[0]
        if rows is not None and not (rows.is_cuda and rows.dtype == torch.int32 and rows.is_contiguous()):
            raise KernelError("streams_step rows: int32 on the GPU")
        slices = p_rows = 0
        if partials is not None:
            if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous() and partials.dim() == 3
                    and partials.shape[2] == width and partials.shape[1] >= x.shape[0]):
                raise KernelError(f"streams_step partials must be float32 [slices, >= {x.shape[0]}, {width}]")
            slices, p_rows = partials.shape[0], partials.shape[1]
            self._f32_vector(mix, copies * copies, "streams_step mix"); self._f32_vector(gain, copies, "streams_step gain")
        if take is not None:
            self._f32_vector(take, copies, "streams_step take")
        dtype, ld_out = torch.float32, 0
        if out is not None:
            _rows_ok(out, "streams_step out")
            if not (out.dtype in DTYPE_CODE and tuple(out.shape) == (n_rows, width) and eps > 0):
                raise KernelError(f"streams_step out must be [{n_rows},{width}], eps positive")
            self._f32_vector(weight, width, "streams_step weight")
            dtype, ld_out = out.dtype, out.stride(0)
        elif partials is None:
            return
        if n_rows == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_streams_step, (
            c_int(DTYPE_CODE[dtype]), _ptr(x), c_long(x.stride(0)), c_int(copies), c_int(width), _ptr(partials),
            c_int(slices), c_int(p_rows), _ptr(mix), _ptr(gain), _ptr(take), _ptr(weight), c_float(eps), _ptr(out),
            c_long(ld_out), _ptr(rows), c_int(n_rows), _stream()))

    # -- attention over a cached latent: the passes around it ----------------------------------------
    def latent_post(self, raw: torch.Tensor, n_tokens: int, q_rank: int, kv_rank: int, rot_dim: int, key_pad: int,
                    has_kv: bool, q_weight, kv_weight, eps: float, cos, sin, rot: int, max_pos: int, tok_seq, tok_pos,
                    seqs, table, q_latent: torch.Tensor, k_pages, v_pages, page_size: int) -> None:
        """Post pass of the down projections ``raw`` (float32, ``a | c | r``): the query latent ``a`` normalised
        with ``q_weight`` into ``q_latent``; with ``has_kv`` the latent ``c`` normalised with ``kv_weight`` into the
        key pages (dimensions ``0 .. kv_rank`` of the one key head of ``key_pad`` elements) and into the value
        pages, and the shared key part ``r``, rotated in neighbouring pairs on its first ``rot`` dimensions,
        behind it in the key pages."""
        _rows_ok(raw, "latent_post raw"); _rows_ok(q_latent, "latent_post q_latent")
        width = q_rank + (kv_rank + rot_dim if has_kv else 0)
        if not (raw.dtype == torch.float32 and raw.shape[0] >= n_tokens and raw.shape[1] >= width):
            raise KernelError(f"latent_post raw must be float32 [>= {n_tokens}, >= {width}]")
        if not (q_latent.dtype in DTYPE_CODE and q_latent.shape[0] >= n_tokens and q_latent.shape[1] == q_rank):
            raise KernelError("latent_post q_latent has the wrong shape or dtype")
        self._f32_vector(q_weight, q_rank, "latent_post q_weight")
        positions = 0
        if has_kv:
            self._f32_vector(kv_weight, kv_rank, "latent_post kv_weight")
            positions = self._rotation_tables(cos, sin, rot, max_pos)
            self._paged_ok(k_pages, v_pages, table, q_latent.dtype, 1, page_size, key_pad, kv_rank)
            if not (key_pad >= kv_rank + rot_dim and max_pos // page_size < table.shape[1]):
                raise KernelError("latent_post: the key head is too short, or a position lies beyond the block table")
            for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
                if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n_tokens):
                    raise KernelError(f"{name} must be int32 with at least {n_tokens} entries")
        if n_tokens == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_latent_post, (
            c_int(DTYPE_CODE[q_latent.dtype]), _ptr(raw), c_long(raw.stride(0)), c_int(n_tokens), c_int(q_rank),
            c_int(kv_rank), c_int(rot_dim), c_int(key_pad), c_int(int(has_kv)), _ptr(q_weight),
            _ptr(kv_weight if has_kv else None), c_float(eps), _ptr(cos if has_kv else None), _ptr(sin if has_kv else None),
            c_int(rot), c_int(positions), c_int(max_pos), _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs),
            _ptr(table if has_kv else None), c_int(table.shape[1] if has_kv else 0), _ptr(q_latent),
            c_long(q_latent.stride(0)), _ptr(k_pages if has_kv else None), _ptr(v_pages if has_kv else None),
            c_int(page_size), _stream()))

    def latent_query(self, qf: torch.Tensor, n_tokens: int, heads: int, dim: int, rot_dim: int, kv_rank: int, key_pad: int,
                     cos, sin, rot: int, max_pos: int, tok_pos, plain: torch.Tensor, q_out: torch.Tensor) -> None:
        """Post pass of the queries' up projection ``qf`` (float32, heads of ``dim`` plain and ``rot_dim`` rotated
        dimensions): the plain parts into ``plain [T, heads*dim]``; the rotated parts, rotated in neighbouring
        pairs on their first ``rot`` dimensions, into ``q_out [T, heads*key_pad]`` behind the ``kv_rank``
        dimensions of each head that the product with the keys' up projection fills (zeros up to ``key_pad``)."""
        _rows_ok(qf, "latent_query qf"); _rows_ok(plain, "latent_query plain"); _rows_ok(q_out, "latent_query q_out")
        if not (qf.dtype == torch.float32 and qf.shape[0] >= n_tokens and qf.shape[1] == heads * (dim + rot_dim)):
            raise KernelError(f"latent_query qf must be float32 [>= {n_tokens}, {heads * (dim + rot_dim)}]")
        if not (plain.dtype in DTYPE_CODE and q_out.dtype == plain.dtype and plain.shape[0] >= n_tokens
                and plain.shape[1] == heads * dim and q_out.shape[0] >= n_tokens and q_out.shape[1] == heads * key_pad
                and key_pad >= kv_rank + rot_dim):
            raise KernelError("latent_query outputs have the wrong shape or dtype")
        positions = self._rotation_tables(cos, sin, rot, max_pos)
        if not (tok_pos.is_cuda and tok_pos.dtype == torch.int32 and tok_pos.is_contiguous() and tok_pos.numel() >= n_tokens):
            raise KernelError("latent_query tok_pos: int32, one position a token")
        if n_tokens == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_latent_query, (
            c_int(DTYPE_CODE[plain.dtype]), _ptr(qf), c_long(qf.stride(0)), c_int(n_tokens), c_int(heads), c_int(dim),
            c_int(rot_dim), c_int(kv_rank), c_int(key_pad), _ptr(cos), _ptr(sin), c_int(rot), c_int(positions),
            c_int(max_pos), _ptr(tok_pos), _ptr(plain), c_long(plain.stride(0)), _ptr(q_out), c_long(q_out.stride(0)),
            _stream()))

    def heads_product(self, x: torch.Tensor, x_stride: int, w: torch.Tensor, out: torch.Tensor, o_stride: int,
                      n_rows: int | None = None) -> None:
        """A product a head: ``out[t, h * o_stride + n] = sum_k w[h, n, k] x[t, h * x_stride + k]`` with
        ``w [heads, N, K]`` contiguous; ``x``, ``w`` and ``out`` in one compute dtype."""
        _rows_ok(x, "heads_product x"); _rows_ok(out, "heads_product out")
        n_rows = x.shape[0] if n_rows is None else n_rows
        if not (w.is_cuda and w.dim() == 3 and w.is_contiguous() and w.dtype in DTYPE_CODE and x.dtype == w.dtype == out.dtype):
            raise KernelError("heads_product w must be [heads, N, K] contiguous, all operands of one dtype")
        heads, n, k = w.shape
        if not (x.shape[0] >= n_rows and out.shape[0] >= n_rows and x.shape[1] >= (heads - 1) * x_stride + k
                and out.shape[1] >= (heads - 1) * o_stride + n and x_stride >= 0 and o_stride >= 0):
            raise KernelError("heads_product: the heads do not fit the rows")
        if n_rows == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_heads_product, (
            c_int(DTYPE_CODE[w.dtype]), _ptr(x), c_long(x.stride(0)), c_int(x_stride), _ptr(w), c_int(heads), c_int(n),
            c_int(k), c_int(n_rows), _ptr(out), c_long(out.stride(0)), c_int(o_stride), _stream()))

    # -- the gated delta rule -----------------------------------------------------------------------
    def delta_max_dim(self) -> int:
        return self._memo(("delta_max_dim",), lambda: int(self.mixers_lib().ls_delta_max_dim()))

    def delta_scratch_floats(self, n_tokens: int, kv_heads: int, heads: int, dim: int, vdim: int, channel: bool = False) -> int:
        lib = self.mixers_lib()
        entry = lib.ls_delta_scratch_floats_channel if channel else lib.ls_delta_scratch_floats
        entry.restype = ctypes.c_long
        return int(entry(c_int(n_tokens), c_int(kv_heads), c_int(heads), c_int(dim), c_int(vdim)))

    def delta_rule(self, raw: torch.Tensor, kv_heads: int, heads: int, dim: int, vdim: int, taps: torch.Tensor, a_log,
                   dt_bias, unit_eps: float, tok_seq, tok_pos, seqs, n_seqs: int, state: torch.Tensor,
                   scratch: torch.Tensor, out: torch.Tensor, channel_decay: torch.Tensor | None = None) -> None:
        """The gated delta rule over the tokens of every request of the step.  ``raw`` float32 holds the
        projections ``q | k`` (``kv_heads`` heads of ``dim``) ``| v`` (``heads`` of ``vdim``) ``| b | a``
        (``heads`` each); every channel of q, k and v passes a causal convolution with ``taps [channels, M]``
        (the last column is the current token's) and silu; q and k become unit vectors (``unit_eps`` inside
        the root), q also times ``dim^-1/2``; ``beta = sigmoid(b)``, ``decay = exp(-exp(a_log) softplus(a +
        dt_bias))``; per head ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.  ``state``
        float32 ``[slots, heads*dim*vdim + (M-1)*channels]``: the matrices, then the convolutions' last inputs;
        read and left for the next step.  ``out`` float32 ``[T, heads*vdim]``.  ``channel_decay`` (float32 rows of
        ``heads*dim`` logits): a decay for every head and key channel instead, ``g = exp(-exp(a_log_h) softplus(logit +
        dt_bias))`` with ``dt_bias [heads*dim]``, which multiplies the rows of ``S``; ``raw`` then ends with ``b``."""
        _rows_ok(raw, "delta_rule raw"); _rows_ok(out, "delta_rule out")
        t = raw.shape[0]
        channels = 2 * kv_heads * dim + heads * vdim
        chan = channel_decay is not None
        ldc = 0
        if chan:
            _rows_ok(channel_decay, "delta_rule channel_decay")
            if not (channel_decay.dtype == torch.float32 and channel_decay.shape[0] >= t and channel_decay.shape[1] == heads * dim):
                raise KernelError(f"delta_rule channel_decay must be float32 [>= {t}, {heads * dim}]")
            ldc = channel_decay.stride(0)
        if not (raw.dtype == torch.float32 and raw.shape[1] >= channels + (1 if chan else 2) * heads and out.dtype == torch.float32
                and tuple(out.shape) == (t, heads * vdim)):
            raise KernelError("delta_rule reads and writes float32 rows, out [T, heads*vdim]")
        if not (heads % kv_heads == 0 and dim <= self.delta_max_dim()):
            raise KernelError(f"delta_rule: {heads} heads over {kv_heads} key heads, keys of at most {self.delta_max_dim()}")
        if not (taps.is_cuda and taps.dtype == torch.float32 and taps.is_contiguous() and taps.dim() == 2
                and taps.shape[0] == channels and taps.shape[1] >= 1):
            raise KernelError(f"delta_rule taps must be float32 [{channels}, M]")
        m = taps.shape[1]
        self._f32_vector(a_log, heads, "delta_rule a_log")
        self._f32_vector(dt_bias, heads * dim if chan else heads, "delta_rule dt_bias")
        if not (state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2
                and state.shape[1] == heads * dim * vdim + (m - 1) * channels):
            raise KernelError(f"delta_rule state must be float32 [slots, {heads * dim * vdim + (m - 1) * channels}]")
        if not (scratch.is_cuda and scratch.dtype == torch.float32 and scratch.is_contiguous()
                and scratch.numel() >= self.delta_scratch_floats(t, kv_heads, heads, dim, vdim, chan)):
            raise KernelError("delta_rule scratch: float32 of delta_scratch_floats elements")
        for name, v in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (v.is_cuda and v.dtype == torch.int32 and v.is_contiguous() and v.numel() >= t):
                raise KernelError(f"delta_rule {name}: int32, one entry a token")
        if n_seqs == 0 or t == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_delta_rule, (
            _ptr(raw), c_long(raw.stride(0)), c_int(t), c_int(kv_heads), c_int(heads), c_int(dim), c_int(vdim), c_int(m),
            _ptr(taps), _ptr(a_log), _ptr(dt_bias), c_float(unit_eps), _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs),
            c_int(n_seqs), _ptr(state), c_long(state.stride(0)), _ptr(scratch), _ptr(out), c_long(out.stride(0)),
            _ptr(channel_decay), c_long(ldc), _stream()))

    # -- an embedding with a table of token pairs, and the shift of a sublayer's input by a token -------------
    def embed_pair(self, tokens: torch.Tensor, tok_seq, tok_pos, seqs, table: torch.Tensor, pairs: torch.Tensor,
                   mul_prev: int, mul_cur: int, state: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
        """``out[t] = table[tokens[t]] * scale + pairs[(token before * mul_prev + tokens[t] * mul_cur) mod buckets]``
        as float32 rows, ``buckets = pairs.shape[0] - 1``; a request's first token takes the last row of ``pairs``.
        ``state`` int32 ``[slots, 1]``: the last token of every request so far, read for the first row of a portion
        and left as the portion's last token."""
        if not (tokens.is_cuda and tokens.dtype == torch.int32 and tokens.dim() == 1 and tokens.is_contiguous()):
            raise KernelError("embed_pair tokens must be a contiguous int32 vector on the GPU")
        t = tokens.shape[0]
        _rows_ok(table, "embed_pair table"); _rows_ok(pairs, "embed_pair pairs"); _rows_ok(out, "embed_pair out")
        if not (table.is_contiguous() and pairs.is_contiguous() and table.dtype in DTYPE_CODE and pairs.dtype == table.dtype
                and pairs.shape[1] == table.shape[1] and pairs.shape[0] >= 2):
            raise KernelError("embed_pair tables must be contiguous, of one dtype and one width, the pairs' with two rows or more")
        if not (out.dtype == torch.float32 and tuple(out.shape) == (t, table.shape[1])):
            raise KernelError(f"embed_pair out must be float32 [{t},{table.shape[1]}]")
        if not (state.is_cuda and state.dtype == torch.int32 and state.dim() == 2 and state.stride(1) == 1):
            raise KernelError("embed_pair state must be int32 [slots, 1] on the GPU")
        for name, v in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (v.is_cuda and v.dtype == torch.int32 and v.is_contiguous() and v.numel() >= t):
                raise KernelError(f"embed_pair {name}: int32, one entry a token")
        if t == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_embed_pair, (
            c_int(DTYPE_CODE[table.dtype]), _ptr(tokens), _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs), _ptr(table),
            c_int(table.shape[0]), _ptr(pairs), c_int(pairs.shape[0] - 1), c_long(mul_prev), c_long(mul_cur), _ptr(state),
            c_long(state.stride(0)), _ptr(out), c_int(t), c_int(table.shape[1]), c_long(out.stride(0)), c_float(scale),
            _stream()))

    def add_rmsnorm_shift(self, h: torch.Tensor, partials, weight: torch.Tensor, eps: float, mu: torch.Tensor, tok_seq,
                          tok_pos, seqs, state: torch.Tensor, out: torch.Tensor) -> None:
        """For a step of single tokens, in one launch: ``h[t] += partials[0][t] + partials[1][t] + ...`` (``partials``
        may be None), ``n = rmsnorm(h[t]) * weight`` as ``rmsnorm`` computes it, ``out[t] = n + (kept - n) * mu`` with
        the request's row of ``state`` (zeros at its first token), which is then left as ``n``."""
        _rows_ok(h, "add_rmsnorm_shift h"); _rows_ok(out, "add_rmsnorm_shift out")
        t, width = h.shape
        if not (h.dtype == torch.float32 and out.dtype in DTYPE_CODE and tuple(out.shape) == (t, width) and width % 4 == 0):
            raise KernelError("add_rmsnorm_shift works on float32 rows of a multiple of four elements")
        self._f32_vector(weight, width, "add_rmsnorm_shift weight"); self._f32_vector(mu, width, "add_rmsnorm_shift mu")
        slices = p_rows = 0
        if partials is not None:
            if not (partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous() and partials.dim() == 3
                    and partials.shape[2] == width and partials.shape[1] >= t):
                raise KernelError("add_rmsnorm_shift partials [slices, rows, width]")
            slices, p_rows = partials.shape[0], partials.shape[1]
        if not (state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
                and state.shape[1] >= width):
            raise KernelError(f"add_rmsnorm_shift state must be float32 [slots, >= {width}]")
        for name, v in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (v.is_cuda and v.dtype == torch.int32 and v.is_contiguous() and v.numel() >= t):
                raise KernelError(f"add_rmsnorm_shift {name}: int32, one entry a token")
        if t == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_add_rmsnorm_shift, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(h), _ptr(partials), c_int(slices), c_int(p_rows), _ptr(weight), _ptr(mu),
            _ptr(tok_seq), _ptr(tok_pos), _ptr(seqs), _ptr(state), c_long(state.stride(0)), _ptr(out), c_int(t), c_int(width),
            c_long(h.stride(0)), c_long(out.stride(0)), c_float(eps), _stream()))

    def token_shift(self, normed: torch.Tensor, mu: torch.Tensor, tok_seq, tok_pos, seqs, state: torch.Tensor,
                    out: torch.Tensor) -> None:
        """``out[t] = n[t] + (n[t-1] - n[t]) * mu`` for the float32 rows ``normed`` of the step, ``n[t-1]`` being the row
        of the same request's token before (zeros at a request's first token); ``state`` float32 ``[slots, width]``
        holds that row for the first token of a portion and is left as the portion's last row."""
        _rows_ok(normed, "token_shift normed"); _rows_ok(out, "token_shift out")
        t, width = normed.shape
        if not (normed.dtype == torch.float32 and out.dtype in DTYPE_CODE and tuple(out.shape) == (t, width)):
            raise KernelError("token_shift reads float32 rows and writes rows of the same shape")
        self._f32_vector(mu, width, "token_shift mu")
        if not (state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
                and state.shape[1] >= width):
            raise KernelError(f"token_shift state must be float32 [slots, >= {width}]")
        for name, v in (("tok_seq", tok_seq), ("tok_pos", tok_pos)):
            if not (v.is_cuda and v.dtype == torch.int32 and v.is_contiguous() and v.numel() >= t):
                raise KernelError(f"token_shift {name}: int32, one entry a token")
        if t == 0:
            return
        lib = self.mixers_lib()
        self._launch(lib, lib.ls_token_shift, (
            c_int(DTYPE_CODE[out.dtype]), _ptr(normed), c_long(normed.stride(0)), _ptr(mu), _ptr(tok_seq), _ptr(tok_pos),
            _ptr(seqs), _ptr(state), c_long(state.stride(0)), _ptr(out), c_long(out.stride(0)), c_int(t), c_int(width),
            _stream()))


ATTENTION_ITEM_INTS = 32
COMBINE_ITEM_INTS = 8


def pack_attention_items(items, seqs, pages=None) -> "np.ndarray":
    """Work items of the attention kernels as the device wants them.  ``items``:
    rows of (seq, row_block, split_begin, split_end, part_base, n_splits,
    split_lo, 0), seq -1 for an item that stands for no work; ``seqs``: the step's rows of (q_off, q_len, q_start, kv_len,
    table_row, 0, 0, 0).  Each item gets a copy of its request's row appended, so
    that a workgroup learns its work from one load, and sixteen more ints: with ``pages`` (an int array
    ``[items, 16]``, or None) the block-table entries of the item's one key tile, which the fused decode kernel
    then takes from the item instead of the block table (the eighth int of the item says so)."""
    import numpy as np

    items = np.asarray(items, dtype=np.int64).reshape(-1, 8)
    seqs = np.asarray(seqs, dtype=np.int64).reshape(-1, 8)
    if not len(items):
        return np.zeros(0, dtype=np.int64)
    null = items[:, 0] < 0
    rows = seqs[np.maximum(items[:, 0], 0)]
    rows[null] = 0                               # a null item is all zeros: a request of no rows, no splits
    items = np.where(null[:, None], 0, items)
    if pages is None:
        ids = np.zeros((len(items), 16), dtype=np.int64)
    else:
        ids = np.asarray(pages, dtype=np.int64).reshape(len(items), 16)
        ids = np.where(null[:, None], 0, ids)
        items = items.copy()
        items[:, 7] = np.where(null, 0, 1)
    return np.concatenate([items, rows, ids], axis=1).reshape(-1)


def pack_combine_items(items, seqs) -> "np.ndarray":
    """Combine items (seq, row_block, part_base, n_splits) with q_off and q_len of their request appended."""
    import numpy as np

    items = np.asarray(items, dtype=np.int64).reshape(-1, 4)
    seqs = np.asarray(seqs, dtype=np.int64).reshape(-1, 8)
    if not len(items):
        return np.zeros(0, dtype=np.int64)
    pad = np.zeros((len(items), 2), dtype=np.int64)
    null = items[:, 0] < 0
    rows = seqs[np.maximum(items[:, 0], 0), :2]
    rows[null] = 0
    items = np.where(null[:, None], 0, items)
    return np.concatenate([items, rows, pad], axis=1).reshape(-1)


_INSTANCE: Kernels | None = None


def kernels() -> Kernels:
    global _INSTANCE
    if _INSTANCE is None:
        _INSTANCE = Kernels()
    return _INSTANCE
