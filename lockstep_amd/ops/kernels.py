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
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
        if not (tokens.is_cuda and tokens.dtype == torch.int32 and tokens.dim() == 1 and tokens.is_contiguous()):
            raise KernelError("embed tokens must be a contiguous int32 vector on the GPU")
        _rows_ok(table, "embed table"); _rows_ok(out, "embed out")
        if not (table.is_contiguous() and table.dtype in DTYPE_CODE):
            raise KernelError("embed table must be contiguous float32/bfloat16")
        if not (out.dtype == torch.float32 and out.shape == (tokens.shape[0], table.shape[1])):
            raise KernelError(f"embed out must be float32 [{tokens.shape[0]},{table.shape[1]}]")
        if tokens.shape[0] == 0:
            return
        self._launch(self.core, self.core.ls_embed, (
            c_int(DTYPE_CODE[table.dtype]), _ptr(tokens), _ptr(table), _ptr(out), c_int(tokens.shape[0]),
            c_int(table.shape[0]), c_int(table.shape[1]), c_long(out.stride(0)), _stream()))

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
