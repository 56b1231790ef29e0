"""The hand-written gfx950 kernels as Python calls on torch tensors.

`HipKernels` loads `libbeholdd_hip.so` (built from csrc/ on first use) through ctypes and
checks every argument on the host (device, dtype, contiguity, shapes) before a kernel is
launched: the kernels themselves trust their arguments.  There is no CPU path: without a GPU
and the library, construction fails.

Every method launches on torch's current HIP stream; results are written into the `out` tensors
that the caller passes (`gemm` may besides return the prepared input of a following norm).
"""

from __future__ import annotations

import ctypes

import torch

from . import build as _build

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    """A kernel refused its arguments or could not be launched."""


class PackedWeight:
    """A bfloat16 weight matrix regrouped into 16-row x 64-column blocks in matrix-core operand
    order (the `tiles` layout of csrc/gemm_bf16.hip).  `shape` and `dtype` are those of the
    matrix it stands for; `data` is the regrouped buffer (rows padded to a multiple of 16)."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.shape, self.dtype = data, (rows, cols), data.dtype

    def dim(self):
        return 2


class NormedRows:
    """The output of an RMSNorm but for each row's factor: `rows` [n, width] bfloat16 holds x * weight and
    `ss` [n, blocks] float32 partial sums of x^2 whose total over `blocks` gives the row's factor
    1 / sqrt(total / width + eps).  Products (`gemm`, `gemm_swiglu`) take it in place of an activation
    matrix and apply the factor to their result; one that cannot (other operand types) runs the norm
    itself from `source`, which must still hold the norm's input then.  `shape` and `dtype` are those of
    the matrix it stands for."""

    def __init__(self, rows: torch.Tensor, ss: torch.Tensor, eps: float, source: torch.Tensor, weight: torch.Tensor):
        self.rows, self.ss, self.eps = rows, ss, float(eps)
        self.source, self.weight = source, weight       # the norm's input and weight, for a product that cannot take this form
        self.shape, self.dtype, self.device = rows.shape, rows.dtype, rows.device

    def dim(self):
        return 2


class PartSums:
    """A bfloat16 matrix [rows, width] that was never written: `sums` [parts, rows, width] float32 holds a product's
    sums over the parts its K was cut into, and an element of the matrix is the sum of its parts in their order,
    rounded to bfloat16.  `HipKernels.gemm_bare` leaves it, `qk_norm_rope_cache` takes it in place of the rows
    (and does what the product's finishing kernel would have done on the way).  `shape` and `dtype` are those of
    the matrix it stands for."""

    def __init__(self, sums: torch.Tensor):
        self.sums, self.parts = sums, int(sums.shape[0])
        self.shape, self.dtype, self.device = sums.shape[1:], torch.bfloat16, sums.device

    def dim(self):
        return 2


class BlockedRows:
    """A bfloat16 activation matrix [rows, width] kept in blocks of `block_rows` (16 or 8) rows x 32 columns, each
    block in the order in which a matrix-core operand lies in a wave's lanes (`bh_rows_index` in csrc/layout.h):
    what the products of many rows and those of up to 32 rows read fastest.  `HipKernels.new_rows` hands one out
    where the product named as the matrix's reader takes it; the kernels that produce activations (`rmsnorm`,
    `gemm_swiglu`, `attention`, a `gemm` that prepares or finishes a norm) write into it, and `gemm` /
    `gemm_swiglu` read it.  `data` holds whole blocks (for more than 32 rows whole tiles of 256 rows); rows the
    matrix does not have hold nothing.  `shape` and `dtype` are those of the matrix."""

    ROWS_PAD = 256

    def __init__(self, data: torch.Tensor, rows: int, width: int, block_rows: int = 16):
        self.data, self.shape, self.dtype, self.device = data, (rows, width), data.dtype, data.device
        self.block_rows = int(block_rows)

    def dim(self):
        return 2

    @staticmethod
    def padded_rows(rows: int, block_rows: int) -> int:
        """Rows that the buffer of a matrix of `rows` rows holds."""
        unit = BlockedRows.ROWS_PAD if rows > 32 else block_rows
        return -(-rows // unit) * unit


def _block_rows(x) -> int:
    """In blocks of how many rows a matrix lies (0: row after row)."""
    return x.block_rows if isinstance(x, BlockedRows) else 0


def _code(tensor, what: str) -> int:
    code = _CODES.get(tensor.dtype)
    if code is None:
        raise KernelError(f"{what}: dtype {tensor.dtype} is not supported (float32 or bfloat16)")
    return code


ALLOCATION_UNIT = 512     # torch's allocator hands out device memory in multiples of this many bytes


def _rounded(n_bytes: int) -> int:
    return -(-int(n_bytes) // ALLOCATION_UNIT) * ALLOCATION_UNIT


class KernelSizes:
    """What the kernels allocate beside their inputs and outputs, from sizes alone: the library's own host-side
    answers (how a product cuts K into parts, how an attention call splits its keys, in what blocks a matrix
    lies), which need the built library but no GPU.  The engine's byte plan asks here before anything is
    allocated; `HipKernels` is one of these and launches as well."""

    def __init__(self, verbose_build: bool = True):
        path = _build.ensure_built(verbose=verbose_build)
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as error:
            raise KernelError(f"cannot load the HIP kernel library {path}: {error}") from None
        self.library_path = path
        self._declare()

    # ---- ctypes declarations ----
    def _declare(self):
        lib = self.lib
        p, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.bh_last_error.restype = ctypes.c_char_p
        lib.bh_page_size.restype = i
        table = {
            "bh_embed": [p, p, p, p, i, p, i, i, i, p],
            "bh_rmsnorm": [p, p, p, i, p, i, i, i, f, i, p],
            "bh_gemm_generic": [p, i, p, i, p, i, i, i, i, i, p],
            "bh_qk_norm_rope_cache": [p, i, p, p, p, i, f, p, p, i, i, p, p, p, p, p, i, i, i, i, i, i, i, i, p],
            "bh_qk_norm_rope_cache_sums": [p, i, p, p, p, i, f, p, p, i, i, p, p, p, p, p, i, i, i, i, i, i, i, i, p],
            "bh_qk_norm_rope_cache_takes_sums": [i, i, i],
            "bh_gemm_bf16_bare_parts": [i, i, i, i],
            "bh_gemm_bf16_bare": [p, p, p, i, i, i, i, i, p],
            "bh_attention_generic": [p, p, i, p, p, p, i, p, p, i, i, i, i, f, i, i, p],
            "bh_swiglu": [p, p, i, i, i, p],
            "bh_sample": [p, p, p, p, p, p, p, p, i, i, p],
            "bh_sample_scratch": [i, i],
            "bh_sample_draw_scratch": [i, i],
            "bh_sample_top_k_scratch": [i, i],
            "bh_gemm_bf16": [p, p, p, i, i, i, i, i, i, i, p, i, f, p, i, p, p, p, i, i, i, p],
            "bh_gemm_bf16_turns": [p, p, p, i, i, i, i, i, i, i, i, i, p],
            "bh_gemm_bf16_then_norm": [p, p, p, i, i, i, i, p, i, f, p, p, i, i, p],
            "bh_rows_blocked": [p, p, i, i, i, i, p],
            "bh_gemm_bf16_finishes_norm": [i, i, i, i],
            "bh_attention_bf16": [p, p, p, p, p, p, p, i, p, p, i, i, i, i, i, i, f, i, i, i, i, p],
            "bh_attention_bf16_splits": [i, i, i, i, i],
            "bh_attention_bf16_writes_blocked": [i, i, i, i, i],
            "bh_attention_decode_fused": [p, p, p, p, p, p, p, i, p, p, i, i, i, i, f, i, i, i, p, p, i, f, p, p, i, i,
                                          i, i, p],
            "bh_kv_order": [i, i],
            "bh_stream_read": [p, ctypes.c_long, i, i, p, p, p],
        }
        for name, argtypes in table.items():
            function = getattr(lib, name)
            function.argtypes = argtypes
            function.restype = i
        lib.bh_gemm_bf16_scratch.argtypes = [i, i, i, i, i]
        lib.bh_gemm_bf16_scratch.restype = ctypes.c_long
        for query in (lib.bh_gemm_bf16_norm_blocks, lib.bh_gemm_bf16_takes_norm, lib.bh_gemm_bf16_turns_blocks,
                      lib.bh_gemm_bf16_reads_blocked, lib.bh_gemm_bf16_writes_blocked):
            query.argtypes, query.restype = [i, i, i, i, i], ctypes.c_int

    def rows_bytes(self, rows, width, act_size, reader_outputs=None, reader_swiglu=False, reader_packed=True) -> int:
        """Bytes of the matrix that `new_rows` hands out for these arguments."""
        rows, width = int(rows), int(width)
        if reader_outputs is not None and reader_packed and act_size == 2 and width % 64 == 0:
            block_rows = int(self.lib.bh_gemm_bf16_reads_blocked(rows, int(reader_outputs), width, 1, int(bool(reader_swiglu))))
            if block_rows:
                return _rounded(BlockedRows.padded_rows(rows, block_rows) * width * 2)
        return _rounded(rows * width * act_size)

    def gemm_working_bytes(self, m, n, k, act_size, packed=True, swiglu=False, then_norm=False) -> int:
        """Bytes that `gemm` (or `gemm_swiglu`) of these sizes allocates for the length of the call or returns
        as a prepared norm: partial sums of K in parts, the rows and sums of a norm behind it, a regrouped copy
        of activations that came in another form than the product reads, SwiGLU's two halves where the fused
        epilogue does not apply."""
        m, n, k = int(m), int(n), int(k)
        if act_size != 2 or k % 8:
            return _rounded(m * 2 * n * act_size) if swiglu else 0
        sizes = (m, n, k, int(bool(packed)), int(bool(swiglu)))
        total = _rounded(int(self.lib.bh_gemm_bf16_scratch(*sizes)))
        if k % 32 == 0:
            total += 2 * _rounded(BlockedRows.padded_rows(m, 16) * k * 2)      # regrouping: out of blocks, into others
        if then_norm:
            blocks = max(int(self.lib.bh_gemm_bf16_norm_blocks(*sizes)), 1)
            total += _rounded(BlockedRows.padded_rows(m, 16) * n * 2) + _rounded(m * blocks * 4)
        if swiglu and n % 16:
            total += _rounded(m * 2 * n * act_size)
        return total

    def attention_working_bytes(self, n_rows, n_seqs, max_rows_per_seq, n_heads, n_kv_heads, head_dim, max_position,
                                act_size) -> int:
        """Bytes that an attention call allocates: the partial results of its key splits."""
        if act_size != 2 or head_dim % 32 or head_dim > 256:
            return 0
        n_splits = int(self.lib.bh_attention_bf16_splits(int(n_seqs), int(max_rows_per_seq), int(n_heads), int(n_kv_heads),
                                                         int(max_position)))
        if n_splits <= 1:
            return 0
        return _rounded(n_rows * n_heads * n_splits * head_dim * 4) + _rounded(n_rows * n_heads * n_splits * 2 * 4)

    def sample_working_bytes(self, n_rows, vocab) -> int:
        words = max(int(self.lib.bh_sample_scratch(int(n_rows), int(vocab))),
                    int(self.lib.bh_sample_draw_scratch(int(n_rows), int(vocab))),
                    int(self.lib.bh_sample_top_k_scratch(int(n_rows), int(vocab))))
        return _rounded(words * 4) + 4 * _rounded(n_rows * 4)

    def packs(self, rows, cols, act_size) -> bool:
        """Whether `pack_weight` regroups a matrix of this shape and element size."""
        return act_size == 2 and cols % 64 == 0

    def packed_bytes(self, rows, cols, act_size) -> int:
        """Device bytes of a weight matrix as `pack_weight` keeps it (rows padded to whole blocks of 16)."""
        if self.packs(rows, cols, act_size):
            return _rounded(-(-rows // 16) * 16 * cols * 2)
        return _rounded(rows * cols * act_size)


class HipKernels(KernelSizes):
    """The kernel set of the product path."""

    def __init__(self, device="cuda:0", verbose_build: bool = True):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to this process: the HIP kernel library has no CPU fallback")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"the HIP kernel library runs on a GPU, not on {device!r}")
        super().__init__(verbose_build)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.device = torch.device("cuda", self._device_index)
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._plans: dict = {}      # (m, n, k, packed, activation) -> what the library says of such a product
        self._bare: dict = {}       # (m, n, k) -> the parts that `gemm_bare` leaves such a product in, or 0
        self.page_size = int(self.lib.bh_page_size())
        if self.page_size != _build.source_page_size():
            raise KernelError(f"{self.library_path} was built for pages of {self.page_size} tokens, the sources say "
                              f"{_build.source_page_size()}: build the library again")

    # ---- helpers ----
    def _stream(self):
        """The current HIP stream of the device as a raw handle (asked of torch without building a stream object:
        a step makes a few hundred launches)."""
        if self._raw_stream is not None:
            return self._raw_stream(self._device_index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check(self, status: int):
        if status != 0:
            raise KernelError(self.lib.bh_last_error().decode("utf-8", "replace"))

    def _ptr(self, tensor, what: str, dtypes=None, optional: bool = False):
        if type(tensor) is torch.Tensor and tensor.device == self.device and tensor.is_contiguous() \
                and (dtypes is None or tensor.dtype in dtypes):
            return tensor.data_ptr()
        if tensor is None:
            if optional:
                return None
            raise KernelError(f"{what}: tensor is required")
        if isinstance(tensor, BlockedRows):
            rows, width = tensor.shape
            if (tensor.block_rows not in (8, 16) or width % 32 or tensor.data.dtype != torch.bfloat16
                    or tensor.data.numel() < BlockedRows.padded_rows(rows, tensor.block_rows) * width):
                raise KernelError(f"{what}: a matrix of {rows} x {width} in blocks of {tensor.block_rows} rows needs a bfloat16 "
                                  f"buffer of {BlockedRows.padded_rows(rows, tensor.block_rows) * width} elements (whole "
                                  f"blocks; whole tiles of {BlockedRows.ROWS_PAD} rows beyond 32 rows), a width that is a "
                                  f"multiple of 32 and blocks of 8 or 16 rows; it has {tensor.data.numel()} elements")
            tensor = tensor.data
        if not isinstance(tensor, torch.Tensor) or tensor.device != self.device:
            raise KernelError(f"{what}: expected a tensor on {self.device}, got "
                              f"{getattr(tensor, 'device', type(tensor))}")
        if not tensor.is_contiguous():
            raise KernelError(f"{what}: tensor must be contiguous")
        if dtypes is not None and tensor.dtype not in dtypes:
            raise KernelError(f"{what}: dtype {tensor.dtype} is not one of {dtypes}")
        return tensor.data_ptr()

    def _product(self, m, n, k, packed, activation):
        """What the library says of a product of these sizes, asked once per shape: (blocks its activations are
        read in, blocks it writes, whether it takes prepared norm rows, the blocks of a norm behind it, scratch
        bytes, whether its finishing kernel finishes a norm)."""
        key = (m, n, k, packed, activation)
        plan = self._plans.get(key)
        if plan is None:
            lib = self.lib
            plan = self._plans[key] = (
                int(lib.bh_gemm_bf16_reads_blocked(*key)), int(lib.bh_gemm_bf16_writes_blocked(*key)),
                bool(lib.bh_gemm_bf16_takes_norm(*key)) if k % 8 == 0 else False, int(lib.bh_gemm_bf16_norm_blocks(*key)),
                int(lib.bh_gemm_bf16_scratch(*key)), bool(packed and lib.bh_gemm_bf16_finishes_norm(m, n, k, 1)))
        return plan

    # ---- kernels ----
    def embed(self, tokens, table, out, token_src=None, fed_tokens=None):
        """out[row] = table[token of the row] widened to float32; tokens int32 [T], table [V, D], out f32 [T, D].
        With `token_src` (int32 [T]) and `fed_tokens` (int32, any length): where token_src[row] >= 0 the row's
        token is fed_tokens[token_src[row]], read on the device."""
        n_rows, width = out.shape
        if tokens.shape != (n_rows,) or table.dim() != 2 or table.shape[1] != width:
            raise KernelError(f"embed: shapes tokens {tuple(tokens.shape)}, table {tuple(table.shape)}, "
                              f"out {tuple(out.shape)} do not fit")
        if (token_src is None) != (fed_tokens is None) or (token_src is not None and token_src.shape != (n_rows,)):
            raise KernelError("embed: fed tokens come with one source index per row")
        self._check(self.lib.bh_embed(
            self._ptr(tokens, "embed tokens", (torch.int32,)), self._ptr(token_src, "embed token_src", (torch.int32,), True),
            self._ptr(fed_tokens, "embed fed tokens", (torch.int32,), True), self._ptr(table, "embed table"),
            _code(table, "embed table"), self._ptr(out, "embed out", (torch.float32,)), n_rows, width,
            table.shape[0], self._stream()))

    def rmsnorm(self, x, weight, eps, out, rows=None):
        """out[r] = x[rows[r] if rows is given else r] * inv_rms * weight; x f32 [*, D], out [n, D]."""
        n_rows, width = out.shape
        if x.dim() != 2 or x.shape[1] != width or (weight is not None and weight.shape != (width,)):
            raise KernelError(f"rmsnorm: shapes x {tuple(x.shape)}, out {tuple(out.shape)} do not fit")
        if rows is None:
            if x.shape[0] != n_rows:
                raise KernelError(f"rmsnorm: {x.shape[0]} input rows for {n_rows} output rows")
        elif rows.shape != (n_rows,):
            raise KernelError(f"rmsnorm: {tuple(rows.shape)} row indices for {n_rows} output rows")
        self._check(self.lib.bh_rmsnorm(
            self._ptr(x, "rmsnorm x", (torch.float32,)), self._ptr(rows, "rmsnorm rows", (torch.int32,), True),
            self._ptr(weight, "rmsnorm weight", None, True), _code(weight, "rmsnorm weight") if weight is not None else F32,
            self._ptr(out, "rmsnorm out"), _code(out, "rmsnorm out"), n_rows, width, float(eps), _block_rows(out),
            self._stream()))

    def new_rows(self, rows, width, dtype, reader_outputs=None, reader_swiglu=False, reader_packed=True):
        """An empty activation matrix [rows, width] for a kernel of this library to fill.  With `reader_outputs`,
        the product that reads it next has that many outputs (`reader_swiglu`: through the gate, so twice as
        many weight rows; `reader_packed`: its weight is a `PackedWeight`): where that product takes `BlockedRows`
        and reads them faster, the matrix is one."""
        rows, width = int(rows), int(width)
        if reader_outputs is not None and reader_packed and dtype == torch.bfloat16 and width % 64 == 0:
            block_rows = self._product(rows, int(reader_outputs), width, 1, int(bool(reader_swiglu)))[0]
            if block_rows:
                return self._new_blocked(rows, width, block_rows)
        return torch.empty((rows, width), dtype=dtype, device=self.device)

    def _new_blocked(self, rows, width, block_rows):
        padded = BlockedRows.padded_rows(rows, block_rows)
        return BlockedRows(torch.empty(padded * width, dtype=torch.bfloat16, device=self.device), rows, width, block_rows)

    def to_blocked(self, x, out=None, block_rows=16):
        """The bfloat16 matrix `x` as `BlockedRows` (into `out` if given, in its blocks)."""
        rows, width = x.shape
        if x.dtype != torch.bfloat16 or width % 32:
            raise KernelError(f"to_blocked: a bfloat16 matrix whose width is a multiple of 32, not {x.dtype} {tuple(x.shape)}")
        if out is None:
            out = self._new_blocked(rows, width, block_rows)
        elif not isinstance(out, BlockedRows) or tuple(out.shape) != (rows, width):
            raise KernelError(f"to_blocked: the output stands for {tuple(out.shape)}, the matrix is {tuple(x.shape)}")
        self._check(self.lib.bh_rows_blocked(self._ptr(x, "rows"), self._ptr(out, "blocks"), rows, width, 1, out.block_rows,
                                             self._stream()))
        return out

    def from_blocked(self, blocked):
        """The matrix that `blocked` stands for, row after row."""
        rows, width = blocked.shape
        out = torch.empty((rows, width), dtype=blocked.dtype, device=self.device)
        self._check(self.lib.bh_rows_blocked(self._ptr(blocked, "blocks"), self._ptr(out, "rows"), rows, width, 0,
                                             blocked.block_rows, self._stream()))
        return out

    def _in_blocks_of(self, x, block_rows):
        """`x` (rows or `BlockedRows`) in blocks of `block_rows` rows (0: as rows), regrouped if it lies otherwise."""
        if _block_rows(x) == block_rows:
            return x
        rows = self.from_blocked(x) if isinstance(x, BlockedRows) else x
        return self.to_blocked(rows, block_rows=block_rows) if block_rows else rows

    def pack_weight(self, w):
        """The form of a weight matrix that the matrix products read fastest: a `PackedWeight` for a
        bfloat16 matrix whose width is a multiple of 64, else the matrix itself."""
        if (isinstance(w, torch.Tensor) and w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[1] % 64 == 0):
            rows, cols = w.shape
            padded = -(-rows // 16) * 16
            if padded != rows:
                w = torch.cat([w, torch.zeros(padded - rows, cols, dtype=w.dtype, device=w.device)])
            # [block of 16 rows][block of 64 k][half u][lane group g][row i][8]
            data = w.view(padded // 16, 16, cols // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()
            return PackedWeight(data, rows, cols)
        return w

    def _gemm_fast(self, a, w, out, accumulate, activation, then_norm=None):
        """Launch the matrix-core product if it takes these operands; say whether it did, and with
        what prepared norm output (None if `then_norm` was not asked for or cannot ride on this product)."""
        fast = self.lib.bh_gemm_bf16
        packed = isinstance(w, PackedWeight)
        ahead = a if isinstance(a, NormedRows) else None
        if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or a.shape[1] % 8:
            if packed:
                raise KernelError("gemm: a packed weight needs bfloat16 activations")
            return False, None
        if activation and (out.shape[1] % 16 or accumulate):
            return False, None
        m, k = a.shape
        n = out.shape[1]
        sizes = (m, n, k, int(packed), int(activation))
        a_block_rows, writes, takes_norm, norm_blocks, scratch_bytes, finishes_norm = self._product(*sizes)
        if a_block_rows == 16 and m > 32 and not scratch_bytes and (ahead is not None or (accumulate and out.dtype != torch.float32)):
            a_block_rows = 0      # the kernel for many rows that reads blocks does not take these operands; the tiles read rows
        # the activations in the form this product reads: whoever produced them for this reader wrote them so
        if ahead is not None:
            if _block_rows(ahead.rows) != a_block_rows:
                ahead = NormedRows(self._in_blocks_of(ahead.rows, a_block_rows), ahead.ss, ahead.eps, ahead.source, ahead.weight)
        else:
            a = self._in_blocks_of(a, a_block_rows)
        c_block_rows = _block_rows(out)       # writes 2: any blocks, 1: SwiGLU's in blocks of 16, 0: rows
        if c_block_rows and not (activation and (writes == 2 or (writes == 1 and c_block_rows == 16))):
            return False, None      # the caller regroups
        if ahead is not None and (ahead.ss.shape[0] != m or ahead.ss.dtype != torch.float32
                                  or not takes_norm):
            raise KernelError(f"gemm: a product of {m} x {n} x {k} does not take these prepared norm rows")
        if (then_norm is not None and ahead is None and accumulate and packed and out.dtype == torch.float32
                and not activation and then_norm.weight.shape == (n,) and then_norm.weight.dtype in _CODES
                and finishes_norm):
            # many rows, K in parts: the finishing kernel owns whole rows and finishes the norm itself
            normed = self.new_rows(m, n, torch.bfloat16, *self._reader_of(then_norm))
            if _block_rows(normed) not in (0, 16):
                normed = torch.empty((m, n), dtype=torch.bfloat16, device=self.device)
            scratch = torch.empty(scratch_bytes // 4, dtype=torch.float32, device=self.device)
            self._check(self.lib.bh_gemm_bf16_then_norm(
                self._ptr(a, "gemm a"), self._ptr(w.data, "gemm w"), self._ptr(out, "gemm out", (torch.float32,)), m, n, k, 1,
                self._ptr(then_norm.weight, "norm weight"), _code(then_norm.weight, "norm weight"), float(then_norm.eps),
                self._ptr(normed, "norm rows"), self._ptr(scratch, "gemm scratch"), int(a_block_rows == 16),
                int(isinstance(normed, BlockedRows)), self._stream()))
            return True, normed
        behind = None
        if (then_norm is not None and out.dtype == torch.float32 and not activation
                and then_norm.weight.shape == (n,) and then_norm.weight.dtype in _CODES):
            blocks = norm_blocks      # 0: this product carries no norm
            if blocks:
                rows = self.new_rows(m, n, torch.bfloat16, *self._reader_of(then_norm)) if writes == 2 else \
                    torch.empty((m, n), dtype=torch.bfloat16, device=self.device)
                behind = NormedRows(rows, torch.empty((m, blocks), dtype=torch.float32, device=self.device), then_norm.eps,
                                    out, then_norm.weight)
        a_rows = ahead.rows if ahead is not None else a
        scratch = None       # products of few tiles add up parts of K through scratch memory
        if scratch_bytes:
            scratch = torch.empty(scratch_bytes // 4, dtype=torch.float32, device=self.device)
        self._check(fast(
            self._ptr(a_rows, "gemm a"), self._ptr(w.data if packed else w, "gemm w"), self._ptr(out, "gemm out"),
            _code(out, "gemm out"), int(bool(accumulate)), m, n, k, int(packed), int(activation),
            self._ptr(ahead.ss, "norm sums") if ahead is not None else None,
            ahead.ss.shape[1] if ahead is not None else 0, ahead.eps if ahead is not None else 0.0,
            self._ptr(then_norm.weight, "norm weight") if behind is not None else None,
            _code(then_norm.weight, "norm weight") if behind is not None else 0,
            self._ptr(behind.rows, "norm rows") if behind is not None else None,
            self._ptr(behind.ss, "norm sums") if behind is not None else None,
            self._ptr(scratch, "gemm scratch", None, True), a_block_rows, c_block_rows,
            _block_rows(behind.rows) if behind is not None else 0, self._stream()))
        return True, behind

    @staticmethod
    def _reader_of(then_norm):
        """The arguments of `new_rows` that name the product reading a norm's output, if the request names one."""
        reader = getattr(then_norm, "reader", None)
        return (reader.outputs, reader.swiglu, getattr(reader, "packed", True)) if reader is not None else ()

    def gemm(self, a, w, out, accumulate=False, then_norm=None):
        """out[M, N] (+)= a[M, K] @ w[N, K]^T with float32 accumulation; `w` may be a PackedWeight and
        `a` the NormedRows an earlier product prepared.  With `then_norm` (an object with `weight` [N] and
        `eps`: an RMSNorm over the rows of `out` as they are after this product) the product may prepare that norm's
        output on its way and return it, as NormedRows or, where it finishes the norm itself, as the bfloat16
        matrix the norm would have given; it returns None when it does neither (then run the norm as usual)."""
        if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
            raise KernelError("gemm: operands must be matrices")
        m, k = a.shape
        n = w.shape[0]
        if w.shape[1] != k or tuple(out.shape) != (m, n):
            raise KernelError(f"gemm: shapes a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        if isinstance(a, NormedRows) and not self._takes_norm(a, w, n, 0):
            a = self._run_norm(a)
        done, prepared = self._gemm_fast(a, w, out, accumulate, 0, then_norm)
        if done:
            return prepared
        if isinstance(a, BlockedRows):
            a = self.from_blocked(a)
        self._check(self.lib.bh_gemm_generic(
            self._ptr(a, "gemm a"), _code(a, "gemm a"), self._ptr(w, "gemm w"), _code(w, "gemm w"),
            self._ptr(out, "gemm out"), _code(out, "gemm out"), int(bool(accumulate)), m, n, k, self._stream()))
        return None

    def gemm_bare(self, a, w):
        """a[M, K] @ w[N, K]^T left as `PartSums`, where the product of these operands is one of many rows whose K the
        library cuts into parts (prompts of a few hundred to about 1,500 rows at the usual widths): the product
        without its finishing kernel, for a consumer that adds the parts up itself.  None where it is not (then call
        `gemm`)."""
        if (not isinstance(w, PackedWeight) or isinstance(a, NormedRows) or a.dim() != 2 or a.dtype != torch.bfloat16
                or a.shape[1] != w.shape[1]):
            return None
        m, k = a.shape
        n = w.shape[0]
        parts = self._bare.get((m, n, k))
        if parts is None:
            parts = self._bare[(m, n, k)] = int(self.lib.bh_gemm_bf16_bare_parts(m, n, k, 1))
        if not parts:
            return None
        a_block_rows = self._product(m, n, k, 1, 0)[0]
        a = self._in_blocks_of(a, a_block_rows)
        sums = torch.empty((parts, m, n), dtype=torch.float32, device=self.device)
        self._check(self.lib.bh_gemm_bf16_bare(self._ptr(a, "gemm a"), self._ptr(w.data, "gemm w"), self._ptr(sums, "gemm sums"),
                                               m, n, k, 1, int(a_block_rows == 16), self._stream()))
        return PartSums(sums)

    def qk_norm_rope_takes_sums(self, n_rows, head_dim, rot) -> bool:
        """Whether `qk_norm_rope_cache` takes `PartSums` for a step of these sizes (`rot`: the rotation's width, 0 for none)."""
        return bool(self.lib.bh_qk_norm_rope_cache_takes_sums(int(n_rows), int(head_dim), int(rot)))

    def gemm_turns(self, a, w, out, blocks, accumulate=False, swiglu=False):
        """The product for many rows whose wave groups take turns, at a given tile width (`blocks` of 16
        weight rows per wave: 8, 6 or 4), whatever `gemm` would choose for these sizes: out[M, N] (+)= a @ w^T,
        or with `swiglu` out[M, F] = silu(a @ w[:F]^T) * (a @ w[F:]^T).  `w` is a PackedWeight."""
        if (not isinstance(w, PackedWeight) or a.dim() != 2 or out.dim() != 2 or a.dtype != torch.bfloat16
                or _block_rows(a) not in (0, 16) or _block_rows(out) not in (0, 16)):
            raise KernelError("gemm_turns: bfloat16 activations [M, K] (rows or `BlockedRows` of 16) and a packed weight")
        m, k = a.shape
        n = out.shape[1]
        if w.shape[1] != k or w.shape[0] != (2 * n if swiglu else n) or out.shape[0] != m:
            raise KernelError(f"gemm_turns: shapes a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_gemm_bf16_turns(
            self._ptr(a, "gemm a"), self._ptr(w.data, "gemm w"), self._ptr(out, "gemm out"), _code(out, "gemm out"),
            int(bool(accumulate)), m, n, k, int(bool(swiglu)), int(blocks), int(_block_rows(a) == 16),
            int(_block_rows(out) == 16), self._stream()))

    def gemm_turns_blocks(self, m, n, k, swiglu=False):
        """The tile width `gemm` uses for a packed product of these sizes (0: another kernel runs it)."""
        return int(self.lib.bh_gemm_bf16_turns_blocks(m, n, k, 1, int(bool(swiglu))))

    def _takes_norm(self, a, w, n, activation):
        """Whether the matrix-core product of these operands applies the row factors of prepared norm rows."""
        m, k = a.shape
        return bool(w.dtype == torch.bfloat16 and k % 8 == 0 and (not activation or n % 16 == 0)
                    and self._product(m, n, k, int(isinstance(w, PackedWeight)), int(activation))[2])

    def _run_norm(self, prepared):
        """The norm that `prepared` stands for, as a step of its own."""
        out = torch.empty(tuple(prepared.shape), dtype=prepared.dtype, device=self.device)
        self.rmsnorm(prepared.source, prepared.weight, prepared.eps, out)
        return out

    def gemm_swiglu(self, a, w, out):
        """out[M, F] = silu(a @ w[:F]^T) * (a @ w[F:]^T) for w [2F, K] = gate rows, then up rows; `a` may
        be NormedRows."""
        if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
            raise KernelError("gemm_swiglu: operands must be matrices")
        m, k = a.shape
        width = out.shape[1]
        if tuple(w.shape) != (2 * width, k) or out.shape[0] != m or out.dtype != a.dtype:
            raise KernelError(f"gemm_swiglu: shapes a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} "
                              "do not fit")
        if isinstance(a, NormedRows) and width % 16 == 0 and not self._takes_norm(a, w, width, 1):
            a = self._run_norm(a)
        if self._gemm_fast(a, w, out, False, 1)[0]:
            return
        if isinstance(out, BlockedRows):      # this product writes rows, or not these blocks: regroup them afterwards
            rows_out = torch.empty((m, width), dtype=out.dtype, device=self.device)
            self.gemm_swiglu(a, w, rows_out)
            self.to_blocked(rows_out, out)
            return
        if isinstance(a, BlockedRows):
            a = self.from_blocked(a)
        both = torch.empty((m, 2 * width), dtype=a.dtype, device=self.device)
        self.gemm(a, w, both)
        self.swiglu(both, out)

    def qk_norm_rope_cache(self, qkv, q_out, q_weight, k_weight, eps, cos, sin, positions, row_seq,
                           k_pages, v_pages, page_table, n_heads, n_kv_heads, head_dim, write_kv, max_position):
        """Per head of the fused [q | k | v] projection rows: RMSNorm (when weights are given),
        split-half rotation at the row's position (when tables are given), then q to `q_out`
        and k, v into the cache pages of (sequence, position).  Rows may come in any order, each
        (sequence, position) once; where eight consecutive positions of a sequence are consecutive rows, as a step
        lays them out, the kernel for many rows writes their values as one piece."""
        n_rows = qkv.shape[0]
        fused = (n_heads + 2 * n_kv_heads) * head_dim
        if qkv.shape != (n_rows, fused) or q_out.shape != (n_rows, n_heads * head_dim) or q_out.dtype != qkv.dtype:
            raise KernelError(f"qk_norm_rope: shapes qkv {tuple(qkv.shape)}, q_out {tuple(q_out.shape)} do not fit "
                              f"{n_heads}+2x{n_kv_heads} heads of {head_dim}")
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,):
            raise KernelError("qk_norm_rope: positions and row_seq must have one entry per row")
        rot, table_positions = 0, 0
        if cos is not None:
            if cos.shape != sin.shape or cos.dim() != 2:
                raise KernelError("qk_norm_rope: cos and sin tables must be matrices of one shape")
            table_positions, rot = cos.shape[0], 2 * cos.shape[1]
        if (q_weight is None) != (k_weight is None):
            raise KernelError("qk_norm_rope: give both norm weights or neither")
        w_code = F32
        if q_weight is not None:
            if q_weight.shape != (head_dim,) or k_weight.shape != (head_dim,) or q_weight.dtype != k_weight.dtype:
                raise KernelError("qk_norm_rope: norm weights must be [head_dim] and of one dtype")
            w_code = _code(q_weight, "qk_norm_rope weight")
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, qkv.dtype, "qk_norm_rope")
        if isinstance(qkv, PartSums):
            if not self.qk_norm_rope_takes_sums(n_rows, head_dim, rot):
                raise KernelError(f"qk_norm_rope: sums in parts are not taken for {n_rows} rows, heads of {head_dim} "
                                  f"and a rotation over {rot} (qk_norm_rope_takes_sums says so beforehand)")
            first, second, entry = self._ptr(qkv.sums, "qkv sums", (torch.float32,)), qkv.parts, self.lib.bh_qk_norm_rope_cache_sums
        else:
            first, second, entry = self._ptr(qkv, "qkv"), _code(qkv, "qkv"), self.lib.bh_qk_norm_rope_cache
        self._check(entry(
            first, second, self._ptr(q_out, "q_out"),
            self._ptr(q_weight, "q_norm", None, True), self._ptr(k_weight, "k_norm", None, True), w_code,
            float(eps), self._ptr(cos, "cos", (torch.float32,), True), self._ptr(sin, "sin", (torch.float32,), True),
            table_positions, rot, self._ptr(positions, "positions", (torch.int32,)),
            self._ptr(row_seq, "row_seq", (torch.int32,)), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1], n_rows, n_heads, n_kv_heads,
            head_dim, int(bool(write_kv)), self.kv_order(k_pages.dtype, head_dim), int(max_position), self._stream()))

    def kv_order(self, dtype, head_dim) -> int:
        """How the elements of one head lie within a cache page of this element type and head size:
        0 = keys [token][dim] and values [dim][token]; 1 = regrouped in 16-byte pieces for the
        matrix-core attention kernel (bfloat16, head sizes in steps of 32).  The kernel that writes
        the cache and both attention kernels follow it, so a cache is only ever read the way it
        was written; whoever fills or inspects pages directly has to follow it too."""
        return int(self.lib.bh_kv_order(BF16 if dtype == torch.bfloat16 else F32, int(head_dim)))

    def _check_pages(self, k_pages, v_pages, page_table, n_kv_heads, head_dim, dtype, what):
        expected = (k_pages.shape[0], n_kv_heads, self.page_size, head_dim)
        expected_v = (k_pages.shape[0], n_kv_heads, head_dim, self.page_size)
        if k_pages.shape != expected or v_pages.shape != expected_v:
            raise KernelError(f"{what}: key pages must be [pages, {n_kv_heads}, {self.page_size}, {head_dim}] and value "
                              f"pages [pages, {n_kv_heads}, {head_dim}, {self.page_size}], got "
                              f"{tuple(k_pages.shape)} and {tuple(v_pages.shape)}")
        if k_pages.dtype != dtype or v_pages.dtype != dtype:
            raise KernelError(f"{what}: cache dtype {k_pages.dtype} differs from the activations' {dtype}")
        if page_table.dim() != 2:
            raise KernelError(f"{what}: the page table must be [sequences, pages]")

    def attention(self, q, out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                  scale, window=0, layout=None):
        """out[row, head] = softmax(q . K * scale) V over the keys of the row's sequence that the row
        may see: positions max(0, p - window + 1) .. p (window 0 = all).  `layout`, when given,
        says how rows group into sequences (seq_start int32 [n_seqs + 1] on the device, n_seqs,
        max_rows_per_seq, max_position), which the matrix-core kernel needs; rows of one sequence
        are consecutive and in position order."""
        n_rows = q.shape[0]
        if q.shape != (n_rows, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape) or out.dtype != q.dtype:
            raise KernelError(f"attention: shapes q {tuple(q.shape)}, out {tuple(out.shape)} do not fit")
        # the matrix-core kernels write blocks themselves: of 16 rows in steps of many columns, of 8 or 16 otherwise
        if isinstance(out, BlockedRows) and not (
                q.dtype == torch.bfloat16 and layout is not None and head_dim % 32 == 0 and head_dim <= 256
                and (out.block_rows == 16 or not self.lib.bh_attention_bf16_writes_blocked(
                    int(layout.n_seqs), int(layout.max_rows_per_seq), n_heads, n_kv_heads, int(layout.max_position)))):
            rows_out = torch.empty(tuple(q.shape), dtype=q.dtype, device=self.device)   # this step's kernel writes rows
            self.attention(q, rows_out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                           scale, window, layout)
            self.to_blocked(rows_out, out)
            return
        if n_heads % n_kv_heads != 0:
            raise KernelError(f"attention: {n_heads} query heads do not group evenly into {n_kv_heads} kv heads")
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,):
            raise KernelError("attention: positions and row_seq must have one entry per row")
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, q.dtype, "attention")
        common = (self._ptr(q, "q"), self._ptr(out, "attention out"))
        fast = self.lib.bh_attention_bf16
        if (q.dtype == torch.bfloat16 and layout is not None and head_dim % 32 == 0
                and head_dim <= 256):
            n_seqs, max_rows = int(layout.n_seqs), int(layout.max_rows_per_seq)
            if layout.seq_start.shape != (n_seqs + 1,) or page_table.shape[0] < n_seqs:
                raise KernelError("attention: seq_start must have one entry per sequence and one more, and the page "
                                  "table a row per sequence")
            n_splits = int(self.lib.bh_attention_bf16_splits(n_seqs, max_rows, n_heads, n_kv_heads,
                                                                      int(layout.max_position)))
            part_o = part_ml = None
            if n_splits > 1:   # partial results of the key splits: scratch for this call only
                part_o = torch.empty(n_rows * n_heads * n_splits * head_dim, dtype=torch.float32, device=self.device)
                part_ml = torch.empty(n_rows * n_heads * n_splits * 2, dtype=torch.float32, device=self.device)
            self._check(fast(*common, self._ptr(part_o, "partial o", None, True),
                             self._ptr(part_ml, "partial sums", None, True), self._ptr(k_pages, "k_pages"),
                             self._ptr(v_pages, "v_pages"), self._ptr(page_table, "page_table", (torch.int32,)),
                             page_table.shape[1], self._ptr(positions, "positions", (torch.int32,)),
                             self._ptr(layout.seq_start, "seq_start", (torch.int32,)), n_seqs, n_rows, max_rows,
                             n_heads, n_kv_heads, head_dim, float(scale), int(window), int(layout.max_position),
                             n_splits, _block_rows(out), self._stream()))
            return
        self._check(self.lib.bh_attention_generic(
            *common, _code(q, "q"), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1],
            self._ptr(row_seq, "row_seq", (torch.int32,)), self._ptr(positions, "positions", (torch.int32,)),
            n_rows, n_heads, n_kv_heads, head_dim, float(scale), int(window), self.kv_order(k_pages.dtype, head_dim),
            self._stream()))

    def attention_decode_fused(self, qkv, out, q_weight, k_weight, eps, cos, sin, positions, k_pages, v_pages,
                               page_table, n_heads, n_kv_heads, head_dim, scale, window, write_kv, layout):
        """`qk_norm_rope_cache` and `attention` in one launch for a step of one row per sequence, from
        the fused projection rows `qkv` [n, (heads + 2 kv_heads) * head_dim]; `out` may be `BlockedRows`.
        Returns False, having done nothing, where the one kernel that does it does not take the operands
        (then call the two)."""
        n_rows = qkv.shape[0]
        rot = 2 * cos.shape[1] if cos is not None else 0
        if (qkv.dtype != torch.bfloat16 or k_pages.dtype != torch.bfloat16 or layout is None
                or int(layout.max_rows_per_seq) != 1 or int(layout.n_seqs) != n_rows
                or head_dim % 32 or head_dim > 256 or n_heads % n_kv_heads or n_heads // n_kv_heads > 16
                or (cos is not None and (rot != head_dim or head_dim % 64))
                or self.kv_order(k_pages.dtype, head_dim) != 1):
            return False
        if qkv.shape != (n_rows, (n_heads + 2 * n_kv_heads) * head_dim) or tuple(out.shape) != (n_rows, n_heads * head_dim) \
                or out.dtype != qkv.dtype:
            raise KernelError(f"attention_decode_fused: shapes qkv {tuple(qkv.shape)}, out {tuple(out.shape)} do not fit "
                              f"{n_heads}+2x{n_kv_heads} heads of {head_dim}")
        if positions.shape != (n_rows,) or layout.seq_start.shape != (n_rows + 1,) or page_table.shape[0] < n_rows:
            raise KernelError("attention_decode_fused: one position and one page-table row per sequence, and seq_start")
        if (q_weight is None) != (k_weight is None) or (cos is None) != (sin is None):
            raise KernelError("attention_decode_fused: norm weights come in pairs, and so do the rotation tables")
        w_code = F32
        if q_weight is not None:
            if q_weight.shape != (head_dim,) or k_weight.shape != (head_dim,) or q_weight.dtype != k_weight.dtype:
                raise KernelError("attention_decode_fused: norm weights must be [head_dim] and of one dtype")
            w_code = _code(q_weight, "norm weight")
        if cos is not None and (cos.shape != sin.shape or cos.dim() != 2):
            raise KernelError("attention_decode_fused: cos and sin tables must be matrices of one shape")
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, head_dim, qkv.dtype, "attention_decode_fused")
        n_splits = int(self.lib.bh_attention_bf16_splits(n_rows, 1, n_heads, n_kv_heads, int(layout.max_position)))
        part_o = part_ml = None
        if n_splits > 1:
            part_o = torch.empty(n_rows * n_heads * n_splits * head_dim, dtype=torch.float32, device=self.device)
            part_ml = torch.empty(n_rows * n_heads * n_splits * 2, dtype=torch.float32, device=self.device)
        self._check(self.lib.bh_attention_decode_fused(
            self._ptr(qkv, "qkv"), self._ptr(out, "attention out"), self._ptr(part_o, "partial o", None, True),
            self._ptr(part_ml, "partial sums", None, True), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1],
            self._ptr(positions, "positions", (torch.int32,)), self._ptr(layout.seq_start, "seq_start", (torch.int32,)),
            n_rows, n_heads, n_kv_heads, head_dim, float(scale), int(window), int(layout.max_position), n_splits,
            self._ptr(q_weight, "q_norm", None, True), self._ptr(k_weight, "k_norm", None, True), w_code, float(eps),
            self._ptr(cos, "cos", (torch.float32,), True), self._ptr(sin, "sin", (torch.float32,), True),
            cos.shape[0] if cos is not None else 0, rot, int(bool(write_kv)), _block_rows(out), self._stream()))
        return True

    def stream_read(self, data, workgroups=256, nontemporal=True) -> int:
        """A yardstick, not a product path: read `data` (any contiguous tensor) once the way the streaming kernels
        read; returns the number of bytes read (whole 64 KB per workgroup)."""
        sink = torch.zeros(1, dtype=torch.int32, device=self.device)
        count = ctypes.c_long(0)
        self._check(self.lib.bh_stream_read(self._ptr(data, "data"), data.numel() * data.element_size(), int(workgroups),
                                            int(bool(nontemporal)), self._ptr(sink, "sink"), ctypes.byref(count), self._stream()))
        return int(count.value)

    def swiglu(self, gate_up, out):
        """out[r, i] = silu(gate_up[r, i]) * gate_up[r, F + i]."""
        n_rows, width = out.shape
        if gate_up.shape != (n_rows, 2 * width) or gate_up.dtype != out.dtype:
            raise KernelError(f"swiglu: shapes {tuple(gate_up.shape)} -> {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_swiglu(self._ptr(gate_up, "gate_up"), self._ptr(out, "swiglu out"),
                                       _code(out, "swiglu out"), n_rows, width, self._stream()))

    def sample(self, logits, tokens, bad, temperature=None, top_k=None, top_p=None, uniform=None):
        """tokens[row] = argmax (temperature absent or <= 0) or a draw from the tempered, filtered
        distribution; bad[row] = 1 where a logit is not finite."""
        n_rows, vocab = logits.shape
        for name, tensor, dtype in (("tokens", tokens, torch.int32), ("bad", bad, torch.int32)):
            if tensor.shape != (n_rows,) or tensor.dtype != dtype:
                raise KernelError(f"sample: {name} must be {dtype} [{n_rows}]")
        for name, tensor, dtype in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                                    ("top_p", top_p, torch.float32), ("uniform", uniform, torch.float32)):
            if tensor is not None and (tensor.shape != (n_rows,) or tensor.dtype != dtype):
                raise KernelError(f"sample: {name} must be {dtype} [{n_rows}]")
        if temperature is not None and uniform is None:
            raise KernelError("sample: temperature sampling needs uniform numbers")
        scratch = None
        if temperature is None:      # greedy rows of a long vocabulary are searched chunk by chunk
            words = int(self.lib.bh_sample_scratch(n_rows, vocab))
            if words:
                scratch = torch.empty(words, dtype=torch.float32, device=self.device)
        elif top_k is None and top_p is None:      # a draw from the whole distribution likewise
            words = int(self.lib.bh_sample_draw_scratch(n_rows, vocab))
            if words:
                scratch = torch.empty(words, dtype=torch.float32, device=self.device)
        else:                                      # and the chunks' candidates for a top-k or a top-p
            words = int(self.lib.bh_sample_top_k_scratch(n_rows, vocab))
            if words:
                scratch = torch.empty(words, dtype=torch.float32, device=self.device)
        self._check(self.lib.bh_sample(
            self._ptr(logits, "logits", (torch.float32,)), self._ptr(temperature, "temperature", None, True),
            self._ptr(top_k, "top_k", None, True), self._ptr(top_p, "top_p", None, True),
            self._ptr(uniform, "uniform", None, True), self._ptr(tokens, "tokens"), self._ptr(bad, "bad"),
            self._ptr(scratch, "sample scratch", None, True), n_rows, vocab, self._stream()))
