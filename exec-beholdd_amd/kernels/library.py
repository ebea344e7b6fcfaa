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
            "bh_attention_generic": [p, p, i, p, p, p, i, p, p, i, i, i, i, f, i, i, p, p],
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
            "bh_attention_bf16": [p, p, p, p, p, p, p, i, p, p, i, i, i, i, i, i, f, i, i, i, i, p, p],
            "bh_attention_bf16_splits": [i, i, i, i, i],
            "bh_attention_bf16_writes_blocked": [i, i, i, i, i],
            "bh_attention_decode_fused": [p, p, p, p, p, p, p, i, p, p, i, i, i, i, f, i, i, i, p, p, i, f, p, p, i, i,
                                          i, i, p],
            "bh_kv_order": [i, i],
            "bh_stream_read": [p, ctypes.c_long, i, i, p, p, p],
            "bh_streams_open": [p, p, i, i, i, p],
            "bh_streams_rmsnorm": [p, p, p, p, p, i, i, i, i, f, i, p],
            "bh_streams_update": [p, p, p, p, p, i, i, i, p],
            "bh_streams_update_rmsnorm": [p, p, p, p, p, p, p, p, i, i, i, i, f, i, p],
            "bh_scale": [p, ctypes.c_long, f, p],
            "bh_relu_squared": [p, p, i, i, i, i, p],
            "bh_lightning_scan": [p, i, i, i, i, i, p, p, p, p, p, i, i, i, i, i, i, p, ctypes.c_long, p],
            "bh_lightning_chunks": [i, i, i, i, i, p],
            "bh_gated_rmsnorm": [p, p, i, i, p, p, i, i, f, i, p],
            "bh_latent_write": [p, i, i, i, p, f, p, i, p, p, p, p, p, i, i, i, i, i, i, p, ctypes.c_long, i, i, i, i, i, p, ctypes.c_long, i, f, p],
            "bh_heads_linear": [p, ctypes.c_long, i, i, p, p, ctypes.c_long, i, i, i, i, i, i, i, i, p],
            "bh_rotate_heads": [p, ctypes.c_long, i, i, p, ctypes.c_long, i, i, i, p, i, p, i, i, i, p],
            "bh_layernorm": [p, p, p, p, p, i, i, i, f, i, p],
            "bh_cast_concat": [p, p, p, i, i, i, i, p],
            "bh_sum_layernorm": [p, p, f, p, p, p, i, i, i, f, i, p],
            "bh_gelu_tanh": [p, p, i, i, i, i, p],
            "bh_head_norm_rope_write": [p, i, i, i, p, p, p, f, p, i, p, p, p, p, p, p, i, i, i, i, i, i, i, i, i, i, f, p],
            "bh_mlstm_gates": [p, p, f, p, ctypes.c_long, i, p, p, p, i, i, p],
            "bh_mlstm_scan": [p, i, i, i, i, i, p, p, ctypes.c_long, p, p, p, i, i, i, i, p],
            "bh_mlstm_finish": [p, p, p, i, i, i, p, f, p, i, i, i, i, p],
            "bh_mlstm_step": [p, i, i, i, i, i, i, p, p, f, p, ctypes.c_long, p, p, f, p, i, i, i, i, i, p],
            "bh_softcap": [p, ctypes.c_long, f, p],
            "bh_rms_scale_add": [p, p, p, i, i, f, p],
            "bh_gelu_gate_table": [p, i, p, p, p, p, i, i, i, p, i, i, i, p],
            "bh_short_conv": [p, i, i, i, p, p, p, ctypes.c_long, p, p, p, p, i, i, i, i, p],
            "bh_short_conv_state": [p, i, i, i, p, ctypes.c_long, p, p, i, i, i, p],
            "bh_whole_norm_rope_write": [p, p, p, f, p, i, p, p, p, i, p, p, p, i, i, i, i, i, i, i, i, i, p],
            "bh_gate_heads": [p, i, i, p, i, i, p, i, i, i, i, i, p],
            "bh_ssm_scan": [p, i, p, i, i, i, p, p, p, p, ctypes.c_long, p, p, p, i, i, i, i, i, p],
            "bh_gated_group_rmsnorm": [p, p, i, i, i, p, f, p, i, i, i, i, i, p],
            "bh_route_top_k": [p, p, p, p, i, i, i, i, p],
            "bh_experts_gate_up": [p, i, p, p, p, i, i, i, i, f, f, f, p, p],
            "bh_experts_down": [p, i, p, p, p, p, i, i, i, i, p],
            "bh_clamped_glu": [p, i, p, i, i, f, f, i, f, p],
            "bh_conv_norm_rope_write": [p, i, i, i, p, i, p, ctypes.c_long, p, p, p, p, f, p, i, p, p, p, p, p, p, i, i, i, i, i, i, i, i, i, p],
            "bh_ssm_scan_fast": [p, i, p, i, i, i, p, p, p, p, ctypes.c_long, p, p, p, p, p, p, i, i, i, i, i, i, i, p],
            "bh_ssm_chunk_rows": [i, i, i],
            "bh_ssm_fast_takes": [i, i],
            "bh_experts_products": [p, p, p, i, p, i, i, i, f, f, f, p],
            "bh_experts_products_takes": [i, i],
            "bh_experts_group": [p, i, p, i, p, i, p],
            "bh_experts_rows": [p, i, i, p, i, p, p, p, i, i, i, i, f, f, f, p, p],
            "bh_experts_gather": [p, i, i, p, i, p, p, p, p, i, i, i, p, p],
            "bh_gla_scan": [p, i, i, i, i, i, p, i, p, f, f, p, ctypes.c_long, p, p, p, i, i, i, i, i, i, i, p, p],
            "bh_gla_chunk_rows": [i, i, i, i, i],
            "bh_slice_rmsnorm": [p, i, i, i, p, f, p, i, i, i, p],
            "bh_weighted_sum": [p, p, f, p, f, ctypes.c_long, p],
            "bh_experts_combine": [p, p, p, p, i, i, i, p],
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

    def ssm_chunk_bytes(self, n_seqs, n_rows, max_rows, n_heads, vdim, n_state) -> int:
        """Bytes of scratch memory that `ssm_scan` allocates for a step of these sizes (sequences cut into chunks)."""
        if not self.lib.bh_ssm_fast_takes(int(vdim), int(n_state)):
            return 0
        chunk_rows = int(self.lib.bh_ssm_chunk_rows(int(n_seqs), int(max_rows), int(n_heads)))
        chunks = -(-int(max_rows) // chunk_rows)
        if chunks <= 1:
            return 0
        return (_rounded(n_seqs * chunks * n_heads * n_state * vdim * 4) + _rounded(n_seqs * chunks * n_heads * 4)
                + _rounded(n_rows * n_heads * 4))

    def gla_chunk_bytes(self, n_seqs, n_rows, max_rows, n_heads, dim, vdim) -> int:
        """Bytes of scratch memory that `gla_scan` allocates for a step of these sizes (long sequences cut into chunks)."""
        chunk_rows = int(self.lib.bh_gla_chunk_rows(int(n_seqs), int(max_rows), int(n_heads), int(dim), int(vdim)))
        if chunk_rows >= max_rows:
            return 0
        chunks = -(-int(max_rows) // chunk_rows)
        return _rounded((n_seqs * chunks * n_heads * dim * (vdim + 1) + n_rows * n_heads * dim) * 4)

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
                  scale, window=0, layout=None, chunk=0, sinks=None):
        """out[row, head] = softmax(q . K * scale) V over the keys of the row's sequence that the row
        may see: positions max(0, p - window + 1) .. p with a window, p - p % chunk .. p with chunks (counted from
        the sequence's position 0), else 0 .. p; not both.  `layout`, when given,
        says how rows group into sequences (seq_start int32 [n_seqs + 1] on the device, n_seqs,
        max_rows_per_seq, max_position), which the matrix-core kernel needs; rows of one sequence
        are consecutive and in position order.  `sinks` (float32 [n_heads]): exp(sinks[head]) is one more term of the
        head's softmax sums, with no key and no value."""
        n_rows = q.shape[0]
        if sinks is not None and (sinks.shape != (n_heads,) or sinks.dtype != torch.float32):
            raise KernelError(f"attention: one float32 sink a head ({n_heads}), got {tuple(sinks.shape)} of {sinks.dtype}")
        if window < 0 or chunk < 0 or (window and chunk):
            raise KernelError(f"attention: a window ({window}) or chunks ({chunk}) of a positive count of positions, not both")
        if chunk:
            window = -int(chunk)      # the kernels' one number for both (csrc/layout.h: bh_first_visible)
        if q.shape != (n_rows, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape) or out.dtype != q.dtype:
            raise KernelError(f"attention: shapes q {tuple(q.shape)}, out {tuple(out.shape)} do not fit")
        # the matrix-core kernels write blocks themselves: of 16 rows in steps of many columns, of 8 or 16 otherwise
        if isinstance(out, BlockedRows) and not (
                q.dtype == torch.bfloat16 and layout is not None and head_dim % 32 == 0 and head_dim <= 256
                and (out.block_rows == 16 or not self.lib.bh_attention_bf16_writes_blocked(
                    int(layout.n_seqs), int(layout.max_rows_per_seq), n_heads, n_kv_heads, int(layout.max_position)))):
            rows_out = torch.empty(tuple(q.shape), dtype=q.dtype, device=self.device)   # this step's kernel writes rows
            self.attention(q, rows_out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                           scale, max(window, 0), layout, chunk, sinks)
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
                             n_splits, _block_rows(out), self._ptr(sinks, "sinks", (torch.float32,), True), self._stream()))
            return
        self._check(self.lib.bh_attention_generic(
            *common, _code(q, "q"), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1],
            self._ptr(row_seq, "row_seq", (torch.int32,)), self._ptr(positions, "positions", (torch.int32,)),
            n_rows, n_heads, n_kv_heads, head_dim, float(scale), int(window), self.kv_order(k_pages.dtype, head_dim),
            self._ptr(sinks, "sinks", (torch.float32,), True), self._stream()))

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

    # ---- several residual streams, and sublayer results kept apart from the residual ----
    def streams_open(self, x, out):
        """out[row, s, :] = x[row, :] for every stream s; x f32 [n, D], out f32 [n, S, D]."""
        n_rows, streams, width = out.shape
        if tuple(x.shape) != (n_rows, width):
            raise KernelError(f"streams_open: shapes x {tuple(x.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_streams_open(self._ptr(x, "streams_open x", (torch.float32,)),
                                             self._ptr(out, "streams_open out", (torch.float32,)), n_rows, width, streams,
                                             self._stream()))

    def streams_rmsnorm(self, x, take, weight, eps, out, rows=None):
        """out[r] = RMSNorm(sum_s take[s] * x[src, s, :]) * weight with src = rows[r] if rows is given else r;
        x f32 [*, S, D], take f32 [S] or None (every stream once), weight f32 [D] or None, out [n, D] (rows or
        `BlockedRows`)."""
        n_rows, width = out.shape
        if x.dim() != 3 or x.shape[2] != width or (weight is not None and weight.shape != (width,)) \
                or (take is not None and take.shape != (x.shape[1],)):
            raise KernelError(f"streams_rmsnorm: shapes x {tuple(x.shape)}, out {tuple(out.shape)} do not fit")
        if rows is None:
            if x.shape[0] != n_rows:
                raise KernelError(f"streams_rmsnorm: {x.shape[0]} input rows for {n_rows} output rows")
        elif rows.shape != (n_rows,):
            raise KernelError(f"streams_rmsnorm: {tuple(rows.shape)} row indices for {n_rows} output rows")
        self._check(self.lib.bh_streams_rmsnorm(
            self._ptr(x, "streams_rmsnorm x", (torch.float32,)), self._ptr(rows, "streams_rmsnorm rows", (torch.int32,), True),
            self._ptr(take, "streams_rmsnorm take", (torch.float32,), True),
            self._ptr(weight, "streams_rmsnorm weight", (torch.float32,), True), self._ptr(out, "streams_rmsnorm out"),
            _code(out, "streams_rmsnorm out"), n_rows, width, x.shape[1], float(eps), _block_rows(out), self._stream()))

    def streams_update(self, x, y, mix=None, give=None, scale=None):
        """x[row, t, :] <- sum_s mix[s, t] * x[row, s, :] + give[t] * scale * y[row, :], all streams at once from the
        old ones; x f32 [n, S, D] in place, y f32 [n, D], mix f32 [S, S] or None (identity), give f32 [S] or None
        (ones), scale f32 [D] or None."""
        n_rows, streams, width = x.shape
        if tuple(y.shape) != (n_rows, width) or (mix is not None and tuple(mix.shape) != (streams, streams)) \
                or (give is not None and tuple(give.shape) != (streams,)) or (scale is not None and tuple(scale.shape) != (width,)):
            raise KernelError(f"streams_update: shapes x {tuple(x.shape)}, y {tuple(y.shape)} do not fit")
        f32 = (torch.float32,)
        self._check(self.lib.bh_streams_update(
            self._ptr(x, "streams_update x", f32), self._ptr(y, "streams_update y", f32),
            self._ptr(mix, "streams_update mix", f32, True), self._ptr(give, "streams_update give", f32, True),
            self._ptr(scale, "streams_update scale", f32, True), n_rows, width, streams, self._stream()))

    def streams_update_rmsnorm(self, x, y, mix, give, scale, take, weight, eps, out):
        """`streams_update(x, y, mix, give, scale)` and then `streams_rmsnorm(x, take, weight, eps, out)` of every row, in one
        pass over the streams."""
        n_rows, streams, width = x.shape
        if tuple(y.shape) != (n_rows, width) or tuple(out.shape) != (n_rows, width) \
                or (mix is not None and tuple(mix.shape) != (streams, streams)) \
                or any(t is not None and tuple(t.shape) != (streams,) for t in (give, take)) \
                or any(t is not None and tuple(t.shape) != (width,) for t in (scale, weight)):
            raise KernelError(f"streams_update_rmsnorm: shapes x {tuple(x.shape)}, y {tuple(y.shape)}, out {tuple(out.shape)} do not fit")
        f32 = (torch.float32,)
        self._check(self.lib.bh_streams_update_rmsnorm(
            self._ptr(x, "streams x", f32), self._ptr(y, "streams y", f32), self._ptr(mix, "streams mix", f32, True),
            self._ptr(give, "streams give", f32, True), self._ptr(scale, "streams scale", f32, True),
            self._ptr(take, "streams take", f32, True), self._ptr(weight, "norm weight", f32, True), self._ptr(out, "norm out"),
            _code(out, "norm out"), n_rows, width, streams, float(eps), _block_rows(out), self._stream()))

    def scale(self, x, factor):
        """x *= factor, in place; x float32."""
        self._check(self.lib.bh_scale(self._ptr(x, "scale x", (torch.float32,)), x.numel(), float(factor), self._stream()))

    def relu_squared(self, x, out=None):
        """out <- max(x, 0)^2; in place without `out`, which may be `BlockedRows` for the product that reads it next."""
        out = x if out is None else out
        if x.dim() != 2 or tuple(out.shape) != tuple(x.shape) or out.dtype != x.dtype:
            raise KernelError(f"relu_squared: shapes {tuple(x.shape)} -> {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_relu_squared(self._ptr(x, "relu_squared x"), self._ptr(out, "relu_squared out"),
                                             _code(x, "relu_squared x"), x.shape[0], x.shape[1], _block_rows(out), self._stream()))

    # ---- linear attention with a decay, as a recurrence over a float32 state ----
    def lightning_chunk_bytes(self, n_seqs, n_rows, max_rows, n_heads, dim, vdim) -> int:
        """Bytes of scratch memory that `lightning_scan` allocates for a step of these sizes (the states of the chunks it cuts
        long sequences into)."""
        rows = ctypes.c_int(0)
        chunks = int(self.lib.bh_lightning_chunks(int(n_seqs), int(n_rows), int(max_rows), int(n_heads), int(vdim), ctypes.byref(rows)))
        return _rounded(n_seqs * chunks * n_heads * dim * vdim * 4) if chunks > 1 else 0

    def lightning_scan(self, proj, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_heads, dim, vdim,
                       max_rows_per_seq=None):
        """For every sequence b of the step (rows seq_start[b] .. seq_start[b + 1] - 1 in order, state row seq_slot[b]) and
        head h: S <- decay[h] * S + k_t v_t^T, out_t = S^T q_t with q, k, v = silu of the row's slices from q_off, k_off,
        v_off of `proj` [n, P].  state f32 [slots, H, dim, vdim] in place, out f32 [n, H * vdim].  `max_rows_per_seq`: no
        sequence of the step brings more rows (the step's total, if it is not given); long sequences that would leave the
        chip idle are cut into chunks that run side by side, whose states take scratch memory for the length of the call."""
        n_rows, stride = proj.shape
        n_seqs = seq_slot.shape[0]
        if (state.dim() != 4 or tuple(state.shape[1:]) != (n_heads, dim, vdim) or tuple(out.shape) != (n_rows, n_heads * vdim)
                or tuple(decay.shape) != (n_heads,) or tuple(seq_start.shape) != (n_seqs + 1,)):
            raise KernelError(f"lightning_scan: shapes proj {tuple(proj.shape)}, state {tuple(state.shape)}, out "
                              f"{tuple(out.shape)} do not fit {n_heads} heads of {dim} x {vdim} and {n_seqs} sequences")
        f32, i32 = (torch.float32,), (torch.int32,)
        most = min(int(max_rows_per_seq), n_rows) if max_rows_per_seq else n_rows
        chunk_rows = ctypes.c_int(0)
        chunks = int(self.lib.bh_lightning_chunks(n_seqs, n_rows, most, n_heads, vdim, ctypes.byref(chunk_rows)))
        scratch = torch.empty(n_seqs * chunks * n_heads * dim * vdim, dtype=torch.float32, device=self.device) if chunks > 1 else None
        self._check(self.lib.bh_lightning_scan(
            self._ptr(proj, "lightning proj"), _code(proj, "lightning proj"), stride, int(q_off), int(k_off), int(v_off),
            self._ptr(state, "lightning state", f32), self._ptr(decay, "lightning decay", f32),
            self._ptr(seq_start, "seq_start", i32), self._ptr(seq_slot, "seq_slot", i32), self._ptr(out, "lightning out", f32),
            n_seqs, n_rows, most, n_heads, dim, vdim, self._ptr(scratch, "chunk states", f32, True),
            scratch.numel() if scratch is not None else 0, self._stream()))

    def gated_rmsnorm(self, o, proj, gate_off, weight, eps, out):
        """out[r] = RMSNorm(o[r]) * weight * sigmoid(proj[r, gate_off : gate_off + W]); o f32 [n, W], out [n, W] in the
        type of `proj` (rows or `BlockedRows`)."""
        n_rows, width = o.shape
        if tuple(out.shape) != (n_rows, width) or proj.shape[0] != n_rows or gate_off < 0 or gate_off + width > proj.shape[1] \
                or out.dtype != proj.dtype or (weight is not None and tuple(weight.shape) != (width,)):
            raise KernelError(f"gated_rmsnorm: shapes o {tuple(o.shape)}, proj {tuple(proj.shape)}, out {tuple(out.shape)} do not fit")
        gate = self._ptr(proj, "gated_rmsnorm gate") + int(gate_off) * proj.element_size()
        self._check(self.lib.bh_gated_rmsnorm(
            self._ptr(o, "gated_rmsnorm o", (torch.float32,)), gate,
            _code(proj, "gated_rmsnorm gate"), proj.shape[1], self._ptr(weight, "gated_rmsnorm weight", (torch.float32,), True),
            self._ptr(out, "gated_rmsnorm out"), n_rows, width, float(eps), _block_rows(out), self._stream()))

    # ---- gated linear attention: a matrix state whose rows decay by factors that the token sets ----
    def gla_scan(self, proj, q_off, k_off, v_off, z, bias, tau, q_scale, state, seq_start, seq_slot, out, n_heads, dim, vdim,
                 max_rows_per_seq=None):
        """Per (sequence, head): S <- diag(alpha_t) S + k_t v_t^T, out_t = S^T (q_scale q_t), alpha_t = sigmoid(z_t + bias)^(1/tau),
        over the sequence's rows in order, from and into state[slot].  proj [n, P] holds q, k (H x dim) and v (H x vdim) from the
        given columns; z f32 [n, H dim]; bias f32 [H dim]; state f32 [slots, H, dim, vdim]; out f32 [n, H vdim].
        `max_rows_per_seq` (the rows of the step's longest sequence; all rows where it is not said) lets long sequences be walked
        in chunks side by side, with scratch memory for this call."""
        n_rows = proj.shape[0]
        n_seqs = seq_slot.shape[0]
        most = int(max_rows_per_seq) if max_rows_per_seq else n_rows
        chunk_rows = int(self.lib.bh_gla_chunk_rows(n_seqs, most, n_heads, dim, vdim))
        scratch = None
        if chunk_rows < most:
            chunks = -(-most // chunk_rows)
            scratch = torch.empty(n_seqs * chunks * n_heads * dim * (vdim + 1) + n_rows * n_heads * dim, dtype=torch.float32, device=self.device)
        if tuple(out.shape) != (n_rows, n_heads * vdim) or z.shape != (n_rows, n_heads * dim) or bias.shape != (n_heads * dim,) \
                or seq_start.shape != (n_seqs + 1,) or state.dim() != 4 or tuple(state.shape[1:]) != (n_heads, dim, vdim):
            raise KernelError(f"gla_scan: shapes proj {tuple(proj.shape)}, z {tuple(z.shape)}, state {tuple(state.shape)}, "
                              f"out {tuple(out.shape)} do not fit")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_gla_scan(
            self._ptr(proj, "gla_scan proj"), _code(proj, "gla_scan proj"), proj.shape[1], int(q_off), int(k_off), int(v_off),
            self._ptr(z, "gla_scan decays", f32), z.shape[1], self._ptr(bias, "gla_scan bias", f32), float(tau), float(q_scale),
            self._ptr(state, "gla_scan state", f32), n_heads * dim * vdim, self._ptr(seq_start, "seq_start", i32),
            self._ptr(seq_slot, "seq_slot", i32), self._ptr(out, "gla_scan out", f32), n_seqs, n_heads, dim, vdim, n_rows, most,
            chunk_rows, self._ptr(scratch, "gla_scan scratch", f32, True), self._stream()))

    def slice_rmsnorm(self, x, first, weight, eps, out):
        """out[r] = x[r, first : first + W] / sqrt(mean of its squares + eps) * weight; x [n, P] and out [n, W] (rows or
        `BlockedRows`) in the activations' type, weight f32 [W]."""
        n_rows, width = out.shape
        if x.shape[0] != n_rows or first < 0 or first + width > x.shape[1] or out.dtype != x.dtype or weight.shape != (width,):
            raise KernelError(f"slice_rmsnorm: shapes x {tuple(x.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_slice_rmsnorm(
            self._ptr(x, "slice_rmsnorm x"), _code(x, "slice_rmsnorm x"), x.shape[1], int(first),
            self._ptr(weight, "slice_rmsnorm weight", (torch.float32,)), float(eps), self._ptr(out, "slice_rmsnorm out"), n_rows, width,
            _block_rows(out), self._stream()))

    def weighted_sum(self, out, x, a, y, b):
        """out = a x + b y, float32 tensors of one shape (out may be x or y)."""
        if x.shape != y.shape or out.shape != x.shape:
            raise KernelError(f"weighted_sum: shapes {tuple(out.shape)}, {tuple(x.shape)}, {tuple(y.shape)} differ")
        f32 = (torch.float32,)
        self._check(self.lib.bh_weighted_sum(self._ptr(out, "weighted_sum out", f32), self._ptr(x, "weighted_sum x", f32), float(a),
                                             self._ptr(y, "weighted_sum y", f32), float(b), x.numel(), self._stream()))

    # ---- attention over a cached latent ----
    def latent_write(self, down, offset, weight, eps, freq, turned, positions, row_seq, k_pages, v_pages, page_table,
                     rank, rot_dim, write=True, query=None, query_head=0, query_first=0, source_head=0, source_first=0, n_heads=0,
                     query_source=None, neighbours=False, magnitude=1.0):
        """From each row of `down` [n, P], at `offset`: c = RMSNorm(rank elements) * weight and the next rot_dim elements
        rotated (the first `turned` of them, pairs (i, i + turned/2), angle position * freq[i]); key [c | rotated] and
        value [c | 0] of ONE kv head of size rank + rot_dim go into the cache pages of (sequence, position) (unless
        `write` is False).  With `query` [n, >= n_heads * query_head] the same launch rotates the rot_dim elements at
        `source_first` of each of the row's `n_heads` heads (`source_head` apart) into query[row, h * query_head + query_first ..];
        the heads are those of `query_source` [n, >= n_heads * source_head] where one is given, else of `down`'s rows.
        `neighbours`: a pair is dimensions (2i, 2i + 1) instead; `magnitude` multiplies every cosine and sine."""
        n_rows = down.shape[0]
        if query_source is not None and (query_source.dim() != 2 or query_source.shape[0] != n_rows or query_source.dtype != down.dtype):
            raise KernelError(f"latent_write: the queries' source {tuple(query_source.shape)} does not fit {n_rows} rows of {down.dtype}")
        head = rank + rot_dim
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,) or (weight is not None and tuple(weight.shape) != (rank,)) \
                or (freq is not None and tuple(freq.shape) != (turned // 2,)):
            raise KernelError("latent_write: one position and one sequence per row, a weight [rank] and a frequency a pair")
        if query is not None and (query.dim() != 2 or query.shape[0] != n_rows or query.dtype != down.dtype):
            raise KernelError(f"latent_write: the queries {tuple(query.shape)} do not fit {n_rows} rows of {down.dtype}")
        self._check_pages(k_pages, v_pages, page_table, 1, head, down.dtype, "latent_write")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_latent_write(
            self._ptr(down, "latent rows"), _code(down, "latent rows"), down.shape[1], int(offset),
            self._ptr(weight, "latent norm weight", f32, True), float(eps), self._ptr(freq, "rotation frequencies", f32, True),
            int(turned), self._ptr(positions, "positions", i32), self._ptr(row_seq, "row_seq", i32),
            self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"), self._ptr(page_table, "page_table", i32),
            page_table.shape[1], n_rows, int(rank), int(rot_dim), self.kv_order(k_pages.dtype, head), int(bool(write)),
            self._ptr(query, "rotated queries", None, True), query.shape[1] if query is not None else 0, int(query_head),
            int(query_first), int(source_head), int(source_first), int(n_heads),
            self._ptr(query_source, "queries' source", None, True), query_source.shape[1] if query_source is not None else 0,
            int(bool(neighbours)), float(magnitude), self._stream()))

    def heads_linear(self, x, x_head, x_first, w, y, y_head, y_first, n_heads):
        """y[row, h, y_first + o] = sum_i w[h, i, o] * x[row, h, x_first + i]: x [n, >= H * x_head] and y [n, >= H * y_head]
        are rows of heads of x_head and y_head elements, w [H, n_in, n_out] of their type; float32 sums.  `y` may be
        `BlockedRows` (for the product that reads it next)."""
        n_rows = x.shape[0]
        if w.dim() != 3 or w.shape[0] != n_heads or y.shape[0] != n_rows or x.dtype != w.dtype or y.dtype != w.dtype:
            raise KernelError(f"heads_linear: shapes x {tuple(x.shape)}, w {tuple(w.shape)}, y {tuple(y.shape)} do not fit")
        self._check(self.lib.bh_heads_linear(
            self._ptr(x, "heads_linear x"), x.shape[1], int(x_head), int(x_first), self._ptr(w, "heads_linear w"),
            self._ptr(y, "heads_linear y"), y.shape[1], int(y_head), int(y_first), _code(w, "heads_linear w"), n_rows, n_heads,
            w.shape[1], w.shape[2], _block_rows(y), self._stream()))

    def rotate_heads(self, x, x_head, x_first, y, y_head, y_first, freq, turned, positions, n_heads, width):
        """y[row, h, y_first + i] = x[row, h, x_first + i] for i < width, the first `turned` of them rotated in pairs
        (i, i + turned/2) by position[row] * freq[i]."""
        n_rows = x.shape[0]
        if y.shape[0] != n_rows or positions.shape != (n_rows,) or x.dtype != y.dtype \
                or (freq is not None and tuple(freq.shape) != (turned // 2,)):
            raise KernelError(f"rotate_heads: shapes x {tuple(x.shape)}, y {tuple(y.shape)} do not fit")
        self._check(self.lib.bh_rotate_heads(
            self._ptr(x, "rotate_heads x"), x.shape[1], int(x_head), int(x_first), self._ptr(y, "rotate_heads y"), y.shape[1],
            int(y_head), int(y_first), _code(x, "rotate_heads x"), self._ptr(freq, "rotation frequencies", (torch.float32,), True),
            int(turned), self._ptr(positions, "positions", (torch.int32,)), n_rows, n_heads, int(width), self._stream()))

    # ---- row-wise operations on the residual and on logits ----
    def layernorm(self, x, weight, bias, eps, out, rows=None):
        """out[r] = (x[row] - mean) / sqrt(var + eps) * weight + bias, row = rows[r] if rows is given else r; x f32 [*, D],
        weight and bias f32 [D] (bias may be None), out [n, D] in rows or blocks of rows."""
        n_rows, width = out.shape
        if x.dim() != 2 or x.shape[1] != width or weight.shape != (width,) or (bias is not None and bias.shape != (width,)):
            raise KernelError(f"layernorm: shapes x {tuple(x.shape)}, out {tuple(out.shape)} do not fit")
        if (rows is None and x.shape[0] != n_rows) or (rows is not None and rows.shape != (n_rows,)):
            raise KernelError(f"layernorm: the input rows do not fit {n_rows} output rows")
        self._check(self.lib.bh_layernorm(
            self._ptr(x, "layernorm x", (torch.float32,)), self._ptr(rows, "layernorm rows", (torch.int32,), True),
            self._ptr(weight, "layernorm weight", (torch.float32,)), self._ptr(bias, "layernorm bias", (torch.float32,), True),
            self._ptr(out, "layernorm out"), _code(out, "layernorm out"), n_rows, width, float(eps), _block_rows(out), self._stream()))

    def sum_layernorm(self, hidden, y, alpha, weight, bias, eps, rounded=None):
        """hidden[r] <- layernorm(alpha * hidden[r] + y[r]) * weight + bias in place (all f32, the variance as the mean of
        the squared deviations); `rounded` [n, D], if given, takes the same in its own type, in rows or blocks of rows."""
        n_rows, width = hidden.shape
        if tuple(y.shape) != (n_rows, width) or weight.shape != (width,) or (bias is not None and bias.shape != (width,)) \
                or (rounded is not None and tuple(rounded.shape) != (n_rows, width)):
            raise KernelError(f"sum_layernorm: shapes hidden {tuple(hidden.shape)}, y {tuple(y.shape)} do not fit")
        self._check(self.lib.bh_sum_layernorm(
            self._ptr(hidden, "sum_layernorm hidden", (torch.float32,)), self._ptr(y, "sum_layernorm y", (torch.float32,)), float(alpha),
            self._ptr(weight, "sum_layernorm weight", (torch.float32,)), self._ptr(bias, "sum_layernorm bias", (torch.float32,), True),
            self._ptr(rounded, "sum_layernorm rounded", None, True), _code(rounded, "sum_layernorm rounded") if rounded is not None else F32,
            n_rows, width, float(eps), _block_rows(rounded) if rounded is not None else 0, self._stream()))

    def gelu_tanh(self, x, out=None):
        """out <- x/2 (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))); in place without `out`, which may be `BlockedRows`."""
        out = x if out is None else out
        if x.dim() != 2 or tuple(out.shape) != tuple(x.shape) or out.dtype != x.dtype:
            raise KernelError(f"gelu_tanh: shapes {tuple(x.shape)} -> {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_gelu_tanh(self._ptr(x, "gelu_tanh x"), self._ptr(out, "gelu_tanh out"), _code(x, "gelu_tanh x"),
                                          x.shape[0], x.shape[1], _block_rows(out), self._stream()))

    def head_norm_rope_write(self, proj, first, bias, q_weight, k_weight, eps, freq, turned, positions, row_seq, q_out, k_pages,
                             v_pages, page_table, n_heads, n_kv_heads, dim, vdim, pad, write_kv, neighbours=False,
                             magnitude=1.0):
        """From column `first` of every row of `proj` [n, P]: q (H heads of dim), k (G of dim), v (G of vdim), plus `bias` (f32
        over those channels, or None); every head of q and k normed by its own root mean square times q_weight / k_weight
        (f32 [dim], both or None); dimensions i and i + turned/2 of every head of q and k turned by position * freq[i];
        (`neighbours`: dimensions 2i and 2i + 1 instead; `magnitude` multiplies every cosine and sine);
        q -> q_out [n, H pad], k and v into the cache pages as heads of `pad` (see csrc/head_norm_attention.hip)."""
        n_rows = proj.shape[0]
        channels = (n_heads + n_kv_heads) * dim + n_kv_heads * vdim
        if tuple(q_out.shape) != (n_rows, n_heads * pad) or q_out.dtype != proj.dtype or first < 0 or first + channels > proj.shape[1]:
            raise KernelError(f"head_norm_rope_write: shapes proj {tuple(proj.shape)}, q_out {tuple(q_out.shape)} do not fit")
        if (q_weight is None) != (k_weight is None) or (q_weight is not None and (q_weight.shape != (dim,) or k_weight.shape != (dim,))):
            raise KernelError("head_norm_rope_write: one norm weight per dimension of a head, for queries and keys alike")
        if bias is not None and bias.shape != (channels,):
            raise KernelError(f"head_norm_rope_write: a bias per channel ({channels}), got {tuple(bias.shape)}")
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,):
            raise KernelError("head_norm_rope_write: positions and row_seq must have one entry per row")
        if turned and (freq is None or freq.shape != (turned // 2,)):
            raise KernelError("head_norm_rope_write: one frequency per turned pair")
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, pad, q_out.dtype, "head_norm_rope_write")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_head_norm_rope_write(
            self._ptr(proj, "proj"), _code(proj, "proj"), proj.shape[1], int(first), self._ptr(bias, "bias", f32, True),
            self._ptr(q_weight, "q norm", f32, True), self._ptr(k_weight, "k norm", f32, True), float(eps),
            self._ptr(freq, "frequencies", f32, True), int(turned), self._ptr(positions, "positions", i32),
            self._ptr(row_seq, "row_seq", i32), self._ptr(q_out, "q_out"), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", i32), page_table.shape[1], n_rows, n_heads, n_kv_heads, dim, vdim, pad,
            self.kv_order(k_pages.dtype, pad), int(bool(write_kv)), int(bool(neighbours)), float(magnitude), self._stream()))

    # ---- a matrix memory with exponential gates, as a recurrence over a float32 state ----
    MLSTM_BESIDE = 4      # floats a row and head beside the read-out: a_t, b_t, m_t, n_t . q_t

    @staticmethod
    def mlstm_state_floats(n_heads, dim, vdim) -> int:
        """Floats of a sequence's state: per head vdim + 1 columns of dim (the last one n), then m."""
        return n_heads * ((vdim + 1) * dim + 1)

    def mlstm_gates(self, pre, bias, cap, state, seq_start, seq_slot, beside, n_heads, dim, vdim):
        """beside[row, head] = (a_t, b_t, m_t, .) from the gates' pre-activations pre f32 [n, 2 H] (input gates, then forget
        gates) plus bias f32 [2 H]: i = cap tanh(x_i / cap), f = logsigmoid(cap tanh(x_f / cap)), m_t = max(f + m_(t-1), i),
        a = exp(f + m_(t-1) - m_t), b = exp(i - m_t); the rows of sequence b (seq_start) in order from the m of state row
        seq_slot[b], which is moved on.  state f32 [slots, mlstm_state_floats]."""
        n_rows = pre.shape[0]
        n_seqs = seq_slot.shape[0]
        if tuple(pre.shape) != (n_rows, 2 * n_heads) or tuple(beside.shape) != (n_rows, n_heads * self.MLSTM_BESIDE) \
                or state.dim() != 2 or state.shape[1] < self.mlstm_state_floats(n_heads, dim, vdim) \
                or tuple(seq_start.shape) != (n_seqs + 1,) or (bias is not None and tuple(bias.shape) != (2 * n_heads,)):
            raise KernelError(f"mlstm_gates: shapes pre {tuple(pre.shape)}, state {tuple(state.shape)}, beside {tuple(beside.shape)} "
                              f"do not fit {n_heads} heads of {dim} x {vdim} and {n_seqs} sequences")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_mlstm_gates(
            self._ptr(pre, "mlstm gates", f32), self._ptr(bias, "mlstm gate bias", f32, True), float(cap),
            self._ptr(state, "mlstm state", f32), state.shape[1], (vdim + 1) * dim + 1, self._ptr(seq_start, "seq_start", i32),
            self._ptr(seq_slot, "seq_slot", i32), self._ptr(beside, "mlstm beside", f32), n_seqs, n_heads, self._stream()))

    def mlstm_scan(self, proj, q_off, k_off, v_off, beside, state, seq_start, seq_slot, read, n_heads, dim, vdim):
        """For every sequence of the step and head: S <- a_t S + b_t k_t [v_t | 1]^T over the sequence's rows in order (a_t, b_t
        from `beside`), read[row, head] = S^T q_t / sqrt(dim) over the vdim value columns and beside[row, head, 3] = the same
        over the column of ones (n . q); q, k, v are the row's slices of `proj` [n, P] from q_off, k_off, v_off."""
        n_rows = proj.shape[0]
        n_seqs = seq_slot.shape[0]
        if tuple(read.shape) != (n_rows, n_heads * vdim) or tuple(beside.shape) != (n_rows, n_heads * self.MLSTM_BESIDE) \
                or state.dim() != 2 or state.shape[1] < self.mlstm_state_floats(n_heads, dim, vdim) \
                or tuple(seq_start.shape) != (n_seqs + 1,):
            raise KernelError(f"mlstm_scan: shapes proj {tuple(proj.shape)}, state {tuple(state.shape)}, read {tuple(read.shape)} "
                              f"do not fit {n_heads} heads of {dim} x {vdim} and {n_seqs} sequences")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_mlstm_scan(
            self._ptr(proj, "mlstm proj"), _code(proj, "mlstm proj"), proj.shape[1], int(q_off), int(k_off), int(v_off),
            self._ptr(beside, "mlstm beside", f32), self._ptr(state, "mlstm state", f32), state.shape[1],
            self._ptr(seq_start, "seq_start", i32), self._ptr(seq_slot, "seq_slot", i32), self._ptr(read, "mlstm read", f32),
            n_seqs, n_heads, dim, vdim, self._stream()))

    def mlstm_finish(self, read, beside, proj, gate_off, weight, eps, out, n_heads, vdim):
        """out[r, h] = rms-normed over vdim (read[r, h] / (max(|n . q|, exp(-m)) + 1e-6)) * weight * sigmoid(proj[r, gate_off ..]);
        out [n, H vdim] in the type of `proj`, rows or `BlockedRows`."""
        n_rows = read.shape[0]
        width = n_heads * vdim
        if tuple(read.shape) != (n_rows, width) or tuple(beside.shape) != (n_rows, n_heads * self.MLSTM_BESIDE) \
                or tuple(out.shape) != (n_rows, width) or proj.shape[0] != n_rows or out.dtype != proj.dtype \
                or (weight is not None and tuple(weight.shape) != (width,)):
            raise KernelError(f"mlstm_finish: shapes read {tuple(read.shape)}, proj {tuple(proj.shape)}, out {tuple(out.shape)} do not fit")
        f32 = (torch.float32,)
        self._check(self.lib.bh_mlstm_finish(
            self._ptr(read, "mlstm read", f32), self._ptr(beside, "mlstm beside", f32), self._ptr(proj, "mlstm gate"),
            _code(proj, "mlstm gate"), proj.shape[1], int(gate_off), self._ptr(weight, "mlstm norm weight", f32, True), float(eps),
            self._ptr(out, "mlstm out"), n_rows, n_heads, vdim, _block_rows(out), self._stream()))

    def mlstm_step(self, proj, q_off, k_off, v_off, gate_off, pre, bias, cap, state, seq_slot, weight, eps, out, n_heads, dim, vdim):
        """`mlstm_gates`, `mlstm_scan` and `mlstm_finish` in one launch for a step in which sequence b brings the one row b
        (a decode step): the same arguments, the same numbers left in the slots' states, out [n, H vdim] in rows or blocks."""
        n_rows = proj.shape[0]
        width = n_heads * vdim
        if seq_slot.shape != (n_rows,) or tuple(pre.shape) != (n_rows, 2 * n_heads) or tuple(out.shape) != (n_rows, width) \
                or out.dtype != proj.dtype or state.dim() != 2 or state.shape[1] < self.mlstm_state_floats(n_heads, dim, vdim) \
                or (bias is not None and tuple(bias.shape) != (2 * n_heads,)) or (weight is not None and tuple(weight.shape) != (width,)):
            raise KernelError(f"mlstm_step: shapes proj {tuple(proj.shape)}, pre {tuple(pre.shape)}, state {tuple(state.shape)}, out "
                              f"{tuple(out.shape)} do not fit {n_heads} heads of {dim} x {vdim} and a row a sequence")
        f32, i32 = (torch.float32,), (torch.int32,)
        self._check(self.lib.bh_mlstm_step(
            self._ptr(proj, "mlstm proj"), _code(proj, "mlstm proj"), proj.shape[1], int(q_off), int(k_off), int(v_off), int(gate_off),
            self._ptr(pre, "mlstm gates", f32), self._ptr(bias, "mlstm gate bias", f32, True), float(cap),
            self._ptr(state, "mlstm state", f32), state.shape[1], self._ptr(seq_slot, "seq_slot", i32),
            self._ptr(weight, "mlstm norm weight", f32, True), float(eps), self._ptr(out, "mlstm out"), n_rows, n_heads, dim, vdim,
            _block_rows(out), self._stream()))

    def cast_concat(self, a, b, out):
        """out[r] = [a[r] | b[r]] in out's type; a, b f32 [n, D] (b may be None), out [n, 2 D] (or [n, D])."""
        n_rows, width = a.shape
        total = 2 * width if b is not None else width
        if tuple(out.shape) != (n_rows, total) or (b is not None and tuple(b.shape) != (n_rows, width)):
            raise KernelError(f"cast_concat: shapes a {tuple(a.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_cast_concat(
            self._ptr(a, "cast_concat a", (torch.float32,)), self._ptr(b, "cast_concat b", (torch.float32,), True),
            self._ptr(out, "cast_concat out"), _code(out, "cast_concat out"), n_rows, width, _block_rows(out), self._stream()))

    def softcap(self, x, cap):
        """x <- cap * tanh(x / cap) in place; x f32."""
        self._check(self.lib.bh_softcap(self._ptr(x, "softcap x", (torch.float32,)), x.numel(), float(cap), self._stream()))

    def rms_scale_add(self, hidden, y, weight, eps):
        """hidden[r] += y[r] / sqrt(mean(y[r]^2) + eps) * weight; all f32."""
        n_rows, width = hidden.shape
        if tuple(y.shape) != (n_rows, width) or weight.shape != (width,):
            raise KernelError(f"rms_scale_add: shapes hidden {tuple(hidden.shape)}, y {tuple(y.shape)} do not fit")
        self._check(self.lib.bh_rms_scale_add(
            self._ptr(hidden, "rms_scale_add hidden", (torch.float32,)), self._ptr(y, "rms_scale_add y", (torch.float32,)),
            self._ptr(weight, "rms_scale_add weight", (torch.float32,)), n_rows, width, float(eps), self._stream()))

    def gelu_gate_table(self, gate, tokens, table, first, out, token_src=None, fed_tokens=None):
        """out[r, i] = gelu_tanh(gate[r, i]) * table[token of r, first + i]; gate, out [n, dim], table [V, W] of one type."""
        n_rows, dim = gate.shape
        if tuple(out.shape) != (n_rows, dim) or tokens.shape != (n_rows,) or table.dim() != 2 or table.dtype != gate.dtype \
                or out.dtype != gate.dtype:
            raise KernelError(f"gelu_gate_table: shapes gate {tuple(gate.shape)}, table {tuple(table.shape)} do not fit")
        if (token_src is None) != (fed_tokens is None) or (token_src is not None and token_src.shape != (n_rows,)):
            raise KernelError("gelu_gate_table: fed tokens come with one source index per row")
        self._check(self.lib.bh_gelu_gate_table(
            self._ptr(gate, "gelu_gate_table gate"), _code(gate, "gelu_gate_table gate"), self._ptr(tokens, "tokens", (torch.int32,)),
            self._ptr(token_src, "token_src", (torch.int32,), True), self._ptr(fed_tokens, "fed tokens", (torch.int32,), True),
            self._ptr(table, "gelu_gate_table table"), table.shape[1], int(first), table.shape[0], self._ptr(out, "gelu_gate_table out"),
            n_rows, dim, _block_rows(out), self._stream()))

    # ---- a short convolution over time, continued through a state ----
    @staticmethod
    def _state_view(state, offset, floats, what):
        """(address of the region at `offset` floats into every slot's row of `state`, floats from slot to slot)."""
        if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() < 2:
            raise KernelError(f"{what}: the state is a contiguous float32 tensor [slots, ...]")
        per_slot = state.numel() // state.shape[0]
        if offset < 0 or offset + floats > per_slot:
            raise KernelError(f"{what}: {floats} floats at {offset} do not lie inside a slot's {per_slot}")
        return state.data_ptr() + 4 * int(offset), per_slot

    def short_conv(self, u, first, weight, bias, state, state_offset, row_seq, seq_start, seq_slot, out, silu=False):
        """out[t, c] = sum_j weight[c, j] * u[t - taps + 1 + j, first + c] (+ bias[c]) (then silu) over the rows of each
        sequence of the step; inputs before the step come from the sequence's state region ([taps - 1, C] f32 at
        `state_offset` floats into state[slot]).  u [n, W], weight f32 [C, taps], out f32 [n, C]."""
        n_rows, channels = out.shape
        taps = weight.shape[1]
        if u.shape[0] != n_rows or weight.shape[0] != channels or (bias is not None and bias.shape != (channels,)):
            raise KernelError(f"short_conv: shapes u {tuple(u.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)} do not fit")
        where, stride = None, 0      # one tap reads no earlier row
        if taps > 1:
            where, stride = self._state_view(state, state_offset, (taps - 1) * channels, "short_conv")
            self._ptr(state, "short_conv state", (torch.float32,))
        self._check(self.lib.bh_short_conv(
            self._ptr(u, "short_conv u"), _code(u, "short_conv u"), u.shape[1], int(first),
            self._ptr(weight, "short_conv weight", (torch.float32,)), self._ptr(bias, "short_conv bias", (torch.float32,), True),
            where, stride, self._ptr(row_seq, "row_seq", (torch.int32,)), self._ptr(seq_start, "seq_start", (torch.int32,)),
            self._ptr(seq_slot, "seq_slot", (torch.int32,)), self._ptr(out, "short_conv out", (torch.float32,)), n_rows, channels,
            taps, int(bool(silu)), self._stream()))

    def short_conv_state(self, u, first, channels, taps, state, state_offset, seq_start, seq_slot):
        """The state after the step: the last taps - 1 inputs of every sequence (old ones where the step brought fewer)."""
        n_seqs = seq_slot.shape[0]
        if seq_start.shape != (n_seqs + 1,):
            raise KernelError("short_conv_state: seq_start has one entry per sequence and one more")
        where, stride = self._state_view(state, state_offset, (taps - 1) * channels, "short_conv_state")
        self._ptr(state, "short_conv state", (torch.float32,))
        self._check(self.lib.bh_short_conv_state(
            self._ptr(u, "short_conv_state u"), _code(u, "short_conv_state u"), u.shape[1], int(first), where, stride,
            self._ptr(seq_start, "seq_start", (torch.int32,)), self._ptr(seq_slot, "seq_slot", (torch.int32,)), n_seqs, int(channels),
            int(taps), self._stream()))

    # ---- attention with queries and keys normed over the whole projection ----
    def whole_norm_rope_write(self, qkv, q_weight, k_weight, eps, freq, turned, positions, row_seq, q_out, k_pages, v_pages,
                              page_table, n_heads, n_kv_heads, dim, vdim, pad, write_kv):
        """qkv f32 [n, H dim + G dim + G vdim] -> q_out [n, H pad] and the cache pages of heads of `pad` (see
        csrc/whole_norm_attention.hip)."""
        n_rows = qkv.shape[0]
        if qkv.shape != (n_rows, (n_heads + n_kv_heads) * dim + n_kv_heads * vdim) or tuple(q_out.shape) != (n_rows, n_heads * pad):
            raise KernelError(f"whole_norm_rope_write: shapes qkv {tuple(qkv.shape)}, q_out {tuple(q_out.shape)} do not fit")
        if q_weight.shape != (n_heads * dim,) or k_weight.shape != (n_kv_heads * dim,):
            raise KernelError("whole_norm_rope_write: one norm weight per query channel and per key channel")
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,):
            raise KernelError("whole_norm_rope_write: positions and row_seq must have one entry per row")
        if turned and (freq is None or freq.shape != (turned // 2,)):
            raise KernelError("whole_norm_rope_write: one frequency per turned pair")
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, pad, q_out.dtype, "whole_norm_rope_write")
        self._check(self.lib.bh_whole_norm_rope_write(
            self._ptr(qkv, "qkv", (torch.float32,)), self._ptr(q_weight, "q norm", (torch.float32,)),
            self._ptr(k_weight, "k norm", (torch.float32,)), float(eps), self._ptr(freq, "frequencies", (torch.float32,), True),
            int(turned), self._ptr(positions, "positions", (torch.int32,)), self._ptr(row_seq, "row_seq", (torch.int32,)),
            self._ptr(q_out, "q_out"), _code(q_out, "q_out"), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1], n_rows, n_heads, n_kv_heads, dim, vdim, pad,
            self.kv_order(k_pages.dtype, pad), int(bool(write_kv)), self._stream()))

    CONV_WALK_ROWS = 128      # from that many rows a step's convolution walks down the rows (csrc/short_conv.hip)
    CONV_ROW_IN_LDS = 30000   # channels of q, k and v together that the one launch keeps in local memory

    def conv_norm_rope_write(self, proj, first, conv_weight, state, state_offset, seq_start, seq_slot, q_weight, k_weight, eps, freq,
                             turned, positions, row_seq, q_out, k_pages, v_pages, page_table, n_heads, n_kv_heads, dim, vdim, pad, write_kv):
        """`short_conv` of the q, k, v channels of `proj` (from column `first`; conv_weight f32 [channels, taps], or None for no
        convolution) and `whole_norm_rope_write` of the result in one launch: the convolved row is never written to memory.  The
        state is read, not updated (`short_conv_state` afterwards).  A step of many rows runs the two kernels after all: the
        convolution that walks down the rows loads every input once, where a workgroup per row loads it once per tap."""
        n_rows = proj.shape[0]
        channels = (n_heads + n_kv_heads) * dim + n_kv_heads * vdim
        walks = n_rows >= self.CONV_WALK_ROWS and conv_weight is not None and 2 <= conv_weight.shape[1] <= 4
        if walks or channels > self.CONV_ROW_IN_LDS:      # (a row of more channels does not fit the one launch's local memory)
            weight = conv_weight if conv_weight is not None else torch.ones((channels, 1), dtype=torch.float32, device=self.device)
            conv = torch.empty((n_rows, channels), dtype=torch.float32, device=self.device)
            self.short_conv(proj, first, weight, None, state if weight.shape[1] > 1 else None, state_offset, row_seq, seq_start, seq_slot, conv)
            self.whole_norm_rope_write(conv, q_weight, k_weight, eps, freq, turned, positions, row_seq, q_out, k_pages, v_pages, page_table,
                                       n_heads, n_kv_heads, dim, vdim, pad, write_kv)
            return
        taps = conv_weight.shape[1] if conv_weight is not None else 0
        if tuple(q_out.shape) != (n_rows, n_heads * pad) or q_out.dtype != proj.dtype or (conv_weight is not None and conv_weight.shape[0] != channels):
            raise KernelError(f"conv_norm_rope_write: shapes proj {tuple(proj.shape)}, q_out {tuple(q_out.shape)} do not fit")
        if q_weight.shape != (n_heads * dim,) or k_weight.shape != (n_kv_heads * dim,):
            raise KernelError("conv_norm_rope_write: one norm weight per query channel and per key channel")
        if positions.shape != (n_rows,) or row_seq.shape != (n_rows,) or seq_start.shape != (seq_slot.shape[0] + 1,):
            raise KernelError("conv_norm_rope_write: positions and row_seq have one entry per row, seq_start one per sequence and one more")
        if turned and (freq is None or freq.shape != (turned // 2,)):
            raise KernelError("conv_norm_rope_write: one frequency per turned pair")
        where, stride = None, 0
        if taps > 1:
            where, stride = self._state_view(state, state_offset, (taps - 1) * channels, "conv_norm_rope_write")
            self._ptr(state, "conv state", (torch.float32,))
        self._check_pages(k_pages, v_pages, page_table, n_kv_heads, pad, q_out.dtype, "conv_norm_rope_write")
        self._check(self.lib.bh_conv_norm_rope_write(
            self._ptr(proj, "proj"), _code(proj, "proj"), proj.shape[1], int(first), self._ptr(conv_weight, "conv weight", (torch.float32,), True),
            taps, where, stride, self._ptr(seq_start, "seq_start", (torch.int32,)), self._ptr(seq_slot, "seq_slot", (torch.int32,)),
            self._ptr(q_weight, "q norm", (torch.float32,)), self._ptr(k_weight, "k norm", (torch.float32,)), float(eps),
            self._ptr(freq, "frequencies", (torch.float32,), True), int(turned), self._ptr(positions, "positions", (torch.int32,)),
            self._ptr(row_seq, "row_seq", (torch.int32,)), self._ptr(q_out, "q_out"), self._ptr(k_pages, "k_pages"), self._ptr(v_pages, "v_pages"),
            self._ptr(page_table, "page_table", (torch.int32,)), page_table.shape[1], n_rows, n_heads, n_kv_heads, dim, vdim, pad,
            self.kv_order(k_pages.dtype, pad), int(bool(write_kv)), self._stream()))

    def gate_heads(self, attended, pad, gate, gate_first, out, n_heads, vdim, per_head=False):
        """out[r, h, i] = attended[r, h, i] * sigmoid(gate[r, gate_first + h vdim + i]), i < vdim; attended [n, H pad].
        `per_head`: one gate a head, gate[r, gate_first + h].  `gate` None: no gate, the heads' first vdim elements side by side."""
        n_rows = attended.shape[0]
        if attended.shape != (n_rows, n_heads * pad) or tuple(out.shape) != (n_rows, n_heads * vdim) or (gate is not None and (gate.shape[0] != n_rows \
                or gate.dtype != attended.dtype)) or out.dtype != attended.dtype:
            raise KernelError(f"gate_heads: shapes attended {tuple(attended.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_gate_heads(
            self._ptr(attended, "gate_heads attended"), _code(attended, "gate_heads attended"), int(pad), self._ptr(gate, "gate_heads gate", None, True),
            gate.shape[1] if gate is not None else 0, int(gate_first), self._ptr(out, "gate_heads out"), n_rows, n_heads, vdim, _block_rows(out), int(bool(per_head)), self._stream()))

    # ---- a state-space recurrence with a scalar decay per head ----
    def ssm_scan(self, xbc, proj, dt_first, dt_bias, a_log, d_skip, state, state_offset, seq_start, seq_slot, out, n_heads, vdim,
                 n_state, n_groups, max_rows_per_seq=None):
        """Per (sequence, head): S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + d_skip x with dt = softplus(proj[:, dt_first
        + head] + dt_bias); xbc f32 [n, H vdim + 2 G N] = [x | B | C], S [H, N, vdim] f32 at `state_offset` floats into
        state[slot], out f32 [n, H vdim].  `max_rows_per_seq` (the most rows any sequence brings; the step's rows if not
        given) decides whether long sequences are cut into chunks that run side by side."""
        n_rows, n_seqs = xbc.shape[0], seq_slot.shape[0]
        inner = n_heads * vdim
        if xbc.shape != (n_rows, inner + 2 * n_groups * n_state) or tuple(out.shape) != (n_rows, inner) or proj.shape[0] != n_rows:
            raise KernelError(f"ssm_scan: shapes xbc {tuple(xbc.shape)}, out {tuple(out.shape)} do not fit")
        if seq_start.shape != (n_seqs + 1,) or any(t.shape != (n_heads,) for t in (dt_bias, a_log, d_skip)):
            raise KernelError("ssm_scan: one dt_bias, A_log and D per head, and seq_start with one entry per sequence and one more")
        where, stride = self._state_view(state, state_offset, n_heads * n_state * vdim, "ssm_scan")
        self._ptr(state, "ssm_scan state", (torch.float32,))
        common = (self._ptr(xbc, "ssm_scan xbc", (torch.float32,)), xbc.shape[1], self._ptr(proj, "ssm_scan proj"), _code(proj, "ssm_scan proj"),
                  proj.shape[1], int(dt_first), self._ptr(dt_bias, "dt_bias", (torch.float32,)), self._ptr(a_log, "A_log", (torch.float32,)),
                  self._ptr(d_skip, "D", (torch.float32,)), where, stride)
        rest = (self._ptr(seq_start, "seq_start", (torch.int32,)), self._ptr(seq_slot, "seq_slot", (torch.int32,)),
                self._ptr(out, "ssm_scan out", (torch.float32,)), n_seqs, n_heads, vdim, n_state, n_groups)
        if not self.lib.bh_ssm_fast_takes(int(vdim), int(n_state)):
            self._check(self.lib.bh_ssm_scan(*common, *rest, self._stream()))
            return
        most = int(max_rows_per_seq) if max_rows_per_seq else n_rows
        chunk_rows = int(self.lib.bh_ssm_chunk_rows(n_seqs, most, n_heads))
        chunks = -(-most // chunk_rows)
        states = decays = cum = None
        if chunks > 1:
            states = torch.empty((n_seqs * chunks, n_heads, n_state, vdim), dtype=torch.float32, device=self.device)
            decays = torch.empty((n_seqs * chunks, n_heads), dtype=torch.float32, device=self.device)
            cum = torch.empty((n_rows, n_heads), dtype=torch.float32, device=self.device)
        self._check(self.lib.bh_ssm_scan_fast(
            *common, self._ptr(states, "chunk states", None, True), self._ptr(decays, "chunk decays", None, True),
            self._ptr(cum, "row decays", None, True), *rest, chunk_rows, chunks, self._stream()))

    def gated_group_rmsnorm(self, y, z, z_first, weight, eps, out, groups, gate_after=False):
        """out = rms_g(y * silu(z[:, z_first : z_first + W])) * weight, the root mean square over each of `groups` equal
        parts of a row; y f32 [n, W], weight f32 [W], out [n, W] of z's type.
        `gate_after`: the statistic is y's alone, out = rms_g(y) * weight * silu(z)."""
        n_rows, width = y.shape
        if tuple(out.shape) != (n_rows, width) or z.shape[0] != n_rows or weight.shape != (width,) or out.dtype != z.dtype:
            raise KernelError(f"gated_group_rmsnorm: shapes y {tuple(y.shape)}, z {tuple(z.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_gated_group_rmsnorm(
            self._ptr(y, "gated_group_rmsnorm y", (torch.float32,)), self._ptr(z, "gated_group_rmsnorm z"), _code(z, "gated_group_rmsnorm z"),
            z.shape[1], int(z_first), self._ptr(weight, "gated_group_rmsnorm weight", (torch.float32,)), float(eps),
            self._ptr(out, "gated_group_rmsnorm out"), n_rows, width, int(groups), _block_rows(out), int(bool(gate_after)), self._stream()))

    # ---- routed experts ----
    def route_top_k(self, logits, bias, chosen, weights, scoring="softmax"):
        """chosen[r] = the `top` largest of logits[r] + bias (largest first, ties to the lower index), weights[r] = softmax over
        those alone; logits f32 [n, E], chosen int32 [n, top], weights f32 [n, top].
        `scoring` "sigmoid": weights[r] = the sigmoid of every chosen logit, each for itself."""
        if scoring not in ("softmax", "sigmoid"):
            raise KernelError(f"route_top_k: scoring is 'softmax' or 'sigmoid', got {scoring!r}")
        n_rows, experts = logits.shape
        top = chosen.shape[1]
        if chosen.shape != (n_rows, top) or weights.shape != (n_rows, top) or (bias is not None and bias.shape != (experts,)):
            raise KernelError(f"route_top_k: shapes logits {tuple(logits.shape)}, chosen {tuple(chosen.shape)} do not fit")
        self._check(self.lib.bh_route_top_k(
            self._ptr(logits, "router logits", (torch.float32,)), self._ptr(bias, "router bias", (torch.float32,), True),
            self._ptr(chosen, "chosen", (torch.int32,)), self._ptr(weights, "route weights", (torch.float32,)), n_rows, experts, top,
            int(scoring == "sigmoid"), self._stream()))

    def experts_gate_up(self, h, chosen, w_gate_up, inner, limit, alpha, shift=1.0, in_weights=None):
        """inner[r * top + j] = act(Wg_e h[r], Wu_e h[r]) for e = chosen[r, j]; w_gate_up [E, 2 ff, K] (gate rows, then up rows).
        `in_weights` float32 [n, top]: a pair's weight multiplies the expert's input (its gate and up sums)."""
        n_rows, k = h.shape
        top = chosen.shape[1]
        experts, twice, k_w = w_gate_up.shape
        ff = twice // 2
        if k_w != k or tuple(inner.shape) != (n_rows * top, ff) or chosen.shape[0] != n_rows or w_gate_up.dtype != h.dtype \
                or inner.dtype != h.dtype:
            raise KernelError(f"experts_gate_up: shapes h {tuple(h.shape)}, weights {tuple(w_gate_up.shape)}, inner {tuple(inner.shape)} do not fit")
        self._check(self.lib.bh_experts_gate_up(
            self._ptr(h, "experts h"), _code(h, "experts h"), self._ptr(chosen, "chosen", (torch.int32,)), self._ptr(w_gate_up, "expert gate/up"),
            self._ptr(inner, "experts inner"), n_rows, top, k, ff, float(limit), float(alpha), float(shift),
            self._ptr(in_weights, "pair weights", (torch.float32,), True), self._stream()))

    def experts_down(self, inner, chosen, weights, w_down, hidden):
        """hidden[r] += sum_j weights[r, j] * Wd_e inner[r * top + j], e = chosen[r, j], j in order; w_down [E, D, ff]."""
        n_rows, top = chosen.shape
        experts, width, ff = w_down.shape
        if tuple(inner.shape) != (n_rows * top, ff) or tuple(hidden.shape) != (n_rows, width) or (weights is not None and weights.shape != (n_rows, top)) \
                or w_down.dtype != inner.dtype:
            raise KernelError(f"experts_down: shapes inner {tuple(inner.shape)}, weights {tuple(w_down.shape)}, hidden {tuple(hidden.shape)} do not fit")
        self._check(self.lib.bh_experts_down(
            self._ptr(inner, "experts inner"), _code(inner, "experts inner"), self._ptr(chosen, "chosen", (torch.int32,)),
            self._ptr(weights, "route weights", (torch.float32,), True), self._ptr(w_down, "expert down"),
            self._ptr(hidden, "experts hidden", (torch.float32,)), n_rows, top, ff, width, self._stream()))

    def experts_group(self, chosen, lists, counts):
        """lists[e, :counts[e]] = the pairs p = row * top + j with chosen[row, j] == e, in ascending order; chosen int32 [n, top],
        lists int32 [E, n], counts int32 [E]."""
        n_rows, top = chosen.shape
        experts = counts.shape[0]
        if lists.shape != (experts, n_rows):
            raise KernelError(f"experts_group: lists {tuple(lists.shape)} for {experts} experts and {n_rows} rows")
        self._check(self.lib.bh_experts_group(self._ptr(chosen, "chosen", (torch.int32,)), n_rows * top, self._ptr(lists, "lists", (torch.int32,)),
                                              n_rows, self._ptr(counts, "counts", (torch.int32,)), experts, self._stream()))

    def experts_rows_take(self, inputs: int) -> bool:
        """Whether `experts_rows` takes rows of that many inputs (16-byte loads)."""
        return inputs % 8 == 0

    def experts_rows(self, rows, rows_per_pair_row, lists, counts, w, out, gated=False, limit=0.0, alpha=0.0, shift=1.0, in_weights=None):
        """For every expert e and each of its pairs p (lists, counts): a product of w[e] with rows[p // rows_per_pair_row], the
        expert's matrix read once per workgroup.  gated: w [E, 2 N, K] (gate rows, then up rows), out [pairs, N] of the rows' type
        = act(gate, up); otherwise w [E, N, K] and out float32 [pairs, N]."""
        experts, w_rows, k = w.shape
        n = w_rows // 2 if gated else w_rows
        if rows.shape[1] != k or out.shape[1] != n or w.dtype != rows.dtype or counts.shape != (experts,) or lists.shape[0] != experts \
                or out.dtype != (rows.dtype if gated else torch.float32):
            raise KernelError(f"experts_rows: shapes rows {tuple(rows.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_experts_rows(
            self._ptr(rows, "experts rows"), _code(rows, "experts rows"), int(rows_per_pair_row), self._ptr(lists, "lists", (torch.int32,)),
            lists.shape[1], self._ptr(counts, "counts", (torch.int32,)), self._ptr(w, "expert weights"), self._ptr(out, "experts out"),
            experts, k, n, int(bool(gated)), float(limit), float(alpha), float(shift),
            self._ptr(in_weights, "pair weights", (torch.float32,), True), self._stream()))

    def experts_products_take(self, dtype, inputs: int, outputs: int) -> bool:
        """Whether `experts_products` takes products of these sizes and element type."""
        return dtype == torch.bfloat16 and bool(self.lib.bh_experts_products_takes(int(inputs), int(outputs)))

    def experts_products(self, rows, w, tiles, out, gated=False, limit=0.0, alpha=0.0, shift=1.0):
        """All experts' products of a prompt in one launch on the matrix cores: rows bf16 [pairs, K] lie expert after expert,
        tiles int32 [n, 3] = (expert, first row, rows of the tile: 1 to 128) names every stretch; gated: w [E, 2 N, K] and out
        bf16 [pairs, N] = act(gate, up); otherwise w [E, N, K] and out float32 [pairs, N]."""
        experts, w_rows, k = w.shape
        n = w_rows // 2 if gated else w_rows
        if rows.shape[1] != k or tuple(out.shape) != (rows.shape[0], n) or rows.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 \
                or out.dtype != (torch.bfloat16 if gated else torch.float32) or tiles.dim() != 2 or tiles.shape[1] != 3:
            raise KernelError(f"experts_products: shapes rows {tuple(rows.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_experts_products(
            self._ptr(rows, "experts rows", (torch.bfloat16,)), self._ptr(w, "expert weights", (torch.bfloat16,)),
            self._ptr(tiles, "tiles", (torch.int32,)), tiles.shape[0], self._ptr(out, "experts out"), k, n, int(bool(gated)), float(limit),
            float(alpha), float(shift), self._stream()))

    def experts_gather(self, x, top, lists, counts, offsets, gathered, place, in_weights=None):
        """gathered[offsets[e] + i] = x[lists[e, i] // top] and place[lists[e, i]] = offsets[e] + i for i < counts[e]: the pairs'
        input rows side by side, expert after expert; with `in_weights` float32 [n, top] every copy times its pair's weight."""
        n_rows, k = x.shape
        experts = counts.shape[0]
        if tuple(gathered.shape) != (n_rows * top, k) or place.shape != (n_rows * top,) or offsets.shape != (experts,) \
                or gathered.dtype != x.dtype:
            raise KernelError(f"experts_gather: shapes x {tuple(x.shape)}, gathered {tuple(gathered.shape)} do not fit")
        self._check(self.lib.bh_experts_gather(
            self._ptr(x, "experts x"), _code(x, "experts x"), int(top), self._ptr(lists, "lists", (torch.int32,)), lists.shape[1],
            self._ptr(counts, "counts", (torch.int32,)), self._ptr(offsets, "offsets", (torch.int32,)), self._ptr(gathered, "gathered"),
            self._ptr(place, "place", (torch.int32,)), experts, k, n_rows,
            self._ptr(in_weights, "pair weights", (torch.float32,), True), self._stream()))

    def experts_combine(self, y, place, weights, hidden, top=None):
        """hidden[r] += sum_j weights[r, j] * y[place[r * top + j]] (place None: y[r * top + j]), j in order; y f32 [pairs, D]."""
        n_rows, top = weights.shape if weights is not None else (hidden.shape[0], int(top))      # no weights: every share counts once
        if tuple(y.shape) != (n_rows * top, hidden.shape[1]) or hidden.shape[0] != n_rows or (place is not None and place.shape != (n_rows * top,)):
            raise KernelError(f"experts_combine: shapes y {tuple(y.shape)}, hidden {tuple(hidden.shape)} do not fit")
        self._check(self.lib.bh_experts_combine(
            self._ptr(y, "experts y", (torch.float32,)), self._ptr(place, "place", (torch.int32,), True),
            self._ptr(weights, "route weights", (torch.float32,), True), self._ptr(hidden, "experts hidden", (torch.float32,)), n_rows, top,
            hidden.shape[1], self._stream()))

    def clamped_glu(self, gate_up, out, limit, alpha, shift=1.0):
        """out = g' * sigmoid(alpha g') * (u' + shift) with g' = min(g, limit), u' = clamp(u, -limit, limit); gate_up [n, 2 ff] = [g | u]."""
        n_rows, twice = gate_up.shape
        if tuple(out.shape) != (n_rows, twice // 2) or twice % 2 or out.dtype != gate_up.dtype:
            raise KernelError(f"clamped_glu: shapes gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)} do not fit")
        self._check(self.lib.bh_clamped_glu(self._ptr(gate_up, "clamped_glu in"), _code(gate_up, "clamped_glu in"), self._ptr(out, "clamped_glu out"),
                                            n_rows, twice // 2, float(limit), float(alpha), _block_rows(out), float(shift), self._stream()))

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
