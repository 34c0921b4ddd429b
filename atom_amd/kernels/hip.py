"""The engine's kernel library: hand-written HIP for gfx950 behind a C interface,
called through ctypes on PyTorch's current stream.

Every method checks on the host that the operands have the shapes, types and
device the kernel and its grid assume, and raises before anything is launched.
There is no fallback: without a GPU or without the built library, construction fails.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch

from . import build as _build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
_STATUS = {
    1: "unsupported element type",
    2: "operand shapes do not fit the kernel",
    3: "unsupported configuration",
    4: "kernel launch failed",
    5: "a size exceeds what the kernel can hold",
}


class KernelError(RuntimeError):
    pass


@dataclass(frozen=True)
class ChipFigures:
    """What was measured on a GPU and decides between two ways of running the same product.  The ways differ in
    speed and, by rounding, in the last bits of their sums; both are tested against the same reference."""

    stream_bytes_per_us: float     # weights the whole chip streams in a few-rows product, bytes per microsecond
    cu_bytes_per_us: float         # what a single CU draws at most
    split_bytes_per_us: float      # the same product with K cut between blocks (more blocks, shorter)
    add_norm_us: float             # the add-norm kernel that a product cut along K needs beside it
    library_tile: int              # rows and columns of the BLAS library's large tiles
    library_slice_k: int           # the least K a slice of a library product keeps ...
    library_slice_k_many: int      # ... and once there are more than library_many_tiles tiles
    library_many_tiles: int
    decode_parts_root: float       # parts of a decode row x sqrt(requests x KV heads) at which attention + merge take least


# by the architecture name the device reports (before its ':' suffixes)
CHIPS = {
    # MI355X, 8 rows: a CU draws 28 GB/s at most (22 when all 256 share the chip's 5.6 TB/s); a kernel costs 3.4 us
    # beside its bytes and the add-norm kernel 5 us.  With tiles of 16 columns: 32B down (320 blocks, 2 on 64 of
    # the CUs): 60.0 us folded against 47.2 + 5.2 the split way; 32B o: 22.5 against 19.2 + 5.2; 4B down (160
    # blocks): 14.6 against 11.2 + 4.7; 8B down (256 blocks): 20.3 against 18.3 + 4.7.  With tiles of 12 columns
    # (427 and 214 blocks): 32B down 52.0 folded, 32B o 20.2, 4B down 13.5.
    "gfx950": ChipFigures(stream_bytes_per_us=5.6e6, cu_bytes_per_us=28e3, split_bytes_per_us=5.5e6, add_norm_us=5.0,
                          library_tile=256, library_slice_k=2048, library_slice_k_many=4096, library_many_tiles=64,
                          # decode attention from the QKV product plus the merge, 2 / 4 / 8 requests of 8 KV heads at
                          # 1,030 to 8,200 keys: least time at 40-64 / 28-48 / 20-28 parts (a part's chain of
                          # dependent steps shortens with more parts, the merge and the waves' set-up grow); a step
                          # of 8 requests at 2,100 keys: 3.853 / 3.816 / 3.790 / 3.837 ms with 32 / 28 / 24 / 20 parts
                          decode_parts_root=192.0),
}


@dataclass
class AttentionMeta:
    """What attention needs to know about a step's batch, on the device, for one
    group of layers that share block tables.

    token_seq[t]      index of the request (row of block_tables) token t belongs to, -1 for padding
    positions[t]      absolute position of token t in its request
    block_tables      [num_seqs, max_blocks] page ids of each request, in order of position
    cu_seqlens_q      [num_seqs + 1] first token of each request in the flat token axis
    context_lens      [num_seqs] keys of each request once this step's tokens are written
    The three ``max_``/``num_`` numbers are host copies used to pick a kernel and its grid.
    """

    token_seq: torch.Tensor
    positions: torch.Tensor
    block_tables: torch.Tensor
    cu_seqlens_q: torch.Tensor
    context_lens: torch.Tensor
    num_seqs: int
    num_tokens: int
    max_q_len: int
    max_context_len: int
    page_size: int
    # requests 0 .. num_prefill-1 bring more than one token (prompt portions), the rest one each;
    # prefill_tiles [num_tiles, 2] lists (request, first row) of every tile of rows_per_tile rows
    num_prefill: int = 0
    prefill_tiles: torch.Tensor | None = None
    rows_per_tile: int = 16
    # the same for other tile heights: rows -> [num_tiles, 2]
    tiles_by_rows: dict | None = None


class DeferredSum:
    """A matrix product that is still a sum of slices: ``partial`` float32 [splits, rows, width], plus an
    optional bias over the width.  The skinny product leaves its result like this when it cuts K; the
    kernel that reads it next (norm, rotation, SiLU-mul) adds the slices in slice order while it reads.
    ``dtype`` is the type the product has once it is a tensor (``HipKernels.materialize``)."""

    def __init__(self, partial: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype):
        self.partial = partial
        self.bias = bias
        self.dtype = dtype

    @property
    def shape(self):
        return self.partial.shape[1:]

    @property
    def device(self):
        return self.partial.device

    @property
    def splits(self) -> int:
        return self.partial.shape[0]

    @property
    def stride(self) -> int:
        return self.partial.shape[1] * self.partial.shape[2]


class PendingNorm:
    """An RMS norm that has not been applied yet: float32 rows ``r`` [*, width]; ``xg`` = bfloat16(r * weight),
    the same rows times the norm's weight; ``ss`` [*, parts], partial sums of squares of the rows of ``r`` (all
    three left by the product that wrote ``r``); eps; and optionally which rows are meant (``rows``, int32).  The
    few-rows product takes ``xg`` as its input and multiplies its float32 sums by the rows' 1 / rms
    (``HipKernels.linear`` / ``linear_silu``); ``HipKernels.materialize`` runs the norm kernel on ``r``."""

    def __init__(self, r, xg, ss, weight, eps: float, rows, dtype: torch.dtype):
        self.r, self.xg, self.ss, self.weight, self.eps, self.rows, self.dtype = r, xg, ss, weight, float(eps), rows, dtype

    @property
    def shape(self):
        return torch.Size((self.rows.numel() if self.rows is not None else self.r.shape[0], self.r.shape[1]))

    @property
    def device(self):
        return self.r.device


class PendingProduct:
    """``x @ weight.T (+ bias)`` of few rows that has not been launched: what follows decides its epilogue (a norm
    with the residual stream adds the sum in place; anything else takes the plain product)."""

    def __init__(self, x, weight, bias, dtype: torch.dtype):
        self.x, self.weight, self.bias, self.dtype = x, weight, bias, dtype
        self.split = False   # set by a norm that wants the product as a sum of K slices (see pending_norm)

    @property
    def shape(self):
        return torch.Size((self.x.shape[0], self.weight.shape[0]))

    @property
    def device(self):
        return self.weight.device


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


class HipKernels:
    """Loads (building first if need be) the kernel library and binds its entry points."""

    name = "hip"

    def __init__(self, device: str | torch.device = "cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError(
                "atom_amd runs on an AMD GPU only: torch.cuda.is_available() is False and there is no CPU path")
        self.device = torch.device(device)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        path = _build.build()
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"could not load the kernel library {path}: {e}") from e
        self.path = path
        for fn in ("atom_embedding", "atom_feed_tokens", "atom_rmsnorm", "atom_silu_mul", "atom_qk_norm_rope_kv_write",
                   "atom_gemm_skinny", "atom_gemm_skinny_splits", "atom_gemm_skinny_supports", "atom_splitk_reduce",
                   "atom_paged_attention_generic", "atom_gemm_f32", "atom_sample", "atom_exponential_noise",
                   "atom_attention_mfma_supports", "atom_attention_decode", "atom_attention_prefill",
                   "atom_attention_prefill_tile_rows", "atom_attention_decode_fused",
                   "atom_attention_decode_fused_supports", "atom_gemm_rows", "atom_gemm_rows_parts",
                   "atom_gemm_rows_supports", "atom_gemm_tile", "atom_gemm_tile_splits", "atom_gemm_tile_supports"):
            getattr(self.lib, fn).restype = ctypes.c_int
        self.allow_library_gemm = True
        # bfloat16 products of few rows run this library's own weight-streaming kernels: up to 64 rows, and
        # up to 128 for the narrow products that atom_gemm_skinny_supports names; the BLAS library takes the rest.
        self.use_skinny_gemm = True
        self.skinny_max_rows = 128
        # up to 8 bfloat16 rows: the product with the norm before it and the residual sum after it folded in
        self.use_rows_gemm = True
        self.split_library_products = True
        # 65 to 256 bfloat16 rows, products no wider than 8,192 columns: the kernel whose grid of tiles and K slices
        # is cut to the chip's CUs (the BLAS library's large tiles leave most of the chip idle there)
        self.use_tile_gemm = True
        self.tile_rows = (65, 256)
        self.tile_max_width = 8192
        self.narrow_row_tiles = True   # tiles of 12 or 8 columns in the few-rows product where they spread better
        self.rows_waves = 0     # 4 or 8 forces the waves a block of that kernel (0: its own choice)
        self.use_mfma_attention = True
        self.use_tiled_prefill = True
        # Its blocks have eight waves whose halves take the key tiles in turn (D <= 128): True, False, or None for the
        # choice by the size of the launch (see _prefill_in_halves)
        self.prefill_key_halves = None
        self.prefill_low_blocks = None   # True / False forces 16 / 32 tokens a wave in the blocks of eight waves
        self.use_fused_decode = True    # decode-only steps of few rows: norm, rotation and cache write inside attention
        self._ws: dict[str, torch.Tensor] = {}
        self._extensions: dict = {}
        self._zeroed: dict[str, torch.Tensor] = {}   # workspaces that every kernel leaves all zero
        props = torch.cuda.get_device_properties(self.device)
        self.num_cus = props.multi_processor_count
        arch = str(getattr(props, "gcnArchName", "")).split(":")[0]
        # the figures of the part these kernels are written for stand in for an unknown one: only speed depends on them
        self.chip = CHIPS.get(arch, CHIPS["gfx950"])

    def workspace(self, name: str, numel: int, dtype=torch.float32) -> torch.Tensor:
        """A scratch tensor that only grows; one per name.  While a HIP graph is being captured the
        tensor comes from the graph's own pool instead, so that the graph never holds memory
        that a later, larger request would free."""
        if torch.cuda.is_current_stream_capturing():
            return torch.empty(max(numel, 1), dtype=dtype, device=self.device)
        t = self._ws.get(name)
        if t is None or t.numel() < numel or t.dtype != dtype:
            t = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._ws[name] = t
        return t

    # the span names of the operations in a profiler trace, the reference's where it has one
    # (atom/model_ops/attention_mha.py:199, 483, 729: "rope_cache", "paged_attention_*", "prefill_attention")
    _SPANS = {"embedding": "embedding", "rmsnorm": "rmsnorm", "silu_mul": "silu_mul",
              "qk_norm_rope_kv_write": "rope_cache", "paged_attention": "paged_attention",
              "linear": "linear", "linear_silu": "linear_silu", "sample": "sample"}

    def mark_trace(self) -> None:
        """Wraps every operation of this object in a ``torch.profiler.record_function`` span, so that a
        profiler trace shows which kernels belong to which operation (the reference's ``--mark-trace``,
        atom/utils/decorators.py:232-257, in its record_function form).  Off by default: a span costs
        host time in every call."""
        for method, span in self._SPANS.items():
            inner = getattr(self, method)
            if getattr(inner, "_marked", False):
                continue

            def marked(*args, _inner=inner, _span=span, **kwargs):
                with torch.profiler.record_function(_span):
                    return _inner(*args, **kwargs)
            marked._marked = True
            setattr(self, method, marked)

    def attention_tile_rows(self, dtype, head_dim: int, page_size: int, group: int, max_q_len: int) -> tuple[int, int]:
        """The heights of the tiles of query rows that ``paged_attention`` wants listed for a step whose
        longest prompt portion has ``max_q_len`` tokens: (of the kernel whose waves load their own keys, of
        the kernel whose waves share key tiles); 0 where a kernel is not used (float32 steps list nothing)."""
        if (dtype != torch.bfloat16 or not self.use_mfma_attention
                or not self.lib.atom_attention_mfma_supports(head_dim, page_size, group)):
            return 0, 0
        tall = 0
        if max_q_len >= 32 and self.use_tiled_prefill:
            tall = int(self.lib.atom_attention_prefill_tile_rows(head_dim, page_size, group))
        return (32 if max_q_len > 16 else 16), tall

    def decode_parts(self, seqs: int, hkv: int, max_context: int) -> int:
        """Over how many waves a decode row's keys are split: enough waves to fill the chip,
        at least 64 keys each."""
        rows = max(1, seqs * hkv)
        want = -(-8 * self.num_cus // rows)
        if want > 8:   # more parts than one block merges itself: the merge kernel's time counts too
            want = min(want, max(9, round(self.chip.decode_parts_root / math.sqrt(rows))))
        return max(1, min(want, 64, -(-max_context // 64)))

    # ------------------------------------------------------------------ helpers

    def load_extension(self, sources: list[str], lib_name: str) -> ctypes.CDLL:
        """For a part that brings HIP kernels of its own: compiles ``sources`` with this library's flags (once;
        ``kernels.build.build_sources``) and loads the result.  The part declares its entry points' types on the
        returned library and calls them with ``pointer(tensor)`` and ``stream()``; ``check`` is the operand test
        every method here uses."""
        key = (tuple(sources), lib_name)
        if key not in self._extensions:
            try:
                self._extensions[key] = ctypes.CDLL(_build.build_sources(list(sources), lib_name))
            except OSError as e:
                raise KernelError(f"could not load the kernels of {lib_name}: {e}") from e
        return self._extensions[key]

    def stream(self):
        """The handle of PyTorch's current stream on this device, as kernels' C entry points take it."""
        return self._stream()

    @staticmethod
    def pointer(t: torch.Tensor | None):
        return _ptr(t)

    def check(self, name: str, t: torch.Tensor, dtype=None, shape=None):
        return self._check(name, t, dtype, shape)

    def _stream(self):
        # the current stream's handle, the short way: these few calls are made hundreds of times a step
        return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _check(self, name: str, t: torch.Tensor, dtype=None, shape=None):
        """Every operand of every call goes through here (a step makes over a thousand such calls):
        the passing case costs a few attribute reads, the failing one says what is wrong."""
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
        if not t.is_cuda:
            raise KernelError(f"{name}: must live on the GPU, is on {t.device}")
        if not t.is_contiguous():
            raise KernelError(f"{name}: must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
        if dtype is not None:
            have = t.dtype
            if have is not dtype and (not isinstance(dtype, (tuple, list)) or have not in dtype):
                raise KernelError(f"{name}: element type {have} not in {dtype}")
        if shape is not None:
            have = t.shape
            ok = len(shape) == len(have)
            if ok:
                for want, got in zip(shape, have):
                    if want is not None and want != got:
                        ok = False
                        break
            if not ok:
                raise KernelError(f"{name}: shape {tuple(have)} does not match {tuple(shape)}")
        return t

    def _done(self, what: str, status: int):
        if status != 0:
            raise KernelError(f"{what}: {_STATUS.get(status, f'status {status}')}")

    @staticmethod
    def _code(t: torch.Tensor) -> int:
        try:
            return _DTYPE_CODE[t.dtype]
        except KeyError:
            raise KernelError(f"element type {t.dtype} is not supported (float32 and bfloat16 are)") from None

    def _sum_args(self, x):
        """The four trailing arguments that say whether an input is a tensor or a sum of slices."""
        if isinstance(x, DeferredSum):
            self._check("slices", x.partial, torch.float32)
            if x.bias is not None:
                self._check("bias of the slices", x.bias, torch.float32, (x.shape[1],))
            return _ptr(x.partial), x.splits, ctypes.c_long(x.stride), _ptr(x.bias)
        return None, 0, ctypes.c_long(0), None

    def materialize(self, x):
        """A tensor from what may still be a sum of slices, a product not launched yet or a norm not applied yet."""
        if isinstance(x, PendingProduct):
            return self._rows_product(x.x, x.weight, x.bias, x.dtype)
        if isinstance(x, PendingNorm):
            out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
            # the float32 rows as a sum of one slice: the norm kernel reads float32 and writes the step's type
            return self.rmsnorm(DeferredSum(x.r.unsqueeze(0), None, x.dtype), x.weight, x.eps, out, rows=x.rows)
        if not isinstance(x, DeferredSum):
            return x
        rows, width = x.shape
        y = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        self._done("splitk_reduce", self.lib.atom_splitk_reduce(
            _ptr(x.partial), _ptr(x.bias), _ptr(y), rows, width, x.splits, int(x.dtype == torch.float32),
            self._stream()))
        return y

    # ---- the few-rows product with the norm before it and the residual sum after it folded in

    def _rows_takes(self, x, weight) -> bool:
        m, k = x.shape
        return bool(self.use_rows_gemm and 1 <= m <= 8 and weight.dtype == torch.bfloat16
                    and (isinstance(x, PendingNorm) or x.dtype == torch.bfloat16)
                    and self.lib.atom_gemm_rows_supports(m, weight.shape[0], k))

    def rows_cols(self, n: int) -> int:
        """Output columns a block of the few-rows product owns for a width of ``n``: 16, or 12 or 8 where that
        takes at least a fifth off the columns of the busiest CU (2,560 columns are 160 tiles of 16 for 256 CUs,
        but 214 of 12; 5,120 and 6,144 are 1.25 and 1.5 tiles of 16 a CU, and 1.67 and 2 of 12).  A block streams
        its columns' rows of w at what one CU draws, so the busiest CU's columns are the product's time wherever
        the chip as a whole is not the limit."""
        if not self.narrow_row_tiles:
            return 16
        def busiest(cols: int) -> int:   # columns of the CU with the most blocks
            tiles = -(-n // cols)
            return -(-tiles // self.num_cus) * cols

        best = 16
        for cols in (12, 8):
            if busiest(cols) * 5 <= busiest(16) * 4 and busiest(cols) < busiest(best):
                best = cols
        return best

    def _rows_residual_pays(self, n: int, k: int) -> bool:
        """Whether the few-rows product with the residual sum folded in beats the product with K cut between
        blocks followed by the add-norm kernel.  The folded one owns ``rows_cols(n)`` columns and all of K per block, so
        its blocks are all the parallelism there is, and it takes as long as its busiest CU needs for its
        blocks' rows of w.  The figures are the chip's (``CHIPS``)."""
        chip = self.chip
        cols = self.rows_cols(n)
        tiles = -(-n // cols)
        folded = max(n * 2 * k / chip.stream_bytes_per_us,                                  # the chip's pace,
                     -(-tiles // self.num_cus) * cols * 2 * k / chip.cu_bytes_per_us)       # the busiest CU's
        split = n * k * 2 / chip.split_bytes_per_us + chip.add_norm_us
        return folded <= split

    def _rows_launch(self, x, weight, bias, mode: int, y=None, res=None, ss_out=None, xg_out=None, g_next=None,
                     out_f32: bool = False):
        m, k = x.shape
        n = weight.shape[0] // 2 if mode == 1 else weight.shape[0]
        self._check("linear weight", weight, torch.bfloat16, (weight.shape[0], k))
        if bias is not None:
            self._check("linear bias", bias, torch.float32, (weight.shape[0],))
        if isinstance(x, PendingNorm):
            self._check("norm input", x.xg, torch.bfloat16, (None, k))
            self._check("sums of squares", x.ss, torch.float32, (x.xg.shape[0], None))
            if x.rows is not None:
                self._check("norm row choice", x.rows, torch.int32, (m,))
            head = (_ptr(x.xg), _ptr(x.rows), _ptr(x.ss), x.ss.shape[1], ctypes.c_float(x.eps))
        else:
            self._check("linear input", x, torch.bfloat16, (m, k))
            head = (_ptr(x), None, None, 0, ctypes.c_float(0.0))
        self._done("gemm_rows", self.lib.atom_gemm_rows(
            *head, _ptr(weight), _ptr(bias), _ptr(y), _ptr(res), _ptr(ss_out), _ptr(xg_out), _ptr(g_next), m, n, k,
            mode, int(out_f32), 16 if mode == 1 else self.rows_cols(n), int(self.rows_waves), self._stream()))

    def _rows_product(self, x, weight, bias, out_dtype):
        y = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=weight.device)
        self._rows_launch(x, weight, bias, 0, y=y, out_f32=out_dtype == torch.float32)
        return y

    def pending_norm(self, x, residual, weight, eps: float, rows=None):
        """``residual += x`` where x is a product that has not been launched (it is launched now, the sum formed
        in place where the product leaves the matrix cores), and the norm of the sum left pending for the product
        that follows.  None if ``x`` is anything else: the caller then takes ``rmsnorm``."""
        if not isinstance(x, PendingProduct) or residual is None:
            return None
        m, n = x.shape
        if not self._rows_residual_pays(n, x.weight.shape[1]) and not isinstance(x.x, PendingNorm):
            x.split = True    # rmsnorm() launches it with K cut between blocks and adds the slices itself
            return None
        self._check("residual", residual, torch.float32, (m, n))
        self._check("norm weight", weight, torch.float32, (n,))
        inner = x.x
        if isinstance(inner, PendingNorm) and inner.r.data_ptr() == residual.data_ptr():
            inner = self.materialize(inner)   # the product may not read the rows it adds to
        ss = torch.empty((m, self.lib.atom_gemm_rows_parts(n, self.rows_cols(n))), dtype=torch.float32,
                         device=residual.device)
        xg = torch.empty((m, n), dtype=torch.bfloat16, device=residual.device)
        self._rows_launch(inner, x.weight, x.bias, 2, res=residual, ss_out=ss, xg_out=xg, g_next=weight)
        return PendingNorm(residual, xg, ss, weight, eps, rows, x.dtype)

    # ------------------------------------------------------------------ kernels

    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        vocab, hidden = table.shape
        tokens = ids.numel()
        self._check("embedding table", table, (torch.float32, torch.bfloat16))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("embedding out", out, (torch.float32, torch.bfloat16), (tokens, hidden))
        self._done("embedding", self.lib.atom_embedding(
            _ptr(table), self._code(table), _ptr(ids), _ptr(out), self._code(out), tokens, hidden, vocab,
            self._stream()))
        return out

    def feed_tokens(self, ids: torch.Tensor, source: torch.Tensor, sampled: torch.Tensor) -> torch.Tensor:
        """``ids[t] = sampled[source[t]]`` where ``source[t] >= 0`` (all int32, in place): token ids that the
        last step's sampler left on the device."""
        n = ids.numel()
        self._check("token ids", ids, torch.int32, (n,))
        self._check("token sources", source, torch.int32, (n,))
        self._check("sampled ids", sampled, torch.int32, (None,))
        self._done("feed_tokens", self.lib.atom_feed_tokens(
            _ptr(ids), _ptr(source), _ptr(sampled), n, sampled.numel(), self._stream()))
        return ids

    def rmsnorm(self, x, weight, eps: float, out, residual=None, mode: str = "plain", rows=None):
        """mode 'plain': out = norm(x); 'init': residual = x, out = norm(x);
        'add': residual += x, out = norm(residual).  With ``rows`` only those source
        rows are normed (into out[0..len(rows))) and the residual is not written."""
        if isinstance(x, PendingProduct) and x.split:
            x = self.linear(x.x, x.weight, x.bias, x.dtype, defer=True, few_rows=False)
        if isinstance(x, (PendingProduct, PendingNorm)):
            x = self.materialize(x)
        width = x.shape[-1]
        code = {"plain": 0, "init": 1, "add": 2}[mode]
        deferred = isinstance(x, DeferredSum)
        if not deferred:
            self._check("norm input", x, (torch.float32, torch.bfloat16), (None, width))
        self._check("norm weight", weight, torch.float32, (width,))
        n_out = rows.numel() if rows is not None else x.shape[0]
        self._check("norm out", out, x.dtype, (n_out, width))
        if code:
            if residual is None:
                raise KernelError("norm: this mode needs the residual stream")
            self._check("residual", residual, torch.float32, tuple(x.shape))
        if rows is not None:
            self._check("norm rows", rows, torch.int32, (n_out,))
        self._done("rmsnorm", self.lib.atom_rmsnorm(
            None if deferred else _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), self._code(out),
            n_out, width, ctypes.c_float(eps), code, *self._sum_args(x), self._stream()))
        return out

    def silu_mul(self, x, out):
        rows, two = x.shape
        if two % 2:
            raise KernelError("silu_mul: the input width must be even (gate | up)")
        deferred = isinstance(x, DeferredSum)
        if not deferred:
            self._check("silu_mul input", x, (torch.float32, torch.bfloat16))
        self._check("silu_mul out", out, x.dtype, (rows, two // 2))
        self._done("silu_mul", self.lib.atom_silu_mul(None if deferred else _ptr(x), _ptr(out), self._code(out), rows,
                                                      two // 2, *self._sum_args(x), self._stream()))
        return out

    def qk_norm_rope_kv_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, cos, sin, positions,
                              slots, num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int,
                              page_size: int, eps: float, write_kv: bool = True):
        if isinstance(qkv, PendingProduct):
            # the float32 product as a sum of one slice: the kernel reads it with the precision it reads slices
            full = self._rows_product(qkv.x, qkv.weight, qkv.bias, torch.float32)
            qkv = DeferredSum(full.unsqueeze(0), None, qkv.dtype)
        tokens = qkv.shape[0]
        dt = qkv.dtype
        deferred = isinstance(qkv, DeferredSum)
        if deferred:
            if tuple(qkv.shape) != (tokens, (num_heads + 2 * num_kv_heads) * head_dim):
                raise KernelError(f"qkv: shape {tuple(qkv.shape)} does not fit the heads")
        else:
            self._check("qkv", qkv, (torch.float32, torch.bfloat16),
                        (tokens, (num_heads + 2 * num_kv_heads) * head_dim))
        self._check("q out", q_out, dt, (tokens, num_heads, head_dim))
        if write_kv:
            self._check("key pages", k_cache, dt, (None, num_kv_heads, page_size, head_dim))
            self._check("value pages", v_cache, dt, (k_cache.shape[0], num_kv_heads, head_dim, page_size))
            self._check("slot mapping", slots, torch.int32, (tokens,))
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                self._check(name, w, torch.float32, (head_dim,))
        if rotary_dim:
            self._check("cos table", cos, torch.float32, (None, rotary_dim // 2))
            self._check("sin table", sin, torch.float32, tuple(cos.shape))
            self._check("positions", positions, torch.int32, (tokens,))
        self._done("qk_norm_rope_kv_write", self.lib.atom_qk_norm_rope_kv_write(
            None if deferred else _ptr(qkv), _ptr(q_out), _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None,
            _ptr(q_weight), _ptr(k_weight), _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
            _ptr(positions) if rotary_dim else None, _ptr(slots) if write_kv else None, self._code(q_out), tokens,
            num_heads, num_kv_heads, head_dim, rotary_dim, page_size, ctypes.c_float(eps), int(bool(write_kv)),
            *self._sum_args(qkv), self._stream()))
        return q_out

    def _attention_mfma(self, q, k_cache, v_cache, out, meta, scale, window, parts=None):
        tokens, hq, d = q.shape
        _, hkv, page_size, _ = k_cache.shape
        self._check("cu_seqlens_q", meta.cu_seqlens_q, torch.int32, (meta.num_seqs + 1,))
        self._check("context_lens", meta.context_lens, torch.int32, (meta.num_seqs,))
        bt = meta.block_tables
        if bt.shape[0] != meta.num_seqs:
            raise KernelError("attention: one block table row per request is needed")
        if meta.num_prefill:
            tiles, rows, tiled = meta.prefill_tiles, meta.rows_per_tile, 0
            if meta.max_q_len >= 32 and meta.tiles_by_rows and self.use_tiled_prefill:
                # long portions: the kernel whose waves share key tiles through LDS
                want = self.lib.atom_attention_prefill_tile_rows(d, page_size, hq // hkv)
                if want and want in meta.tiles_by_rows:
                    tiles, rows = meta.tiles_by_rows[want], want
                    blocks = tiles.shape[0] * hq * 32 // (4 * want)
                    tiled = 2 if self._prefill_in_halves(blocks, meta) else 1
                    if tiled == 2 and self._prefill_low_blocks(blocks, d, meta):
                        tiled = 3
            self._check("prefill tiles", tiles, torch.int32, (None, 2))
            if not tiled and rows not in (16, 32):
                raise KernelError("attention: tiles hold 16 or 32 rows")
            self._done("attention_prefill", self.lib.atom_attention_prefill(
                _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q), _ptr(meta.context_lens),
                _ptr(bt), bt.shape[1], _ptr(tiles), tiles.shape[0], rows, tiled, hq, hkv, d, page_size,
                ctypes.c_float(scale), int(window or 0), self._stream()))
        seqs = meta.num_seqs - meta.num_prefill
        if seqs:
            if parts is None:
                visible = min(meta.max_context_len, window) if window else meta.max_context_len
                parts = self.decode_parts(seqs, hkv, visible)
            ws_o = ws_ml = None
            if parts > 1:
                ws_o = self.workspace("attn_o", seqs * hq * parts * d)
                ws_ml = self.workspace("attn_ml", seqs * hq * parts * 2)
            self._done("attention_decode", self.lib.atom_attention_decode(
                _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q), _ptr(meta.context_lens),
                _ptr(bt), bt.shape[1], meta.num_prefill, seqs, hq, hkv, d, page_size, ctypes.c_float(scale),
                int(window or 0), parts, _ptr(ws_o), _ptr(ws_ml), self._stream()))
        return out

    def _prefill_in_halves(self, blocks: int, meta) -> bool:
        """Whether the prefill kernel with shared key tiles runs blocks of eight waves (one a CU, the key tiles taken
        in turn by the block's halves) rather than of four (two a CU, each on its own).  Measured on an MI355X with
        32 / 8 heads of 128: two blocks of four waves keep each other's SIMDs busy as long as both run, so they win
        when a CU has a queue of them (8,192 fresh tokens: 640 against 690 us) or when all blocks are about as long
        (2,048 tokens behind 8,192 cached: 355 against 390 us); a block of eight waves does not depend on a
        neighbour, and wins when there is none (a portion of 512 tokens behind 3,072 cached, 128 blocks: 74 against
        99 us) or when the long blocks of a fresh prompt outlive their short neighbours (2,048 tokens: 64 against
        72 us)."""
        if self.prefill_key_halves is not None:
            return bool(self.prefill_key_halves)
        if blocks <= self.num_cus:
            return True
        return blocks <= 2 * self.num_cus and 2 * meta.max_context_len < 3 * meta.max_q_len

    def _prefill_low_blocks(self, blocks: int, head_dim: int, meta) -> bool:
        """Whether the blocks of eight waves take 16 query tokens a wave instead of 32 (twice the blocks, each with
        half the products per key tile it stages): when the launch would otherwise leave half of the CUs without a
        block (512 tokens behind 3,072 cached: 65 against 78 us), and for fresh prompts of up to a block a CU, whose
        blocks are mostly short (549 / 768 / 1,024 tokens: 16 / 20 / 29 against 21 / 24 / 30 us; behind 2,048 cached
        tokens the same launches take 82-90 against 62-68 us, so those keep 32 tokens a wave)."""
        if self.prefill_low_blocks is not None:
            return bool(self.prefill_low_blocks) and head_dim <= 128
        if head_dim > 128:
            return False
        return 2 * blocks <= self.num_cus or (blocks <= self.num_cus and 2 * meta.max_context_len < 3 * meta.max_q_len)

    def fused_decode_attention(self, qkv, k_cache, v_cache, out, meta: AttentionMeta, scale: float, window, q_weight,
                               k_weight, cos, sin, slots, num_heads: int, num_kv_heads: int, head_dim: int,
                               rotary_dim: int, eps: float, write_kv: bool = True, parts: int | None = None):
        """For a step in which every request brings one token: per-head norm of q and k, rotation, the write of the
        new keys and values and attention over the pages in one kernel (and the merge of the key ranges), starting
        from the QKV product, which has to be one that has not been launched yet (a few-rows ``PendingProduct``; it is
        launched here with float32 output).  Returns ``out``, or None when this case is not taken: the caller then
        runs ``qk_norm_rope_kv_write`` and ``paged_attention``."""
        page_size = meta.page_size
        if (not self.use_fused_decode or not isinstance(qkv, PendingProduct) or meta.num_prefill or out.dtype != torch.bfloat16
                or rotary_dim != head_dim or cos is None
                or not self.lib.atom_attention_decode_fused_supports(head_dim, page_size, num_heads // num_kv_heads)):
            return None
        tokens = qkv.shape[0]
        if meta.num_seqs != tokens or tuple(qkv.shape) != (tokens, (num_heads + 2 * num_kv_heads) * head_dim):
            return None
        self._check("key pages", k_cache, torch.bfloat16, (None, num_kv_heads, page_size, head_dim))
        self._check("value pages", v_cache, torch.bfloat16, (k_cache.shape[0], num_kv_heads, head_dim, page_size))
        self._check("attention out", out, torch.bfloat16, (tokens, num_heads, head_dim))
        self._check("cu_seqlens_q", meta.cu_seqlens_q, torch.int32, (tokens + 1,))
        self._check("context_lens", meta.context_lens, torch.int32, (tokens,))
        self._check("block tables", meta.block_tables, torch.int32, (tokens, None))
        self._check("cos table", cos, torch.float32, (None, head_dim // 2))
        self._check("sin table", sin, torch.float32, tuple(cos.shape))
        if meta.max_context_len > cos.shape[0]:
            raise KernelError("attention: a position lies beyond the rotation tables")
        if meta.max_context_len > meta.block_tables.shape[1] * page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                self._check(name, w, torch.float32, (head_dim,))
        if write_kv:
            self._check("slot mapping", slots, torch.int32, (tokens,))
        full = self._rows_product(qkv.x, qkv.weight, qkv.bias, torch.float32)
        if parts is None:
            visible = min(meta.max_context_len, window) if window else meta.max_context_len
            parts = self.decode_parts(tokens, num_kv_heads, visible)
        ws_o = ws_ml = None
        if parts > 1:
            ws_o = self.workspace("attn_o", tokens * num_heads * parts * head_dim)
            ws_ml = self.workspace("attn_ml", tokens * num_heads * parts * 2)
        bt = meta.block_tables
        self._done("attention_decode_fused", self.lib.atom_attention_decode_fused(
            _ptr(full), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin), _ptr(slots) if write_kv else None,
            ctypes.c_float(eps), int(bool(write_kv)), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q),
            _ptr(meta.context_lens), _ptr(bt), bt.shape[1], 0, tokens, num_heads, num_kv_heads, head_dim, page_size,
            ctypes.c_float(scale), int(window or 0), parts, _ptr(ws_o), _ptr(ws_ml), self._stream()))
        return out

    def paged_attention(self, q, k_cache, v_cache, out, meta: AttentionMeta, scale: float,
                        window: int | None = None, parts: int | None = None):
        tokens, hq, d = q.shape
        _, hkv, page_size, _ = k_cache.shape
        dt = q.dtype
        if hq % hkv:
            raise KernelError(f"attention: {hq} query heads are not a multiple of {hkv} key/value heads")
        self._check("q", q, (torch.float32, torch.bfloat16))
        self._check("key pages", k_cache, dt, (None, hkv, page_size, d))
        self._check("value pages", v_cache, dt, (k_cache.shape[0], hkv, d, page_size))
        self._check("attention out", out, dt, (tokens, hq, d))
        self._check("token_seq", meta.token_seq, torch.int32, (tokens,))
        self._check("positions", meta.positions, torch.int32, (tokens,))
        self._check("block tables", meta.block_tables, torch.int32, (None, None))
        if meta.page_size != page_size:
            raise KernelError("attention: the batch's page size differs from the cache's")
        if meta.max_context_len > meta.block_tables.shape[1] * page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        group = hq // hkv
        if (dt == torch.bfloat16 and self.use_mfma_attention
                and self.lib.atom_attention_mfma_supports(d, page_size, group)):
            return self._attention_mfma(q, k_cache, v_cache, out, meta, scale, window, parts)
        self._done("paged_attention", self.lib.atom_paged_attention_generic(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.token_seq), _ptr(meta.positions),
            _ptr(meta.block_tables), meta.block_tables.shape[1], self._code(q), tokens, hq, hkv, d, page_size,
            ctypes.c_float(scale), int(window or 0), self._stream()))
        return out

    def _library_slices(self, m: int, n: int, k: int) -> int:
        """Into how many slices of K a product that goes to the BLAS library is cut when its reader can add
        slices.  Measured on an MI355X with the o and down products of the 4B, 8B and 32B shapes at 544 to 4,096
        rows, the add-norm that reads the slices included: the library's kernels leave much of the chip idle
        while a product has fewer tiles of 256 x 256 than the chip has CUs, and the most slices that keep
        tiles x slices within the CUs win (8B down: 96 -> 58 us at 544 rows, 140 -> 108 at 1,024, 210 -> 197 at
        2,048; 32B down 373 -> 247 at 1,024), as long as a slice keeps 2,048 of K, and 4,096 once there are more
        than 64 tiles.  Products that widen (whose reader here is the rotation kernel, which wants a tensor for
        many rows) are left whole."""
        if not self.split_library_products or n > k:
            return 1
        chip = self.chip
        tiles = -(-m // chip.library_tile) * -(-n // chip.library_tile)
        for slices in (4, 2):
            per = k // slices
            if (k % (slices * 8) == 0 and tiles * slices <= self.num_cus and per >= chip.library_slice_k
                    and (tiles <= chip.library_many_tiles or per >= chip.library_slice_k_many)):
                return slices
        return 1

    def _tile(self, x, weight) -> bool:
        m, k = x.shape
        n = weight.shape[0]
        return bool(self.use_tile_gemm and self.tile_rows[0] <= m <= self.tile_rows[1] and n <= self.tile_max_width
                    and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                    and self.lib.atom_gemm_tile_supports(m, n, k))

    def _skinny(self, x, weight) -> bool:
        m, k = x.shape
        return bool(self.use_skinny_gemm and m <= self.skinny_max_rows and x.dtype == torch.bfloat16
                    and weight.dtype == torch.bfloat16 and self.lib.atom_gemm_skinny_supports(m, weight.shape[0], k))

    def linear(self, x, weight, bias=None, out_dtype=None, defer: bool = False, few_rows: bool = True):
        """``x @ weight.T (+ bias)``.  bfloat16 operands with at most 64 rows (narrow products: 128) run this
        library's own weight-streaming kernels, 65 to 256 rows of products up to 8,192 columns wide its kernel of
        tiles and K slices cut to the chip; the rest goes to the BLAS library, as the reference's engine
        does for its matrix products; anything with a float32 operand runs this library's float32
        kernel (plain FMA, no reduced-precision mode).  With ``defer`` the result may come back as a
        ``DeferredSum`` for a kernel that adds the slices while it reads them."""
        if isinstance(x, (DeferredSum, PendingProduct)):
            x = self.materialize(x)
        m, k = x.shape
        n = weight.shape[0]
        if m and few_rows and self._rows_takes(x, weight):
            if defer:
                return PendingProduct(x, weight, bias, out_dtype or x.dtype)
            return self._rows_product(x, weight, bias, out_dtype or x.dtype)
        x = self.materialize(x)
        self._check("linear input", x, (torch.float32, torch.bfloat16))
        self._check("linear weight", weight, (torch.float32, torch.bfloat16), (n, k))
        out_dtype = out_dtype or x.dtype
        if bias is not None:
            self._check("linear bias", bias, torch.float32, (n,))
        if self._tile(x, weight):
            splits = self.lib.atom_gemm_tile_splits(m, n, k, self.num_cus)
            if splits == 1:
                y = torch.empty((m, n), dtype=out_dtype, device=x.device)
                self._done("gemm_tile", self.lib.atom_gemm_tile(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(y), None, m, n, k, 1, int(out_dtype == torch.float32),
                    self._stream()))
                return y
            partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            self._done("gemm_tile", self.lib.atom_gemm_tile(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, n, k, splits, 0, self._stream()))
            result = DeferredSum(partial, bias, out_dtype)
            # a product that widens is read next by the rotation kernel, which wants a tensor for this many rows
            return result if defer and n <= k else self.materialize(result)
        if m and self._skinny(x, weight):
            splits = self.lib.atom_gemm_skinny_splits(m, n, k, 0)
            if splits == 1:
                y = torch.empty((m, n), dtype=out_dtype, device=x.device)
                self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(y), None, m, n, k, int(out_dtype == torch.float32), 0,
                    self._stream()))
                return y
            partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, n, k, 0, 0, self._stream()))
            result = DeferredSum(partial, bias, out_dtype)
            return result if defer else self.materialize(result)
        if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and self.allow_library_gemm:
            slices = self._library_slices(m, n, k) if defer else 1
            if slices > 1:
                # a product with too few tiles to fill the chip: K in slices as one batched product with float32
                # output, left as a sum that the norm behind it adds while it reads
                part = k // slices
                partial = torch.bmm(x.view(m, slices, part).transpose(0, 1),
                                    weight.view(n, slices, part).permute(1, 2, 0), out_dtype=torch.float32)
                return DeferredSum(partial, bias, out_dtype)
            if bias is None and out_dtype == torch.bfloat16:
                return torch.nn.functional.linear(x, weight)
            # float32 out, or a bias: the library writes its float32 sums as they are, so that logits have the
            # same precision whatever the number of rows, and a bias is added before anything is rounded
            y = torch.mm(x, weight.t(), out_dtype=torch.float32)
            if bias is not None:
                y += bias
            return y if out_dtype == torch.float32 else y.to(out_dtype)
        y = torch.empty((m, n), dtype=out_dtype, device=x.device)
        self._done("gemm_f32", self.lib.atom_gemm_f32(
            _ptr(x), self._code(x), _ptr(weight), self._code(weight), _ptr(bias), _ptr(y), self._code(y), m, n, k,
            self._stream()))
        return y

    def linear_silu(self, x, weight, bias=None):
        """``silu(x @ Wg.T + bg) * (x @ Wu.T + bu)`` for ``weight`` = gate rows then up rows: one kernel
        where the skinny product does not cut K, else the product and SiLU-mul over its slices."""
        m, k = x.shape
        two = weight.shape[0]
        if two % 2:
            raise KernelError("linear_silu: the weight must hold as many gate rows as up rows")
        inter = two // 2
        if m and self._rows_takes(x, weight):
            act = torch.empty((m, inter), dtype=x.dtype, device=weight.device)
            self._rows_launch(x, weight, bias, 1, y=act)
            return act
        x = self.materialize(x)
        if m and self._skinny(x, weight):
            self._check("linear input", x, torch.bfloat16)
            self._check("linear weight", weight, torch.bfloat16, (two, k))
            if bias is not None:
                self._check("linear bias", bias, torch.float32, (two,))
            act = torch.empty((m, inter), dtype=x.dtype, device=x.device)
            splits = self.lib.atom_gemm_skinny_splits(m, inter, k, 1)
            if splits == 1:
                self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(act), None, m, inter, k, 0, 1, self._stream()))
                return act
            partial = torch.empty((splits, m, two), dtype=torch.float32, device=x.device)
            self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, inter, k, 0, 1, self._stream()))
            return self.silu_mul(DeferredSum(partial, bias, x.dtype), act)
        gate_up = self.linear(x, weight, bias)
        act = torch.empty((m, inter), dtype=x.dtype, device=x.device)
        return self.silu_mul(gate_up, act)

    def sample(self, logits, temperatures, out, top_ks=None, top_ps=None, noise=None, seeds=None, counters=None,
               eps: float = 1e-10):
        rows, vocab = logits.shape
        self._check("logits", logits, torch.float32)
        self._check("sampled ids", out, torch.int32, (rows,))
        if temperatures is not None:
            self._check("temperatures", temperatures, torch.float32, (rows,))
        if top_ks is not None:
            self._check("top_ks", top_ks, torch.int32, (rows,))
        if top_ps is not None:
            self._check("top_ps", top_ps, torch.float32, (rows,))
        stride = 0
        if noise is not None:
            self._check("noise", noise, torch.float32, (None, vocab))
            if noise.shape[0] not in (1, rows):
                raise KernelError("noise must have one row or one per logits row")
            stride = vocab if noise.shape[0] == rows and rows > 1 else 0
        else:
            if temperatures is not None and (seeds is None or counters is None):
                raise KernelError("sampling without given noise needs seeds and counters")
        if seeds is not None:
            self._check("seeds", seeds, torch.int64, (rows,))
            self._check("counters", counters, torch.int64, (rows,))
        # every row's maximum (and, without filters, its race) is spread over 64 blocks: chunk maxima, chunk winners
        ws_vals = self.workspace("sample_vals", rows * 128)
        ws_idx = self.workspace("sample_idx", rows * 128, torch.int32)
        ws_filter = None
        if temperatures is not None and (top_ks is not None or top_ps is not None) and vocab >= 16384:
            # histograms of the threshold search: zero when made, and left zero by every call
            need = rows * (4096 * 12 + 32)
            ws_filter = self._zeroed.get("sample_filter")
            if ws_filter is None or ws_filter.numel() < need:
                if torch.cuda.is_current_stream_capturing():
                    # making it would record a fill node into the graph; the caller samples these rows once
                    # outside a capture first, which leaves the workspace in place
                    raise KernelError("sample: the top-k / top-p workspace has to exist before a graph is captured "
                                      f"({rows} rows need {need} bytes)")
                ws_filter = torch.zeros(need, dtype=torch.uint8, device=self.device)
                self._zeroed["sample_filter"] = ws_filter
        self._done("sample", self.lib.atom_sample(
            _ptr(logits), _ptr(temperatures), _ptr(top_ks), _ptr(top_ps), _ptr(noise), ctypes.c_long(stride),
            _ptr(seeds), _ptr(counters), _ptr(out), rows, vocab, ctypes.c_float(eps), _ptr(ws_vals), _ptr(ws_idx),
            _ptr(ws_filter), self._stream()))
        return out

    def exponential_noise(self, seeds, counters, vocab: int):
        rows = seeds.numel()
        self._check("seeds", seeds, torch.int64, (rows,))
        self._check("counters", counters, torch.int64, (rows,))
        out = torch.empty((rows, vocab), dtype=torch.float32, device=seeds.device)
        self._done("exponential_noise", self.lib.atom_exponential_noise(
            _ptr(out), _ptr(seeds), _ptr(counters), rows, vocab, self._stream()))
        return out
