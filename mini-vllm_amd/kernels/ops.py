"""Operations of the decoder on device tensors, bound to one activation type.

Each method checks shapes, types and placement on the host and then launches a kernel of
the HIP library on the current stream. Tensors must live on the GPU: there is no CPU path.
"""
from __future__ import annotations

from typing import Optional

import os

import torch

from . import library
from .library import DTYPE_BF16, DTYPE_F32, KernelLibraryError

_CODES = {torch.float32: DTYPE_F32, torch.bfloat16: DTYPE_BF16}
_NAMES = {torch.float32: "float32", torch.bfloat16: "bfloat16"}

# largest number of rows the weight-streaming product takes in one launch
SKINNY_MAX_M = 64
# ... and up to this many rows against small weights (the layers of a 0.6B-sized model): between 65 and
# 96 rows the engine's products, with the norms and the activation folded into them, still beat the
# library's with kernels of their own between them (a step of 72 / 80 / 96 sequences 3.2 / 4.4 / 2.3 %
# faster; at 112 and 128 rows nothing is gained)
SKINNY_WIDE_MAX_M = 96
SKINNY_WIDE_MAX_WEIGHT = 8 * 1024 * 1024
# most rows of one launch of it
SKINNY_LAUNCH_ROWS = 512
# the kernel that shares activation rows through LDS and splits K over workgroups takes over from
# this many rows on for weights of at least MID_MIN_WEIGHT elements, and at any number of rows for
# weights of at least MID_ALWAYS_WEIGHT elements with rows of at least MID_ALWAYS_K (measured on
# MI355X: below these the second kernel that adds its partial sums costs more than its better use of
# the memory system brings; with short rows, as in the output head of a narrow model, nothing is gained)
MID_MIN_M = 9
MID_MIN_WEIGHT = 12 * 1024 * 1024
MID_ALWAYS_WEIGHT = 120 * 1000 * 1000
MID_ALWAYS_K = 2048
# A weight with at least four times as many rows as columns and this many elements (gate/up of a large
# model, the output head of a large vocabulary) goes to the library's product at any number of rows:
# it streams such a weight at the memory's speed, 5.0 to 5.9 TB/s, where the engine's kernels reach
# 3.5 to 5 (0.6B-sized head: 51 against 65 us at one row, 83 against 136 at 64 rows; 32B-sized gate/up:
# 89 against 105 and 98 against 153). Weights with long rows it serves badly (32B-sized down: 134 us
# against 56).
LIBRARY_TALL_WEIGHT = 96 * 1000 * 1000
# The gated pair in one pass (no [M, 2I] intermediate, no second kernel) keeps the smaller of these
# weights for fewer than 16 rows (8B-sized: 44 against 46 us at 8 rows, 49 against 46 at 16); from
# this size on the library and a separate activation kernel win at every number of rows
LIBRARY_TALL_WEIGHT_GATED = 240 * 1000 * 1000
# The tiled MFMA product (gemm_tile.hip) takes the steps between the weight-streaming kernels and the
# library, where it is ahead of both (measured on MI355X, weights rotating so that they come from memory):
# a gated pair with the activation in its epilogue from 32 rows on (0.6B sizes at 64 rows: 7.7 us
# against the weight-streaming kernel's 11.4 and the library's 13.8 with the activation as a kernel of
# its own; at 1,024 rows 21.6 against 24.6; level from 1,536 on), for weights of 64 MB and more up to 128
# rows (8B sizes at 64 rows 44 against 51 us; at 256 the library is ahead); a plain product against a
# small weight with at least 4,096 rows (enough tiles without splitting K) from 40 to 512 rows (0.6B qkv
# at 64 rows 6.8 against 7.8 us, at 256 rows 7.2 against the library's 9.0; weights with fewer rows go to
# the library, which is a tenth ahead there); any plain product against a weight of 16 MB and more from
# 33 to 256 rows (8B sizes at 128 rows: down 33 against the library's 67 us, o 16 against 23, qkv 22 against 25).
# Below 33 rows it is ahead of the kernel that splits K over workgroups wherever that one was used (9 rows and
# more: 8B sizes at 16 rows o 11.6 against 13.6 us, down 23.7 against 28.7, gate/up 41.9 against 47.7; 32B o at
# 12 rows 19.7 against 23.3; in the model 8B decode at 12 / 16 / 32 sequences 9 / 10 / 3 % faster, 32B at 16
# sequences 8 %), and at 8 rows against weights of 96 MB and more (32B down 53 against 64 us, 32B qkv 23 against
# 29; 32B decode at batch 8 2.4 % faster) unless a norm can be folded into the weight-streaming product instead
# (8B down: 24.9 us with the norm in it against 23.7 and a norm kernel of 5). Fewer rows stay where they were:
# in the model a 32B step of one sequence was 2 % slower with the tiled product, and the gated 8B pair behind a
# folded norm at 8 rows made the step 4 % slower although the product alone was 4 us faster. The largest weights
# (MID_ALWAYS_WEIGHT: 32B down) take it from the first row on: 48 us in the model against the K-splitting kernel's
# 58, 32B decode at 1 / 4 / 8 sequences 1-6 / 3-6 / 6 % faster.
TILE_MIN_WEIGHT = 4 * 1024 * 1024             # bytes: smaller weights were not measured and stay where they were
TILE_GATED_MIN_M = 32
TILE_GATED_MAX_M = 1536
TILE_GATED_BIG_WEIGHT = 64 * 1024 * 1024      # bytes
TILE_GATED_BIG_MIN_M = 9
TILE_GATED_BIG_MAX_M = 128
TILE_SMALL_MIN_M = 40
TILE_SMALL_MAX_M = 512
TILE_SMALL_MIN_N = 4096
TILE_BIG_WEIGHT = 16 * 1024 * 1024            # bytes
TILE_BIG_MIN_M = 9
TILE_BIG_MAX_M = 256
TILE_HUGE_WEIGHT = 96 * 1024 * 1024           # bytes
TILE_HUGE_MIN_M = 8
# weights with long rows (the down matrices of a mixture's experts side by side: K = experts x width): the
# weight-streaming product splits such a K over few waves and reaches 2.2 TB/s on them, the tiled one splits it over
# workgroups, sixteen ways for such rows (``tile_plan``). Measured with MV_TILE_LONG_ROWS=0 and 1, decode at batch 8 of the
# 0.6B-sized mixtures (K = 25,344, N = 1,024): Furanex 3.375 -> 3.22 ms a step (3.32 with eight splits), Dutilix 2.467 -> 2.40
TILE_LONG_ROWS_K = 16384
TILE_LONG_ROWS_RATIO = 8                      # K >= ratio * N
# most rows for which residual add and norm are fused into the following product
FUSED_NORM_MAX_M = 16
# the fused kernel keeps the rows in registers: at most 8 waves x 4 chunks of 512 columns
FUSED_NORM_MAX_CHUNKS = 32
# the sampler's first pass: workgroups that share a row, and the rows its scratch is made for
SAMPLE_CHUNKS = 32
SAMPLE_WORK_ROWS = 1024
# compute units of the device the launch heuristics were tuned on; an ``Ops`` asks its device
COMPUTE_UNITS = 256
# context length from which the prompt attention uses two key groups per workgroup
PREFILL_TWO_GROUPS_FROM = 1024
# waves per workgroup of the decode attention
DECODE_ATTENTION_WAVES = 4
# the workgroup kernel splits a sequence's keys until about one workgroup for every compute unit is
# in flight (``Ops.compute_units``)
# (sequence, kv head) pairs of one decode step whose keys may be split over workgroups
SPLIT_COUNTERS = 1 << 16
# from this many tokens on, value rows are written to their pages 16 tokens of a kv head at a time
STORE_V_SPLIT_TOKENS = 64


def dtype_from_name(name: str) -> torch.dtype:
    if name in ("float32", "fp32", "f32"):
        return torch.float32
    if name in ("bfloat16", "bf16"):
        return torch.bfloat16
    raise ValueError(f"compute dtype must be 'bfloat16' or 'float32', got {name!r}")


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _dev(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelLibraryError(f"{what} is on {t.device}; the engine's kernels run on the GPU only")


def _weight_code(w: torch.Tensor, what: str) -> int:
    code = _CODES.get(w.dtype)
    if code is None:
        raise KernelLibraryError(f"{what} has dtype {w.dtype}; weights are float32 or bfloat16")
    return code


class SplitSum:
    """The output of a matrix product that exists only as the float partial sums of its splits of K
    so far: ``out[m, n] = round(sum_f work[f, m, n] + bias[n])``. The next residual add + norm can
    take it as its delta and add the sums up itself (``Ops.add_rmsnorm``), which saves the kernel
    that would; anything else calls ``materialize``. The sums live in the work area all such
    products share, so the next of them adds this one up first if nobody has asked for it yet."""

    def __init__(self, ops: "Ops", out: torch.Tensor, work: torch.Tensor, splits: int, bias: Optional[torch.Tensor]):
        self.ops, self.out, self.work, self.splits, self.bias = ops, out, work, splits, bias
        self.shape = out.shape
        self.done = False          # the sums were added up into ``out``, or are no longer needed

    def materialize(self) -> torch.Tensor:
        if not self.done:
            M, N = self.out.shape
            self.ops.lib.call("mv_gemm_mid_reduce", self.work.data_ptr(), _ptr(self.bias), self.out.data_ptr(),
                              self.out.stride(0) if M > 1 else N, _CODES[self.out.dtype], M, N, self.splits, 0,
                              self.ops._stream())
            self.discard()
        return self.out

    def discard(self) -> None:
        """The sums will not be asked for again (they were consumed, or the step is over)."""
        self.done = True
        if self.ops._split_pending is self:
            self.ops._split_pending = None


class WeightedRows:
    """What ``Ops.gemm(..., fold=...)`` returns when it took the residual add and the norm into its
    product: the rows of the new residual times the norm's weight (``weighted``, the activation
    type) and, per row, ``P`` partial sums of squares. ``Ops.gemm`` / ``Ops.gemm_swiglu`` take it as
    their input and divide their output rows by the root mean square; ``materialize()`` gives the
    normalised rows to anything else. Used once."""
    is_weighted_rows = True

    def __init__(self, ops: "Ops", fold, P: int):
        self.ops, self.norm = ops, fold.norm
        self.weighted, self.partial, self.P, self.eps = fold.weighted, fold.partial, P, float(fold.eps)
        self.normed = fold.normed
        self.shape = fold.weighted.shape
        self.used = False
        self._done = False

    def take(self) -> None:
        if self.used:
            raise RuntimeError("half-normalised rows were used twice")
        self.used = True

    def materialize(self) -> torch.Tensor:
        """Runs the second half of the norm (once) and returns the normalised rows."""
        if not self._done:
            self.take()
            self.ops.scale_rows(self.weighted, self.partial, self.P, self.eps, self.normed)
            self._done = True
        return self.normed


class Ops:
    def __init__(self, dtype: torch.dtype):
        if dtype not in _CODES:
            raise ValueError(f"unsupported compute dtype {dtype}")
        self.dtype = dtype
        self.code = _CODES[dtype]
        self.lib = library.load(library.variant_of(_NAMES[dtype]))
        self.use_fast_kernels = dtype == torch.bfloat16
        self.use_library_gemm = dtype == torch.bfloat16
        self.use_tiled_gemm = dtype == torch.bfloat16     # (a test of the kernels behind it switches it off)
        # compute units of the device: grids are sized in rounds of one workgroup each
        self.compute_units = int(self.lib.dll.mv_device_compute_units()) if torch.cuda.is_available() else COMPUTE_UNITS
        # set by the executor while it records a graph; library products take part in a recording
        # while ``library_in_graphs`` holds (see _library_allowed)
        self.for_graph = False
        self.library_in_graphs = True
        self.stream_handle: Optional[int] = None
        self._transposed = {}
        self._mid_work: Optional[torch.Tensor] = None
        self._lt_work: Optional[torch.Tensor] = None        # the library's workspace
        self._split_pending: Optional[SplitSum] = None     # partial sums in the work area nobody has used yet
        self._mid_retired: list = []
        self._tile_work: Optional[torch.Tensor] = None     # partial sums of the tiled product when it splits K
        self._sample_work: Optional[torch.Tensor] = None
        self._latent_work: Optional[torch.Tensor] = None   # per-run results of the latent attention's single-token kernel
        self._attn_counters: Optional[torch.Tensor] = None
        # measurement: with a list here, every launch leaves (entry point, bytes it has to move,
        # floating-point operations) in it; the benchmark sets it for one eager step and prices the
        # kernels of a profile with the totals (engine/roofline.py)
        self.ledger: Optional[list] = None

    def _note(self, entry: str, nbytes, flops=0) -> None:
        if self.ledger is not None:
            self.ledger.append((entry, int(nbytes), int(flops)))

    @staticmethod
    def _size(*tensors) -> int:
        return sum(t.numel() * t.element_size() for t in tensors if t is not None)

    # ------------------------------------------------------------------------------------
    def bind_stream(self) -> None:
        """Looks the current stream up once; until ``unbind_stream`` every launch goes there.
        (Asking for the current stream costs more than a launch; a step asks once.)"""
        self.stream_handle = torch.cuda.current_stream().cuda_stream

    def unbind_stream(self) -> None:
        self.stream_handle = None

    def _stream(self) -> int:
        h = self.stream_handle
        return h if h is not None else torch.cuda.current_stream().cuda_stream

    def _act(self, t: torch.Tensor, what: str) -> None:
        _dev(t, what)
        if t.dtype != self.dtype:
            raise KernelLibraryError(f"{what} has dtype {t.dtype}, expected {self.dtype}")

    # ------------------------------------------------------------------------------------
    def embedding(self, ids: torch.Tensor, table: torch.Tensor, resid: torch.Tensor, scale: float = 1.0,
                  gather: Optional[tuple] = None) -> None:
        """resid[n] = table[ids[n]] * scale; ids int32 [n], resid float32 [n, h].

        ``gather`` = (index int32 [>= n], float32 table [rows, w], float32 out [n, w]) rides on the same
        launch: out[n] = table[index[n]] (rows outside the table give zeros)."""
        _dev(ids, "ids"); _dev(table, "embedding table"); _dev(resid, "residual")
        n, h = resid.shape
        if ids.dtype != torch.int32 or ids.numel() < n or resid.dtype != torch.float32:
            raise KernelLibraryError("embedding: ids must be int32 [>= n] and the residual float32 [n, h]")
        if table.dim() != 2 or table.shape[1] != h or not table.is_contiguous() or not resid.is_contiguous():
            raise KernelLibraryError(f"embedding: table {tuple(table.shape)} does not fit residual {tuple(resid.shape)}")
        if gather is not None:
            index, table2, out2 = gather
            self._check_gather(index, table2, out2, n)
            self._note("mv_embedding", n * h * (table.element_size() + 4) + n * 4 + n * (8 * out2.shape[1] + 4))
            self.lib.call("mv_embedding_gather", ids.data_ptr(), table.data_ptr(), _weight_code(table, "embedding table"),
                          resid.data_ptr(), n, h, table.shape[0], float(scale), index.data_ptr(), table2.data_ptr(),
                          out2.data_ptr(), table2.shape[1], table2.shape[0], self._stream())
            return
        self._note("mv_embedding", n * h * (table.element_size() + 4) + n * 4)
        self.lib.call("mv_embedding", ids.data_ptr(), table.data_ptr(), _weight_code(table, "embedding table"),
                      resid.data_ptr(), n, h, table.shape[0], float(scale), self._stream())

    @staticmethod
    def _check_gather(index: torch.Tensor, table: torch.Tensor, out: torch.Tensor, n: int) -> None:
        _dev(index, "gather index"); _dev(table, "gather table"); _dev(out, "gathered rows")
        if index.dtype != torch.int32 or index.numel() < n:
            raise KernelLibraryError("gather: the index must be int32 with a row for every token")
        if (table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or out.dtype != torch.float32
                or out.shape != (n, table.shape[1]) or not out.is_contiguous()):
            raise KernelLibraryError(f"gather: float32 table {tuple(table.shape)} does not fit float32 rows {tuple(out.shape)}")

    def gather_rows(self, index: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
        """out[n] = table[index[n]] for a float32 table (rows outside it give zeros)."""
        n = out.shape[0]
        self._check_gather(index, table, out, n)
        self._note("mv_gather_rows", n * (8 * out.shape[1] + 4))      # (a name of its own: "mv_embedding" starts a model step)
        self.lib.call("mv_embedding", index.data_ptr(), table.data_ptr(), DTYPE_F32, out.data_ptr(), n, table.shape[1],
                      table.shape[0], 1.0, self._stream())

    def add_rmsnorm(self, resid: torch.Tensor, delta: Optional[torch.Tensor], weight: Optional[torch.Tensor],
                    eps: float, out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                    unit_offset: bool = False) -> None:
        """resid += delta (when ``rows`` is None), out = rmsnorm(resid + delta) * weight.

        With ``rows`` (int32 [n_out]) only those rows are normalised into ``out`` and the
        residual is left unchanged. ``out`` None does the add alone."""
        _dev(resid, "residual")
        if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
            raise KernelLibraryError("add_rmsnorm: the residual must be a contiguous float32 [n, h]")
        n, h = resid.shape
        if isinstance(delta, SplitSum):
            if self._add_rmsnorm_split(resid, delta, weight, eps, out, rows, unit_offset):
                return
            delta = delta.materialize()
        if delta is not None:
            self._act(delta, "delta")
            if delta.shape != resid.shape or not delta.is_contiguous():
                raise KernelLibraryError(f"add_rmsnorm: delta {tuple(delta.shape)} does not match {tuple(resid.shape)}")
        n_out = n
        if rows is not None:
            _dev(rows, "rows")
            if rows.dtype != torch.int32:
                raise KernelLibraryError("add_rmsnorm: rows must be int32")
            n_out = rows.numel()
        wcode = DTYPE_F32
        if out is not None:
            self._act(out, "norm output")
            if weight is None:
                raise KernelLibraryError("add_rmsnorm: a norm needs its weight")
            _dev(weight, "norm weight")
            wcode = _weight_code(weight, "norm weight")
            if weight.numel() != h or not weight.is_contiguous():
                raise KernelLibraryError(f"add_rmsnorm: weight of {weight.numel()} elements for rows of {h}")
            if out.dim() != 2 or out.shape[0] < n_out or out.shape[1] != h or not out.is_contiguous():
                raise KernelLibraryError(f"add_rmsnorm: output {tuple(out.shape)} does not fit [{n_out}, {h}]")
        self._note("mv_add_rmsnorm", (n * h * (8 if rows is None and delta is not None else 4) if rows is None else n_out * h * 4)
                   + (0 if delta is None else (n if rows is None else n_out) * h * delta.element_size())
                   + (0 if out is None else n_out * h * out.element_size()), 4 * n_out * h)
        self.lib.call("mv_add_rmsnorm", resid.data_ptr(), _ptr(delta), _ptr(weight), wcode, float(eps),
                      int(unit_offset), _ptr(out), _ptr(rows), n_out, h, self.code, self._stream())

    def _add_rmsnorm_split(self, resid: torch.Tensor, delta: "SplitSum", weight: Optional[torch.Tensor], eps: float,
                           out: Optional[torch.Tensor], rows: Optional[torch.Tensor], unit_offset: bool) -> bool:
        """add + norm straight from a product's partial sums; False (nothing done) when the sizes
        are not served. With ``rows`` the delta stays pending in the stream, so the sums are kept."""
        n, h = resid.shape
        if (delta.done or out is None or weight is None or tuple(delta.shape) != (n, h) or h % 8 or h > 8192
                or out.dtype != self.dtype or out.dim() != 2 or out.shape[1] != h or not out.is_contiguous()
                or not weight.is_contiguous() or weight.numel() != h or weight.data_ptr() % 16
                or (rows is not None and (rows.dtype != torch.int32 or out.shape[0] < rows.numel()))
                or (rows is None and out.shape[0] < n)):
            return False
        n_out = n if rows is None else rows.numel()
        self._note("mv_add_rmsnorm_split", n_out * h * (4 * delta.splits + (8 if rows is None else 4) + out.element_size()),
                   (4 + delta.splits) * n_out * h)
        self.lib.call("mv_add_rmsnorm_split", resid.data_ptr(), delta.work.data_ptr(), delta.splits, n * h,
                      _ptr(delta.bias), weight.data_ptr(), _weight_code(weight, "norm weight"), float(eps),
                      int(unit_offset), out.data_ptr(), _ptr(rows), n_out, h, self.code, self._stream())
        if rows is None:
            delta.discard()
        return True

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                unit_offset: bool = False) -> None:
        """out = rmsnorm(x) * weight over the last dimension of 2-d views (rows may be strided)."""
        self._act(x, "rmsnorm input"); self._act(out, "rmsnorm output"); _dev(weight, "norm weight")
        if x.dim() != 2 or out.shape != x.shape or x.stride(1) != 1 or out.stride(1) != 1:
            raise KernelLibraryError("rmsnorm: input and output must be 2-d with a contiguous last dimension")
        n, h = x.shape
        if weight.numel() != h or not weight.is_contiguous():
            raise KernelLibraryError(f"rmsnorm: weight of {weight.numel()} elements for rows of {h}")
        self._note("mv_rmsnorm", self._size(x, out), 4 * n * h)
        self.lib.call("mv_rmsnorm", x.data_ptr(), x.stride(0) if n > 1 else h, weight.data_ptr(),
                      _weight_code(weight, "norm weight"), float(eps), int(unit_offset), out.data_ptr(),
                      out.stride(0) if n > 1 else h, n, h, self.code, self._stream())

    def rope_table(self, inv_freq: torch.Tensor, max_pos: int) -> torch.Tensor:
        """float32 [max_pos, 2 * len(inv_freq)] = cat(cos, sin) of position * inv_freq."""
        _dev(inv_freq, "inv_freq")
        if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
            raise KernelLibraryError("rope_table: inv_freq must be a contiguous float32 vector")
        rot = 2 * inv_freq.numel()
        table = torch.empty((max_pos, rot), dtype=torch.float32, device=inv_freq.device)
        self.lib.call("mv_rope_table", inv_freq.data_ptr(), table.data_ptr(), max_pos, rot, self._stream())
        return table

    def qk_norm_rope_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                           positions: torch.Tensor, token_seq: torch.Tensor,
                           q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                           rope_table: Optional[torch.Tensor], interleaved: bool,
                           k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
                           block_table: Optional[torch.Tensor], page_size: int,
                           unit_offset: bool = False, value_dim: Optional[int] = None, value_from_key: bool = False,
                           extra_columns: int = 0) -> None:
        """In place on the rows of ``qkv`` = [q | k | v]: per-head RMSNorm of q and k (when
        weights are given), rotary embedding (when a table is given); k and v are written to
        the cache pages when pages are given. Without pages the rows hold only q. With
        ``value_dim`` a value row has that size instead of ``head_dim``, and the rows may hold
        further columns behind v (nothing touches them). With ``value_from_key`` the rows are
        [q | k] and the value pages take the keys as the rows hold them, before norm and rotation
        (the key columns themselves are never rewritten: rotated keys go to the key pages only).
        ``extra_columns``: columns behind these that nothing touches."""
        self._act(qkv, "qkv")
        n = qkv.shape[0]
        store = k_pages is not None
        vdim = head_dim if value_dim is None else int(value_dim)
        if value_from_key and (vdim != head_dim or not store):
            raise KernelLibraryError("qk_norm_rope_store: values taken from the keys have the keys' size and go to pages")
        width = num_heads * head_dim + (num_kv_heads * (head_dim + (0 if value_from_key else vdim)) if store else 0)
        if qkv.dim() != 2 or qkv.stride(1) != 1 or (qkv.shape[1] != width + extra_columns if value_dim is None and not extra_columns
                                                    else qkv.shape[1] < width + extra_columns):
            raise KernelLibraryError(f"qk_norm_rope_store: qkv {tuple(qkv.shape)} does not hold {width} columns")
        for t, what in ((positions, "positions"), (token_seq, "token_seq")):
            _dev(t, what)
            if t.dtype != torch.int32 or t.numel() < n:
                raise KernelLibraryError(f"qk_norm_rope_store: {what} must be int32 with at least {n} elements")
        wcode = DTYPE_F32
        if q_weight is not None:
            wcode = _weight_code(q_weight, "q_norm weight")
            if q_weight.numel() != head_dim or (store and (k_weight is None or k_weight.numel() != head_dim
                                                          or k_weight.dtype != q_weight.dtype)):
                raise KernelLibraryError("qk_norm_rope_store: q/k norm weights must both hold head_dim elements")
        rot = 0
        if rope_table is not None:
            _dev(rope_table, "rope table")
            if rope_table.dtype != torch.float32 or rope_table.dim() != 2 or not rope_table.is_contiguous():
                raise KernelLibraryError("qk_norm_rope_store: the rope table must be a contiguous float32 matrix")
            rot = rope_table.shape[1]
        bt_width = 0
        if store:
            assert v_pages is not None and block_table is not None
            self._act(k_pages, "key pages"); self._act(v_pages, "value pages"); _dev(block_table, "block table")
            if tuple(k_pages.shape[1:]) != (num_kv_heads, page_size, head_dim) or \
                    tuple(v_pages.shape[1:]) != (num_kv_heads, vdim, page_size) or \
                    not k_pages.is_contiguous() or not v_pages.is_contiguous():
                raise KernelLibraryError(
                    f"qk_norm_rope_store: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not match "
                    f"[pages, {num_kv_heads}, {page_size}, {head_dim}] / [pages, {num_kv_heads}, {head_dim}, {page_size}]")
            if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
                raise KernelLibraryError("qk_norm_rope_store: the block table must be a contiguous int32 matrix")
            bt_width = block_table.shape[1]
        q_dim = num_heads * head_dim
        kv_dim = num_kv_heads * head_dim
        stride = qkv.stride(0) if n > 1 else qkv.shape[1]
        if store and vdim != head_dim:
            # values of another size than keys: the keys with the queries, the value rows as a launch of their own
            self._note("mv_qk_norm_rope_store", n * (2 * q_dim + 2 * kv_dim + 2 * num_kv_heads * vdim) * qkv.element_size()
                       + (n * rot * 4 if rope_table is not None else 0), 10 * n * (q_dim + kv_dim))
            self.lib.call("mv_qk_norm_rope_store", qkv.data_ptr(), stride, 0, q_dim, q_dim + kv_dim, positions.data_ptr(),
                          token_seq.data_ptr(), _ptr(block_table), bt_width, page_size, _ptr(k_pages), _ptr(v_pages), n,
                          num_heads, num_kv_heads, head_dim, _ptr(q_weight), _ptr(k_weight), wcode, float(eps),
                          int(unit_offset), _ptr(rope_table), rot, int(interleaved), 2, self.code, self._stream())
            self.lib.call("mv_store_v_pages", qkv.data_ptr(), stride, q_dim + kv_dim, positions.data_ptr(),
                          token_seq.data_ptr(), block_table.data_ptr(), bt_width, page_size, v_pages.data_ptr(), n,
                          num_kv_heads, vdim, self.code, self._stream())
            return
        # with many tokens the values go to their transposed pages tile by tile, so that
        # neighbouring tokens write neighbouring slots (mode 3); with few, a store per token and head
        mode = 0 if not store else (3 if n >= STORE_V_SPLIT_TOKENS else 1)
        self._note("mv_qk_norm_rope_store", n * (width + q_dim + (2 * kv_dim if store else 0)) * qkv.element_size()
                   + (n * rot * 4 if rope_table is not None else 0), 10 * n * (q_dim + (kv_dim if store else 0)))
        self.lib.call("mv_qk_norm_rope_store", qkv.data_ptr(), stride, 0, q_dim,
                      q_dim if value_from_key else q_dim + kv_dim, positions.data_ptr(), token_seq.data_ptr(), _ptr(block_table), bt_width,
                      page_size, _ptr(k_pages), _ptr(v_pages), n, num_heads, num_kv_heads, head_dim,
                      _ptr(q_weight), _ptr(k_weight), wcode, float(eps), int(unit_offset), _ptr(rope_table), rot,
                      int(interleaved), mode, self.code, self._stream())

    # ------------------------------------------------------------------------------------
    # parts with a state per request, sandwich norms, capped logits
    # ------------------------------------------------------------------------------------
    @staticmethod
    def _ints(n: int, **tensors) -> None:
        for what, (t, least) in tensors.items():
            _dev(t, what)
            if t.dtype != torch.int32 or t.numel() < least or not t.is_contiguous():
                raise KernelLibraryError(f"{what} must be contiguous int32 with at least {least} elements")

    def token_shift(self, h: torch.Tensor, mix: torch.Tensor, state: torch.Tensor, token_seq: torch.Tensor,
                    cu_seqlens: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor) -> None:
        """out[t] = h[t] + (h[t-1] - h[t]) * mix; the row in front of a request's first row of the step
        is state[slot], which then takes the request's last row. h, out [n, w]; state [slots, w]."""
        self._act(h, "shift input"); self._act(out, "shift output"); self._act(state, "shift state"); _dev(mix, "shift weight")
        n, w = h.shape
        if out.shape != h.shape or h.stride(1) != 1 or out.stride(1) != 1 or out.data_ptr() == h.data_ptr():
            raise KernelLibraryError("token_shift: input and output must be two [n, w] buffers")
        if state.dim() != 2 or state.shape[1] != w or not state.is_contiguous() or mix.numel() != w or not mix.is_contiguous():
            raise KernelLibraryError(f"token_shift: state {tuple(state.shape)} / weight {tuple(mix.shape)} do not fit rows of {w}")
        self._ints(n, token_seq=(token_seq, n), cu_seqlens=(cu_seqlens, 2), state_slots=(state_slots, 1))
        self._note("mv_token_shift", 2 * self._size(h) + self._size(out), 3 * n * w)
        self.lib.call("mv_token_shift", h.data_ptr(), h.stride(0) if n > 1 else w, out.data_ptr(),
                      out.stride(0) if n > 1 else w, mix.data_ptr(), _weight_code(mix, "shift weight"), state.data_ptr(),
                      token_seq.data_ptr(), cu_seqlens.data_ptr(), state_slots.data_ptr(), n, w, self.code, self._stream())

    def input_conv(self, h: torch.Tensor, taps: torch.Tensor, state: Optional[torch.Tensor], token_seq: torch.Tensor,
                   cu_seqlens: torch.Tensor, state_slots: torch.Tensor, n_seqs: int, out: torch.Tensor,
                   taps_t: Optional[torch.Tensor] = None) -> None:
        """out[t] = h[t] + sum_j taps[:, j] * h[t - T + 1 + j] along each request's rows (T = taps.shape[1], the last tap
        multiplies h[t]); the rows in front of a request's first row of the step are state[slot] [T - 1, w], which then
        takes the request's last T - 1 rows. h, out [n, w]; taps [w, T]; state [slots, T - 1, w] (None with one tap).
        ``taps_t`` [T, w]: the same taps tap by tap, which lets the kernel take eight channels a thread."""
        self._act(h, "convolution input"); self._act(out, "convolution output"); _dev(taps, "convolution taps")
        n, w = h.shape
        if out.shape != h.shape or h.stride(1) != 1 or out.stride(1) != 1 or out.data_ptr() == h.data_ptr():
            raise KernelLibraryError("input_conv: input and output must be two [n, w] buffers")
        if taps.dim() != 2 or taps.shape[0] != w or not taps.is_contiguous():
            raise KernelLibraryError(f"input_conv: taps {tuple(taps.shape)} do not fit rows of {w}")
        T = taps.shape[1]
        if T > 1:
            self._act(state, "convolution state")
            if tuple(state.shape[1:]) != (T - 1, w) or not state.is_contiguous():
                raise KernelLibraryError(f"input_conv: state {tuple(state.shape)} does not hold {T - 1} rows of {w}")
        self._ints(n, token_seq=(token_seq, n), cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        self._note("mv_input_conv", self._size(h, out) + (T - 1) * n_seqs * w * h.element_size() * 2, 2 * T * n * w)
        taps_t = self._taps_by_tap(taps, taps_t, "input_conv")
        self.lib.call("mv_input_conv", h.data_ptr(), h.stride(0) if n > 1 else w, out.data_ptr(), out.stride(0) if n > 1 else w,
                      taps.data_ptr(), _ptr(taps_t), _weight_code(taps, "convolution taps"), T, _ptr(state) if T > 1 else 0,
                      token_seq.data_ptr(), cu_seqlens.data_ptr(), state_slots.data_ptr(), n, n_seqs, w, self.code, self._stream())

    @staticmethod
    def _taps_by_tap(taps: torch.Tensor, taps_t: Optional[torch.Tensor], what: str) -> Optional[torch.Tensor]:
        if taps_t is None:
            return None
        _dev(taps_t, "convolution taps, tap by tap")
        if tuple(taps_t.shape) != (taps.shape[1], taps.shape[0]) or taps_t.dtype != taps.dtype or not taps_t.is_contiguous():
            raise KernelLibraryError(f"{what}: taps given tap by tap {tuple(taps_t.shape)} do not mirror the taps {tuple(taps.shape)}")
        return taps_t

    def group_norm(self, weight: torch.Tensor, eps: float, groups: int, out: torch.Tensor, resid: Optional[torch.Tensor] = None,
                   x: Optional[torch.Tensor] = None, delta: Optional[torch.Tensor] = None,
                   rows: Optional[torch.Tensor] = None) -> None:
        """RMS norm in ``groups`` equal runs of neighbouring columns, times ``weight``. Either of the float32 residual
        ``resid`` [n, h] (plus ``delta``; without ``rows`` the sum goes back to ``resid``; with ``rows`` int32 only those rows
        are normalised and nothing is written back) or of the activation rows ``x`` [n, h]."""
        if (resid is None) == (x is None):
            raise KernelLibraryError("group_norm: either the residual or activation rows")
        src = resid if resid is not None else x
        _dev(src, "norm input"); self._act(out, "norm output"); _dev(weight, "norm weight")
        n, h = src.shape
        if resid is not None and (resid.dtype != torch.float32 or not resid.is_contiguous()):
            raise KernelLibraryError("group_norm: the residual must be a contiguous float32 [n, h]")
        if x is not None:
            self._act(x, "norm input")
            if x.dim() != 2 or x.stride(1) != 1 or delta is not None or rows is not None:
                raise KernelLibraryError("group_norm: activation rows are normalised as they are")
        if delta is not None:
            self._act(delta, "delta")
            if delta.shape != src.shape or not delta.is_contiguous():
                raise KernelLibraryError(f"group_norm: delta {tuple(delta.shape)} does not match {tuple(src.shape)}")
        n_out = n
        if rows is not None:
            _dev(rows, "rows")
            if rows.dtype != torch.int32:
                raise KernelLibraryError("group_norm: rows must be int32")
            n_out = rows.numel()
        if weight.numel() != h or not weight.is_contiguous() or groups < 1 or h % groups:
            raise KernelLibraryError(f"group_norm: weight of {weight.numel()} elements / {groups} groups for rows of {h}")
        if out.dim() != 2 or out.shape[0] < n_out or out.shape[1] != h or out.stride(1) != 1:
            raise KernelLibraryError(f"group_norm: output {tuple(out.shape)} does not fit [{n_out}, {h}]")
        self._note("mv_group_norm_rows", n_out * h * (src.element_size() * (2 if resid is not None and delta is not None and rows is None else 1)
                                                      + (delta.element_size() if delta is not None else 0) + out.element_size()),
                   4 * n_out * h)
        self.lib.call("mv_group_norm_rows", _ptr(resid), _ptr(x), (x.stride(0) if n > 1 else h) if x is not None else 0,
                      _ptr(delta), weight.data_ptr(), _weight_code(weight, "norm weight"), float(eps), int(groups),
                      out.data_ptr(), out.stride(0) if out.shape[0] > 1 else h, _ptr(rows), n_out, h, self.code, self._stream())

    def group_norm_add_norm(self, y: torch.Tensor, norm_y, resid: torch.Tensor, norm_next, out: Optional[torch.Tensor],
                            groups: int, conv: Optional[tuple] = None) -> None:
        """resid += gnorm(y) * w (``norm_y`` = (weight, eps)); with ``norm_next`` of the same form, out = gnorm(resid) * w'.
        Both norms work in ``groups`` runs of columns; the sum stays float32 in between.

        ``conv`` = (taps [h, T], state [slots, T - 1, h] or None, token_seq, state_slots[, taps tap by tap [T, h]]), for steps
        in which every request brings one token: ``out`` gets the rows after the input convolution that ``input_conv`` would
        apply to them."""
        self._act(y, "sublayer output"); _dev(resid, "residual")
        n, h = resid.shape
        if resid.dtype != torch.float32 or not resid.is_contiguous() or tuple(y.shape) != (n, h) or y.stride(1) != 1:
            raise KernelLibraryError("group_norm_add_norm: a float32 residual [n, h] and an output of the same shape are needed")
        wa, eps_a = norm_y
        _dev(wa, "norm weight")
        if wa.numel() != h or not wa.is_contiguous() or groups < 1 or h % groups:
            raise KernelLibraryError(f"group_norm_add_norm: weight of {wa.numel()} elements / {groups} groups for rows of {h}")
        wb, eps_b, wb_code = None, 1.0, DTYPE_F32
        if out is not None:
            if norm_next is None:
                raise KernelLibraryError("group_norm_add_norm: an output needs the second norm")
            self._act(out, "norm output")
            wb, eps_b = norm_next
            _dev(wb, "norm weight")
            wb_code = _weight_code(wb, "norm weight")
            if wb.numel() != h or not wb.is_contiguous() or tuple(out.shape) != (n, h) or not out.is_contiguous():
                raise KernelLibraryError("group_norm_add_norm: the second norm's weight or output does not fit")
        taps = taps_t = state = tsq = slots = None
        T, taps_code = 0, DTYPE_F32
        if conv is not None:
            taps, state, tsq, slots = conv[:4]
            if out is None:
                raise KernelLibraryError("group_norm_add_norm: a convolution needs the second norm and its output")
            _dev(taps, "convolution taps")
            taps_code = _weight_code(taps, "convolution taps")
            if taps.dim() != 2 or taps.shape[0] != h or not taps.is_contiguous():
                raise KernelLibraryError(f"group_norm_add_norm: taps {tuple(taps.shape)} do not fit rows of {h}")
            T = taps.shape[1]
            if T > 1:
                self._act(state, "convolution state")
                if tuple(state.shape[1:]) != (T - 1, h) or not state.is_contiguous():
                    raise KernelLibraryError(f"group_norm_add_norm: state {tuple(state.shape)} does not hold {T - 1} rows of {h}")
            self._ints(n, token_seq=(tsq, n), state_slots=(slots, 1))
            taps_t = self._taps_by_tap(taps, conv[4] if len(conv) > 4 else None, "group_norm_add_norm")
        self._note("mv_group_norm_add_norm", self._size(y, out) + 2 * self._size(resid), 8 * n * h)
        self.lib.call("mv_group_norm_add_norm", y.data_ptr(), y.stride(0) if n > 1 else h, wa.data_ptr(),
                      _weight_code(wa, "norm weight"), float(eps_a), resid.data_ptr(), _ptr(wb), wb_code, float(eps_b), int(groups),
                      _ptr(out), n, h, T, _ptr(taps), _ptr(taps_t), taps_code, _ptr(state) if T > 1 else 0, _ptr(tsq), _ptr(slots),
                      self.code, self._stream())

    def xielu(self, x: torch.Tensor, a_pos: float, a_neg: float, out: torch.Tensor) -> None:
        """out = a_pos x^2 + x / 2 where x > 0, a_neg (exp(x) - 1 - x) + x / 2 elsewhere; x, out [n, cols] (may be the same)."""
        self._act(x, "activation input"); self._act(out, "activation output")
        if x.dim() != 2 or out.shape != x.shape or x.stride(1) != 1 or out.stride(1) != 1:
            raise KernelLibraryError("xielu: input and output must be [n, cols] with a contiguous last dimension")
        n, cols = x.shape
        self._note("mv_xielu", self._size(x, out), 6 * n * cols)
        self.lib.call("mv_xielu", x.data_ptr(), x.stride(0) if n > 1 else cols, out.data_ptr(), out.stride(0) if n > 1 else cols,
                      n, cols, float(a_pos), float(a_neg), self.code, self._stream())

    def _delta_weights(self, heads: int, dim: int, rank: int, w2t: torch.Tensor, w0: torch.Tensor, a_bias: torch.Tensor,
                       what: str) -> int:
        inner = heads * dim
        for t, shape, name in ((w2t, (rank, inner), "w2 (transposed)"), (w0, (inner,), "w0"), (a_bias, (inner,), "a_bias")):
            _dev(t, name)
            if tuple(t.shape) != shape or not t.is_contiguous() or t.dtype != w2t.dtype:
                raise KernelLibraryError(f"{what}: {name} must be a contiguous {shape} tensor of w2's dtype")
        return _weight_code(w2t, "w2")

    def delta_prepare(self, packed: torch.Tensor, heads: int, dim: int, rank: int, w2t: torch.Tensor, w0: torch.Tensor,
                      a_bias: torch.Tensor, decay_rate: float, key_eps: float, coef: torch.Tensor) -> None:
        """From rows [r | k | v | g | a | w1] (heads*dim columns each, ``rank`` for w1) the float32
        vectors of the delta rule, coef [n, heads, 5, dim]: the decay
        exp(-decay_rate * sigmoid(w2 tanh(w1) + w0)), rate * unit key with rate = sigmoid(a + a_bias),
        the unit key k / sqrt(sum(k^2) + key_eps) of each head, k and r. ``w2t`` is w2 transposed, [rank, heads*dim]."""
        self._act(packed, "delta rows")
        n, inner = packed.shape[0], heads * dim
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < 5 * inner + rank:
            raise KernelLibraryError(f"delta_prepare: rows {tuple(packed.shape)} do not hold 5 x {inner} + {rank} columns")
        if coef.dtype != torch.float32 or tuple(coef.shape) != (n, heads, 5, dim) or not coef.is_contiguous():
            raise KernelLibraryError(f"delta_prepare: coefficients must be float32 [{n}, {heads}, 5, {dim}]")
        wcode = self._delta_weights(heads, dim, rank, w2t, w0, a_bias, "delta_prepare")
        self._note("mv_delta_prepare", n * (3 * inner + rank) * packed.element_size() + self._size(w2t, coef), 2 * n * inner * rank)
        self.lib.call("mv_delta_prepare", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], n, heads, dim,
                      rank, w2t.data_ptr(), w0.data_ptr(), a_bias.data_ptr(), wcode, float(decay_rate),
                      float(key_eps), coef.data_ptr(), self.code, self._stream())

    def _delta_state(self, state: torch.Tensor, heads: int, dim: int, what: str) -> None:
        _dev(state, "delta state")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, dim) or not state.is_contiguous():
            raise KernelLibraryError(f"{what}: the state must be float32 [slots, {heads}, {dim}, {dim}]")

    def delta_scan(self, packed: torch.Tensor, coef: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor,
                   state_slots: torch.Tensor, n_seqs: int, heads: int, dim: int, out: torch.Tensor) -> None:
        """The delta rule over the step's rows, request by request (rows cu_seqlens[s] .. cu_seqlens[s+1]
        of request s, state row state_slots[s]): S <- diag(w) S - (a*u)(u^T S) + k v^T, out = S^T r, with
        v from the packed rows and w, a*u, u, k, r from ``coef``. state float32 [slots, heads, dim, dim]
        holds each head's matrix column by column (state[.., j, i] = S[i][j], i the key channel); it is
        read and left advanced. out float32 [n, heads*dim]."""
        self._act(packed, "delta rows")
        n, inner = packed.shape[0], heads * dim
        if coef.dtype != torch.float32 or tuple(coef.shape) != (n, heads, 5, dim) or not coef.is_contiguous():
            raise KernelLibraryError(f"delta_scan: coefficients must be float32 [{n}, {heads}, 5, {dim}]")
        if out.dtype != torch.float32 or tuple(out.shape) != (n, inner) or not out.is_contiguous():
            raise KernelLibraryError(f"delta_scan: the output must be float32 [{n}, {inner}]")
        self._delta_state(state, heads, dim, "delta_scan")
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < 3 * inner:
            raise KernelLibraryError(f"delta_scan: rows {tuple(packed.shape)} do not hold r, k and v")
        self._ints(n, cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        self._note("mv_delta_scan", n * inner * packed.element_size() + self._size(coef, out)
                   + 2 * min(n_seqs, max(n, 1)) * inner * dim * 4, 8 * n * inner * dim)
        self.lib.call("mv_delta_scan", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], coef.data_ptr(),
                      state.data_ptr(), cu_seqlens.data_ptr(), state_slots.data_ptr(), n_seqs, n, heads, dim,
                      out.data_ptr(), self.code, self._stream())

    def delta_step(self, packed: torch.Tensor, heads: int, dim: int, rank: int, w2t: torch.Tensor, w0: torch.Tensor,
                   a_bias: torch.Tensor, norm_weight: torch.Tensor, decay_rate: float, key_eps: float, eps: float,
                   state: torch.Tensor, token_seq: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor) -> None:
        """``delta_prepare``, ``delta_scan`` and ``delta_finish`` in one kernel for a step in which every
        request brings one token: row t belongs to request token_seq[t] (negative: a padding row)."""
        self._act(packed, "delta rows"); self._act(out, "delta output"); _dev(norm_weight, "delta norm weight")
        n, inner = packed.shape[0], heads * dim
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < 5 * inner + rank:
            raise KernelLibraryError(f"delta_step: rows {tuple(packed.shape)} do not hold 5 x {inner} + {rank} columns")
        if tuple(out.shape) != (n, inner) or out.stride(1) != 1 or norm_weight.numel() != inner \
                or not norm_weight.is_contiguous() or norm_weight.dtype != w2t.dtype:
            raise KernelLibraryError("delta_step: output or norm weight do not fit")
        wcode = self._delta_weights(heads, dim, rank, w2t, w0, a_bias, "delta_step")
        self._delta_state(state, heads, dim, "delta_step")
        self._ints(n, token_seq=(token_seq, n), state_slots=(state_slots, 1))
        self._note("mv_delta_step", n * (5 * inner + rank) * packed.element_size() + self._size(w2t, out)
                   + 2 * n * inner * dim * 4, 8 * n * inner * dim + 2 * n * inner * rank)
        self.lib.call("mv_delta_step", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], n, heads, dim, rank,
                      w2t.data_ptr(), w0.data_ptr(), a_bias.data_ptr(), norm_weight.data_ptr(), wcode, float(decay_rate),
                      float(key_eps), float(eps), state.data_ptr(), token_seq.data_ptr(), state_slots.data_ptr(),
                      out.data_ptr(), out.stride(0) if n > 1 else inner, self.code, self._stream())

    def delta_finish(self, raw: torch.Tensor, packed: torch.Tensor, weight: torch.Tensor, heads: int, dim: int,
                     eps: float, out: torch.Tensor) -> None:
        """out = raw / rms(raw over each head) * weight * sigmoid(g), g the fourth block of the packed rows."""
        self._act(packed, "delta rows"); self._act(out, "delta output"); _dev(weight, "delta norm weight")
        n, inner = packed.shape[0], heads * dim
        if raw.dtype != torch.float32 or tuple(raw.shape) != (n, inner) or not raw.is_contiguous():
            raise KernelLibraryError(f"delta_finish: the scan's output must be float32 [{n}, {inner}]")
        if tuple(out.shape) != (n, inner) or out.stride(1) != 1 or packed.shape[1] < 4 * inner or weight.numel() != inner \
                or not weight.is_contiguous():
            raise KernelLibraryError("delta_finish: operands do not fit")
        self._note("mv_delta_finish", self._size(raw, out) + n * inner * packed.element_size(), 8 * n * inner)
        self.lib.call("mv_delta_finish", raw.data_ptr(), packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1],
                      weight.data_ptr(), _weight_code(weight, "delta norm weight"), n, heads, dim, float(eps),
                      out.data_ptr(), out.stride(0) if n > 1 else inner, self.code, self._stream())

    # ------------------------------------------------------------------------------------
    # mixers with a decayed matrix state per head and scalar gates (gated delta rule, mLSTM)
    def _state_vectors(self, n: int, heads: int, groups: int, dk: int, dvs: int, qk: torch.Tensor, vals: torch.Tensor,
                       gates: torch.Tensor, what: str) -> None:
        for t, shape, name in ((qk, (n, groups, 2, dk), "queries and keys"), (vals, (n, heads, dvs), "values"),
                               (gates, (n, heads, 4), "gates")):
            _dev(t, name)
            if t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous():
                raise KernelLibraryError(f"{what}: {name} must be contiguous float32 {shape}, got {tuple(t.shape)} {t.dtype}")

    def gated_delta_prepare(self, packed: torch.Tensor, heads: int, groups: int, dk: int, dv: int, taps: int,
                            conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                            conv_state: Optional[torch.Tensor], unit_eps: float, token_seq: torch.Tensor,
                            cu_seqlens: torch.Tensor, state_slots: torch.Tensor, n_seqs: int, qk: torch.Tensor,
                            vals: torch.Tensor, gates: torch.Tensor) -> None:
        """From rows [q (groups*dk) | k (groups*dk) | v (heads*dv) | g | b (heads) | a (heads)]: q, k, v through a
        causal convolution of ``taps`` taps per channel (conv_w [channels, taps], last tap the current token) and
        SiLU; q and k unit vectors per group (q times dk^-1/2); gates[..., 0] = exp(-exp(a_log) softplus(a + dt_bias)),
        gates[..., 1] = sigmoid(b). conv_state [slots, taps-1, channels] holds each request's last inputs: read for
        the rows in front of the step, then advanced."""
        self._act(packed, "delta rows")
        n, C = packed.shape[0], 2 * groups * dk + heads * dv
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < C + heads * dv + 2 * heads:
            raise KernelLibraryError(f"gated_delta_prepare: rows {tuple(packed.shape)} are too short")
        self._state_vectors(n, heads, groups, dk, dv, qk, vals, gates, "gated_delta_prepare")
        for t, shape, name in ((conv_w, (C, taps), "convolution taps"), (a_log, (heads,), "A_log"), (dt_bias, (heads,), "dt_bias")):
            _dev(t, name)
            if tuple(t.shape) != shape or not t.is_contiguous() or t.dtype != conv_w.dtype:
                raise KernelLibraryError(f"gated_delta_prepare: {name} must be a contiguous {shape} tensor of the taps' dtype")
        if taps > 1:
            self._act(conv_state, "convolution state")
            if conv_state.dim() != 3 or tuple(conv_state.shape[1:]) != (taps - 1, C) or not conv_state.is_contiguous():
                raise KernelLibraryError(f"gated_delta_prepare: the convolution's state must be [slots, {taps - 1}, {C}]")
        self._ints(n, token_seq=(token_seq, n), cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        self._note("mv_gdelta_prepare", n * (C + 2 * heads) * packed.element_size() + self._size(qk, vals, gates), 2 * n * C * taps + 8 * n * C)
        self.lib.call("mv_gdelta_prepare", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], n, n_seqs, heads,
                      groups, dk, dv, taps, conv_w.data_ptr(), a_log.data_ptr(), dt_bias.data_ptr(),
                      _weight_code(conv_w, "convolution taps"), _ptr(conv_state), float(unit_eps), token_seq.data_ptr(),
                      cu_seqlens.data_ptr(), state_slots.data_ptr(), qk.data_ptr(), vals.data_ptr(), gates.data_ptr(),
                      self.code, self._stream())

    def mlstm_prepare(self, packed: torch.Tensor, heads: int, dk: int, dv: int, i_bias: torch.Tensor, f_bias: torch.Tensor,
                      cap: float, max_state: torch.Tensor, token_seq: torch.Tensor, cu_seqlens: torch.Tensor,
                      state_slots: torch.Tensor, n_seqs: int, qk: torch.Tensor, vals: torch.Tensor, gates: torch.Tensor) -> None:
        """From rows [q | k (heads*dk each) | v | g (heads*dv each) | i | f (heads each)]: q * dk^-1/2 and k as floats,
        the values with a one behind them (vals [n, heads, dv + 1]), and the stabilised gates: with
        i' = cap tanh((i + i_bias)/cap), f' = logsigmoid(cap tanh((f + f_bias)/cap)) and the running maximum
        m' = max(f' + m, i') (max_state [slots, heads], read and advanced), gates = (exp(f' + m - m'), exp(i' - m'), exp(-m'), 0)."""
        self._act(packed, "mlstm rows")
        n = packed.shape[0]
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < 2 * heads * (dk + dv) + 2 * heads:
            raise KernelLibraryError(f"mlstm_prepare: rows {tuple(packed.shape)} are too short")
        self._state_vectors(n, heads, heads, dk, dv + 1, qk, vals, gates, "mlstm_prepare")
        for t, name in ((i_bias, "input gate bias"), (f_bias, "forget gate bias")):
            _dev(t, name)
            if t.numel() != heads or not t.is_contiguous() or t.dtype != i_bias.dtype:
                raise KernelLibraryError(f"mlstm_prepare: the {name} must hold {heads} numbers")
        _dev(max_state, "running maximum")
        if max_state.dtype != torch.float32 or max_state.dim() != 2 or max_state.shape[1] != heads or not max_state.is_contiguous():
            raise KernelLibraryError(f"mlstm_prepare: the running maximum must be float32 [slots, {heads}]")
        self._ints(n, token_seq=(token_seq, n), cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        self._note("mv_mlstm_prepare", n * (2 * heads * dk + heads * dv + 2 * heads) * packed.element_size() + self._size(qk, vals, gates),
                   40 * n * heads)
        self.lib.call("mv_mlstm_prepare", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], n, n_seqs, heads, dk,
                      dv, i_bias.data_ptr(), f_bias.data_ptr(), _weight_code(i_bias, "gate bias"), float(cap),
                      max_state.data_ptr(), token_seq.data_ptr(), cu_seqlens.data_ptr(), state_slots.data_ptr(), qk.data_ptr(),
                      vals.data_ptr(), gates.data_ptr(), self.code, self._stream())

    def state_scan(self, qk: torch.Tensor, vals: torch.Tensor, gates: torch.Tensor, state: torch.Tensor,
                   cu_seqlens: torch.Tensor, state_slots: torch.Tensor, n_seqs: int, heads: int, groups: int, dk: int,
                   dvs: int, read: bool, out: torch.Tensor) -> None:
        """Per request and head, token by token: S <- a S; u = b (v - [read] S^T k); S <- S + k u^T; out = S^T q, with
        (a, b) = gates[..., :2]. state float32 [slots, heads, dvs, dk] (a head's matrix column by column) is read and
        left advanced; out float32 [n, heads, dvs]."""
        n = vals.shape[0]
        self._state_vectors(n, heads, groups, dk, dvs, qk, vals, gates, "state_scan")
        _dev(state, "matrix state"); _dev(out, "scan output")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dvs, dk) or not state.is_contiguous():
            raise KernelLibraryError(f"state_scan: the state must be float32 [slots, {heads}, {dvs}, {dk}]")
        if out.dtype != torch.float32 or tuple(out.shape) != (n, heads, dvs) or not out.is_contiguous():
            raise KernelLibraryError(f"state_scan: the output must be float32 [{n}, {heads}, {dvs}]")
        self._ints(n, cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        self._note("mv_state_scan", self._size(qk, vals, gates, out) + 2 * min(n_seqs, max(n, 1)) * heads * dvs * dk * 4,
                   (6 if read else 4) * n * heads * dvs * dk)
        self.lib.call("mv_state_scan", qk.data_ptr(), vals.data_ptr(), gates.data_ptr(), state.data_ptr(), cu_seqlens.data_ptr(),
                      state_slots.data_ptr(), n_seqs, n, heads, groups, dk, dvs, int(bool(read)), out.data_ptr(), self._stream())

    def state_finish(self, raw: torch.Tensor, gates: torch.Tensor, packed: torch.Tensor, gate_offset: int, weight: torch.Tensor,
                     heads: int, dv: int, eps: float, token_seq: torch.Tensor, out: torch.Tensor, shared_weight: bool,
                     silu_gate: bool, normaliser: bool = False, denom_eps: float = 0.0) -> None:
        """out[t, h] = o / rms(o) * weight * act(g) per head, o = raw[t, h, :dv]; with ``normaliser`` o is first divided
        by max(|raw[t, h, dv]|, gates[t, h, 2]) + denom_eps. ``weight`` holds dv numbers shared by the heads or
        heads*dv; act is SiLU or the logistic function; g are ``heads*dv`` columns of ``packed`` from ``gate_offset``."""
        self._act(packed, "mixer rows"); self._act(out, "mixer output"); _dev(weight, "output norm weight")
        n, dvs = packed.shape[0], dv + (1 if normaliser else 0)
        if raw.dtype != torch.float32 or tuple(raw.shape) != (n, heads, dvs) or not raw.is_contiguous():
            raise KernelLibraryError(f"state_finish: the scan's output must be float32 [{n}, {heads}, {dvs}]")
        if gates.dtype != torch.float32 or tuple(gates.shape) != (n, heads, 4) or not gates.is_contiguous():
            raise KernelLibraryError("state_finish: gates must be float32 [n, heads, 4]")
        if tuple(out.shape) != (n, heads * dv) or out.stride(1) != 1 or packed.shape[1] < gate_offset + heads * dv \
                or weight.numel() != (dv if shared_weight else heads * dv) or not weight.is_contiguous():
            raise KernelLibraryError("state_finish: operands do not fit")
        self._ints(n, token_seq=(token_seq, n))
        self._note("mv_state_finish", self._size(raw, out) + n * heads * dv * packed.element_size(), 8 * n * heads * dv)
        self.lib.call("mv_state_finish", raw.data_ptr(), gates.data_ptr(), packed.data_ptr(),
                      packed.stride(0) if n > 1 else packed.shape[1], int(gate_offset), weight.data_ptr(),
                      _weight_code(weight, "output norm weight"), int(shared_weight), int(silu_gate), int(normaliser),
                      float(denom_eps), n, heads, dv, float(eps), token_seq.data_ptr(), out.data_ptr(),
                      out.stride(0) if n > 1 else heads * dv, self.code, self._stream())

    def state_step(self, delta: bool, packed: torch.Tensor, heads: int, groups: int, dk: int, dv: int, norm_weight: torch.Tensor,
                   eps: float, state: torch.Tensor, token_seq: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor,
                   n_seqs: int, out: torch.Tensor, taps: int = 1, conv_w: Optional[torch.Tensor] = None,
                   a_log: Optional[torch.Tensor] = None, dt_bias: Optional[torch.Tensor] = None,
                   conv_state: Optional[torch.Tensor] = None, unit_eps: float = 1e-6, i_bias: Optional[torch.Tensor] = None,
                   f_bias: Optional[torch.Tensor] = None, cap: float = 1.0, max_state: Optional[torch.Tensor] = None,
                   denom_eps: float = 0.0) -> bool:
        """For a step in which every request brings one token: the prepare kernel, ``state_scan`` and ``state_finish`` of
        the gated delta rule (``delta``) or of the mLSTM as one kernel per (row, head), with the same sums in the same
        order. False when the sizes are not served (nothing was done)."""
        self._act(packed, "mixer rows"); self._act(out, "mixer output"); _dev(norm_weight, "output norm weight")
        n = packed.shape[0]
        dvs = dv if delta else dv + 1
        width = (2 * groups * dk + 2 * heads * dv + 2 * heads) if delta else (2 * heads * (dk + dv) + 2 * heads)
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < width or tuple(out.shape) != (n, heads * dv) \
                or out.stride(1) != 1 or norm_weight.numel() != (dv if delta else heads * dv) or not norm_weight.is_contiguous():
            raise KernelLibraryError("state_step: operands do not fit")
        _dev(state, "matrix state")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dvs, dk) or not state.is_contiguous():
            raise KernelLibraryError(f"state_step: the state must be float32 [slots, {heads}, {dvs}, {dk}]")
        wcode = _weight_code(norm_weight, "output norm weight")
        if delta:
            C = 2 * groups * dk + heads * dv
            for t, shape, name in ((conv_w, (C, taps), "convolution taps"), (a_log, (heads,), "A_log"), (dt_bias, (heads,), "dt_bias")):
                _dev(t, name)
                if tuple(t.shape) != shape or not t.is_contiguous() or t.dtype != norm_weight.dtype:
                    raise KernelLibraryError(f"state_step: {name} must be a contiguous {shape} tensor of the norm weight's dtype")
            if taps > 1:
                self._act(conv_state, "convolution state")
                if conv_state.dim() != 3 or tuple(conv_state.shape[1:]) != (taps - 1, C) or not conv_state.is_contiguous():
                    raise KernelLibraryError(f"state_step: the convolution's state must be [slots, {taps - 1}, {C}]")
        else:
            for t, name in ((i_bias, "input gate bias"), (f_bias, "forget gate bias")):
                _dev(t, name)
                if t.numel() != heads or not t.is_contiguous() or t.dtype != norm_weight.dtype:
                    raise KernelLibraryError(f"state_step: the {name} must hold {heads} numbers of the norm weight's dtype")
            _dev(max_state, "running maximum")
            if max_state.dtype != torch.float32 or max_state.dim() != 2 or max_state.shape[1] != heads or not max_state.is_contiguous():
                raise KernelLibraryError(f"state_step: the running maximum must be float32 [slots, {heads}]")
        self._ints(n, token_seq=(token_seq, n), cu_seqlens=(cu_seqlens, n_seqs + 1), state_slots=(state_slots, n_seqs))
        if not self.lib.offer("mv_state_step", int(bool(delta)), packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1],
                              n, n_seqs, heads, groups, dk, dv, taps, _ptr(conv_w), _ptr(a_log), _ptr(dt_bias), _ptr(i_bias),
                              _ptr(f_bias), norm_weight.data_ptr(), wcode, _ptr(conv_state), _ptr(max_state), state.data_ptr(),
                              float(unit_eps), float(cap), float(denom_eps), float(eps), token_seq.data_ptr(),
                              cu_seqlens.data_ptr(), state_slots.data_ptr(), out.data_ptr(),
                              out.stride(0) if n > 1 else heads * dv, self.code, self._stream()):
            return False
        self._note("mv_state_step", n * width * packed.element_size() + self._size(out) + 2 * n * heads * dvs * dk * 4,
                   (6 if delta else 4) * n * heads * dvs * dk)
        return True

    # ------------------------------------------------------------------------------------
    # attention over a cached latent
    def latent_prepare(self, packed: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, q_norm: torch.Tensor,
                       kv_norm: torch.Tensor, eps: float, table: Optional[torch.Tensor], positions: torch.Tensor,
                       token_seq: torch.Tensor, block_table: torch.Tensor, page_size: int, q_latent: torch.Tensor,
                       pages: torch.Tensor, pages_t: Optional[torch.Tensor] = None) -> None:
        """From rows [dq (q_rank) | dkv (kv_rank + rot_dim) | ...]: q_latent = rmsnorm(dq) * q_norm; the row's cache
        entry [rmsnorm(dkv[:kv_rank]) * kv_norm | rot(dkv[kv_rank:])] goes to pages [pages, page_size, kv_rank + rot_dim]
        at the row's position (``table``: float32 [positions, rot_dim] = cat(cos, sin), pairs i, i + rot_dim/2).
        ``pages_t`` [pages, kv_rank, page_size], when given, gets the latent once more, a page's slots side by side."""
        self._act(packed, "latent rows"); self._act(q_latent, "query latent"); self._act(pages, "latent pages")
        n = packed.shape[0]
        if packed.dim() != 2 or packed.stride(1) != 1 or packed.shape[1] < q_rank + kv_rank + rot_dim:
            raise KernelLibraryError(f"latent_prepare: rows {tuple(packed.shape)} are too short")
        if tuple(q_latent.shape) != (n, q_rank) or q_latent.stride(1) != 1:
            raise KernelLibraryError(f"latent_prepare: the query latent must be [{n}, {q_rank}]")
        if pages.dim() != 3 or tuple(pages.shape[1:]) != (page_size, kv_rank + rot_dim) or not pages.is_contiguous():
            raise KernelLibraryError(f"latent_prepare: pages must be [pages, {page_size}, {kv_rank + rot_dim}]")
        for t, size, name in ((q_norm, q_rank, "query latent norm"), (kv_norm, kv_rank, "latent norm")):
            _dev(t, name)
            if t.numel() != size or not t.is_contiguous() or t.dtype != q_norm.dtype:
                raise KernelLibraryError(f"latent_prepare: the {name} weight must hold {size} numbers")
        if pages_t is not None:
            self._act(pages_t, "slot-contiguous latent pages")
            if tuple(pages_t.shape) != (pages.shape[0], kv_rank, page_size) or not pages_t.is_contiguous():
                raise KernelLibraryError(f"latent_prepare: the slot-contiguous pages must be [{pages.shape[0]}, {kv_rank}, {page_size}]")
        rows = 0
        if rot_dim:
            _dev(table, "rotary table")
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise KernelLibraryError(f"latent_prepare: the rotary table must be float32 [positions, {rot_dim}]")
            rows = table.shape[0]
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("latent_prepare: the block table must be contiguous int32 [sequences, width]")
        self._ints(n, positions=(positions, n), token_seq=(token_seq, n))
        self._note("mv_latent_prepare", n * (q_rank + kv_rank + rot_dim) * 2 * packed.element_size(), 8 * n * (q_rank + kv_rank + rot_dim))
        self.lib.call("mv_latent_prepare", packed.data_ptr(), packed.stride(0) if n > 1 else packed.shape[1], n, q_rank, kv_rank,
                      rot_dim, q_norm.data_ptr(), kv_norm.data_ptr(), _weight_code(q_norm, "latent norm"), float(eps),
                      _ptr(table), rows, positions.data_ptr(), token_seq.data_ptr(), block_table.data_ptr(),
                      block_table.shape[1], page_size, q_latent.data_ptr(), q_latent.stride(0) if n > 1 else q_rank,
                      pages.data_ptr(), _ptr(pages_t), self.code, self._stream())

    def head_linear(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, token_seq: torch.Tensor, tail: int = 0,
                    table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                    gate: Optional[torch.Tensor] = None, w_rows: Optional[torch.Tensor] = None,
                    gate_per_head: bool = False) -> None:
        """Per head h: out[t, h, :OUT] = x[t, h, :IN] @ w[h] with w [heads, IN, OUT]. (With ``gate_per_head`` the gate is
        [n, >= heads] rows, one number for all outputs of a head.) x [n, heads, IN + tail] in the
        activation type gives out float32 [n, heads, OUT + tail], the ``tail`` last inputs copied behind the outputs
        and rotated by the row's position (``table`` as for ``latent_prepare``); x float32 [n, heads, IN] gives out
        [n, heads * OUT] in the activation type, multiplied by sigmoid(gate [n, heads * OUT]) when a gate is given.
        ``w_rows`` is the same weight as [heads, OUT, IN]: in bfloat16, steps of more than 64 rows whose IN is a multiple
        of 32 take the MFMA kernel, which reads that layout (and rounds float32 inputs to bfloat16 as it reads them)."""
        _dev(x, "head_linear input"); _dev(w, "head_linear weight"); _dev(out, "head_linear output")
        if w.dim() != 3 or not w.is_contiguous() or x.dim() != 3 or x.stride(2) != 1 or x.stride(1) != x.shape[2]:
            raise KernelLibraryError("head_linear: x [n, heads, width] and a contiguous w [heads, IN, OUT] are needed")
        n, H = x.shape[0], w.shape[0]
        IN, OUT = w.shape[1], w.shape[2]
        self._ints(n, token_seq=(token_seq, n))
        if out.dim() == 3 and x.dtype == self.dtype and out.dtype == torch.float32 and gate is None:
            mode = 0
            if tuple(x.shape) != (n, H, IN + tail) or tuple(out.shape) != (n, H, OUT + tail) or not out.is_contiguous():
                raise KernelLibraryError(f"head_linear: {tuple(x.shape)} x {tuple(w.shape)} -> {tuple(out.shape)} does not fit")
            ldy, ldy_head = out.stride(0) if n > 1 else H * (OUT + tail), OUT + tail
            if tail:
                _dev(table, "rotary table")
                if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != tail or not table.is_contiguous():
                    raise KernelLibraryError(f"head_linear: the rotary table must be float32 [positions, {tail}]")
                self._ints(n, positions=(positions, n))
        elif out.dim() == 2 and x.dtype == torch.float32 and out.dtype == self.dtype and tail == 0:
            mode = 1
            if tuple(x.shape) != (n, H, IN) or tuple(out.shape) != (n, H * OUT) or out.stride(1) != 1:
                raise KernelLibraryError(f"head_linear: {tuple(x.shape)} x {tuple(w.shape)} -> {tuple(out.shape)} does not fit")
            ldy, ldy_head = out.stride(0) if n > 1 else H * OUT, OUT
            if gate is not None:
                self._act(gate, "output gate")
                if gate.dim() != 2 or gate.shape[0] != n or gate.stride(1) != 1 \
                        or (gate.shape[1] < H if gate_per_head else gate.shape[1] != H * OUT):
                    raise KernelLibraryError("head_linear: the gate must be [n, heads * OUT], or [n, >= heads] with one number a head")
        else:
            raise KernelLibraryError(f"head_linear: {x.dtype} -> {out.dtype} with these options is not served")
        if w_rows is not None and n > 64 and self.use_fast_kernels and w_rows.dtype == torch.bfloat16 \
                and self.lib.has("mv_head_linear_mfma"):
            _dev(w_rows, "head_linear weight")
            if tuple(w_rows.shape) != (H, OUT, IN) or not w_rows.is_contiguous():
                raise KernelLibraryError(f"head_linear: the row layout of the weight must be [{H}, {OUT}, {IN}]")
            if self.lib.offer("mv_head_linear_mfma", x.data_ptr(), x.stride(0), x.shape[2], w_rows.data_ptr(), n, H, IN, OUT,
                              out.data_ptr(), ldy, ldy_head, tail, _ptr(table), _ptr(positions), _ptr(gate),
                              gate.stride(0) if gate is not None else 0, int(gate_per_head), token_seq.data_ptr(), mode,
                              self._stream()):
                self._note("mv_head_linear_mfma", self._size(x, w, out), 2 * n * H * IN * OUT)
                return
        self._note("mv_head_linear", self._size(x, w, out), 2 * n * H * IN * OUT)
        self.lib.call("mv_head_linear", x.data_ptr(), x.stride(0) if n > 1 else H * x.shape[2], x.shape[2], w.data_ptr(),
                      _weight_code(w, "head_linear weight"), n, H, IN, OUT, out.data_ptr(), ldy, ldy_head, tail, _ptr(table),
                      _ptr(positions), _ptr(gate), (gate.stride(0) if n > 1 else gate.shape[1]) if gate is not None else 0,
                      int(gate_per_head), token_seq.data_ptr(), mode, self.code, self._stream())

    def attention_latent(self, q: torch.Tensor, out: torch.Tensor, pages: torch.Tensor, block_table: torch.Tensor,
                         page_size: int, positions: torch.Tensor, token_seq: torch.Tensor, heads: int, kv_rank: int,
                         rot_dim: int, scale: float, plan=None, pages_t: Optional[torch.Tensor] = None) -> None:
        """Causal softmax attention of q float32 [n, heads, kv_rank + rot_dim] over the cached rows [latent | rotated
        key part] of each row's request (pages [pages, page_size, kv_rank + rot_dim]); out float32 [n, heads, kv_rank] is
        the weighted sum of the latents. Steps of single tokens take the kernel that deals a row's keys out over workgroups;
        in bfloat16 other steps take the MFMA kernel where it serves the sizes (it reads the values from ``pages_t``
        [pages, kv_rank, page_size], the latents with a page's slots side by side); everything else the general kernel."""
        _dev(q, "latent queries"); _dev(out, "latent attention output"); self._act(pages, "latent pages")
        n, dk = q.shape[0], kv_rank + rot_dim
        if q.dtype != torch.float32 or tuple(q.shape) != (n, heads, dk) or not q.is_contiguous():
            raise KernelLibraryError(f"attention_latent: queries must be float32 [{n}, {heads}, {dk}]")
        if out.dtype != torch.float32 or tuple(out.shape) != (n, heads, kv_rank) or not out.is_contiguous():
            raise KernelLibraryError(f"attention_latent: the output must be float32 [{n}, {heads}, {kv_rank}]")
        if pages.dim() != 3 or tuple(pages.shape[1:]) != (page_size, dk) or not pages.is_contiguous():
            raise KernelLibraryError(f"attention_latent: pages must be [pages, {page_size}, {dk}]")
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("attention_latent: the block table must be contiguous int32 [sequences, width]")
        self._ints(n, positions=(positions, n), token_seq=(token_seq, n))
        kv_tokens = plan.kv_tokens if plan is not None else 0
        pairs = plan.attention_pairs if plan is not None else 0
        if plan is not None and plan.decode_only and plan.max_context_len > 0 and self._attention_latent_split(
                q, out, pages, block_table, page_size, positions, token_seq, n, heads, kv_rank, rot_dim, scale,
                plan.max_context_len, kv_tokens):
            return
        if pages_t is not None and self.use_fast_kernels and self.lib.has("mv_attention_latent_mfma") \
                and not (plan is not None and plan.decode_only):
            self._act(pages_t, "slot-contiguous latent pages")
            if tuple(pages_t.shape) != (pages.shape[0], kv_rank, page_size) or not pages_t.is_contiguous():
                raise KernelLibraryError(f"attention_latent: the slot-contiguous pages must be [{pages.shape[0]}, {kv_rank}, {page_size}]")
            if self.lib.offer("mv_attention_latent_mfma", q.data_ptr(), heads * dk, out.data_ptr(), heads * kv_rank, pages.data_ptr(),
                              pages_t.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size, positions.data_ptr(),
                              token_seq.data_ptr(), n, heads, kv_rank, rot_dim, float(scale), self._stream()):
                self._note("mv_attention_latent_mfma", self._size(q, out) + kv_tokens * (dk + kv_rank) * pages.element_size(),
                           2 * pairs * heads * (dk + kv_rank))
                return
        self._note("mv_attention_latent", self._size(q, out) + kv_tokens * dk * pages.element_size(),
                   2 * pairs * heads * (dk + kv_rank))
        self.lib.call("mv_attention_latent", q.data_ptr(), heads * dk, out.data_ptr(), heads * kv_rank, pages.data_ptr(),
                      block_table.data_ptr(), block_table.shape[1], page_size, positions.data_ptr(), token_seq.data_ptr(),
                      n, heads, kv_rank, rot_dim, float(scale), self.code, self._stream())

    def _attention_latent_split(self, q, out, pages, block_table, page_size, positions, token_seq, n, heads, kv_rank, rot_dim,
                                scale, max_context, kv_tokens) -> bool:
        """Steps of single tokens: each row's keys dealt out to workgroups in runs of 256 positions, every workgroup
        serving 16 heads from key rows staged in LDS; False when the sizes are not served (the general kernel runs)."""
        need = int(self.lib.dll.mv_attention_latent_split_workspace(n, heads, kv_rank, max_context))
        if self._latent_work is None or self._latent_work.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                return False                                   # no allocation inside a capture
            if self._latent_work is not None:
                self._mid_retired.append(self._latent_work)    # captured graphs may hold its address
            self._latent_work = torch.empty(max(need, 1 << 20), dtype=torch.float32, device=q.device)
        dk = kv_rank + rot_dim
        if not self.lib.offer("mv_attention_latent_split", q.data_ptr(), heads * dk, out.data_ptr(), heads * kv_rank,
                              pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size, positions.data_ptr(),
                              token_seq.data_ptr(), n, heads, kv_rank, rot_dim, float(scale), int(max_context),
                              self._latent_work.data_ptr(), self._latent_work.numel(), self.code, self._stream()):
            return False
        self._note("mv_attention_latent_split", self._size(q, out) + kv_tokens * dk * pages.element_size(), 0)
        return True

    # ------------------------------------------------------------------------------------
    # mixture of experts
    def moe_route(self, logits: torch.Tensor, correction: Optional[torch.Tensor], groups: int, keep: int, top: int,
                  sum_eps: float, dense: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, scoring: str = "softmax",
                  group_worth: str = "max", normalize: bool = True) -> None:
        """From float32 router logits [n, E]: scores = softmax over E; the ``top`` largest of scores + correction among the
        experts of the ``keep`` groups (of ``groups`` equal runs of neighbours) whose largest such number is largest are
        chosen; a chosen expert's weight is its score / (sum of the chosen scores + sum_eps). dense float32 [n, E] gets the
        weights (zero elsewhere), ids int32 / weights float32 [n, top] the chosen experts in the order of choice.
        ``scoring`` "sigmoid": scores = sigmoid(logit); ``group_worth`` "top2": a group is worth the sum of its two
        largest numbers; ``normalize`` False: the weights are the chosen scores themselves."""
        if scoring not in ("softmax", "sigmoid") or group_worth not in ("max", "top2"):
            raise KernelLibraryError(f"moe_route: unknown scoring {scoring!r} or group worth {group_worth!r}")
        flags = (1 if scoring == "sigmoid" else 0) | (2 if group_worth == "top2" else 0) | (0 if normalize else 4)
        _dev(logits, "router logits")
        n, E = logits.shape
        if logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise KernelLibraryError("moe_route: float32 logits [n, E] are needed")
        for t, shape, dt, name in ((dense, (n, E), torch.float32, "dense weights"), (ids, (n, top), torch.int32, "ids"),
                                   (weights, (n, top), torch.float32, "weights")):
            _dev(t, name)
            if t.dtype != dt or tuple(t.shape) != shape or not t.is_contiguous():
                raise KernelLibraryError(f"moe_route: {name} must be contiguous {dt} {shape}")
        if correction is not None:
            _dev(correction, "router correction")
            if correction.numel() != E or not correction.is_contiguous():
                raise KernelLibraryError(f"moe_route: the correction must hold {E} numbers")
        self._note("mv_moe_route", self._size(logits, dense, ids, weights), 20 * n * E)
        self.lib.call("mv_moe_route", logits.data_ptr(), logits.stride(0) if n > 1 else E, n, E, _ptr(correction),
                      _weight_code(correction, "router correction") if correction is not None else DTYPE_F32, groups, keep,
                      top, float(sum_eps), flags, dense.data_ptr(), ids.data_ptr(), weights.data_ptr(), self._stream())

    def moe_swiglu_scale(self, gate_up: torch.Tensor, dense: Optional[torch.Tensor], experts: int, ff: int, out: torch.Tensor,
                         limit: float = 0.0, slope: float = 1.0, shared: int = 0, table=None) -> None:
        """out[t, e, c] = dense[t, e] * silu(gate_up[t, e*ff + c]) * gate_up[t, experts*ff + e*ff + c] (zero where the
        weight is zero, whatever the products hold). With ``limit`` > 0 the clamped pair instead: g = min(gate, limit),
        u = clamp(up, -limit, limit), out = dense * g * sigmoid(slope * g) * (u + 1). With ``shared`` > 0 the rows hold
        that many gate and as many up columns of a shared expert behind the others', and out gets its pair, with the
        weight one, behind the experts' columns. ``table`` = (token ids int32 [>= n], int32 [rows, top]) instead of
        ``dense``: row t's experts are table[token_ids[t]], each with the weight 1 / top (what ``moe_table_route`` would
        leave in ``dense``, looked up here instead)."""
        self._act(gate_up, "gate_up"); self._act(out, "expert activations")
        n = gate_up.shape[0]
        if tuple(gate_up.shape) != (n, 2 * experts * ff + 2 * shared) or gate_up.stride(1) != 1 \
                or tuple(out.shape) != (n, experts * ff + shared) or not out.is_contiguous():
            raise KernelLibraryError("moe_swiglu_scale: operands do not fit")
        tokens = rows = None
        if table is not None:
            tokens, rows = table
            for t, name in ((tokens, "token ids"), (rows, "expert table")):
                _dev(t, name)
                if t.dtype != torch.int32 or not t.is_contiguous():
                    raise KernelLibraryError(f"moe_swiglu_scale: {name} must be contiguous int32")
            if tokens.numel() < n or rows.dim() != 2:
                raise KernelLibraryError("moe_swiglu_scale: a token id for every row and a table [rows, top] are needed")
        else:
            _dev(dense, "dense weights")
            if dense.dtype != torch.float32 or dense.shape[0] != n or dense.shape[1] < experts or dense.stride(1) != 1:
                raise KernelLibraryError("moe_swiglu_scale: operands do not fit")
        self._note("mv_moe_swiglu_scale", self._size(gate_up, out), 8 * out.numel())
        self.lib.call("mv_moe_swiglu_scale", gate_up.data_ptr(), gate_up.stride(0) if n > 1 else gate_up.shape[1], _ptr(dense),
                      (dense.stride(0) if n > 1 else dense.shape[1]) if dense is not None else 0, n, experts, ff, int(shared),
                      out.data_ptr(), float(limit), float(slope), _ptr(tokens), _ptr(rows),
                      rows.shape[0] if rows is not None else 0, rows.shape[1] if rows is not None else 0, self.code, self._stream())

    def moe_table_route(self, token_ids: torch.Tensor, table: torch.Tensor, experts: int, dense: torch.Tensor, ids: torch.Tensor,
                        weights: torch.Tensor) -> None:
        """Experts named by a table: row t uses table[token_ids[t]] (int32 [rows, top]), each with the weight 1 / top.
        dense float32 [n, >= experts], ids int32 / weights float32 [n, top] are left as ``moe_route`` leaves them."""
        n, top = ids.shape
        for t, name in ((token_ids, "token ids"), (table, "expert table"), (ids, "ids")):
            _dev(t, name)
            if t.dtype != torch.int32 or not t.is_contiguous():
                raise KernelLibraryError(f"moe_table_route: {name} must be contiguous int32")
        _dev(dense, "dense weights"); _dev(weights, "weights")
        if token_ids.numel() < n or table.dim() != 2 or table.shape[1] != top or dense.dtype != torch.float32 or dense.dim() != 2 \
                or dense.shape[0] != n or dense.shape[1] < experts or dense.stride(1) != 1 or weights.dtype != torch.float32 \
                or tuple(weights.shape) != (n, top) or not weights.is_contiguous():
            raise KernelLibraryError("moe_table_route: operands do not fit")
        self._note("mv_moe_table_route", self._size(dense, ids, weights) + n * (top + 1) * 4, n * experts)
        self.lib.call("mv_moe_table_route", token_ids.data_ptr(), table.data_ptr(), table.shape[0], n, experts, top, dense.data_ptr(),
                      dense.stride(0) if n > 1 else dense.shape[1], ids.data_ptr(), weights.data_ptr(), self._stream())

    def moe_identity_add(self, y: torch.Tensor, h: torch.Tensor, dense: torch.Tensor, first: int, count: int,
                         overwrite: bool = False) -> None:
        """y[t] += (dense[t, first:first+count] summed) * h[t]; with ``overwrite`` y is set instead."""
        self._act(y, "feed-forward output"); self._act(h, "feed-forward input"); _dev(dense, "dense weights")
        n, width = y.shape
        if tuple(h.shape) != (n, width) or y.stride(1) != 1 or h.stride(1) != 1 or dense.dtype != torch.float32 \
                or dense.shape[0] != n or dense.shape[1] < first + count or dense.stride(1) != 1:
            raise KernelLibraryError("moe_identity_add: operands do not fit")
        self._note("mv_moe_identity_add", 2 * self._size(y) + self._size(h), 2 * n * width)
        self.lib.call("mv_moe_identity_add", y.data_ptr(), y.stride(0) if n > 1 else width, h.data_ptr(),
                      h.stride(0) if n > 1 else width, dense.data_ptr(), dense.stride(0) if n > 1 else dense.shape[1], first,
                      count, n, width, int(overwrite), self.code, self._stream())

    def moe_grouped(self, x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, experts: int, identity: int, ff: int,
                    ids: torch.Tensor, weights: torch.Tensor, dense: torch.Tensor, ints: torch.Tensor, act: torch.Tensor,
                    out: torch.Tensor, y: torch.Tensor, limit: float = 0.0, slope: float = 1.0) -> bool:
        """The experts' products over the chosen (token, expert) pairs only (bfloat16): y[t] = sum over t's chosen experts
        of weight * down_e(silu(gate_e x) * up_e x) + (its identity experts' weights) * x[t]; with ``limit`` > 0 the pair
        is the clamped one, g = min(gate, limit), u = clamp(up, -limit, limit), g * sigmoid(slope * g) * (u + 1). ``w_gate_up`` is
        [2 * experts * ff, hidden] (all gate blocks, then all up blocks), ``w_down`` [hidden, experts * ff]; ids / weights
        [n, top] and dense [n, experts + identity] as ``moe_route`` leaves them; ``ints`` (int32), ``act`` [n * top, ff]
        and ``out`` float32 [n * top, hidden] are scratch. False when the sizes are not served (nothing was done)."""
        if self.dtype != torch.bfloat16 or not self.lib.has("mv_moe_grouped") or w_gate_up.dtype != torch.bfloat16 \
                or w_down.dtype != torch.bfloat16:
            return False
        self._act(x, "feed-forward input"); self._act(y, "feed-forward output"); self._act(act, "expert activations")
        n, hidden = x.shape
        top = ids.shape[1]
        if tuple(w_gate_up.shape) != (2 * experts * ff, hidden) or tuple(w_down.shape) != (hidden, experts * ff) \
                or not w_gate_up.is_contiguous() or not w_down.is_contiguous() or x.stride(1) != 1 or y.stride(1) != 1 \
                or tuple(y.shape) != (n, hidden) or tuple(act.shape) != (n * top, ff) or not act.is_contiguous() \
                or out.dtype != torch.float32 or tuple(out.shape) != (n * top, hidden) or not out.is_contiguous() \
                or ids.dtype != torch.int32 or tuple(weights.shape) != (n, top) or weights.dtype != torch.float32 \
                or not ids.is_contiguous() or not weights.is_contiguous() or dense.dtype != torch.float32 \
                or dense.shape[0] != n or dense.shape[1] < experts + identity or dense.stride(1) != 1 \
                or ints.dtype != torch.int32 or ints.numel() < int(self.lib.dll.mv_moe_grouped_ints(n, top, experts)):
            raise KernelLibraryError("moe_grouped: operands do not fit")
        for t in (w_gate_up, w_down, ids, weights, dense, ints, out):
            _dev(t, "moe_grouped operand")
        if not self.lib.offer("mv_moe_grouped", x.data_ptr(), x.stride(0) if n > 1 else hidden, n, hidden, w_gate_up.data_ptr(),
                              w_down.data_ptr(), experts, identity, ff, ids.data_ptr(), weights.data_ptr(), top, dense.data_ptr(),
                              dense.stride(0) if n > 1 else dense.shape[1], ints.data_ptr(), act.data_ptr(), out.data_ptr(),
                              y.data_ptr(), y.stride(0) if n > 1 else hidden, float(limit), float(slope), self._stream()):
            return False
        used = min(experts, n * top)
        self._note("mv_moe_grouped", self._size(x, y) + used * 3 * ff * hidden * 2 + self._size(act, out) * 2,
                   2 * n * top * 3 * ff * hidden)
        return True

    def hyper_step(self, lanes: torch.Tensor, out: Optional[torch.Tensor] = None, first: Optional[torch.Tensor] = None,
                   write=None, read=None, total: Optional[torch.Tensor] = None) -> None:
        """Several residual streams, float32 ``lanes`` [S, n, W]. ``write`` = (y [n, W] of the activation type, mix float32
        [S, S] indexed [from, to], out_weights float32 [S]): lane t <- sum_s mix[s, t] lane s + out_weights[t] y, all from
        the old lanes. ``read`` = (in_weights float32 [S], norm weight [W], eps): ``out`` [n, W] (activation type) =
        rmsnorm(sum_s in_weights[s] lane s) * weight, from the lanes as the write leaves them. ``first`` float32 [n, W]:
        the lanes do not exist yet, every one of them is this row. ``total`` float32 [n, W] gets the sum of the lanes
        (behind a write without a read the lanes themselves are then not stored)."""
        _dev(lanes, "residual lanes")
        if lanes.dtype != torch.float32 or lanes.dim() != 3 or lanes.stride(2) != 1 or lanes.stride(1) != lanes.shape[2]:
            raise KernelLibraryError("hyper_step: the lanes must be float32 [streams, n, width] with contiguous rows")
        S, n, W = lanes.shape
        for t, name in ((first, "first rows"), (total, "summed rows")):
            if t is not None:
                _dev(t, name)
                if t.dtype != torch.float32 or tuple(t.shape) != (n, W) or not t.is_contiguous():
                    raise KernelLibraryError(f"hyper_step: the {name} must be contiguous float32 [{n}, {W}]")
        y = w_mix = w_out = w_in = w_norm = None
        eps = 1.0
        if write is not None:
            y, w_mix, w_out = write
            self._act(y, "sublayer output")
            if y.dim() != 2 or y.shape[0] != n or y.shape[1] < W or y.stride(1) != 1:
                raise KernelLibraryError(f"hyper_step: the sublayer output must be [{n}, {W}]")
            for t, shape in ((w_mix, (S, S)), (w_out, (S,))):
                _dev(t, "stream weights")
                if t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous():
                    raise KernelLibraryError(f"hyper_step: stream weights must be contiguous float32 {shape}")
        if read is not None:
            w_in, w_norm, eps = read
            _dev(w_in, "stream weights"); _dev(w_norm, "norm weight")
            if w_in.dtype != torch.float32 or tuple(w_in.shape) != (S,) or not w_in.is_contiguous() or w_norm.numel() != W \
                    or not w_norm.is_contiguous():
                raise KernelLibraryError(f"hyper_step: the read needs float32 [{S}] stream weights and a norm weight of {W}")
            self._act(out, "normed rows")
            if tuple(out.shape) != (n, W) or out.stride(1) != 1:
                raise KernelLibraryError(f"hyper_step: the normed rows must be [{n}, {W}]")
        if n == 0:
            return
        moved = (S if first is None else 1) + (S if (read is not None or total is None) else 0) + (1 if total is not None else 0)
        self._note("mv_hyper_step", n * W * (4 * moved + (y.element_size() if y is not None else 0)
                                               + (out.element_size() if read is not None else 0)), n * W * (2 * S * S + 2 * S + 4))
        self.lib.call("mv_hyper_step", lanes.data_ptr(), lanes.stride(0), _ptr(first), S, n, W, _ptr(y),
                      (y.stride(0) if n > 1 else y.shape[1]) if y is not None else 0, _ptr(w_mix), _ptr(w_out), _ptr(w_in),
                      _ptr(w_norm), _weight_code(w_norm, "norm weight") if w_norm is not None else DTYPE_F32, float(eps),
                      _ptr(out) if read is not None else 0, (out.stride(0) if n > 1 else W) if read is not None else 0,
                      _ptr(total), self.code, self._stream())

    def qkv_rotate_norm_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                              positions: torch.Tensor, token_seq: torch.Tensor, rope_table: Optional[torch.Tensor],
                              interleaved: bool, unit_norm: bool, eps: float, k_pages: torch.Tensor, v_pages: torch.Tensor,
                              block_table: torch.Tensor, page_size: int, q_weight: Optional[torch.Tensor] = None,
                              k_weight: Optional[torch.Tensor] = None, mix_rows: Optional[torch.Tensor] = None,
                              mix_weight: Optional[torch.Tensor] = None) -> None:
        """On the rows ``qkv`` = [q | k | v | ...] of a step: q and k heads are rotated over their first channels by the
        row's position (``rope_table`` float32 [positions, rot] = cat(cos, sin)) and, with ``unit_norm``, divided by their
        root mean square afterwards (times ``q_weight`` / ``k_weight`` where given); q stays in the rows, k goes to the key
        pages [pages, kv_heads, page_size, head_dim]. The values go to the value pages [pages, kv_heads, value_dim,
        page_size]; with ``mix_rows`` [n, >= kv_heads * value_dim] and ``mix_weight`` (one number on the device, m) they
        are (1 - m) v + m mix_rows first."""
        self._act(qkv, "qkv"); self._act(k_pages, "key pages"); self._act(v_pages, "value pages")
        n = qkv.shape[0]
        q_dim, kv_dim, v_dim = num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * value_dim
        if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < q_dim + kv_dim + v_dim:
            raise KernelLibraryError(f"qkv_rotate_norm_store: rows {tuple(qkv.shape)} do not hold {q_dim + kv_dim + v_dim} columns")
        if tuple(k_pages.shape[1:]) != (num_kv_heads, page_size, head_dim) or tuple(v_pages.shape[1:]) != (num_kv_heads, value_dim, page_size) \
                or not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelLibraryError(f"qkv_rotate_norm_store: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not match "
                                     f"[pages, {num_kv_heads}, {page_size}, {head_dim}] / [pages, {num_kv_heads}, {value_dim}, {page_size}]")
        self._ints(n, positions=(positions, n), token_seq=(token_seq, n))
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("qkv_rotate_norm_store: the block table must be a contiguous int32 matrix")
        rot = 0
        if rope_table is not None:
            _dev(rope_table, "rope table")
            if rope_table.dtype != torch.float32 or rope_table.dim() != 2 or not rope_table.is_contiguous() \
                    or rope_table.shape[1] > head_dim or rope_table.shape[1] % 2:
                raise KernelLibraryError("qkv_rotate_norm_store: the rope table must be contiguous float32 [positions, rot <= head_dim]")
            rot = rope_table.shape[1]
        wcode = DTYPE_F32
        if (q_weight is None) != (k_weight is None):
            raise KernelLibraryError("qkv_rotate_norm_store: norm weights come in pairs")
        if q_weight is not None:
            wcode = _weight_code(q_weight, "q norm weight")
            if q_weight.numel() != head_dim or k_weight.numel() != head_dim or k_weight.dtype != q_weight.dtype:
                raise KernelLibraryError("qkv_rotate_norm_store: norm weights must both hold head_dim elements")
        mcode, mstride = DTYPE_F32, 0
        if mix_rows is not None:
            self._act(mix_rows, "rows blended into the values"); _dev(mix_weight, "blend weight")
            if mix_rows.dim() != 2 or mix_rows.shape[0] != n or mix_rows.shape[1] < v_dim or mix_rows.stride(1) != 1 \
                    or mix_weight is None or mix_weight.numel() != 1:
                raise KernelLibraryError(f"qkv_rotate_norm_store: blending needs rows [{n}, >= {v_dim}] and one weight")
            mcode = _weight_code(mix_weight, "blend weight")
            mstride = mix_rows.stride(0) if n > 1 else mix_rows.shape[1]
        if n == 0:
            return
        self._note("mv_qkv_rotate_norm_store", n * (2 * q_dim + 2 * kv_dim + (3 if mix_rows is not None else 2) * v_dim) * qkv.element_size()
                   + n * rot * 4, 10 * n * (q_dim + kv_dim))
        self.lib.call("mv_qkv_rotate_norm_store", qkv.data_ptr(), qkv.stride(0) if n > 1 else qkv.shape[1], 0, q_dim, q_dim + kv_dim,
                      positions.data_ptr(), token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      k_pages.data_ptr(), v_pages.data_ptr(), n, num_heads, num_kv_heads, head_dim, value_dim, _ptr(q_weight),
                      _ptr(k_weight), wcode, int(unit_norm), float(eps), _ptr(rope_table), rot, int(interleaved), _ptr(mix_rows),
                      mstride, _ptr(mix_weight), mcode, self.code, self._stream())

    def add_rows(self, y: torch.Tensor, x: torch.Tensor) -> None:
        """In place on rows of the activation type: y <- y + x (added in float32, rounded once)."""
        self._act(y, "rows"); self._act(x, "rows to add")
        if y.dim() != 2 or tuple(x.shape) != tuple(y.shape) or y.stride(1) != 1 or x.stride(1) != 1:
            raise KernelLibraryError("add_rows: two matrices of one shape with contiguous rows are needed")
        rows, cols = y.shape
        if rows == 0:
            return
        self._note("mv_add_rows", 3 * self._size(y), rows * cols)
        self.lib.call("mv_add_rows", y.data_ptr(), y.stride(0) if rows > 1 else cols, x.data_ptr(), x.stride(0) if rows > 1 else cols,
                      rows, cols, self.code, self._stream())

    def scale_f32(self, x: torch.Tensor, factor: float) -> None:
        """In place on float32 [rows, cols]: x <- x * factor."""
        _dev(x, "rows")
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelLibraryError("scale_f32: float32 rows with a contiguous last dimension are needed")
        rows, cols = x.shape
        if rows == 0:
            return
        self._note("mv_scale_f32", 2 * self._size(x), rows * cols)
        self.lib.call("mv_scale_f32", x.data_ptr(), x.stride(0) if rows > 1 else cols, rows, cols, float(factor), self._stream())

    def norm_add_norm(self, y: torch.Tensor, norm_y, resid: torch.Tensor, norm_next, out: Optional[torch.Tensor],
                      shift: Optional[tuple] = None) -> None:
        """resid += rmsnorm(y) * w (``norm_y`` = (weight, eps, unit_offset)); with ``norm_next`` of the same
        form, out = rmsnorm(resid) * w'. The sum stays float32 in between.

        ``shift`` = (mix, state [slots, h], token_seq, state_slots), for steps in which every request brings
        one token: ``out`` gets the rows after the token shift that ``token_shift`` would apply to them (row r
        belongs to request token_seq[r]; the state takes the unshifted row)."""
        self._act(y, "sublayer output"); _dev(resid, "residual")
        n, h = resid.shape
        if resid.dtype != torch.float32 or not resid.is_contiguous() or tuple(y.shape) != (n, h) or y.stride(1) != 1:
            raise KernelLibraryError("norm_add_norm: a float32 residual [n, h] and an output of the same shape are needed")
        wa, eps_a, unit_a = norm_y
        _dev(wa, "norm weight")
        if wa.numel() != h or not wa.is_contiguous():
            raise KernelLibraryError(f"norm_add_norm: weight of {wa.numel()} elements for rows of {h}")
        wb, eps_b, unit_b, wb_code = None, 1.0, False, DTYPE_F32
        if out is not None:
            if norm_next is None:
                raise KernelLibraryError("norm_add_norm: an output needs the second norm")
            self._act(out, "norm output")
            wb, eps_b, unit_b = norm_next
            _dev(wb, "norm weight")
            wb_code = _weight_code(wb, "norm weight")
            if wb.numel() != h or not wb.is_contiguous() or tuple(out.shape) != (n, h) or not out.is_contiguous():
                raise KernelLibraryError("norm_add_norm: the second norm's weight or output does not fit")
        mix = state = tsq = slots = None
        mix_code = DTYPE_F32
        if shift is not None:
            mix, state, tsq, slots = shift
            if out is None:
                raise KernelLibraryError("norm_add_norm: a token shift needs the second norm and its output")
            self._act(state, "shift state"); _dev(mix, "shift weight")
            mix_code = _weight_code(mix, "shift weight")
            if state.dim() != 2 or state.shape[1] != h or not state.is_contiguous() or mix.numel() != h or not mix.is_contiguous():
                raise KernelLibraryError(f"norm_add_norm: shift state {tuple(state.shape)} / weight do not fit rows of {h}")
            self._ints(n, token_seq=(tsq, n), state_slots=(slots, 1))
        self._note("mv_norm_add_norm", self._size(y, out) + 2 * self._size(resid) + (2 * self._size(out) if shift else 0), 8 * n * h)
        self.lib.call("mv_norm_add_norm", y.data_ptr(), y.stride(0) if n > 1 else h, wa.data_ptr(),
                      _weight_code(wa, "norm weight"), float(eps_a), int(unit_a), resid.data_ptr(), _ptr(wb), wb_code,
                      float(eps_b), int(unit_b), _ptr(out), n, h, _ptr(mix), mix_code, _ptr(state), _ptr(tsq), _ptr(slots),
                      self.code, self._stream())

    def soft_cap(self, logits: torch.Tensor, cap: float) -> None:
        """In place on float32 [rows, cols]: x <- cap * tanh(x / cap)."""
        _dev(logits, "logits")
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise KernelLibraryError("soft_cap: float32 rows with a contiguous last dimension are needed")
        rows, cols = logits.shape
        if rows == 0:
            return
        self._note("mv_soft_cap", 2 * self._size(logits), 4 * rows * cols)
        self.lib.call("mv_soft_cap", logits.data_ptr(), logits.stride(0) if rows > 1 else cols, rows, cols, float(cap),
                      self._stream())

    @staticmethod
    def _chunk_priced(plan, chunk: int):
        """For the ledger: with chunks a request's queries read at most the keys of the chunks they stand in,
        not its whole context; the plan's key and pair counts are capped accordingly (an upper bound still)."""
        if plan is None or chunk <= 0:
            return plan
        import copy
        seqs = max(1, len(plan.q_lens) if plan.q_lens else plan.n_seqs)
        tokens = sum(plan.q_lens) if plan.q_lens else seqs
        priced = copy.copy(plan)
        priced.kv_tokens = min(plan.kv_tokens, seqs * chunk + tokens)
        priced.attention_pairs = min(plan.attention_pairs, tokens * chunk)
        return priced

    @staticmethod
    def _window_priced(plan, window: int, first: int):
        """For the ledger: under a window (``window`` positions behind the query, beside the first ``first``) a
        request's queries read the keys from the window of its first query on and the kept ones, and a query at
        position p makes min(p, window) + 1 pairs and one for each kept position that the window has let go of."""
        if plan is None or window < 0 or not plan.starts or len(plan.starts) != len(plan.step_q_lens):
            return plan
        import copy
        keys = pairs = 0
        for start, ql in zip(plan.starts, plan.step_q_lens):
            lo = max(0, start - window)
            keys += start + ql - lo + min(first, lo)
            for p in range(start, start + ql):
                pairs += min(p, window) + 1 + max(0, min(first, p - window))
        priced = copy.copy(plan)
        priced.kv_tokens, priced.attention_pairs = keys, pairs
        return priced

    def attention_sigmoid(self, q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                          block_table: torch.Tensor, page_size: int, positions: torch.Tensor, token_seq: torch.Tensor,
                          num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                          chunk: Optional[int], window: Optional[int], bias: Optional[torch.Tensor],
                          gate: Optional[torch.Tensor], plan: Optional["AttentionPlan"] = None) -> None:
        """Causal attention with sigmoid weights over the paged cache: the query at position p sees the
        keys of its request from max(start of p's chunk, p - window, 0) to p, each with the weight
        sigmoid(q.k * scale + bias[head]), not normalised. q [n, >= H*D] rows, out [n, H*Dv]; bias float32
        [H] or None; gate [n, >= H] rows of the activation type or None (head h's output times
        sigmoid(gate[t, h]))."""
        self._act(q, "queries"); self._act(out, "attention output")
        self._act(k_pages, "key pages"); self._act(v_pages, "value pages")
        n = q.shape[0]
        if q.dim() != 2 or q.shape[1] < num_heads * head_dim or q.stride(1) != 1 \
                or tuple(out.shape) != (n, num_heads * value_dim) or out.stride(1) != 1:
            raise KernelLibraryError(f"attention_sigmoid: q {tuple(q.shape)} / out {tuple(out.shape)} do not hold "
                                     f"{num_heads} heads of {head_dim} / {value_dim}")
        if tuple(k_pages.shape[1:]) != (num_kv_heads, page_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (num_kv_heads, value_dim, page_size) or \
                not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelLibraryError(f"attention_sigmoid: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} have the "
                                     f"wrong layout for {num_kv_heads} heads of {head_dim} / {value_dim}, page {page_size}")
        self._ints(n, positions=(positions, n), token_seq=(token_seq, n))
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("attention_sigmoid: the block table must be a contiguous int32 matrix")
        if num_heads % num_kv_heads:
            raise KernelLibraryError(f"attention_sigmoid: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if bias is not None:
            _dev(bias, "score bias")
            if bias.dtype != torch.float32 or bias.numel() != num_heads or not bias.is_contiguous():
                raise KernelLibraryError(f"attention_sigmoid: the score bias must be float32 [{num_heads}]")
        gate_stride = 0
        if gate is not None:
            self._act(gate, "head gates")
            if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < num_heads or gate.stride(1) != 1:
                raise KernelLibraryError(f"attention_sigmoid: gates {tuple(gate.shape)} do not hold {num_heads} per row")
            gate_stride = gate.stride(0) if n > 1 else gate.shape[1]
        if n == 0:
            return
        c = 0 if chunk is None else int(chunk)
        w = -1 if window is None else int(window)
        qs = q.stride(0) if n > 1 else q.shape[1]
        os_ = out.stride(0) if n > 1 else num_heads * value_dim
        group = num_heads // num_kv_heads
        if (self.use_fast_kernels and plan is not None and self.lib.has("mv_attention_prefill_sigmoid")
                and head_dim == value_dim and head_dim in (64, 128) and page_size >= 16 and not page_size & (page_size - 1)
                and qs % 8 == 0 and os_ % 4 == 0 and q.data_ptr() % 16 == 0 and out.data_ptr() % 8 == 0):
            nt, kw, n_units, n_busy = self._prefill_variant(plan, group, num_kv_heads)
            if nt:
                self._note_attention("mv_attention_prefill_sigmoid", self._chunk_priced(plan, c), n, num_heads, num_kv_heads,
                                     head_dim, 2)
                self.lib.call("mv_attention_prefill_sigmoid", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                              v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                              positions.data_ptr(), plan.cu_seqlens.data_ptr(), plan.n_seqs, n_units, n_busy, nt, kw,
                              num_heads, num_kv_heads, head_dim, float(scale), w, c, _ptr(bias), _ptr(gate), gate_stride,
                              self._stream())
                return
        self._note_attention("mv_attention_sigmoid_ref", self._chunk_priced(plan, c), n, num_heads, num_kv_heads, head_dim,
                             q.element_size())
        self.lib.call("mv_attention_sigmoid_ref", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                      v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size, positions.data_ptr(),
                      token_seq.data_ptr(), n, num_heads, num_kv_heads, head_dim, value_dim, float(scale), c, w,
                      _ptr(bias), _ptr(gate), gate_stride, self.code, self._stream())

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> None:
        """out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i]."""
        self._act(gate_up, "gate_up"); self._act(out, "swiglu output")
        n, two_i = gate_up.shape
        if two_i % 2 or out.shape != (n, two_i // 2) or not gate_up.is_contiguous() or not out.is_contiguous():
            raise KernelLibraryError(f"swiglu: {tuple(gate_up.shape)} -> {tuple(out.shape)} is not [n, 2I] -> [n, I]")
        self._note("mv_swiglu", self._size(gate_up, out), 6 * out.numel())
        self.lib.call("mv_swiglu", gate_up.data_ptr(), out.data_ptr(), n, two_i // 2, self.code, self._stream())

    # ------------------------------------------------------------------------------------
    def gemm(self, a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
             exact: bool = False, defer_sum: bool = False, fold=None):
        """out[M, N] = a[M, K] @ w[N, K]^T (+ bias). ``out`` is the activation type or float32.

        With ``defer_sum`` the caller can take a ``SplitSum`` instead of the finished ``out``: when
        the product runs on the kernel that splits K, its partial sums are left to whoever uses the
        result (a residual add + norm adds them up on the way; ``materialize()`` gives ``out``).
        The return value is that object, or None when ``out`` is complete.

        float32 compute always takes the exact kernel. bfloat16 compute takes the
        weight-streaming MFMA kernel for up to SKINNY_MAX_M rows, the library's matrix product
        for more rows, and the exact kernel when the weight is stored in float32, when
        ``exact`` is set or when no other kernel takes the shape.

        ``a`` may be a pending norm (parts.base.PendingNorm): then the residual add, the norm and
        the product run as one kernel when the step has at most 16 rows, else the norm runs first.
        ``a`` may also be ``WeightedRows``: the output rows are then divided by the rows' root mean
        square where the weight-streaming kernel takes the shape, else the rows are normalised first.

        ``fold`` (parts.base.NormFold) offers the residual add and the norm behind this product: when
        the weight-streaming kernel takes the shape it adds the product to the residual, leaves the
        rows weighted for the norm, and ``WeightedRows`` is returned; ``out`` is not written then."""
        if not isinstance(a, torch.Tensor):
            if isinstance(a, WeightedRows):
                if not exact and self._gemm_scaled(a, w, out, bias, swiglu=False):
                    return None
            elif not exact and self._gemm_fused_norm(a, w, out, bias, swiglu=False):
                return None
            a = a.materialize()
        self._act(a, "gemm input"); _dev(w, "gemm weight"); _dev(out, "gemm output")
        if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
            raise KernelLibraryError("gemm: operands must be matrices")
        M, K = a.shape
        N = w.shape[0]
        if w.shape[1] != K or out.shape != (M, N):
            raise KernelLibraryError(f"gemm: [{M}, {K}] x {tuple(w.shape)}^T -> {tuple(out.shape)} does not fit")
        if a.stride(1) != 1 or out.stride(1) != 1 or not w.is_contiguous():
            raise KernelLibraryError("gemm: operands need a contiguous last dimension")
        if out.dtype not in (self.dtype, torch.float32):
            raise KernelLibraryError(f"gemm: output dtype {out.dtype} must be {self.dtype} or float32")
        wcode = _weight_code(w, "gemm weight")
        if bias is not None:
            _dev(bias, "bias")
            if bias.dtype != w.dtype or bias.numel() != N:
                raise KernelLibraryError("gemm: the bias must have the weight's dtype and N elements")
        if M == 0:
            return None
        lda = a.stride(0) if M > 1 else K
        ldc = out.stride(0) if M > 1 else N
        fast = self.use_fast_kernels and not exact and wcode == DTYPE_BF16
        if (fast and self.prefers_library(M, N, K) and self._library_serves(out)
                and self._library_allowed(M, N, K, bias is not None, out.dtype)
                and self._library_product(a, w, bias, out)):
            return None
        if fast and lda % 8 == 0 and a.data_ptr() % 16 == 0 and self.wants_tile(
                M, N, K, fold_offered=(fold is not None and self._fold_serves(fold, out, M, N)
                                       and not (self.wants_mid(M, N, K) and self.lib.has("mv_gemm_mid")))):
            if defer_sum and out.dtype == self.dtype and out.is_contiguous():
                pending = self._gemm_tile_sums(a, lda, w, bias, out, M, N, K)
                if pending is not None:
                    return pending
            if self.gemm_tile(a, w, out, bias):
                return None
        if fast and K % 32 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and self.lib.has("mv_gemm_skinny"):
            done = self._gemm_mid(a, lda, w, bias, out, ldc, M, N, K, swiglu=False,
                                  defer_sum=defer_sum and out.dtype == self.dtype and out.is_contiguous())
            if done:
                return done if isinstance(done, SplitSum) else None
            if not self.streams_rows(M, N, K) and self._library_serves(out) and \
                    self._library_allowed(M, N, K, bias is not None, out.dtype) and self._library_product(a, w, bias, out):
                return
            if fold is not None and self._fold_serves(fold, out, M, N):
                P = int(self.lib.dll.mv_gemm_skinny_fold_parts(M, N, K))
                resid = fold.stream.resid
                self._note("mv_gemm_skinny_fold", M * K * 2 + N * K * 2 + M * N * (8 + 2) + M * P * 4, 2 * M * N * K + 4 * M * N)
                self.lib.call("mv_gemm_skinny_fold", a.data_ptr(), lda, w.data_ptr(), _ptr(bias), resid.data_ptr(),
                              resid.stride(0) if M > 1 else N, fold.weight.data_ptr(),
                              _weight_code(fold.weight, "norm weight"), int(fold.unit_offset), fold.weighted.data_ptr(),
                              fold.weighted.stride(0) if M > 1 else N, fold.partial.data_ptr(), P, M, N, K,
                              self._stream())
                return WeightedRows(self, fold, P)
            # more rows than one workgroup takes are dealt out to groups of workgroups by the kernel
            for m0 in range(0, M, SKINNY_LAUNCH_ROWS):
                m = min(SKINNY_LAUNCH_ROWS, M - m0)
                self._note("mv_gemm_skinny", m * K * 2 + (N * K * 2 if m0 == 0 else 0) + m * N * out.element_size(), 2 * m * N * K)
                self.lib.call("mv_gemm_skinny", a.data_ptr() + m0 * lda * 2, lda, w.data_ptr(), K, _ptr(bias),
                              out.data_ptr() + m0 * ldc * out.element_size(), ldc, _CODES[out.dtype], m, N, K,
                              self._stream())
            return
        if fast and M > SKINNY_MAX_M and self._library_serves(out) and \
                self._library_allowed(M, N, K, bias is not None, out.dtype) and self._library_product(a, w, bias, out):
            return
        self._note("mv_gemm_ref", self._size(a, w, out), 2 * M * N * K)
        self.lib.call("mv_gemm_ref", a.data_ptr(), lda, self.code, w.data_ptr(), K, wcode, _ptr(bias),
                      out.data_ptr(), ldc, _CODES[out.dtype], M, N, K, self._stream())

    @staticmethod
    def streams_rows(M: int, N: int, K: int) -> bool:
        """Whether the weight-streaming product is the engine's choice for M rows against an [N, K]
        weight (before the library and the K-splitting kernel have had their say)."""
        return M <= SKINNY_MAX_M or (M <= SKINNY_WIDE_MAX_M and N * K <= SKINNY_WIDE_MAX_WEIGHT)

    def prefers_library(self, M: int, N: int, K: int, gated: bool = False) -> bool:
        """Whether a product of few rows against this weight is left to the library (see
        LIBRARY_TALL_WEIGHT); ``gated``: the alternative is the gated pair in one pass."""
        if not (self.use_library_gemm and self.lib.has("mv_gemm_lt")) or N < 4 * K or N * K < LIBRARY_TALL_WEIGHT:
            return False
        return not gated or N * K >= LIBRARY_TALL_WEIGHT_GATED or M >= 16

    def _library_serves(self, out: torch.Tensor) -> bool:
        """The library's product writes the activation type; called directly it also writes float32
        (the logits of a step of more than 64 rows)."""
        return out.dtype == self.dtype or (out.dtype == torch.float32 and self.lib.has("mv_gemm_lt")
                                           and out.data_ptr() % 16 == 0)

    def _library_product(self, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor) -> bool:
        """out = a @ w^T (+ bias) by the library (hipBLASLt), bf16 in, bf16 or float32 out. It is
        called directly where the kernel library was built with it (a call costs a third of the host
        time of the tensor library's dispatcher, which matters for prompt steps of small models);
        else, for bf16 output, through ``torch.mm``. False, with nothing done, when the library has
        no algorithm for the shape."""
        M, K = a.shape
        N = w.shape[0]
        if self.lib.has("mv_gemm_lt") and a.stride(1) == 1 and out.stride(1) == 1 and a.data_ptr() % 16 == 0 \
                and out.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0:
            if self._lt_work is None:
                if torch.cuda.is_current_stream_capturing():
                    raise KernelLibraryError("the library's workspace must be made before a capture")
                self._lt_work = torch.empty(int(self.lib.dll.mv_gemm_lt_workspace()), dtype=torch.uint8, device=a.device)
            self._note("mv_gemm_lt", self._size(a, w, out), 2 * M * N * K)
            return self.lib.offer("mv_gemm_lt", a.data_ptr(), a.stride(0) if M > 1 else K, w.data_ptr(), _ptr(bias),
                                  out.data_ptr(), out.stride(0) if M > 1 else N, _CODES[out.dtype], M, N, K,
                                  self._lt_work.data_ptr(), self._lt_work.numel(), self._stream())
        if out.dtype != self.dtype:
            return False                 # float32 comes only from the direct call
        wt = self._transposed.get(w.data_ptr())
        if wt is None or wt.shape != (K, N):
            wt = self._transposed[w.data_ptr()] = w.t()      # the view is made once per weight
        if bias is None:
            torch.mm(a, wt, out=out)
        else:
            torch.addmm(bias, a, wt, out=out)
        return True

    def _library_allowed(self, M: int, N: int, K: int, with_bias: bool, out_dtype: torch.dtype = torch.bfloat16) -> bool:
        """Whether the library's matrix product may serve this shape now: whenever it is switched
        on, and while a graph is being recorded only as long as ``library_in_graphs`` holds. The
        executor looks at every graph it has recorded (``graph_census``) and records it again
        without library products should one of them have left a memset node in it."""
        return self.use_library_gemm and (self.library_in_graphs or not self.for_graph)

    def graph_census(self, raw_graph: int) -> dict:
        """Nodes of a recorded graph by kind: {"kernel", "memset", "copy", "other"}."""
        import ctypes
        counts = (ctypes.c_int * 4)()
        self.lib.call("mv_graph_census", raw_graph, ctypes.addressof(counts))
        return dict(kernel=counts[0], memset=counts[1], copy=counts[2], other=counts[3])

    def _gemm_mid(self, a: torch.Tensor, lda: int, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  ldc: int, M: int, N: int, K: int, swiglu: bool, defer_sum: bool = False):
        """The kernel for up to 64 rows against a large weight (activation rows shared through LDS,
        K split over workgroups); False when the shape is left to the weight-streaming kernel.
        With ``defer_sum`` the partial sums are not added up: a ``SplitSum`` is returned."""
        if not (self.wants_mid(M, N, K) and self.lib.has("mv_gemm_mid")):
            return False
        need = int(self.lib.dll.mv_gemm_mid_workspace(M, N, K))
        if need <= 0:
            return False
        if self._mid_work is None or self._mid_work.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                return False                                   # no allocation inside a capture
            if self._split_pending is not None:
                self._split_pending.materialize()
            if self._mid_work is not None:
                self._mid_retired.append(self._mid_work)       # captured graphs may hold its address
            self._mid_work = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=a.device)
        if self._split_pending is not None:
            self._split_pending.materialize()                  # its sums are about to be overwritten
        if defer_sum and not swiglu and self.lib.has("mv_add_rmsnorm_split"):
            self._note("mv_gemm_mid", self._size(a, w) + 4 * M * N * int(self.lib.dll.mv_gemm_mid_splits(N, K)), 2 * M * N * K)
            self.lib.call("mv_gemm_mid_sums", a.data_ptr(), lda, w.data_ptr(), M, N, K, self._mid_work.data_ptr(),
                          self._mid_work.numel(), self._stream())
            pending = SplitSum(self, out, self._mid_work, int(self.lib.dll.mv_gemm_mid_splits(N, K)), bias)
            self._split_pending = pending
            return pending
        self._note("mv_gemm_mid", self._size(a, w, out) + 8 * M * N * int(self.lib.dll.mv_gemm_mid_splits(N, K)), 2 * M * N * K)
        self.lib.call("mv_gemm_mid", a.data_ptr(), lda, w.data_ptr(), _ptr(bias), out.data_ptr(), ldc,
                      _CODES[out.dtype], M, N, K, int(swiglu), self._mid_work.data_ptr(), self._mid_work.numel(),
                      self._stream())
        return True

    def wants_tile(self, M: int, N: int, K: int, gated: bool = False, fold_offered: bool = False) -> bool:
        """Whether M rows against an [N, K] weight (``gated``: the packed gate/up pair) go to the tiled
        product (see TILE_GATED_MIN_M). ``fold_offered``: the caller could fold a norm into the
        weight-streaming product instead, which keeps the few-row steps of the largest weights."""
        if not (self.use_fast_kernels and self.use_tiled_gemm and self.lib.has("mv_gemm_tile")) or K % 64 or M * N >= 1 << 31:
            return False
        weight_bytes = 2 * N * K
        if weight_bytes < TILE_MIN_WEIGHT:
            return False
        if gated:
            # (the largest pairs, 32B-sized ones, stream faster through the library at any number of rows)
            if N % 2 or N * K >= LIBRARY_TALL_WEIGHT_GATED:
                return False
            if weight_bytes >= TILE_GATED_BIG_WEIGHT:
                return TILE_GATED_BIG_MIN_M <= M <= TILE_GATED_BIG_MAX_M
            return TILE_GATED_MIN_M <= M <= TILE_GATED_MAX_M
        if self.prefers_library(M, N, K):
            return False
        if weight_bytes >= TILE_BIG_WEIGHT:
            if M < TILE_BIG_MIN_M:
                if N * K >= MID_ALWAYS_WEIGHT:
                    return True
                if K >= TILE_LONG_ROWS_K and K >= TILE_LONG_ROWS_RATIO * N and os.environ.get("MV_TILE_LONG_ROWS", "1") != "0":
                    return True
                return M >= TILE_HUGE_MIN_M and weight_bytes >= TILE_HUGE_WEIGHT and not fold_offered
            return M <= TILE_BIG_MAX_M
        return N >= TILE_SMALL_MIN_N and TILE_SMALL_MIN_M <= M <= TILE_SMALL_MAX_M

    def _gemm_tile_sums(self, a: torch.Tensor, lda: int, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                        M: int, N: int, K: int):
        """The tiled product of a shape whose K is split, left as partial sums (``SplitSum``) for the
        residual add + norm behind it; None when the shape is not split or the sums cannot be kept."""
        splits = int(self.lib.dll.mv_gemm_tile_splits(M, N, K, 0, 0))
        if splits <= 1 or not self.lib.has("mv_add_rmsnorm_split"):
            return None
        need = splits * M * N
        if self._mid_work is None or self._mid_work.numel() < need:
            if torch.cuda.is_current_stream_capturing():
                return None                                    # no allocation inside a capture
            if self._split_pending is not None:
                self._split_pending.materialize()
            if self._mid_work is not None:
                self._mid_retired.append(self._mid_work)       # captured graphs may hold its address
            self._mid_work = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=a.device)
        if self._split_pending is not None:
            self._split_pending.materialize()                  # its sums are about to be overwritten
        self._note("mv_gemm_tile", self._size(a, w) + 4 * M * N * splits, 2 * M * N * K)
        self.lib.call("mv_gemm_tile_sums", a.data_ptr(), lda, w.data_ptr(), M, N, K, self._mid_work.data_ptr(),
                      self._mid_work.numel(), 0, self._stream())
        pending = SplitSum(self, out, self._mid_work, splits, bias)
        self._split_pending = pending
        return pending

    def gemm_tile(self, a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
                  gated: bool = False, force: int = 0) -> bool:
        """out[M, N] = a @ w^T (+ bias), or with ``gated`` out[M, N / 2] = silu(a Wg^T) * (a Wu^T), by the
        engine's tiled MFMA product for many rows. False, with nothing done, when the shape is not taken.
        ``force`` fixes the tile and the split of K (measurements)."""
        if not (self.use_fast_kernels and self.lib.has("mv_gemm_tile")):
            return False
        M, K = a.shape
        N = w.shape[0]
        n_out = N // 2 if gated else N
        if (M == 0 or K % 64 or a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not w.is_contiguous()
                or w.shape[1] != K or a.stride(1) != 1 or (M > 1 and a.stride(0) % 8) or a.data_ptr() % 16
                or w.data_ptr() % 16 or out.shape != (M, n_out) or out.stride(1) != 1
                or out.dtype not in (torch.bfloat16, torch.float32) or (gated and (N % 2 or bias is not None))
                or (bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N))
                or M * N >= 1 << 31):
            return False
        need = int(self.lib.dll.mv_gemm_tile_workspace(M, N, K, int(gated), force))
        if need < 0:
            return False
        work = None
        if need > 0:
            if self._tile_work is None or self._tile_work.numel() < need:
                if torch.cuda.is_current_stream_capturing():
                    return False                               # no allocation inside a capture
                if self._tile_work is not None:
                    self._mid_retired.append(self._tile_work)  # captured graphs may hold its address
                self._tile_work = torch.empty(max(need, 1 << 22), dtype=torch.float32, device=a.device)
            work = self._tile_work
        self._note("mv_gemm_tile", self._size(a, w, out) + 8 * need, 2 * M * N * K)
        self.lib.call("mv_gemm_tile", a.data_ptr(), a.stride(0) if M > 1 else K, w.data_ptr(), _ptr(bias), out.data_ptr(),
                      out.stride(0) if M > 1 else n_out, _CODES[out.dtype], M, N, K, int(gated), _ptr(work),
                      0 if work is None else work.numel(), force, self._stream())
        return True

    @staticmethod
    def wants_mid(M: int, N: int, K: int) -> bool:
        """Whether a product of M rows with an [N, K] weight goes to the kernel that splits K (it takes
        up to 64 rows)."""
        if M > SKINNY_MAX_M or K % 128:
            return False
        return (N * K >= MID_ALWAYS_WEIGHT and K >= MID_ALWAYS_K) or (N * K >= MID_MIN_WEIGHT and M >= MID_MIN_M)

    def can_fold_norm(self, rows: int, width: int, consumer=None) -> bool:
        """Whether a residual add and a norm over ``rows`` x ``width`` may be offered to the product in
        front of them (``gemm(..., fold=...)``): steps of up to SKINNY_MAX_M rows, when the product
        behind the norm (``consumer`` = (weight rows, weight columns, gated)) is one the
        weight-streaming kernel takes — behind any other the rows would have to be normalised by a
        kernel of their own, and nothing is gained (32B sizes, where gate/up goes to the library: 2 %
        slower). Where both this and the fused add + norm + product kernel could serve (up to 16
        rows), this is taken: the product behind reads finished bf16 rows instead of normalising
        them in every workgroup (0.6B sizes: a step of 1, 8, 16 sequences 5, 3, 4 % faster)."""
        if not (self.use_fast_kernels and self.dtype == torch.bfloat16 and self.lib.has("mv_gemm_skinny_fold")
                and self.lib.has("mv_gemm_skinny_scaled") and 0 < rows <= SKINNY_WIDE_MAX_M and width % 4 == 0):
            return False
        if consumer is None:
            return rows <= SKINNY_MAX_M
        n, k, gated = consumer
        return (k == width and self.streams_rows(rows, n, k) and k % 32 == 0 and not (gated and n % 2)
                and not (self.wants_mid(rows, n, k) and self.lib.has("mv_gemm_mid"))
                and not self.prefers_library(rows, n, k, gated=gated))

    def _fold_serves(self, fold, out: torch.Tensor, M: int, N: int) -> bool:
        resid = fold.stream.resid
        return (M <= SKINNY_WIDE_MAX_M and out.dtype == self.dtype and self.lib.has("mv_gemm_skinny_fold")
                and resid.dtype == torch.float32 and resid.shape == (M, N) and resid.stride(1) == 1
                and fold.weight.numel() == N and fold.weight.is_contiguous()
                and fold.weighted.shape == (M, N) and fold.weighted.stride(1) == 1 and fold.weighted.dtype == self.dtype
                and N % 4 == 0 and (M == 1 or (resid.stride(0) % 4 == 0 and fold.weighted.stride(0) % 4 == 0))
                and resid.data_ptr() % 16 == 0 and fold.weighted.data_ptr() % 8 == 0 and fold.weight.data_ptr() % 16 == 0
                and fold.partial.numel() >= M * ((N + 3) // 4) and fold.stream.delta is None
                and fold.stream.weighted is None)

    def _gemm_scaled(self, rows: "WeightedRows", w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor],
                     swiglu: bool) -> bool:
        """The product (or gated pair) behind a folded norm: output rows divided by the input rows' root
        mean square; False if the shape is not taken (nothing has been done then)."""
        a = rows.weighted
        M, K = a.shape
        if (not self.use_fast_kernels or not self.lib.has("mv_gemm_skinny_scaled") or M == 0
                or not self.streams_rows(M, w.shape[0], K)
                or w.dtype != torch.bfloat16 or not w.is_contiguous() or w.shape[1] != K or K % 32
                or a.stride(1) != 1 or (M > 1 and a.stride(0) % 8) or a.data_ptr() % 16
                or out.stride(1) != 1 or out.dtype != torch.bfloat16 or (swiglu and w.shape[0] % 2)):
            return False
        N = w.shape[0] // 2 if swiglu else w.shape[0]
        if out.shape != (M, N):
            return False
        if self.wants_mid(M, w.shape[0], K) and self.lib.has("mv_gemm_mid"):
            return False
        if self.prefers_library(M, w.shape[0], K, gated=swiglu) and self._library_allowed(M, w.shape[0], K, bias is not None):
            return False
        if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N):
            return False
        if (self.wants_tile(M, w.shape[0], K, gated=swiglu) and self.lib.has("mv_gemm_tile_scaled") and w.data_ptr() % 16 == 0
                and int(self.lib.dll.mv_gemm_tile_splits(M, w.shape[0], K, int(swiglu), 0)) == 1):
            rows.take()
            self._note("mv_gemm_tile", self._size(a, w, out) + M * rows.P * 4, 2 * M * w.shape[0] * K)
            self.lib.call("mv_gemm_tile_scaled", a.data_ptr(), a.stride(0) if M > 1 else K, w.data_ptr(), _ptr(bias),
                          out.data_ptr(), out.stride(0) if M > 1 else N, _CODES[out.dtype], M, w.shape[0], K, int(swiglu),
                          rows.partial.data_ptr(), rows.P, rows.eps, self._stream())
            return True
        rows.take()
        self._note("mv_gemm_skinny_scaled", self._size(a, w, out) + M * rows.P * 4, 2 * M * w.shape[0] * K)
        self.lib.call("mv_gemm_skinny_scaled", a.data_ptr(), a.stride(0) if M > 1 else K, w.data_ptr(), _ptr(bias),
                      out.data_ptr(), out.stride(0) if M > 1 else N, rows.partial.data_ptr(), rows.P, rows.eps, M, N, K,
                      int(swiglu), self._stream())
        return True

    def scale_rows(self, weighted: torch.Tensor, partial: torch.Tensor, P: int, eps: float, out: torch.Tensor) -> None:
        """out[m] = weighted[m] / sqrt(sum_p partial[m][p] / width + eps): the norm of rows that a product
        left half normalised, for whatever cannot divide its own output rows."""
        M, width = weighted.shape
        self._act(weighted, "weighted rows"); self._act(out, "normed rows")
        if out.shape != (M, width) or out.stride(1) != 1 or weighted.stride(1) != 1 or partial.numel() < M * P:
            raise KernelLibraryError("scale_rows: shapes do not fit")
        self._note("mv_scale_rows", self._size(weighted, out) + M * P * 4, 2 * M * width)
        self.lib.call("mv_scale_rows", weighted.data_ptr(), weighted.stride(0) if M > 1 else width, partial.data_ptr(), P,
                      float(eps), out.data_ptr(), out.stride(0) if M > 1 else width, self.code, M, width, self._stream())

    def can_fuse_norm(self, rows: int, width: int) -> bool:
        """Whether a norm over ``rows`` x ``width`` may be deferred into the next product."""
        return (self.use_fast_kernels and self.lib.has("mv_gemm_skinny_norm") and 0 < rows <= FUSED_NORM_MAX_M
                and width % 64 == 0 and rows * ((width + 511) // 512) <= FUSED_NORM_MAX_CHUNKS
                and rows * (width + 8) * 2 <= 44 * 1024)

    def _gemm_fused_norm(self, pending, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor],
                         swiglu: bool) -> bool:
        """add + RMSNorm + product (or gated pair) in one kernel; False if the shape is not taken
        (nothing has been done then)."""
        M, K = pending.shape
        form = pending.norm.as_scaled_rms()     # None: the norm computes something the fused kernel does not
        if form is None:
            return False
        weight, eps, unit_offset = form
        if (not self.can_fuse_norm(M, K) or weight.numel() != K or not weight.is_contiguous()
                or weight.data_ptr() % 16
                or w.dtype != torch.bfloat16 or not w.is_contiguous() or w.shape[1] != K
                or out.stride(1) != 1 or (swiglu and (w.shape[0] % 2 or out.dtype != torch.bfloat16))):
            return False
        N = w.shape[0] // 2 if swiglu else w.shape[0]
        if out.shape != (M, N) or out.dtype not in (torch.bfloat16, torch.float32):
            return False
        if self.wants_mid(M, w.shape[0], K) and self.lib.has("mv_gemm_mid"):
            return False    # the norm as a kernel of its own and the K-splitting product are faster here
        if self.prefers_library(M, w.shape[0], K, gated=swiglu):
            return False    # as are the norm and the library's product
        if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N):
            return False
        resid_in, delta, resid_out = pending.fused()
        if isinstance(delta, SplitSum):
            delta = delta.materialize()
        self._note("mv_gemm_skinny_norm", M * K * (4 + (2 + 4 if delta is not None else 0)) + self._size(w, out),
                   2 * M * w.shape[0] * K + 4 * M * K)
        self.lib.call("mv_gemm_skinny_norm", resid_in.data_ptr(), _ptr(delta), _ptr(resid_out), weight.data_ptr(),
                      _weight_code(weight, "norm weight"), float(eps), int(unit_offset), w.data_ptr(),
                      _ptr(bias), out.data_ptr(), out.stride(0) if M > 1 else N, _CODES[out.dtype], M, N, K,
                      int(swiglu), self._stream())
        return True

    def gemm_swiglu(self, a: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor) -> bool:
        """out[M, I] = silu(a Wg^T) * (a Wu^T) for the packed weight [2I, K] in one pass over the
        weight, when the weight-streaming kernel takes the shape. Returns False (and does nothing)
        otherwise; the caller then runs the product and the activation separately. ``a`` may be a
        pending norm, as in ``gemm``."""
        if not isinstance(a, torch.Tensor):
            if isinstance(a, WeightedRows):
                if self._gemm_scaled(a, w_gate_up, out, None, swiglu=True):
                    return True
            elif self._gemm_fused_norm(a, w_gate_up, out, None, swiglu=True):
                return True
            a = a.materialize()
        if not (self.use_fast_kernels and self.lib.has("mv_gemm_skinny_swiglu")):
            return False
        M, K = a.shape
        two_i = w_gate_up.shape[0]
        if self.wants_tile(M, two_i, K, gated=True) and self.gemm_tile(a, w_gate_up, out, None, gated=True):
            return True
        if self.prefers_library(M, two_i, K, gated=True) and self._library_allowed(M, two_i, K, False):
            return False
        # with the library's product at hand, more rows than one workgroup takes go there
        if (M > SKINNY_LAUNCH_ROWS or M == 0
                or (not self.streams_rows(M, two_i, K) and self._library_allowed(M, two_i, K, False))
                or w_gate_up.dtype != torch.bfloat16 or K % 32 or two_i % 2
                or a.stride(1) != 1 or (M > 1 and a.stride(0) % 8) or a.data_ptr() % 16
                or not w_gate_up.is_contiguous() or w_gate_up.shape[1] != K):
            return False
        self._act(a, "gemm input"); self._act(out, "swiglu output"); _dev(w_gate_up, "gate_up weight")
        if out.shape != (M, two_i // 2) or out.stride(1) != 1:
            raise KernelLibraryError(f"gemm_swiglu: output {tuple(out.shape)} is not [{M}, {two_i // 2}]")
        if self._gemm_mid(a, a.stride(0) if M > 1 else K, w_gate_up, None, out, out.stride(0) if M > 1 else two_i // 2,
                          M, two_i, K, swiglu=True):
            return True
        self._note("mv_gemm_skinny_swiglu", self._size(a, w_gate_up, out), 2 * M * two_i * K)
        self.lib.call("mv_gemm_skinny_swiglu", a.data_ptr(), a.stride(0) if M > 1 else K, w_gate_up.data_ptr(),
                      out.data_ptr(), out.stride(0) if M > 1 else two_i // 2, M, two_i // 2, K, self._stream())
        return True

    # ------------------------------------------------------------------------------------
    def attention(self, q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  block_table: torch.Tensor, page_size: int, positions: torch.Tensor, token_seq: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, scale: float, window: Optional[int],
                  plan: Optional["AttentionPlan"] = None, keep_first: int = 0, gate: Optional[torch.Tensor] = None,
                  value_dim: Optional[int] = None) -> None:
        """Causal attention of the step's queries over the paged cache.

        q: [n, >= H*D] rows (a view into the qkv rows), out: [n, H*Dv] (``value_dim`` Dv: the size of a value row
        where it differs from a key's; such sizes take the general kernel). The query at position p
        of sequence s sees keys max(0, p - window) .. p of s and, with ``keep_first``, the first
        ``keep_first`` positions of s however far back they lie. ``gate`` [n, >= H] (a view into the
        packed rows): head h's output is multiplied by sigmoid(gate[:, h]). ``plan`` carries what the faster
        kernels need to know about the step (see AttentionPlan); without it, or in float32, the
        general kernel runs."""
        self._act(q, "queries"); self._act(out, "attention output")
        self._act(k_pages, "key pages"); self._act(v_pages, "value pages")
        n = q.shape[0]
        vdim = head_dim if value_dim is None else int(value_dim)
        hd = num_heads * vdim
        if q.dim() != 2 or q.shape[1] < num_heads * head_dim or q.stride(1) != 1 or out.shape != (n, hd) or out.stride(1) != 1:
            raise KernelLibraryError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not hold "
                                     f"{num_heads} heads of {head_dim} / {vdim}")
        if tuple(k_pages.shape[1:]) != (num_kv_heads, page_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (num_kv_heads, vdim, page_size) or \
                not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelLibraryError(f"attention: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} have the "
                                     f"wrong layout for {num_kv_heads} heads of {head_dim}, page {page_size}")
        for t, what in ((positions, "positions"), (token_seq, "token_seq")):
            _dev(t, what)
            if t.dtype != torch.int32 or t.numel() < n:
                raise KernelLibraryError(f"attention: {what} must be int32 with at least {n} elements")
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("attention: the block table must be a contiguous int32 matrix")
        if num_heads % num_kv_heads:
            raise KernelLibraryError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if n == 0:
            return
        w = -1 if window is None else int(window)
        first = 0 if window is None else max(0, int(keep_first))      # without a window every key is seen anyway
        qs = q.stride(0) if n > 1 else q.shape[1]
        os_ = out.stride(0) if n > 1 else hd
        gs = 0
        if gate is not None:
            self._act(gate, "head gates")
            if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < num_heads or gate.stride(1) != 1:
                raise KernelLibraryError(f"attention: gates {tuple(gate.shape)} do not hold {num_heads} numbers a row")
            gs = gate.stride(0) if n > 1 else gate.shape[1]
        if vdim == head_dim and self._attention_fast(q, qs, out, os_, k_pages, v_pages, block_table, page_size, positions,
                                                     token_seq, num_heads, num_kv_heads, head_dim, scale, w, plan, first, gate, gs):
            return
        self._note_attention("mv_attention_ref", plan, n, num_heads, num_kv_heads, head_dim, q.element_size())
        self.lib.call("mv_attention_ref", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                      v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      positions.data_ptr(), token_seq.data_ptr(), n, num_heads, num_kv_heads, head_dim, vdim,
                      float(scale), w, first, _ptr(gate), gs, self.code, self._stream())

    def _note_attention(self, entry: str, plan, n_tokens: int, H: int, Hkv: int, D: int, item: int, splits: int = 1) -> None:
        """Bytes: the keys and values of every sequence once (per key, so that the line can be priced
        at another context length), queries and outputs, the partial results of split keys written and
        read back. Operations: two products over every (query, visible key) pair."""
        if self.ledger is None:
            return
        keys = getattr(plan, "kv_tokens", 0) if plan is not None else 0
        pairs = getattr(plan, "attention_pairs", 0) if plan is not None else 0
        fixed = 2 * n_tokens * H * D * item
        if splits > 1:
            fixed += 2 * n_tokens * H * splits * (D + 2) * 4
        self.ledger.append((entry, fixed, 0, keys, pairs, 2 * Hkv * D * item, 4 * H * D))

    def _split_counters(self, n: int, partials) -> Optional[int]:
        """One counter for every (sequence, kv head) of a decode step whose keys are split over
        workgroups: the workgroups count themselves in and the last one adds the partial results up.
        The counters are zero between launches (the last workgroup puts its counter back), so they are
        cleared once, here; launches that share them must follow each other on one stream. They belong
        to this ``Ops`` (an engine has its own), and a launch that fails clears them again
        (``_decode_launch``)."""
        if partials is None:
            return None
        if self._attn_counters is None:
            self._attn_counters = torch.zeros(SPLIT_COUNTERS, dtype=torch.int32, device=partials.device)
        if n > SPLIT_COUNTERS:
            raise ValueError(f"a decode step of {n} (sequence, kv head) pairs exceeds the {SPLIT_COUNTERS} split counters")
        return self._attn_counters.data_ptr()

    def _decode_launch(self, entry: str, *args) -> None:
        """Launches a decode attention; should the launch fail, the split counters are put back to
        zero (outside a capture) before the error goes on: a launch that stopped half-way may have
        left some counted."""
        try:
            self.lib.call(entry, *args)
        except Exception:
            if self._attn_counters is not None and not torch.cuda.is_current_stream_capturing():
                try:
                    torch.cuda.synchronize()
                    self._attn_counters.zero_()
                except Exception:
                    pass
            raise

    def _decode_split(self, plan, n_seqs: int, H: int, Hkv: int, D: int, context: Optional[int] = None):
        """Over how many workgroups a decode step deals a sequence's keys out, and the work area for
        their partial results: (nsplit, partials). The keys go round in groups of 128 (a block of 32
        to each of a workgroup's four waves), so a split beyond the number of such groups in the
        planned context would only add workgroups that end at once. The count is a property of the
        plan (a captured graph keeps it): about one workgroup in flight for every compute unit (measured on MI355X with 8 kv heads at contexts of 1,100: 512 and 1,024
        workgroups are 5 and 18 % slower at batch 8; batch 64 is fastest without a split)."""
        # (``context``: the keys a query reads at most, where a window makes that fewer than the planned context)
        ctx = max(1, plan.max_context_len if context is None else min(context, plan.max_context_len))
        forced = getattr(plan, "decode_splits", None)
        nsplit = forced if forced else max(1, min(self.compute_units // max(1, n_seqs * Hkv), -(-ctx // 128), 64))
        partials = None
        if nsplit > 1:
            rows = max(n_seqs * nsplit, 2048 // Hkv, 256)      # one size serves every batch of a graph set
            partials = plan.workspace.get("attn.partials", (rows * H * (D + 2),), torch.float32)
        return nsplit, partials

    def attention_decode_fused(self, qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor,
                               v_pages: torch.Tensor, block_table: torch.Tensor, page_size: int,
                               positions: torch.Tensor, token_seq: torch.Tensor, num_heads: int, num_kv_heads: int,
                               head_dim: int, scale: float, window: Optional[int], plan,
                               q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                               rope_table: Optional[torch.Tensor], interleaved: bool, store_kv: bool,
                               unit_offset: bool = False, rope_rows: Optional[torch.Tensor] = None) -> bool:
        """A decode step's attention straight from the raw rows ``qkv`` = [q | k | v] (or [q] alone
        without ``store_kv``): per-head norm, rotation, cache write and attention in one kernel.
        Returns False, having done nothing, when the step or the sizes are not taken; the caller
        then runs ``qk_norm_rope_store`` and ``attention``. ``rope_rows`` float32 [tokens, D]: the rows of
        ``rope_table`` at the step's positions, when something gathered them earlier in the step."""
        if (not self.use_fast_kernels or plan is None or not plan.decode_only
                or not self.lib.has("mv_attention_decode_fused")):
            return False
        H, Hkv, D = num_heads, num_kv_heads, head_dim
        n = qkv.shape[0]
        width = (H + (2 * Hkv if store_kv else 0)) * D
        stride = qkv.stride(0) if n > 1 else qkv.shape[1]
        os_ = out.stride(0) if n > 1 else H * D
        if (D not in (64, 128) or page_size % 16 or H % Hkv or H // Hkv > 16 or n != plan.n_seqs or n == 0
                or qkv.dim() != 2 or qkv.shape[1] < width or qkv.stride(1) != 1 or stride % 8 or qkv.data_ptr() % 16
                or out.shape != (n, H * D) or out.stride(1) != 1 or os_ % 4 or out.data_ptr() % 8
                or interleaved or (rope_table is not None and (rope_table.dim() != 2 or rope_table.shape[1] != D
                                                               or rope_table.dtype != torch.float32
                                                               or not rope_table.is_contiguous()))
                or (q_weight is None and k_weight is not None)):
            return False
        wcode = DTYPE_F32
        if q_weight is not None:
            if q_weight.numel() != D or q_weight.data_ptr() % 16 or (
                    store_kv and (k_weight is None or k_weight.numel() != D or k_weight.dtype != q_weight.dtype
                                  or k_weight.data_ptr() % 16)):
                return False
            wcode = _weight_code(q_weight, "q_norm weight")
        self._act(qkv, "qkv"); self._act(out, "attention output")
        self._act(k_pages, "key pages"); self._act(v_pages, "value pages")
        if tuple(k_pages.shape[1:]) != (Hkv, page_size, D) or tuple(v_pages.shape[1:]) != (Hkv, D, page_size) or \
                not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelLibraryError(f"attention: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} have the "
                                     f"wrong layout for {Hkv} heads of {D}, page {page_size}")
        for t, what in ((positions, "positions"), (token_seq, "token_seq")):
            _dev(t, what)
            if t.dtype != torch.int32 or t.numel() < n:
                raise KernelLibraryError(f"attention: {what} must be int32 with at least {n} elements")
        _dev(block_table, "block table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
            raise KernelLibraryError("attention: the block table must be a contiguous int32 matrix")
        if rope_rows is not None and (rope_table is None or rope_rows.dtype != torch.float32 or not rope_rows.is_cuda
                                      or rope_rows.shape != (n, D) or not rope_rows.is_contiguous()
                                      or rope_rows.data_ptr() % 16):
            rope_rows = None
        nsplit, partials = self._decode_split(plan, n, H, Hkv, D)
        self._note_attention("mv_attention_decode_fused", plan, n, H, Hkv, D, 2, splits=nsplit)
        self._decode_launch("mv_attention_decode_fused", qkv.data_ptr(), stride, 0, H * D, (H + Hkv) * D, out.data_ptr(), os_,
                      k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      positions.data_ptr(), plan.cu_seqlens.data_ptr(), n, H, Hkv, D, float(scale),
                      -1 if window is None else int(window), _ptr(q_weight), _ptr(k_weight), wcode, float(eps),
                      int(unit_offset), _ptr(rope_table), _ptr(rope_rows), int(store_kv), _ptr(partials),
                      self._split_counters(n * Hkv, partials), nsplit, -(-max(1, plan.max_context_len) // page_size),
                      DECODE_ATTENTION_WAVES, token_seq.data_ptr(), self._stream())
        return True

    def _prefill_variant(self, plan, group: int, Hkv: int):
        """(column tiles per wave, key groups per workgroup, units, busy units) of the MFMA prompt
        attention for this step; column tiles 0: the kernel does not serve ``group`` heads per kv head."""
        # 128 columns per workgroup (each operand read from LDS feeds two MFMAs) when that still leaves
        # two workgroups for every compute unit, else 64 (measured on MI355X: 2048 tokens of one
        # sequence with 8 kv heads are faster with 64, 4096 tokens or 8 x 512 with 128)
        nt, n_units, n_busy = 0, 0, 0
        for cand in (2, 1):
            u = self.lib.dll.mv_attention_prefill_unit_tokens(group, cand)
            if u > 0:
                units, busy = plan.units(u), plan.busy_units(u)
                if cand == 2 and busy * Hkv < 2 * self.compute_units and \
                        self.lib.dll.mv_attention_prefill_unit_tokens(group, 1) > 0:
                    continue
                nt, n_units, n_busy = cand, units, busy
                break
        if plan.prefill_variant is not None:
            nt = int(plan.prefill_variant[0])
            u = self.lib.dll.mv_attention_prefill_unit_tokens(group, nt)
            if u <= 0:
                raise KernelLibraryError(f"attention: {nt} column tiles a wave do not serve {group} heads per kv head")
            n_units, n_busy = plan.units(u), plan.busy_units(u)
        if nt == 0:
            return 0, 0, 0, 0
        # two key groups per workgroup (eight waves) halve the walk over long contexts; they pay while
        # the grid leaves compute units waiting for the longest walk (measured on MI355X, 8 kv heads:
        # faster below two four-wave workgroups per compute unit, 33.9 against 35.3 us at 1,792 tokens,
        # slower from there on, 44.0 against 40.8 us at 2,048)
        # (a recorded step's grid is sized for the most units its size class can have; the rule goes by
        # the units its tokens fill, as an eager step's does)
        kw = 2 if plan.max_context_len >= PREFILL_TWO_GROUPS_FROM and n_busy * Hkv < 2 * self.compute_units else 1
        if plan.prefill_variant is not None:
            kw = int(plan.prefill_variant[1])
        return nt, kw, n_units, n_busy

    def _attention_fast(self, q, qs, out, os_, k_pages, v_pages, block_table, page_size, positions, token_seq,
                        H, Hkv, D, scale, window, plan, first: int = 0, gate=None, gs: int = 0) -> bool:
        """The MFMA kernels, when the step and the sizes allow them."""
        if not self.use_fast_kernels or plan is None or not self.lib.has("mv_attention_decode"):
            return False
        if D not in (64, 128) or page_size % 16 or qs % 8 or os_ % 4 or q.data_ptr() % 16 or out.data_ptr() % 8:
            return False
        group = H // Hkv
        n_seqs = plan.n_seqs
        priced = self._window_priced(plan, window, first) if self.ledger is not None else plan
        if plan.decode_only and group <= 16:
            # under a window a query reads the window, the kept positions and what the blocks of 32 add at both ends
            nsplit, partials = self._decode_split(plan, n_seqs, H, Hkv, D,
                                                  context=None if window < 0 else window + 1 + first + 64)
            self._note_attention("mv_attention_decode", priced, q.shape[0], H, Hkv, D, 2, splits=nsplit)
            self._decode_launch("mv_attention_decode", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                          v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                          positions.data_ptr(), plan.cu_seqlens.data_ptr(), n_seqs, H, Hkv, D, float(scale), window,
                          _ptr(partials), self._split_counters(n_seqs * Hkv, partials), nsplit,
                          -(-max(1, plan.max_context_len) // page_size), DECODE_ATTENTION_WAVES, token_seq.data_ptr(),
                          first, _ptr(gate), gs, self._stream())
            return True
        if page_size & (page_size - 1):
            return False
        nt, kw, n_units, n_busy = self._prefill_variant(plan, group, Hkv)
        if nt == 0:
            return False
        self._note_attention("mv_attention_prefill", priced, q.shape[0], H, Hkv, D, 2)
        self.lib.call("mv_attention_prefill", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                      v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      positions.data_ptr(), plan.cu_seqlens.data_ptr(), n_seqs, n_units, n_busy, nt, kw, H, Hkv, D,
                      float(scale), window, first, _ptr(gate), gs, self._stream())
        return True

    # ------------------------------------------------------------------------------------
    def sample(self, logits: torch.Tensor, out: torch.Tensor, temperature: Optional[torch.Tensor] = None,
               top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
               rng: Optional[torch.Tensor] = None, advance: Optional[tuple] = None) -> None:
        """One token id per row of float32 ``logits`` into int32 ``out``.

        temperature float32 [M] (None or 0: arg-max), top_k int32 [M], top_p float32 [M],
        rng int64 [M, 2] = (seed, counter) of each row's random stream.

        ``advance`` = (token_ids, positions, context_lens), int32 [>= M] each, makes the kernel
        prepare the same step's next run on the device: row m's token also goes to token_ids[m],
        positions[m] and context_lens[m] grow by one and so does the counter in ``rng``."""
        _dev(logits, "logits"); _dev(out, "sampled ids")
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise KernelLibraryError("sample: logits must be float32 [M, V] with a contiguous last dimension")
        M, V = logits.shape
        if out.dtype != torch.int32 or out.numel() < M:
            raise KernelLibraryError("sample: the output must be int32 with at least M elements")
        for t, dt, what in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                            (top_p, torch.float32, "top_p")):
            if t is not None:
                _dev(t, what)
                if t.dtype != dt or t.numel() < M or not t.is_contiguous():
                    raise KernelLibraryError(f"sample: {what} must be {dt} with at least M elements")
        if temperature is not None:
            if rng is None or rng.dtype != torch.int64 or rng.shape != (M, 2) or not rng.is_contiguous():
                raise KernelLibraryError("sample: rng must be int64 [M, 2] when temperatures are given")
            _dev(rng, "rng")
        if M == 0:
            return
        # rows without thresholds are shared by SAMPLE_CHUNKS workgroups each (two short launches);
        # the scratch for their partial results is made once
        work = None
        if M <= SAMPLE_WORK_ROWS and V >= 4096:
            if self._sample_work is None:
                self._sample_work = torch.empty(SAMPLE_WORK_ROWS * SAMPLE_CHUNKS * 2, dtype=torch.int32,
                                                device=logits.device)
            work = self._sample_work
        self._note("mv_sample", M * V * 4, 2 * M * V)
        if advance is not None:
            for t, what in zip(advance, ("next token ids", "positions", "context lengths")):
                _dev(t, what)
                if t.dtype != torch.int32 or t.numel() < M or not t.is_contiguous():
                    raise KernelLibraryError(f"sample: {what} must be contiguous int32 with at least M elements")
            self.lib.call("mv_sample_advance", logits.data_ptr(), logits.stride(0) if M > 1 else V, M, V,
                          _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(rng), out.data_ptr(), _ptr(work),
                          SAMPLE_CHUNKS, advance[0].data_ptr(), advance[1].data_ptr(), advance[2].data_ptr(),
                          self._stream())
            return
        self.lib.call("mv_sample", logits.data_ptr(), logits.stride(0) if M > 1 else V, M, V, _ptr(temperature),
                      _ptr(top_k), _ptr(top_p), _ptr(rng), out.data_ptr(), _ptr(work), SAMPLE_CHUNKS, self._stream())


_OPS = {}


def get_ops(dtype: torch.dtype) -> Ops:
    """A front end shared by code outside any engine (tools, tests of single kernels). An engine makes
    its own (``Ops(dtype)``): launches that share one must follow each other on one stream."""
    ops = _OPS.get(dtype)
    if ops is None:
        ops = _OPS[dtype] = Ops(dtype)
    return ops
