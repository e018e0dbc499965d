"""Operations of the decoder on device tensors, bound to one activation type.

Each method checks shapes, types and placement on the host and then launches a kernel of
the HIP library on the current stream. Tensors must live on the GPU: there is no CPU path.
"""
from __future__ import annotations

from typing import Optional

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
        self._note("mv_embedding", n * (8 * out.shape[1] + 4))
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
                           unit_offset: bool = False) -> None:
        """In place on the rows of ``qkv`` = [q | k | v]: per-head RMSNorm of q and k (when
        weights are given), rotary embedding (when a table is given); k and v are written to
        the cache pages when pages are given. Without pages the rows hold only q."""
        self._act(qkv, "qkv")
        n = qkv.shape[0]
        store = k_pages is not None
        width = (num_heads + (2 * num_kv_heads if store else 0)) * head_dim
        if qkv.dim() != 2 or qkv.shape[1] != width or qkv.stride(1) != 1:
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
                    tuple(v_pages.shape[1:]) != (num_kv_heads, head_dim, page_size) or \
                    not k_pages.is_contiguous() or not v_pages.is_contiguous():
                raise KernelLibraryError(
                    f"qk_norm_rope_store: pages {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not match "
                    f"[pages, {num_kv_heads}, {page_size}, {head_dim}] / [pages, {num_kv_heads}, {head_dim}, {page_size}]")
            if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
                raise KernelLibraryError("qk_norm_rope_store: the block table must be a contiguous int32 matrix")
            bt_width = block_table.shape[1]
        q_dim = num_heads * head_dim
        kv_dim = num_kv_heads * head_dim
        stride = qkv.stride(0) if n > 1 else width
        # with many tokens the values go to their transposed pages tile by tile, so that
        # neighbouring tokens write neighbouring slots (mode 3); with few, a store per token and head
        mode = 0 if not store else (3 if n >= STORE_V_SPLIT_TOKENS else 1)
        self._note("mv_qk_norm_rope_store", n * (width + q_dim + (2 * kv_dim if store else 0)) * qkv.element_size()
                   + (n * rot * 4 if rope_table is not None else 0), 10 * n * (q_dim + (kv_dim if store else 0)))
        self.lib.call("mv_qk_norm_rope_store", qkv.data_ptr(), stride, 0, q_dim,
                      q_dim + kv_dim, positions.data_ptr(), token_seq.data_ptr(), _ptr(block_table), bt_width,
                      page_size, _ptr(k_pages), _ptr(v_pages), n, num_heads, num_kv_heads, head_dim,
                      _ptr(q_weight), _ptr(k_weight), wcode, float(eps), int(unit_offset), _ptr(rope_table), rot,
                      int(interleaved), mode, self.code, self._stream())

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
                  plan: Optional["AttentionPlan"] = None) -> None:
        """Causal attention of the step's queries over the paged cache.

        q: [n, >= H*D] rows (a view into the qkv rows), out: [n, H*D]. The query at position p
        of sequence s sees keys max(0, p - window) .. p of s. ``plan`` carries what the faster
        kernels need to know about the step (see AttentionPlan); without it, or in float32, the
        general kernel runs."""
        self._act(q, "queries"); self._act(out, "attention output")
        self._act(k_pages, "key pages"); self._act(v_pages, "value pages")
        n = q.shape[0]
        hd = num_heads * head_dim
        if q.dim() != 2 or q.shape[1] < hd or q.stride(1) != 1 or out.shape != (n, hd) or out.stride(1) != 1:
            raise KernelLibraryError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not hold "
                                     f"{num_heads} heads of {head_dim}")
        if tuple(k_pages.shape[1:]) != (num_kv_heads, page_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (num_kv_heads, head_dim, page_size) or \
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
        qs = q.stride(0) if n > 1 else q.shape[1]
        os_ = out.stride(0) if n > 1 else hd
        if self._attention_fast(q, qs, out, os_, k_pages, v_pages, block_table, page_size, positions, token_seq,
                                num_heads, num_kv_heads, head_dim, scale, w, plan):
            return
        self._note_attention("mv_attention_ref", plan, n, num_heads, num_kv_heads, head_dim, q.element_size())
        self.lib.call("mv_attention_ref", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                      v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      positions.data_ptr(), token_seq.data_ptr(), n, num_heads, num_kv_heads, head_dim,
                      float(scale), w, self.code, self._stream())

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

    def _decode_split(self, plan, n_seqs: int, H: int, Hkv: int, D: int):
        """Over how many workgroups a decode step deals a sequence's keys out, and the work area for
        their partial results: (nsplit, partials). The keys go round in groups of 128 (a block of 32
        to each of a workgroup's four waves), so a split beyond the number of such groups in the
        planned context would only add workgroups that end at once. The count is a property of the
        plan (a captured graph keeps it): about one workgroup in flight for every compute unit (measured on MI355X with 8 kv heads at contexts of 1,100: 512 and 1,024
        workgroups are 5 and 18 % slower at batch 8; batch 64 is fastest without a split)."""
        ctx = max(1, plan.max_context_len)
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

    def _attention_fast(self, q, qs, out, os_, k_pages, v_pages, block_table, page_size, positions, token_seq,
                        H, Hkv, D, scale, window, plan) -> bool:
        """The MFMA kernels, when the step and the sizes allow them."""
        if not self.use_fast_kernels or plan is None or not self.lib.has("mv_attention_decode"):
            return False
        if D not in (64, 128) or page_size % 16 or qs % 8 or os_ % 4 or q.data_ptr() % 16 or out.data_ptr() % 8:
            return False
        group = H // Hkv
        n_seqs = plan.n_seqs
        if plan.decode_only and group <= 16:
            nsplit, partials = self._decode_split(plan, n_seqs, H, Hkv, D)
            self._note_attention("mv_attention_decode", plan, q.shape[0], H, Hkv, D, 2, splits=nsplit)
            self._decode_launch("mv_attention_decode", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                          v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                          positions.data_ptr(), plan.cu_seqlens.data_ptr(), n_seqs, H, Hkv, D, float(scale), window,
                          _ptr(partials), self._split_counters(n_seqs * Hkv, partials), nsplit,
                          -(-max(1, plan.max_context_len) // page_size), DECODE_ATTENTION_WAVES, token_seq.data_ptr(),
                          self._stream())
            return True
        if page_size & (page_size - 1):
            return False
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
            return False
        # two key groups per workgroup (eight waves) halve the walk over long contexts; they pay while
        # the grid leaves compute units waiting for the longest walk (measured on MI355X, 8 kv heads:
        # faster below two four-wave workgroups per compute unit, 33.9 against 35.3 us at 1,792 tokens,
        # slower from there on, 44.0 against 40.8 us at 2,048)
        # (a recorded step's grid is sized for the most units its size class can have; the rule goes by
        # the units its tokens fill, as an eager step's does)
        kw = 2 if plan.max_context_len >= PREFILL_TWO_GROUPS_FROM and n_busy * Hkv < 2 * self.compute_units else 1
        if plan.prefill_variant is not None:
            kw = int(plan.prefill_variant[1])
        self._note_attention("mv_attention_prefill", plan, q.shape[0], H, Hkv, D, 2)
        self.lib.call("mv_attention_prefill", q.data_ptr(), qs, out.data_ptr(), os_, k_pages.data_ptr(),
                      v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
                      positions.data_ptr(), plan.cu_seqlens.data_ptr(), n_seqs, n_units, n_busy, nt, kw, H, Hkv, D,
                      float(scale), window, self._stream())
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
