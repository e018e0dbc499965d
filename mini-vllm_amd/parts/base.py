"""What a layer is made of, and how a part is declared, registered and built.

A model is data: a ``ModelPlan`` lists layers, each layer names the kind and the sizes of
its mixer, feed-forward, norms and the block arrangement that wires them. A part never
learns which model it is in; it sees its own spec, its own tensors and the step's context.

A part class has three duties:

* ``tensors(spec)`` declares the tensors it needs, by logical name (``"q"``, ``"gate"``),
  with shape and the law random weights are drawn from. The architecture maps logical
  names to names on disk; the loader checks shapes and hands the tensors over.
* ``__init__(spec, tensors, runtime)`` takes them (it may pack several into one).
* ``forward(...)`` launches its kernels on the step's tensors.

Mixers additionally state what memory they need per request: ``cache_need(spec)`` for pages
of keys and values, ``state_shape(spec)`` for a fixed-size state.

New kinds are added with ``register_mixer`` / ``register_feed_forward`` / ``register_norm`` /
``register_position_encoding`` / ``register_block`` / ``register_embedding`` / ``register_head``;
nothing else in the engine changes.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Dict, List, Optional, Sequence, Tuple

import torch


# ---------------------------------------------------------------------------------------
# Declarations
# ---------------------------------------------------------------------------------------
@dataclass(frozen=True)
class TensorDecl:
    """One tensor a part needs. ``init``: "normal" = N(0, std), "ones_normal" = 1 + N(0, std),
    "zeros_normal" = N(0, std) for biases. ``integer`` tensors are kept as int32."""
    shape: Tuple[int, ...]
    init: str = "normal"
    integer: bool = False


class PartSpec:
    """Base of the frozen dataclasses that describe one part; ``kind`` selects the class."""
    kind: ClassVar[str] = ""


class Retention:
    """How long a cache group keeps a position of a request. The cache manager and the executor ask
    only these questions of it, so a mixer with another rule brings a class of its own (frozen
    dataclasses make good ones: equal rules compare equal and hash alike)."""

    # every position stays for the whole life of the request: only then can pages that hold a
    # prompt's prefix be shared between requests
    keeps_everything: ClassVar[bool] = False

    def first_kept_page(self, next_position: int, page_size: int) -> int:
        """Index of the first page the request still needs when its next query stands at
        ``next_position``; pages before it are given back, and no kernel may touch them."""
        raise NotImplementedError

    def first_kept_pages(self, next_positions, page_size: int):
        """The same for an int64 array of positions (one per sequence of a step)."""
        import numpy as np
        return np.fromiter((self.first_kept_page(int(p), page_size) for p in next_positions), dtype=np.int64,
                           count=len(next_positions))

    def most_pages(self, length: int, page_size: int) -> Optional[int]:
        """Most pages a request of ``length`` tokens holds at one time, if the rule can tell
        (a request that needs more than its pool has is refused when it is submitted)."""
        return None

    def most_pages_held(self, length: int, page_size: int, portion: int) -> Optional[int]:
        """Most pages a request that grows to ``length`` tokens holds at one time when a step brings at
        most ``portion`` of its tokens, if the rule can tell: the executor then gives the group's pool no
        more pages than that for every request that can be live (a group that gives pages back early
        needs a smaller pool than one that keeps everything). None: as many as ``length`` fills."""
        return None

    def key(self) -> Tuple:
        """Calls whose needs have equal keys share a group: a pool and block tables of their own."""
        return (type(self).__name__,) + tuple(sorted(vars(self).items()))


@dataclass(frozen=True)
class KeepAll(Retention):
    keeps_everything: ClassVar[bool] = True

    def first_kept_page(self, next_position: int, page_size: int) -> int:
        return 0

    def first_kept_pages(self, next_positions, page_size: int):
        import numpy as np
        return np.zeros(len(next_positions), dtype=np.int64)

    def most_pages(self, length: int, page_size: int) -> Optional[int]:
        return -(-length // page_size)

    def most_pages_held(self, length: int, page_size: int, portion: int) -> Optional[int]:
        return -(-length // page_size)


@dataclass(frozen=True)
class KeepWindow(Retention):
    """The last ``window`` positions besides the query's own stay; older pages go back to the pool."""
    window: int = 0

    def __post_init__(self):
        if self.window < 0:
            raise ValueError(f"a window must be >= 0, got {self.window}")

    def first_kept_page(self, next_position: int, page_size: int) -> int:
        return max(0, next_position - self.window) // page_size

    def first_kept_pages(self, next_positions, page_size: int):
        import numpy as np
        return np.maximum(0, np.asarray(next_positions, dtype=np.int64) - self.window) // page_size

    def most_pages_held(self, length: int, page_size: int, portion: int) -> Optional[int]:
        # while a portion runs: the window behind its first token, the portion itself, and the two
        # pages that the ends of that range may only touch
        return min(-(-length // page_size), (self.window + max(1, portion)) // page_size + 2)


class CacheNeed:
    """Paged memory a mixer needs for each token of a request: which tensors a page consists of
    and how long positions are kept. The executor allocates ``[pages, *shape]`` per named tensor
    for every call with this need and hands them to the mixer as ``ctx.kv(call).pages[name]``."""

    retention: Retention

    def page_shapes(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        """Name -> shape of one page of ``page_size`` token slots."""
        raise NotImplementedError

    def page_dtypes(self, activation_dtype: torch.dtype) -> Dict[str, torch.dtype]:
        """Name -> element type of each page tensor; the default keeps everything in the activation
        type. A mixer that pages float32 or integer state names the type here."""
        return {name: activation_dtype for name in self.page_shapes(1)}

    def group_key(self) -> Tuple:
        return self.retention.key()

    def bytes_per_token(self, activation_dtype) -> int:
        """Bytes of cache one token takes in one call. (An ``int`` is read as the size of an element
        of every tensor.)"""
        if isinstance(activation_dtype, int):
            sizes = {name: activation_dtype for name in self.page_shapes(1)}
        else:
            sizes = {name: torch.empty((), dtype=dt).element_size()
                     for name, dt in self.page_dtypes(activation_dtype).items()}
        total = 0
        for name, shape in self.page_shapes(1).items():
            n = 1
            for d in shape:
                n *= int(d)
            total += n * sizes[name]
        return total


@dataclass(frozen=True)
class KeyValueNeed(CacheNeed):
    """Keys and values of softmax attention: K pages ``[kv_heads, slot, head_dim]`` and V pages
    transposed, ``[kv_heads, head_dim, slot]``, so that both matrix products of the attention
    kernels read their first operand straight from a page."""
    retention: Retention
    num_kv_heads: int
    head_dim: int

    def page_shapes(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        return {"k": (self.num_kv_heads, page_size, self.head_dim), "v": (self.num_kv_heads, self.head_dim, page_size)}


# ---------------------------------------------------------------------------------------
# Registries
# ---------------------------------------------------------------------------------------
class Registry:
    def __init__(self, what: str):
        self.what = what
        self._classes: Dict[str, type] = {}

    def register(self, kind: str, cls: Optional[type] = None):
        def deco(c):
            if kind in self._classes and self._classes[kind] is not c:
                raise ValueError(f"{self.what} kind {kind!r} is already registered")
            self._classes[kind] = c
            return c
        return deco(cls) if cls is not None else deco

    def unregister(self, kind: str) -> None:
        self._classes.pop(kind, None)

    def get(self, kind: str) -> type:
        try:
            return self._classes[kind]
        except KeyError:
            raise KeyError(f"no {self.what} of kind {kind!r} is registered "
                           f"(known: {sorted(self._classes)})") from None

    def kinds(self) -> List[str]:
        return sorted(self._classes)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position_encoding = POSITION_ENCODINGS.register
register_block = BLOCKS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register


# ---------------------------------------------------------------------------------------
# Runtime handed to every part
# ---------------------------------------------------------------------------------------
class Workspace:
    """Named device buffers that live across steps and are shared between layers.

    ``get`` returns a view of the wanted shape; the backing buffer grows when a step needs
    more. While a graph is being captured nothing may be allocated, so the buffers have to be
    grown (``reserve``) before."""

    def __init__(self, device: torch.device, retain: bool = False):
        """``retain`` keeps a buffer alive after a larger one has replaced it: captured graphs that
        hold its address go on working."""
        self.device = device
        self._buffers: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: Dict[Tuple, torch.Tensor] = {}
        self._retired: List[torch.Tensor] = []
        self.retain = retain
        self.frozen = False

    def get(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        vkey = (name, dtype, tuple(shape))
        view = self._views.get(vkey)          # making a view costs as much as a launch: keep them
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            if self.frozen:
                raise RuntimeError(f"workspace buffer {name!r} would have to grow to {n} elements while frozen")
            if buf is not None and self.retain:
                self._retired.append(buf)
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]             # views of the replaced buffer
        view = buf[:n].view(*shape)
        if len(self._views) > 4096:
            self._views.clear()
        self._views[vkey] = view
        return view

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in list(self._buffers.values()) + self._retired)


@dataclass
class Runtime:
    """What parts share: the device, the activation type, the kernels and scratch memory."""
    device: torch.device
    dtype: torch.dtype
    ops: Any
    workspace: Workspace
    max_positions: int          # longest sequence the engine serves (rows of position tables)


class HiddenStream:
    """The residual stream of a step: a float32 sum ``resid`` and the last part's output
    ``delta`` that has not been added yet. A norm consumes the pending delta (one fused
    kernel adds it and normalises the sum). ``delta`` is a tensor, or whatever ``ops.gemm(...,
    defer_sum=True)`` returned in its place (an output whose partial sums the norm's kernel adds
    up itself; it has ``shape``, ``materialize()`` and ``discard()``)."""

    __slots__ = ("resid", "delta", "spare", "weighted")

    def __init__(self, resid: torch.Tensor, spare: Optional[torch.Tensor] = None):
        self.resid = resid
        self.delta: Optional[torch.Tensor] = None
        # rows that the last product already added to ``resid`` and left half normalised for the
        # norm that comes next (see NormFold); that norm takes them from here
        self.weighted = None
        # a second buffer of the same shape: a kernel that adds the delta while other workgroups
        # still read the old sum writes the new sum here, and the two change places
        self.spare = spare


class PendingNorm:
    """A norm that has not run yet: the stream whose pending delta it will add, and its weight
    and constants. A part whose first operation is one matrix product over its input may take
    this instead of a tensor (it declares ``accepts_pending_norm = True``) and hand it to
    ``ops.gemm`` / ``ops.gemm_swiglu``, which fuse add, norm and product into one kernel when the
    step is small enough, and otherwise call ``materialize`` and go on as usual. It must be used
    exactly once."""

    def __init__(self, norm, stream: HiddenStream, ctx):
        self.norm, self.stream, self.ctx = norm, stream, ctx
        self.shape = stream.resid.shape
        self.used = False
        self._tensor: Optional[torch.Tensor] = None

    def materialize(self) -> torch.Tensor:
        """Runs the norm (once) and returns the normalised activations."""
        if self._tensor is None:
            if self.used:
                raise RuntimeError("a pending norm was already consumed by a fused kernel")
            self.used = True
            self._tensor = self.norm.forward(self.stream, self.ctx)
        return self._tensor

    def fused(self) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
        """For a kernel that does the add and the norm itself: (residual in, delta or None,
        residual out or None). The stream is updated as if the norm had run."""
        if self.used:
            raise RuntimeError("a pending norm was used twice")
        self.used = True
        st = self.stream
        resid_in, delta = st.resid, st.delta
        resid_out = None
        if delta is not None:
            resid_out = st.spare
            st.resid, st.spare = resid_out, resid_in
            st.delta = None
        return resid_in, delta, resid_out


class NormFold:
    """A residual add and the norm behind it, offered to the product in front of them. With too many
    rows to normalise them inside every workgroup of the next product (``PendingNorm``), the add and
    the norm can still go without a kernel of their own: the product that makes the delta owns each
    element once, so it adds it to ``stream.resid`` there, writes the sum times the norm's weight to
    ``weighted`` and the sums of squares of its column slices to ``partial``; the product behind the
    norm divides its output rows by the root mean square it gets from those sums.

    It is offered only when the part behind the norm says what its first product is
    (``first_product() -> (weight rows, weight columns, gated)``, beside ``accepts_pending_norm``)
    and the kernels take that product from such rows.

    A part that declares ``accepts_fold = True`` gets one as ``fold=`` (or None), hands it to
    ``ops.gemm(..., fold=fold)`` with its last product and returns whatever that returns: the delta
    as before when the shape was not taken, else the half-normalised rows (``ops.WeightedRows``),
    which the block leaves in ``stream.weighted`` for the norm."""

    __slots__ = ("norm", "stream", "weight", "eps", "unit_offset", "weighted", "partial", "normed")

    def __init__(self, norm, stream: HiddenStream, weight: torch.Tensor, eps: float, unit_offset: bool,
                 weighted: torch.Tensor, partial: torch.Tensor, normed: torch.Tensor):
        self.norm, self.stream = norm, stream
        self.weight, self.eps, self.unit_offset = weight, eps, unit_offset
        self.weighted, self.partial, self.normed = weighted, partial, normed


# ---------------------------------------------------------------------------------------
# Part base classes (interfaces)
# ---------------------------------------------------------------------------------------
class Part:
    spec_class: ClassVar[Optional[type]] = None
    # A part whose ``forward`` only launches device work that depends on the step's sizes may be
    # captured in a graph and replayed with other data. A part that looks at host-side values of
    # the step (``ctx.q_lens``, ``ctx.starts``, ``ctx.host_state_slots``) must say False: the
    # executor then runs every step eagerly.
    graph_safe: ClassVar[bool] = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorDecl]:
        """Logical name -> declaration of every tensor this part reads from the model folder."""
        return {}


class Norm(Part):
    """forward(stream, rows=None) -> normalised activations [n or len(rows), h]; adds the
    stream's pending delta first (and keeps the sum in the stream unless ``rows`` is given).
    apply(x, out) normalises a plain tensor. ``pending(stream, ctx)`` may return a PendingNorm
    (see there) instead of running; the default runs at once."""

    def pending(self, stream: HiddenStream, ctx):
        return self.forward(stream, ctx)

    def as_scaled_rms(self) -> Optional[Tuple[torch.Tensor, float, bool]]:
        """(weight, eps, unit_offset) when this norm computes ``x / sqrt(mean(x^2) + eps) * w`` (or
        ``* (1 + w)`` with ``unit_offset``) over the whole row, the form that the fused add + norm +
        product kernel computes itself; None (the default) keeps the norm a kernel of its own."""
        return None

    def forward(self, stream: HiddenStream, ctx, rows: Optional[torch.Tensor] = None,
                tag: str = "normed") -> torch.Tensor:
        raise NotImplementedError

    def apply(self, x: torch.Tensor, out: torch.Tensor) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    """Either hands a rotary table to the mixer's fused kernel (``rotary()``) or rewrites q and
    k itself (``apply``)."""

    def rotary(self) -> Optional[Tuple[torch.Tensor, bool]]:
        """(float32 table [positions, rotary_dim] = cat(cos, sin), interleaved) or None."""
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], ctx) -> None:
        """In place on q [n, H, D] and k [n, Hkv, D] views, for encodings without a table."""
        raise NotImplementedError

    def step_gather(self, ctx):
        """Asked once per step, in front of the layers: (index int32 [tokens], float32 table [rows, w],
        float32 out [tokens, w]) when the encoding wants ``out[t] = table[index[t]]`` prepared for the
        step (it leaves ``out`` in ``ctx.position_rows[self]`` for its mixers), else None. The
        model lets the step's first kernel carry the gather."""
        return None


class Mixer(Part):
    """forward(x, ctx, call) -> y: mixes information along the sequence. ``call`` identifies
    this execution of the layer in the model's order; ``ctx.kv(call)`` and ``ctx.state(call)``
    give its cache pages and its per-request state."""

    @classmethod
    def cache_need(cls, spec) -> Optional[CacheNeed]:
        return None

    @classmethod
    def state_shape(cls, spec) -> Optional[Tuple[Tuple[int, ...], torch.dtype]]:
        """Shape and dtype of the fixed-size state each request holds for this mixer."""
        return None

    def forward(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(x, ctx) -> y, token by token."""

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Embedding(Part):
    """forward(ctx, resid): fills the float32 residual stream [tokens, hidden] from ``ctx.token_ids``.
    An embedding that declares ``carries_gather = True`` takes ``gather=`` (see
    ``PositionEncoding.step_gather``) and runs it in its own launch; for any other the model runs
    the gather as a kernel of its own."""
    carries_gather: ClassVar[bool] = False

    def forward(self, ctx, resid: torch.Tensor) -> None:
        raise NotImplementedError


class Head(Part):
    """forward(h, ctx) -> float32 logits [rows, vocab] from the normalised rows whose logits are wanted."""

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Wires the parts of one layer: forward(stream, ctx, call) updates the stream.

    A block that declares ``accepts_next_norm = True`` is also given ``next_norm=`` and ``next_part=``:
    the norm that the block called next applies first to the stream and the part that takes its
    output (``entry_norm()``, ``entry_part()``), or None. It may offer that norm to its last part
    (``NormFold``)."""
    accepts_next_norm: ClassVar[bool] = False

    def __init__(self, spec, norms: Dict[str, Norm], mixer: Mixer, ffn: FeedForward):
        raise NotImplementedError

    def entry_norm(self) -> Optional["Norm"]:
        """The norm this block applies to the stream before anything else, if it starts with one."""
        return None

    def entry_part(self):
        """The part that takes the output of ``entry_norm()``."""
        return None

    def forward(self, stream: HiddenStream, ctx, call: int) -> None:
        raise NotImplementedError
