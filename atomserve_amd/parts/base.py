"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from its spec alone (`parts.plan`), declares the tensors it needs
(`weight_decls`), is given them (`bind`) and then computes on flat batches of tokens.
Kinds of parts:

  norm          forward(x, delta, rows) -> normalised rows, optionally adding `delta`
                into the fp32 residual stream first
  position      prepare(step) once per step; mixers ask it for what their kernel needs
  mixer         forward(h, step, cache) -> [T, hidden]; says which cache it wants
                through `cache_request()`
  feed_forward  forward(h, step) -> [T, hidden]
  arrangement   runs one layer: owns the order of norms, mixer, feed-forward and
                residual sums

Registering another kind of any of these is one `register(...)` call; the model
builder, the loader, the cache manager and the step function only speak these
interfaces.
"""

from dataclasses import dataclass
from typing import Any, Callable, Optional

import torch

# ---- what a part tells the loader -------------------------------------------------


@dataclass(frozen=True)
class WeightDecl:
    """shape: expected shape after stacking.
    role:  "matrix" is cast to the compute dtype; "vector" (gains and the like) keeps
           32-bit storage if the checkpoint stores it so, else follows the compute dtype;
           "table_int" is kept as int32."""

    shape: tuple
    role: str = "matrix"


# ---- what a mixer tells the cache manager -----------------------------------------


@dataclass(frozen=True)
class PagedCacheRequest:
    """Keys and values of every token (or of the last `window` tokens) in pages."""

    num_kv_heads: int
    head_dim: int
    window: int = 0  # 0: all keys are kept; > 0: pages wholly behind the window are given back


@dataclass(frozen=True)
class StateCacheRequest:
    """A fixed-size state per running request: `shape` elements of `dtype` per slot."""

    shape: tuple
    dtype: torch.dtype = torch.float32


class Part:
    """Common behaviour: declare tensors, receive them."""

    # Whether a decode step through this part may be captured once and replayed as a graph: its
    # work is launches on the current stream whose shapes and order depend only on the shapes of
    # the step's tensors, with no copy to the host and no wait for the device.  A part says so
    # itself; one that does not is run step by step.
    capturable = False

    def __init__(self, spec: Any, env: "BuildEnv"):
        self.spec = spec
        self.env = env

    def weight_decls(self) -> dict:
        return {}

    def bind(self, tensors: dict) -> None:
        for name, t in tensors.items():
            setattr(self, name.replace(".", "_"), t)

    def streamed(self) -> list:
        """The `ops.Streamed` matrices this part owns (their copies in wave order are memory beside the
        checkpoint's tensors, which the model reports); none for most parts."""
        return []


@dataclass
class BuildEnv:
    """What every part may know about where it runs: never which model."""

    dtype: torch.dtype  # compute dtype: torch.bfloat16 or torch.float32
    device: torch.device
    # whether matrices that decode steps stream are kept a second time in the order their kernels read
    # them (faster steps for the weights' bytes again); a part asks `ops.Streamed(w, env.stream_copies)`
    stream_copies: bool = True
    # which of the library's kernels the model's matrix products run (`ops.ProductChoices`): the model's own
    # object, which its parts hand to `ops.gemm`; None: the one the process shares
    products: Any = None


class PendingNorm:
    """A norm of the fp32 stream `x` whose last step is still due: the part before has added its
    output into `x` and left what the norm's consumer needs to finish the norm inside its first
    matrix product (`gemm`, `gemm_gated`).  `rows()` runs the norm's own kernel on `x` for a
    consumer that wants the normalised rows themselves."""

    def __init__(self, norm: "Norm", x: torch.Tensor):
        self.norm = norm
        self.x = x

    def rows(self) -> torch.Tensor:
        return self.norm.forward(self.x)

    def gemm(self, w: torch.Tensor, out: torch.Tensor) -> None:
        """out = norm(x) @ w^T"""
        raise NotImplementedError

    def gemm_gated(self, w: torch.Tensor, out: torch.Tensor, activation: str) -> bool:
        """out = act(norm(x) @ w[:I]^T) * (norm(x) @ w[I:]^T) in one kernel, if there is one for this
        activation; else False and nothing done (the caller takes `rows()` and its own kernels)."""
        return False


class SplitSums:
    """The output of a part's last matrix product as fp32 partial sums [splits, T, hidden] over
    ranges of K, still to be added up and into the stream: a norm that says `takes_split_sums`
    does both in its own kernel."""

    def __init__(self, sums: torch.Tensor):
        self.sums = sums


class Mixer(Part):
    # Two optional shortcuts an arrangement may take with a part that declares them:
    # takes_pending_norm: `h` may arrive as a PendingNorm instead of normalised rows;
    # adds_to_residual: forward accepts `residual=` (the fp32 stream) and `next_norm=` (the norm
    #   that follows); where its last product can add into the stream and leave that norm
    #   pending (`Norm.absorb`), it returns the PendingNorm instead of its output; where that norm
    #   `takes_split_sums` it may return its output as `SplitSums`.
    takes_pending_norm = False
    adds_to_residual = False

    def cache_request(self) -> Optional[Any]:
        return None

    def row_split(self) -> Optional[tuple]:
        """(short, tile) if this mixer's kernels want the step's rows sorted: the tokens of rows with
        at most `short` tokens listed as single queries (`step.short_tokens`), longer rows cut into
        work items of up to `tile` consecutive tokens (`step.long_tiles`).  None: it reads rows as
        they come (`step.row_first`, `step.row_len`)."""
        return None

    def forward(self, h: torch.Tensor, step: Any, cache: Any) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    takes_pending_norm = False  # as for a Mixer
    adds_to_residual = False

    def forward(self, h: torch.Tensor, step: Any) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    takes_split_sums = False  # whether `forward` accepts a SplitSums as `delta`

    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        raise NotImplementedError

    def absorb(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor) -> Optional[PendingNorm]:
        """x += a @ w^T (rounded as the product alone would be) with this norm of the sum left
        pending, in one kernel; None where there is no such kernel (then the caller computes the
        product and `forward` adds and normalises)."""
        return None


class Position(Part):
    # How a mixer is to apply what `prepare` returns.  "half": an fp32 table [T, R/2, 2] of (cos, sin) by which
    # the pairs (i, i + R/2) of a head's first R coordinates turn (scaled, partial or slowed rotations are
    # other tables of the same kind).  A part of another layout (neighbouring pairs, something added to the
    # scores) names it here, and a mixer whose kernels do not compute that layout refuses the part.
    pairs: Optional[str] = None

    def prepare(self, step: Any) -> Any:
        raise NotImplementedError


class Arrangement:
    """Runs one layer over the residual stream `x` (fp32, updated in place) and the
    not-yet-added output `delta` of the layer before (or the PendingNorm that layer left for
    this one's `first_norm`); returns the new pending delta (or PendingNorm of `next_norm`)."""

    def __init__(self, spec: Any, env: BuildEnv):
        self.spec = spec
        self.env = env

    def parts(self) -> dict:
        raise NotImplementedError

    @property
    def capturable(self) -> bool:
        """Every part of the layer is (see Part.capturable)."""
        return all(part.capturable for part in self.parts().values())

    def first_norm(self) -> Optional["Norm"]:
        """The norm this layer applies to the stream first, for the layer before to leave pending."""
        return None

    def forward(self, x, delta, step, cache, next_norm=None):
        raise NotImplementedError


# ---- registries --------------------------------------------------------------------

_REGISTRIES: dict = {"norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "arrangement": {}}


def register(family: str, kind: str, builder: Callable, replace: bool = False) -> None:
    """Make `builder(spec, env)` the part for specs of this `kind`."""
    table = _REGISTRIES[family]
    if kind in table and not replace:
        raise ValueError(f"{family} kind {kind!r} is already registered")
    table[kind] = builder


def build(family: str, spec: Any, env: BuildEnv):
    _load_builtin()
    kind = spec.arrangement if family == "arrangement" else spec.kind
    table = _REGISTRIES[family]
    if kind not in table:
        raise ValueError(f"no {family} part of kind {kind!r}; registered: {sorted(table)}")
    return table[kind](spec, env)


def _load_builtin() -> None:
    from atomserve_amd.parts import attention, block, mlp, norm, rope  # noqa: F401
