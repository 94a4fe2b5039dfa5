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

    def __init__(self, spec: Any, env: "BuildEnv"):
        self.spec = spec
        self.env = env

    def weight_decls(self) -> dict:
        return {}

    def bind(self, tensors: dict) -> None:
        for name, t in tensors.items():
            setattr(self, name.replace(".", "_"), t)


@dataclass
class BuildEnv:
    """What every part may know about where it runs: never which model."""

    dtype: torch.dtype  # compute dtype: torch.bfloat16 or torch.float32
    device: torch.device


class Mixer(Part):
    def cache_request(self) -> Optional[Any]:
        return None

    def forward(self, h: torch.Tensor, step: Any, cache: Any) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, step: Any) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        raise NotImplementedError


class Position(Part):
    def prepare(self, step: Any) -> Any:
        raise NotImplementedError


class Arrangement:
    """Runs one layer over the residual stream `x` (fp32, updated in place) and the
    not-yet-added output `delta` of the layer before; returns the new pending delta."""

    def __init__(self, spec: Any, env: BuildEnv):
        self.spec = spec
        self.env = env

    def parts(self) -> dict:
        raise NotImplementedError

    def forward(self, x, delta, step, cache):
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
