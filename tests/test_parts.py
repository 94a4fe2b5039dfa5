"""What the parts refuse at build time, without a GPU: a plan that names a per-head norm or a position
encoding that the attention kernels do not compute is an error that names it, never a wrong rotation."""

import dataclasses

import pytest
import torch

from atomserve_amd.config.registry import architecture_for
from atomserve_amd.parts.base import BuildEnv, Position, build, register
from atomserve_amd.parts.plan import NormSpec
from tests.conftest import TINY_A, TINY_B

ENV = BuildEnv(dtype=torch.float32, device=torch.device("cpu"))


def attention_spec(raw=TINY_B):
    arch = architecture_for(raw)
    return arch.build_plan(arch.parse_config(raw)).layers[0].mixer


def test_attention_builds_from_the_architectures_own_spec():
    spec = attention_spec()
    mixer = build("mixer", spec, ENV)
    assert mixer.position.pairs == "half" and mixer.row_split() == (8, 64)
    assert spec.qk_norm.kind == "rmsnorm" and spec.qk_norm.size == spec.head_dim


def test_attention_refuses_a_per_head_norm_it_does_not_compute():
    spec = attention_spec()
    other = dataclasses.replace(spec, qk_norm=NormSpec("layernorm", spec.head_dim, 1e-5))
    with pytest.raises(ValueError, match="layernorm"):
        build("mixer", other, ENV)
    with pytest.raises(ValueError, match="gains"):
        build("mixer", dataclasses.replace(spec, qk_norm=NormSpec("rmsnorm", spec.head_dim // 2, 1e-5)), ENV)
    assert build("mixer", dataclasses.replace(spec, qk_norm=None), ENV).q_norm_weight is None  # none at all is fine


def test_attention_refuses_a_position_part_of_another_layout():
    @dataclasses.dataclass(frozen=True)
    class NeighbourSpec:
        kind: str
        rotary_dim: int
        theta: float

    class NeighbourPairs(Position):
        """Turns the pairs (2i, 2i + 1): a table of the same shape that means something else."""

        pairs = "neighbours"

        def prepare(self, step):
            raise AssertionError("never asked: the mixer refuses the part when it is built")

    class Undeclared(Position):
        def prepare(self, step):
            raise AssertionError("never asked")

    register("position", "toy_neighbours", NeighbourPairs, replace=True)
    register("position", "toy_undeclared", Undeclared, replace=True)
    spec = attention_spec(TINY_A)
    for kind, named in (("toy_neighbours", "neighbours"), ("toy_undeclared", "None")):
        with pytest.raises(ValueError, match=named):
            build("mixer", dataclasses.replace(spec, position=NeighbourSpec(kind, spec.head_dim, 1e4)), ENV)
    assert build("mixer", dataclasses.replace(spec, position=None), ENV).position is None  # no rotation at all is fine
