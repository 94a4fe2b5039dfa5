"""Weights from safetensors, by tensor name (reference atomserve/loader.py:63-148).

The architecture says how each tensor of the plan is made of checkpoint tensors: a name,
names stacked along the rows (q, k, v into one projection, gate and up into one), rows cut
out of a fused tensor, a transposed matrix, or matrices stacked along a new axis (`Take`,
`Stack`); the parts say what shape and role each plan tensor has.  Everything that is wrong with a checkpoint is collected
and reported in one error: missing tensors, unexpected ones, wrong shapes.

Storage: matrices in the compute dtype (bfloat16 when serving); vectors such as norm
gains keep 32-bit storage when the checkpoint stores them so; integer tables int32.
"""

import glob
import json
import os
from contextlib import ExitStack
from dataclasses import dataclass
from typing import Optional

import torch

_SAFETENSORS_DTYPES = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
                       "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
                       "U8": torch.uint8, "BOOL": torch.bool}  # fmt: skip


@dataclass(frozen=True)
class Take:
    """One checkpoint tensor, or a piece of it, as a part of a plan tensor.

    transpose: a matrix stored [in, out] is turned to this package's [out, in] first.
    rows: (start, stop) keeps these rows only (after the transposition), for a checkpoint that
    stores several plan tensors fused in one."""

    name: str
    transpose: bool = False
    rows: Optional[tuple] = None

    def shape_from(self, stored: tuple) -> tuple:
        shape = tuple(stored)
        if self.transpose:
            if len(shape) != 2:
                raise ValueError(f"{self.name}: only a matrix can be transposed, this has shape {shape}")
            shape = shape[::-1]
        if self.rows is not None:
            start, stop = self.rows
            if not 0 <= start < stop <= shape[0]:
                raise ValueError(f"{self.name}: rows {start}:{stop} lie outside its {shape[0]} rows")
            shape = (stop - start, *shape[1:])
        return shape

    def apply(self, tensor):
        if self.transpose:
            tensor = tensor.t()
        if self.rows is not None:
            tensor = tensor[self.rows[0] : self.rows[1]]
        return tensor


@dataclass(frozen=True)
class Stack:
    """Several pieces as one plan tensor: laid one after the other along the rows (q, k and v
    into one projection), or with `new_axis` as the slices of a new first axis (one matrix per
    expert into [experts, out, in])."""

    parts: tuple
    new_axis: bool = False


def as_stack(entry) -> Stack:
    """A checkpoint map's entry in its general form.  An entry may be a checkpoint name, a `Take`,
    a list of either (stacked along the rows), or a `Stack`."""
    if isinstance(entry, Stack):
        parts, new_axis = entry.parts, entry.new_axis
    elif isinstance(entry, (str, Take)):
        parts, new_axis = (entry,), False
    else:
        parts, new_axis = tuple(entry), False
    return Stack(tuple(Take(p) if isinstance(p, str) else p for p in parts), new_axis)


class WeightsError(ValueError):
    """The checkpoint does not fit the model; lists every problem found."""

    def __init__(self, missing, unexpected, wrong_shapes, where=""):
        self.missing, self.unexpected, self.wrong_shapes = list(missing), list(unexpected), list(wrong_shapes)
        lines = [f"checkpoint {where} does not fit the model:".replace("  ", " ")]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shapes:
            lines.append(f"  wrong shape: {name} is {tuple(got)}, expected {tuple(want)}")
        super().__init__("\n".join(lines))


class DictSource:
    """Checkpoint tensors held in memory (random weights, tests)."""

    def __init__(self, tensors: dict):
        self.tensors = tensors

    def names(self):
        return list(self.tensors)

    def shape(self, name):
        return tuple(self.tensors[name].shape)

    def dtype(self, name):
        return self.tensors[name].dtype

    def get(self, name):
        return self.tensors[name]


def missing_shards(model_dir: str) -> list:
    """The weight files that a folder's index (model.safetensors.index.json, if it has one) names and the
    folder does not hold: a partly copied or partly downloaded checkpoint is reported by its files, before
    any tensor is looked for (reference atomserve/loader.py:28-40)."""
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if not os.path.isfile(index):
        return []
    with open(index) as f:
        named = set(json.load(f).get("weight_map", {}).values())
    return sorted(name for name in named if not os.path.isfile(os.path.join(model_dir, name)))


class SafetensorsSource:
    """Every *.safetensors file of a folder, memory-mapped; tensors are read one at a time."""

    def __init__(self, model_dir: str, stack: ExitStack):
        from safetensors import safe_open

        absent = missing_shards(model_dir)
        if absent:
            raise FileNotFoundError(f"{model_dir} lacks {', '.join(absent)}, which its model.safetensors.index.json names")
        shards = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
        if not shards:
            raise FileNotFoundError(f"no *.safetensors files in {model_dir}")
        self.where = {}
        for path in shards:
            f = stack.enter_context(safe_open(path, framework="pt", device="cpu"))
            for name in f.keys():  # noqa: SIM118
                self.where[name] = f

    def names(self):
        return list(self.where)

    def shape(self, name):
        return tuple(self.where[name].get_slice(name).get_shape())

    def dtype(self, name):
        return _SAFETENSORS_DTYPES.get(self.where[name].get_slice(name).get_dtype(), torch.float32)

    def get(self, name):
        return self.where[name].get_tensor(name)


def _storage_dtype(role: str, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if role == "table_int":
        return torch.int32
    if role == "vector" and stored in (torch.float32, torch.float64):
        return torch.float32
    return compute


def bind_checkpoint(model, arch, config, source, where: str = "") -> dict:
    """Check `source` against the model, then stack, convert, move and bind its tensors.
    Returns {plan tensor name: tensor}."""
    decls = model.weight_decls()
    mapping = arch.checkpoint_map(config)
    expected_shapes = arch.checkpoint_shapes(config)
    undeclared = sorted(set(decls) - set(mapping))
    if undeclared:
        raise KeyError(f"architecture {arch.name} maps no checkpoint tensors to {undeclared}")
    present = set(source.names())
    used, missing, wrong = set(), [], []
    recipes = {target: as_stack(mapping[target]) for target in decls}
    for target, decl in decls.items():
        takes = recipes[target].parts
        names = [t.name for t in takes]
        used.update(names)
        absent = [n for n in names if n not in present]
        missing.extend(absent)
        bad = False
        for n in names:
            if n in present and n in expected_shapes and source.shape(n) != tuple(expected_shapes[n][0]):
                if not any(w[0] == n for w in wrong):
                    wrong.append((n, source.shape(n), expected_shapes[n][0]))
                bad = True
        if absent or bad:
            continue
        shapes = [t.shape_from(source.shape(t.name)) for t in takes]
        label = "+".join(dict.fromkeys(names))
        if recipes[target].new_axis:
            made = (len(shapes), *shapes[0])
            alike = all(sh == shapes[0] for sh in shapes)
        else:
            made = (sum(sh[0] for sh in shapes), *shapes[0][1:])
            alike = all(sh[1:] == shapes[0][1:] for sh in shapes)
        if not alike or made != tuple(decl.shape):
            wrong.append((label, made, decl.shape))
    unexpected = sorted(present - used - set(arch.ignored(config)))
    if missing or unexpected or wrong:
        raise WeightsError(sorted(set(missing)), unexpected, wrong, where)

    env = model.env
    tensors = {}
    for target, decl in decls.items():
        recipe = recipes[target]
        stored = source.dtype(recipe.parts[0].name)
        dtype = _storage_dtype(decl.role, stored, env.dtype)
        pieces = [t.apply(source.get(t.name)).to(device=env.device, dtype=dtype) for t in recipe.parts]
        if recipe.new_axis:
            made = torch.stack(pieces, dim=0)
        else:
            made = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=0)
        tensors[target] = made.contiguous()
    model.bind(tensors)
    return tensors


def load_weights(model_dir: str, model, arch, config) -> dict:
    """Read `<model_dir>/*.safetensors` into `model` (already built for a dtype and device)."""
    with ExitStack() as stack:
        return bind_checkpoint(model, arch, config, SafetensorsSource(model_dir, stack), where=f"in {model_dir}")


def load_model(model_dir: str, dtype: torch.dtype, device, stream_copies: bool = True):
    """config.json -> architecture -> plan -> model with its weights: (model, arch, config)."""
    from atomserve_amd.config.registry import load_model_config
    from atomserve_amd.models.decoder import DecoderModel

    arch, config = load_model_config(model_dir)
    model = DecoderModel(arch.build_plan(config), dtype, device, stream_copies=stream_copies)
    load_weights(model_dir, model, arch, config)
    return model, arch, config
