"""Weights from safetensors, by tensor name (reference atomserve/loader.py:63-148).

The architecture says which checkpoint tensors make up each tensor of the plan (q, k,
v stacked into one projection, gate and up into one); the parts say what shape and
role each plan tensor has.  Everything that is wrong with a checkpoint is collected
and reported in one error: missing tensors, unexpected ones, wrong shapes.

Storage: matrices in the compute dtype (bfloat16 when serving); vectors such as norm
gains keep 32-bit storage when the checkpoint stores them so; integer tables int32.
"""

import glob
import os
from contextlib import ExitStack

import torch

_SAFETENSORS_DTYPES = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
                       "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
                       "U8": torch.uint8, "BOOL": torch.bool}  # fmt: skip


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


class SafetensorsSource:
    """Every *.safetensors file of a folder, memory-mapped; tensors are read one at a time."""

    def __init__(self, model_dir: str, stack: ExitStack):
        from safetensors import safe_open

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
    for target, decl in decls.items():
        sources = mapping[target]
        used.update(sources)
        absent = [n for n in sources if n not in present]
        missing.extend(absent)
        for n in sources:
            if n in present and n in expected_shapes and source.shape(n) != tuple(expected_shapes[n][0]):
                wrong.append((n, source.shape(n), expected_shapes[n][0]))
        if not absent and not any(w[0] in sources for w in wrong):
            shapes = [source.shape(n) for n in sources]
            stacked = (sum(s[0] for s in shapes), *shapes[0][1:])
            if any(s[1:] != shapes[0][1:] for s in shapes) or stacked != tuple(decl.shape):
                wrong.append(("+".join(sources), stacked, decl.shape))
    unexpected = sorted(present - used - set(arch.ignored(config)))
    if missing or unexpected or wrong:
        raise WeightsError(sorted(set(missing)), unexpected, wrong, where)

    env = model.env
    tensors = {}
    for target, decl in decls.items():
        sources = mapping[target]
        stored = source.dtype(sources[0])
        dtype = _storage_dtype(decl.role, stored, env.dtype)
        parts = [source.get(n).to(device=env.device, dtype=dtype) for n in sources]
        tensors[target] = (parts[0] if len(parts) == 1 else torch.cat(parts, dim=0)).contiguous()
    model.bind(tensors)
    return tensors


def load_weights(model_dir: str, model, arch, config) -> dict:
    """Read `<model_dir>/*.safetensors` into `model` (already built for a dtype and device)."""
    with ExitStack() as stack:
        return bind_checkpoint(model, arch, config, SafetensorsSource(model_dir, stack), where=f"in {model_dir}")


def load_model(model_dir: str, dtype: torch.dtype, device):
    """config.json -> architecture -> plan -> model with its weights: (model, arch, config)."""
    from atomserve_amd.config.registry import load_model_config
    from atomserve_amd.models.decoder import DecoderModel

    arch, config = load_model_config(model_dir)
    model = DecoderModel(arch.build_plan(config), dtype, device)
    load_weights(model_dir, model, arch, config)
    return model, arch, config
