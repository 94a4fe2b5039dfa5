"""Random weights from a configuration and a seed, as a model folder or in memory.

One seeded generator draws every tensor in the order the architecture lists them:
matrices N(0, std), gains 1 + N(0, gain_std).  Values are drawn in fp32 and rounded
to the storage dtype, so a bfloat16 folder read back in float32 holds the same numbers.
"""

import json
import os

import torch


def random_checkpoint(arch, config, seed: int, dtype=torch.bfloat16, device="cpu", std: float = 0.02,
                      gain_std: float = 0.1) -> dict:  # fmt: skip
    """{checkpoint name: tensor} on `device`, drawn tensor by tensor."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name, (shape, role) in arch.checkpoint_shapes(config).items():
        t = torch.randn(tuple(shape), generator=gen, device=device, dtype=torch.float32)
        t = t.mul_(gain_std).add_(1.0) if role == "vector" else t.mul_(std)
        out[name] = t.to(dtype)
    return out


def write_random_model(path: str, config, seed: int, dtype=torch.bfloat16, std: float = 0.02,
                       gain_std: float = 0.1) -> str:  # fmt: skip
    """Write `path/config.json` and `path/model.safetensors` for a typed configuration."""
    from safetensors.torch import save_file

    from atomserve_amd.config.registry import architecture_for

    raw = config.to_dict()
    raw["torch_dtype"] = str(dtype).replace("torch.", "")  # what the file holds
    arch = architecture_for(raw)
    os.makedirs(path, exist_ok=True)
    tensors = random_checkpoint(arch, config, seed, dtype=dtype, std=std, gain_std=gain_std)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    return path
