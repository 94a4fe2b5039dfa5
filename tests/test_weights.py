"""Weights by tensor name, their storage, the one error that lists everything wrong, and
the random-weights folder (reference atomserve/loader.py:63-148)."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from atomserve_amd.config import Qwen3Config
from atomserve_amd.weights import WeightsError, load_model, write_random_model
from tests.conftest import TINY_A, TINY_B, plain_random_weights, write_model_dir


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_tensors_are_found_stacked_and_stored(raw, dtype, tmp_path):
    w = plain_random_weights(raw, seed=1)
    path = write_model_dir(str(tmp_path), raw, w, torch.bfloat16)
    model, arch, c = load_model(path, dtype, "cpu")
    t = model._tensors
    H, KV, D = c.num_heads, c.num_kv_heads, c.head_dim
    assert t["layers.1.mixer.qkv.weight"].shape == ((H + 2 * KV) * D, c.hidden_size)
    q, k, v = t["layers.1.mixer.qkv.weight"].split([H * D, KV * D, KV * D])
    assert torch.equal(q.float(), w["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(k.float(), w["model.layers.1.self_attn.k_proj.weight"])
    assert torch.equal(v.float(), w["model.layers.1.self_attn.v_proj.weight"])
    gate, up = t["layers.0.ffn.gate_up.weight"].chunk(2)
    assert torch.equal(gate.float(), w["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(up.float(), w["model.layers.0.mlp.up_proj.weight"])
    assert all(x.dtype == dtype for x in t.values())
    if c.tie_word_embeddings:
        assert model.head_weight is model.embed_weight and "head.weight" not in t
    else:
        assert torch.equal(model.head_weight.float(), w["lm_head.weight"])
    assert model.blocks[0].mixer.q_norm_weight.shape == (D,)


def test_gains_stored_in_32_bit_stay_so_and_matrices_follow_the_compute_dtype(tmp_path):
    w = plain_random_weights(TINY_A, seed=2)
    path = write_model_dir(str(tmp_path), TINY_A, w, torch.float32)
    model, _, _ = load_model(path, torch.bfloat16, "cpu")
    t = model._tensors
    assert t["layers.0.mixer_norm.weight"].dtype == torch.float32
    assert t["layers.0.mixer.q_norm.weight"].dtype == torch.float32
    assert t["final_norm.weight"].dtype == torch.float32
    assert t["layers.0.mixer.qkv.weight"].dtype == torch.bfloat16 and t["embed.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_misshapen_tensors(tmp_path):
    w = plain_random_weights(TINY_B, seed=3)
    del w["model.layers.2.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(192)
    w["extra.weight"] = torch.zeros(3)
    w["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(64, 95)
    w["model.layers.1.self_attn.q_norm.weight"] = torch.zeros(16)
    path = write_model_dir(str(tmp_path), TINY_B, w)
    with pytest.raises(WeightsError) as info:
        load_model(path, torch.float32, "cpu")
    e = info.value
    assert e.missing == ["model.layers.2.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["extra.weight", "model.layers.0.self_attn.q_proj.bias"]
    assert {name for name, _, _ in e.wrong_shapes} == {"model.layers.1.self_attn.k_proj.weight", "model.layers.1.self_attn.q_norm.weight"}
    text = str(e)
    for fragment in ("missing tensors (2)", "unexpected tensors (2)", "(64, 95)", "expected (64, 96)", "extra.weight"):
        assert fragment in text


def test_untied_model_needs_its_head_and_tied_model_ignores_a_shipped_one(tmp_path):
    w = plain_random_weights(TINY_B, seed=4)
    del w["lm_head.weight"]
    with pytest.raises(WeightsError, match="lm_head.weight"):
        load_model(write_model_dir(str(tmp_path / "b"), TINY_B, w), torch.float32, "cpu")
    wa = plain_random_weights(TINY_A, seed=4)
    wa["lm_head.weight"] = torch.ones(256, 64)  # a tied checkpoint may ship a copy; the configuration decides
    model, _, _ = load_model(write_model_dir(str(tmp_path / "a"), TINY_A, wa), torch.float32, "cpu")
    assert model.head_weight is model.embed_weight


def test_no_weight_files(tmp_path):
    import json

    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load_model(str(tmp_path), torch.float32, "cpu")


def test_random_weights_folder(tmp_path):
    c = Qwen3Config.from_dict(TINY_B)
    a = write_random_model(str(tmp_path / "a"), c, seed=5)
    b = write_random_model(str(tmp_path / "b"), c, seed=5)
    other = write_random_model(str(tmp_path / "c"), c, seed=6)
    ta, tb, tc = (load_file(os.path.join(p, "model.safetensors")) for p in (a, b, other))
    assert sorted(os.listdir(a)) == ["config.json", "model.safetensors"]
    assert all(torch.equal(ta[k], tb[k]) for k in ta) and any(not torch.equal(ta[k], tc[k]) for k in ta)
    assert all(v.dtype == torch.bfloat16 for v in ta.values())
    mat = ta["model.layers.0.mlp.gate_proj.weight"].float()
    gain = torch.cat([ta[f"model.layers.{i}.input_layernorm.weight"].float() for i in range(3)])
    assert abs(float(mat.std()) - 0.02) < 0.002 and abs(float(mat.mean())) < 0.002
    assert abs(float(gain.mean()) - 1.0) < 0.03 and abs(float(gain.std()) - 0.1) < 0.03
    model, _, c2 = load_model(a, torch.float32, "cpu")  # and it loads back as a model
    assert c2 == c and "lm_head.weight" in ta


def test_sharded_folder_is_read_across_files(tmp_path):
    w = plain_random_weights(TINY_A, seed=7)
    path = write_model_dir(str(tmp_path), TINY_A, w)
    os.remove(os.path.join(path, "model.safetensors"))
    names = sorted(w)
    save_file({k: w[k].bfloat16() for k in names[::2]}, os.path.join(path, "model-00001-of-00002.safetensors"))
    save_file({k: w[k].bfloat16() for k in names[1::2]}, os.path.join(path, "model-00002-of-00002.safetensors"))
    model, _, _ = load_model(path, torch.float32, "cpu")
    assert torch.equal(model.embed_weight, w["model.embed_tokens.weight"])
    # a folder whose index names a file that is not there says which file (reference atomserve/loader.py:28-40,
    # tests/test_cli.py:54-75), not which tensors
    shards = {k: f"model-0000{1 + i % 2}-of-00002.safetensors" for i, k in enumerate(names)}
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": shards}, f)
    load_model(path, torch.float32, "cpu")
    os.remove(os.path.join(path, "model-00002-of-00002.safetensors"))
    with pytest.raises(FileNotFoundError, match="lacks model-00002-of-00002.safetensors"):
        load_model(path, torch.float32, "cpu")


def test_a_checkpoint_of_another_layout_is_a_matter_of_the_map_alone():
    """The same model from a checkpoint that fuses q, k and v in one tensor, stores gate and up fused
    in the other order, keeps the output projection transposed ([in, out]) and, for a part with
    experts, one matrix per expert: the architecture's map names slices, a transposition and a stack
    along a new axis; the loader itself does not change."""
    import dataclasses

    from atomserve_amd.config.registry import Architecture, architecture_for
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights import Stack, Take
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint

    raw = dict(TINY_B, num_hidden_layers=1)
    qwen = architecture_for(raw)
    c = qwen.parse_config(raw)
    w = plain_random_weights(raw, seed=3)
    p, inter = "model.layers.0.", c.intermediate_size
    other = {k: v for k, v in w.items() if "_proj" not in k}
    other[p + "attn.c_attn"] = torch.cat([w[p + f"self_attn.{x}_proj.weight"] for x in "qkv"])
    other[p + "attn.c_proj"] = w[p + "self_attn.o_proj.weight"].t().contiguous()
    other[p + "mlp.up_gate"] = torch.cat([w[p + "mlp.up_proj.weight"], w[p + "mlp.gate_proj.weight"]])
    other[p + "mlp.down_proj.weight"] = w[p + "mlp.down_proj.weight"]

    def checkpoint_map(cfg):
        names = qwen.checkpoint_map(cfg)
        names["layers.0.mixer.qkv.weight"] = p + "attn.c_attn"
        names["layers.0.mixer.o.weight"] = Take(p + "attn.c_proj", transpose=True)
        names["layers.0.ffn.gate_up.weight"] = [Take(p + "mlp.up_gate", rows=(inter, 2 * inter)),
                                                Take(p + "mlp.up_gate", rows=(0, inter))]  # fmt: skip
        return names

    arch = Architecture("Other", qwen.parse_config, qwen.build_plan, checkpoint_map, lambda cfg: {})
    model = DecoderModel(arch.build_plan(c), torch.float32, "cpu")
    bind_checkpoint(model, arch, c, DictSource(other))
    reference = DecoderModel(qwen.build_plan(c), torch.float32, "cpu")
    bind_checkpoint(reference, qwen, c, DictSource(w))
    assert model._tensors.keys() == reference._tensors.keys()
    for name, t in reference._tensors.items():
        assert torch.equal(model._tensors[name], t), name

    # a transposed tensor of the wrong size and a slice beyond the tensor are named in the one error
    broken = dict(other)
    broken[p + "attn.c_proj"] = torch.zeros(5, 7)
    with pytest.raises(WeightsError, match="attn.c_proj is \\(7, 5\\), expected"):
        bind_checkpoint(DecoderModel(arch.build_plan(c), torch.float32, "cpu"), arch, c, DictSource(broken))

    # matrices of three experts stacked along a new first axis
    class Experts:
        env = model.env

        def weight_decls(self):
            from atomserve_amd.parts.base import WeightDecl

            return {"experts.weight": WeightDecl((3, 4, 6))}

        def bind(self, tensors):
            self.tensors = tensors

    mats = {f"expert.{i}.w": torch.randn(4, 6) for i in range(3)}
    toy = dataclasses.replace(arch, checkpoint_map=lambda cfg: {"experts.weight": Stack(tuple(mats), new_axis=True)})
    holder = Experts()
    bind_checkpoint(holder, toy, c, DictSource(mats))
    assert torch.equal(holder.tensors["experts.weight"], torch.stack(list(mats.values())))
