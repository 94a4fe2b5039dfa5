"""The command-line surface (argument parsing only; no model is loaded;
reference tests/test_cli.py:9-51)."""

import pytest

from atomserve_amd import __version__
from atomserve_amd.engine.cli import build_parser, engine_config_for, main, parse_ids


def test_help_version_and_required_model(capsys):
    with pytest.raises(SystemExit) as exc:
        main(["--help"])
    assert exc.value.code == 0 and "usage: atomserve" in capsys.readouterr().out
    with pytest.raises(SystemExit) as exc:
        main(["--version"])
    assert exc.value.code == 0 and __version__ in capsys.readouterr().out
    with pytest.raises(SystemExit) as exc:
        build_parser().parse_args([])
    assert exc.value.code == 2
    assert build_parser().parse_args(["Qwen/Qwen3-0.6B"]).model == "Qwen/Qwen3-0.6B"


def test_reference_option_names_and_defaults():
    a = build_parser().parse_args(["m"])
    assert (a.dtype, a.kv_mem_gb, a.block_size, a.max_num_seqs, a.max_batched_tokens, a.no_prefix_caching) == (
        "bf16", 4.0, 16, 32, 512, False)  # fmt: skip
    assert (a.temperature, a.top_k, a.top_p) == (0.6, 20, 0.95)


def test_pool_is_sized_from_the_memory_budget():
    """4 GiB of bf16 cache at 1.75 MiB per 16-token block of Qwen3-0.6B is 2340 blocks."""
    block_bytes = 28 * 2 * 8 * 128 * 2 * 16
    cfg = engine_config_for(build_parser().parse_args(["m", "--kv-mem-gb", "4"]), block_bytes, 40960)
    assert cfg.num_blocks == 2340 and cfg.max_model_len == 2340 * 16
    small = engine_config_for(build_parser().parse_args(["m", "--kv-mem-gb", "1"]), block_bytes, 40960)
    assert small.max_model_len == small.num_blocks * 16 < 40960
    capped = engine_config_for(build_parser().parse_args(["m", "--kv-mem-gb", "64"]), block_bytes, 40960)
    assert capped.max_model_len == 40960


def test_bytes_per_block_of_a_model():
    import torch

    from atomserve_amd.cache import CachePools
    from atomserve_amd.parts.base import PagedCacheRequest

    requests = {i: PagedCacheRequest(8, 128) for i in range(28)}
    assert CachePools.bytes_per_block(requests, 16, torch.bfloat16) == 28 * 2 * 8 * 128 * 2 * 16


def test_prompt_ids_are_parsed():
    assert parse_ids("1, 2,3  4") == [1, 2, 3, 4]


def test_the_budget_is_fitted_to_what_the_gpu_has_left():
    """reference atomserve/cli.py:122-136: the budget shrinks to the room, with a note; no room is an error."""
    from atomserve_amd.engine.cli import fit_kv_budget, kv_budget

    gib = 2**30
    notes = []
    assert fit_kv_budget(4.0, 100 * gib, 2 * gib, notes.append) == 4.0 and not notes
    assert fit_kv_budget(4.0, 5 * gib, 2 * gib, notes.append) == 3.0 and "reduced from 4.0 to 3.0" in notes[0]
    assert fit_kv_budget("auto", 100 * gib, 2 * gib, notes.append) == 98.0 and len(notes) == 1
    with pytest.raises(SystemExit, match="no room for a KV cache"):
        fit_kv_budget(4.0, 2 * gib, 2 * gib, notes.append)
    assert kv_budget("auto") == "auto" and kv_budget("2.5") == 2.5
    assert build_parser().parse_args(["m", "--kv-mem-gb", "auto"]).kv_mem_gb == "auto"
    with pytest.raises(SystemExit):
        build_parser().parse_args(["m", "--kv-mem-gb", "-1"])


def test_the_reserve_of_a_step_grows_with_its_budget_and_the_vocabulary():
    from atomserve_amd.config.model_config import Qwen3Config
    from atomserve_amd.engine.cli import step_reserve_bytes
    from atomserve_amd.models.qwen3 import build_plan

    cfg = dict(vocab_size=151936, hidden_size=4096, intermediate_size=12288, num_layers=2, num_heads=32, num_kv_heads=8,
               head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False, max_position_embeddings=4096)  # fmt: skip
    plan = build_plan(Qwen3Config(**cfg))
    small, large = step_reserve_bytes(plan, 512, 32), step_reserve_bytes(plan, 8192, 32)
    assert 2**30 < small < large < 8 * 2**30
    assert step_reserve_bytes(build_plan(Qwen3Config(**{**cfg, "vocab_size": 1000})), 512, 32) < small


def test_limits_that_contradict_each_other_are_a_message():
    """A token budget smaller than the number of running requests (one decoded token each) or a pool of no
    pages ends with a message that names it, as an exit of the program, not as a traceback."""
    block_bytes = 28 * 2 * 8 * 128 * 2 * 16
    with pytest.raises(SystemExit, match="max_num_batched_tokens"):
        engine_config_for(build_parser().parse_args(["m", "--max-batched-tokens", "8", "--max-num-seqs", "16"]), block_bytes, 40960)
    with pytest.raises(SystemExit, match="positive"):
        engine_config_for(build_parser().parse_args(["m", "--block-size", "0"]), block_bytes, 40960)
    with pytest.raises(SystemExit, match="no room for a single KV block"):
        engine_config_for(build_parser().parse_args(["m", "--kv-mem-gb", "0.000001"]), block_bytes, 40960)
    # a --max-model-len above what pool and model allow is cut down to it, not an error
    cut = engine_config_for(build_parser().parse_args(["m", "--kv-mem-gb", "1", "--max-model-len", "1000000"]), block_bytes, 40960)
    assert cut.max_model_len == cut.num_blocks * 16
    assert build_parser().parse_args(["m", "--no-stream-copies"]).no_stream_copies is True
