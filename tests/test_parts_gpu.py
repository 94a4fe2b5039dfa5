"""Parts alone and composed: each part of a layer against its plain reference, and models
that are not Qwen3, registered from here without a change to the package: a mixer with a
fixed-size state of its own in some layers, a feed-forward that routes each token to one of
several experts, a position encoding that turns half of each head by slowed positions, a layer
that runs twice, a run that reads the cache another run wrote, a mixer that keeps nothing and sorts
a step's rows its own way, another norm and another arrangement of a layer."""

import dataclasses
import math

import pytest
import torch

from tests import plain_kernels as pk
from tests import plain_qwen3 as plain
from tests.conftest import TINY_A, TINY_B, plain_random_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ---- a toy mixer, defined here ----------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class DecaySpec:
    kind: str
    hidden_size: int
    decay: float


def make_decay_mixer():
    from atomserve_amd.parts.base import Mixer, StateCacheRequest, WeightDecl

    class DecayMixer(Mixer):
        """y_t = gain * s_t with s_t = decay * s_{t-1} + h_t: a running sum kept per request in a
        fixed-size state slot, so a prompt cut anywhere continues where it stopped."""

        def weight_decls(self):
            return {"gain": WeightDecl((self.spec.hidden_size,), role="vector")}

        def cache_request(self):
            return StateCacheRequest((self.spec.hidden_size,), torch.float32)

        def forward(self, h, step, cache):
            out = torch.empty_like(h)
            flat = 0
            for row in step.host_rows:
                n = len(row.tokens)
                s = cache.state[row.state_slot]
                if row.start == 0:
                    s.zero_()
                for t in range(flat, flat + n):
                    s.mul_(self.spec.decay).add_(h[t].float())
                    out[t] = (s * self.gain.float()).to(h.dtype)
                flat += n
            return out

    return DecayMixer


def register_toy_architecture():
    """Qwen3's layers with the mixer of every odd layer replaced by the decay mixer."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture
    from atomserve_amd.parts.base import register

    register("mixer", "toy_decay", make_decay_mixer(), replace=True)
    qwen = architecture_for(TINY_A)

    def build_plan(c):
        plan = qwen.build_plan(c)
        layers = tuple(
            dataclasses.replace(layer, mixer=DecaySpec("toy_decay", c.hidden_size, 0.5 + 0.1 * i)) if i % 2 else layer
            for i, layer in enumerate(plan.layers)
        )
        return dataclasses.replace(plan, layers=layers)

    def checkpoint_map(c):
        names = {k: v for k, v in qwen.checkpoint_map(c).items()
                 if not any(k.startswith(f"layers.{i}.mixer.") for i in range(1, c.num_layers, 2))}  # fmt: skip
        for i in range(1, c.num_layers, 2):
            names[f"layers.{i}.mixer.gain"] = [f"model.layers.{i}.decay.gain"]
        return names

    def checkpoint_shapes(c):
        shapes = {k: v for k, v in qwen.checkpoint_shapes(c).items()
                  if not any(k.startswith(f"model.layers.{i}.self_attn.") for i in range(1, c.num_layers, 2))}  # fmt: skip
        for i in range(1, c.num_layers, 2):
            shapes[f"model.layers.{i}.decay.gain"] = ((c.hidden_size,), "vector")
        return shapes

    return register_architecture(
        Architecture("ToyDecayForCausalLM", qwen.parse_config, build_plan, checkpoint_map, checkpoint_shapes), replace=True
    )


def plain_toy_logits(raw, w, ids):
    """The toy model, whole sequence, no cache, from the plain functions."""
    cfg = plain.normalise_config(raw)
    wd = {k: v.double() for k, v in w.items()}
    ids = torch.as_tensor(ids)
    pos = torch.arange(len(ids))
    x = plain.embed(wd["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = plain.rms_norm(x, wd[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
        if i % 2:
            s, ys = torch.zeros_like(h[0]), []
            for t in range(len(ids)):
                s = (0.5 + 0.1 * i) * s + h[t]
                ys.append(s * wd[p + "decay.gain"])
            x = x + torch.stack(ys)
        else:
            x = x + plain.attention_layer(h, wd, p, cfg, pos)
        h = plain.rms_norm(x, wd[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
    x = plain.rms_norm(x, wd["model.norm.weight"], cfg["rms_norm_eps"])
    head = "model.embed_tokens.weight" if cfg["tie_word_embeddings"] else "lm_head.weight"
    return (x @ wd[head].T).float()


def build_engine(arch, raw, weights, dtype, device=DEV, **engine):
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint

    config = arch.parse_config(raw)
    model = DecoderModel(arch.build_plan(config), dtype, device)
    bind_checkpoint(model, arch, config, DictSource(weights))
    cfg = {"block_size": 16, "num_blocks": 32, "max_model_len": 256, "max_num_seqs": 4, "max_num_batched_tokens": 64, **engine}
    return create_engine(model, EngineConfig(**cfg))


def step_rows(engine, caches, entries):
    """entries: (name, tokens, want) -> logits; requests keep their pages and slots in `caches`;
    after the step, pages that a window has passed are given back."""
    from atomserve_amd.engine.batch import Row

    m = engine.scheduler.manager
    rows = []
    for name, tokens, want in entries:
        rc, done = caches.setdefault(name, [m.new_request(), 0])
        assert m.reserve(rc, done, len(tokens))
        rows.append(Row(tokens, done, rc.tables, want, rc.state_slot))
        caches[name][1] += len(tokens)
    logits = engine.runner.step(rows).float().cpu()
    for name, _, _ in entries:
        m.release_behind_window(*caches[name])
    return logits


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_mixer_with_state_of_its_own(dtype, device=DEV):
    arch = register_toy_architecture()
    raw = {**TINY_B, "architectures": ["ToyDecayForCausalLM"], "num_hidden_layers": 4}
    w = plain_random_weights(raw, seed=5, std=0.2, gain_std=0.2)
    for i in (1, 3):
        for k in [k for k in w if k.startswith(f"model.layers.{i}.self_attn.")]:
            del w[k]
        w[f"model.layers.{i}.decay.gain"] = (1 + 0.2 * torch.randn(raw["hidden_size"])).bfloat16().float()
    engine = build_engine(arch, raw, w, dtype, device)
    manager = engine.scheduler.manager
    assert len(manager.state_groups) == 1 and len(manager.paged_groups) == 1 and not manager.prefix_reuse_possible
    assert manager.paged_groups[0].cache_ids == [0, 2] and manager.state_groups[0].cache_ids == [1, 3]
    a = torch.randint(0, 1000, (45,), generator=torch.Generator().manual_seed(1)).tolist()
    b = torch.randint(0, 1000, (23,), generator=torch.Generator().manual_seed(2)).tolist()
    ref_a, ref_b = plain_toy_logits(raw, w, a), plain_toy_logits(raw, w, b)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    caches = {}
    whole = step_rows(engine, caches, [("a", a, list(range(45)))])
    assert (whole - ref_a).abs().max() <= tol * max(1.0, ref_a.abs().max())
    # the same request cut anywhere, beside another one: the state carries over between steps
    caches2 = {}
    got_a, got_b = [], []
    got = step_rows(engine, caches2, [("a2", a[:10], list(range(10))), ("b", b[:2], [0, 1])])
    got_a.append(got[:10]); got_b.append(got[10:])  # noqa: E702
    got = step_rows(engine, caches2, [("b", b[2:20], list(range(18))), ("a2", a[10:11], [0])])
    got_b.append(got[:18]); got_a.append(got[18:])  # noqa: E702
    got = step_rows(engine, caches2, [("a2", a[11:45], list(range(34))), ("b", b[20:], [0, 1, 2])])
    got_a.append(got[:34]); got_b.append(got[34:])  # noqa: E702
    assert (torch.cat(got_a) - ref_a).abs().max() <= tol * max(1.0, ref_a.abs().max())
    assert (torch.cat(got_b) - ref_b).abs().max() <= tol * max(1.0, ref_b.abs().max())
    for rc, _ in list(caches.values()) + list(caches2.values()):
        manager.release(rc)
    assert manager.num_free == manager.num_blocks and manager.num_free_slots == 4
    # and through the scheduler: greedy generation equals the plain model's
    from atomserve_amd.engine.sequence import SamplingParams

    if dtype == torch.float32:
        outs = engine.generate([a[:7], b[:12]], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
        for prompt, out in zip((a[:7], b[:12]), outs):
            seq = list(prompt)
            for t in out:
                assert t == int(plain_toy_logits(raw, w, seq)[-1].argmax())
                seq.append(t)


def plain_looped_logits(raw, w, ids):
    """Run list [0, 1, 1 again reading the cache of its first run]: the second run of layer 1
    takes its queries from the current hidden state and its keys and values from the first run."""
    cfg = plain.normalise_config(raw)
    wd = {k: v.double() for k, v in w.items()}
    ids = torch.as_tensor(ids)
    pos = torch.arange(len(ids))
    T, H, KV, D = len(ids), cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    x = plain.embed(wd["model.embed_tokens.weight"], ids)
    kept = None
    for layer, reuse in ((0, False), (1, False), (1, True)):
        p = f"model.layers.{layer}."
        h = plain.rms_norm(x, wd[p + "input_layernorm.weight"], eps)
        q = plain.rope(plain.rms_norm((h @ wd[p + "self_attn.q_proj.weight"].T).view(T, H, D), wd[p + "self_attn.q_norm.weight"], eps), pos, theta)
        if reuse:
            k, v = kept
        else:
            k = plain.rope(plain.rms_norm((h @ wd[p + "self_attn.k_proj.weight"].T).view(T, KV, D), wd[p + "self_attn.k_norm.weight"], eps), pos, theta)
            v = (h @ wd[p + "self_attn.v_proj.weight"].T).view(T, KV, D)
            kept = (k, v)
        o = plain.causal_attention(q, k, v, pos)
        x = x + o.reshape(T, H * D) @ wd[p + "self_attn.o_proj.weight"].T
        h = plain.rms_norm(x, wd[p + "post_attention_layernorm.weight"], eps)
        x = x + plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
    x = plain.rms_norm(x, wd["model.norm.weight"], eps)
    return (x @ wd["model.embed_tokens.weight"].T).float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_layer_runs_twice_and_reads_the_cache_of_its_first_run(dtype, device=DEV):
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture
    from atomserve_amd.parts.plan import Run

    qwen = architecture_for(TINY_A)

    def build_plan(c):
        return dataclasses.replace(qwen.build_plan(c), run=(Run(0), Run(1), Run(1, cache=1, writes=False)))

    arch = register_architecture(
        Architecture("LoopedForCausalLM", qwen.parse_config, build_plan, qwen.checkpoint_map, qwen.checkpoint_shapes), replace=True
    )
    raw = {**TINY_A, "architectures": ["LoopedForCausalLM"]}
    w = plain_random_weights(raw, seed=6, std=0.2, gain_std=0.2)
    engine = build_engine(arch, raw, w, dtype, device)
    assert engine.scheduler.manager.paged_groups[0].cache_ids == [0, 1]  # three runs, two caches
    ids = torch.randint(0, 256, (40,), generator=torch.Generator().manual_seed(3)).tolist()
    ref = plain_looped_logits(raw, w, ids)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    caches = {}
    got = [step_rows(engine, caches, [("a", ids[:21], list(range(21)))])]
    got += [step_rows(engine, caches, [("a", [ids[i]], [0])]) for i in range(21, 30)]
    got.append(step_rows(engine, caches, [("a", ids[30:], list(range(10)))]))
    assert (torch.cat(got) - ref).abs().max() <= tol * max(1.0, ref.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layers_with_a_window_have_pages_of_their_own_and_give_them_back(dtype, device=DEV):
    """Odd layers see the last 24 keys only: two cache groups, each with its pool and tables.
    The windowed group's pool is smaller than one request's length, so it only works because
    pages behind the window return to the pool and are handed out again, to the same and to
    the other request; what they held before must never show."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture

    qwen = architecture_for(TINY_B)
    window = 24

    def build_plan(c):
        plan = qwen.build_plan(c)
        layers = tuple(dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, window=window)) if i % 2 else layer
                       for i, layer in enumerate(plan.layers))  # fmt: skip
        return dataclasses.replace(plan, layers=layers)

    arch = register_architecture(
        Architecture("WindowedForCausalLM", qwen.parse_config, build_plan, qwen.checkpoint_map, qwen.checkpoint_shapes), replace=True
    )
    raw = {**TINY_B, "architectures": ["WindowedForCausalLM"], "num_hidden_layers": 4}
    w = plain_random_weights(raw, seed=8, std=0.2, gain_std=0.2)
    engine = build_engine(arch, raw, w, dtype, device, num_blocks=24, max_model_len=384)
    m = engine.scheduler.manager
    assert [(g.window, g.cache_ids) for g in m.paged_groups] == [(0, [0, 2]), (window, [1, 3])]
    a = torch.randint(0, 1000, (170,), generator=torch.Generator().manual_seed(4)).tolist()
    b = torch.randint(0, 1000, (150,), generator=torch.Generator().manual_seed(5)).tolist()

    def reference(ids):
        cfg = plain.normalise_config(raw)
        wd = {k: v.double() for k, v in w.items()}
        pos = torch.arange(len(ids))
        x = plain.embed(wd["model.embed_tokens.weight"], torch.as_tensor(ids))
        for i in range(4):
            p = f"model.layers.{i}."
            h = plain.rms_norm(x, wd[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
            x = x + plain.attention_layer(h, wd, p, {**cfg, "window": window if i % 2 else 0}, pos)
            h = plain.rms_norm(x, wd[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
            x = x + plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
        x = plain.rms_norm(x, wd["model.norm.weight"], cfg["rms_norm_eps"])
        return (x @ wd["lm_head.weight"].T).float()

    ref = {"a": reference(a), "b": reference(b)}
    caches, got, at = {}, {"a": [], "b": []}, {"a": 0, "b": 0}
    held_most = 0
    plan = [("a", 50), ("b", 3), ("a", 1), ("b", 70), ("a", 1), ("a", 30), ("b", 1), ("a", 2), ("b", 40), ("a", 66), ("b", 36), ("a", 20)]
    ids = {"a": a, "b": b}
    i = 0
    while i < len(plan):
        entries = []
        for name, n in plan[i : i + 2] if plan[i][0] != plan[min(i + 1, len(plan) - 1)][0] else plan[i : i + 1]:
            entries.append((name, ids[name][at[name] : at[name] + n], list(range(n))))
            at[name] += n
        i += len(entries)
        logits = step_rows(engine, caches, entries)
        k = 0
        for name, tokens, _ in entries:
            got[name].append(logits[k : k + len(tokens)])
            k += len(tokens)
        windowed = m.paged_groups[1].allocator
        held_most = max(held_most, windowed.num_pages - windowed.num_free)
    assert at == {"a": 170, "b": 150}
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for name in "ab":
        assert (torch.cat(got[name]) - ref[name]).abs().max() <= tol * max(1.0, ref[name].abs().max()), name
    # 320 tokens went through the windowed layers on at most a handful of pages at a time
    assert held_most <= 2 * (-(-(window + 70) // 16) + 1)
    assert sum(1 for p in caches["a"][0].tables[1] if p == -1) >= 8  # given back as the window moved on
    for rc, _ in caches.values():
        m.release(rc)
    assert all(g.allocator.num_free == 24 for g in m.paged_groups)


# ---- a toy feed-forward with routing and a toy position encoding, defined here ---------------


@dataclasses.dataclass(frozen=True)
class RoutedSpec:
    kind: str
    hidden_size: int
    intermediate_size: int
    num_experts: int


@dataclasses.dataclass(frozen=True)
class SlowedRotarySpec:
    kind: str
    rotary_dim: int  # the first coordinates of a head that turn; the rest stay
    theta: float
    slowdown: float  # positions are divided by this before the angles are formed


def make_routed_feed_forward():
    from atomserve_amd.parts.base import FeedForward, WeightDecl

    class RoutedFeedForward(FeedForward):
        """Each token goes to the one expert with the largest router logit (32-bit) and comes back
        scaled by that expert's softmax weight: y = p_e * relu(h up_e^T) down_e^T."""

        def weight_decls(self):
            s = self.spec
            return {
                "router": WeightDecl((s.num_experts, s.hidden_size)),
                "up": WeightDecl((s.num_experts * s.intermediate_size, s.hidden_size)),
                "down": WeightDecl((s.num_experts * s.hidden_size, s.intermediate_size)),
            }

        def forward(self, h, step):
            s = self.spec
            probs = torch.softmax(h.float() @ self.router.float().T, dim=-1)
            weight, expert = probs.max(dim=-1)
            out = torch.zeros_like(h)
            up = self.up.view(s.num_experts, s.intermediate_size, s.hidden_size)
            down = self.down.view(s.num_experts, s.hidden_size, s.intermediate_size)
            for e in range(s.num_experts):
                rows = (expert == e).nonzero().flatten()
                if len(rows):
                    y = torch.relu(h[rows] @ up[e].T) @ down[e].T
                    out[rows] = (weight[rows, None] * y.float()).to(h.dtype)
            return out

    return RoutedFeedForward


def make_slowed_rotary():
    from atomserve_amd.parts.base import Position

    class SlowedRotary(Position):
        """Rotation of half of each head, by angles of position / slowdown: the table the attention
        part hands to its kernel, computed here with library calls."""

        pairs = "half"  # a table of (cos, sin) for the pairs (i, i + R/2), as the attention kernels rotate

        def prepare(self, step):
            s = self.spec
            key = ("toy_slowed", s.rotary_dim, s.theta, s.slowdown)
            if key not in step.shared:
                i = torch.arange(0, s.rotary_dim, 2, dtype=torch.float64, device=self.env.device)
                angle = (step.positions.double() / s.slowdown)[:, None] / (s.theta ** (i / s.rotary_dim))[None, :]
                step.shared[key] = torch.stack([angle.cos(), angle.sin()], dim=-1).float().contiguous()
            return step.shared[key]

    return SlowedRotary


NUM_EXPERTS, EXPERT_WIDTH, SLOWDOWN = 3, 40, 4.0


def register_routed_architecture():
    """Qwen3's layers; the feed-forward of every even layer is the routed one, and the attention of
    every odd layer turns half of each head with slowed positions."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture
    from atomserve_amd.parts.base import register

    register("feed_forward", "toy_routed", make_routed_feed_forward(), replace=True)
    register("position", "toy_slowed", make_slowed_rotary(), replace=True)
    qwen = architecture_for(TINY_B)

    def build_plan(c):
        plan = qwen.build_plan(c)
        layers = []
        for i, layer in enumerate(plan.layers):
            if i % 2:
                position = SlowedRotarySpec("toy_slowed", c.head_dim // 2, c.rope_theta, SLOWDOWN)
                layer = dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, position=position))
            else:
                layer = dataclasses.replace(layer, ffn=RoutedSpec("toy_routed", c.hidden_size, EXPERT_WIDTH, NUM_EXPERTS))
            layers.append(layer)
        return dataclasses.replace(plan, layers=tuple(layers))

    def routed(c):
        return range(0, c.num_layers, 2)

    def checkpoint_map(c):
        names = {k: v for k, v in qwen.checkpoint_map(c).items()
                 if not any(k.startswith(f"layers.{i}.ffn.") for i in routed(c))}  # fmt: skip
        for i in routed(c):
            names[f"layers.{i}.ffn.router"] = [f"model.layers.{i}.moe.router.weight"]
            names[f"layers.{i}.ffn.up"] = [f"model.layers.{i}.moe.experts.{e}.up.weight" for e in range(NUM_EXPERTS)]
            names[f"layers.{i}.ffn.down"] = [f"model.layers.{i}.moe.experts.{e}.down.weight" for e in range(NUM_EXPERTS)]
        return names

    def checkpoint_shapes(c):
        shapes = {k: v for k, v in qwen.checkpoint_shapes(c).items()
                  if not any(k.startswith(f"model.layers.{i}.mlp.") for i in routed(c))}  # fmt: skip
        for i in routed(c):
            shapes[f"model.layers.{i}.moe.router.weight"] = ((NUM_EXPERTS, c.hidden_size), "matrix")
            for e in range(NUM_EXPERTS):
                shapes[f"model.layers.{i}.moe.experts.{e}.up.weight"] = ((EXPERT_WIDTH, c.hidden_size), "matrix")
                shapes[f"model.layers.{i}.moe.experts.{e}.down.weight"] = ((c.hidden_size, EXPERT_WIDTH), "matrix")
        return shapes

    return register_architecture(
        Architecture("ToyRoutedForCausalLM", qwen.parse_config, build_plan, checkpoint_map, checkpoint_shapes), replace=True
    )


def routed_weights(raw, seed):
    w = plain_random_weights(raw, seed=seed, std=0.2, gain_std=0.2)
    g = torch.Generator().manual_seed(seed + 100)
    h = raw["hidden_size"]
    for i in range(0, raw["num_hidden_layers"], 2):
        for k in [k for k in w if k.startswith(f"model.layers.{i}.mlp.")]:
            del w[k]
        w[f"model.layers.{i}.moe.router.weight"] = torch.randn(NUM_EXPERTS, h, generator=g).bfloat16().float()
        for e in range(NUM_EXPERTS):
            w[f"model.layers.{i}.moe.experts.{e}.up.weight"] = (0.2 * torch.randn(EXPERT_WIDTH, h, generator=g)).bfloat16().float()
            w[f"model.layers.{i}.moe.experts.{e}.down.weight"] = (0.2 * torch.randn(h, EXPERT_WIDTH, generator=g)).bfloat16().float()
    return w


def plain_routed_logits(raw, w, ids, slowdown=SLOWDOWN):
    """The routed toy model, whole sequence, no cache; also the smallest lead of a chosen expert's
    router logit over the runner-up, which says how safe the choices are from rounding."""
    cfg = plain.normalise_config(raw)
    wd = {k: v.double() for k, v in w.items()}
    ids = torch.as_tensor(ids)
    pos = torch.arange(len(ids))
    T, H, KV, D = len(ids), cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    x = plain.embed(wd["model.embed_tokens.weight"], ids)
    lead = math.inf
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = plain.rms_norm(x, wd[p + "input_layernorm.weight"], eps)
        if i % 2:  # half of each head turns, by a quarter of the position
            q = plain.rms_norm((h @ wd[p + "self_attn.q_proj.weight"].T).view(T, H, D), wd[p + "self_attn.q_norm.weight"], eps)
            k = plain.rms_norm((h @ wd[p + "self_attn.k_proj.weight"].T).view(T, KV, D), wd[p + "self_attn.k_norm.weight"], eps)
            v = (h @ wd[p + "self_attn.v_proj.weight"].T).view(T, KV, D)
            R = D // 2
            q = torch.cat([plain.rope(q[..., :R], pos.double() / slowdown, theta), q[..., R:]], dim=-1)
            k = torch.cat([plain.rope(k[..., :R], pos.double() / slowdown, theta), k[..., R:]], dim=-1)
            o = plain.causal_attention(q, k, v, pos)
            x = x + o.reshape(T, H * D) @ wd[p + "self_attn.o_proj.weight"].T
        else:
            x = x + plain.attention_layer(h, wd, p, cfg, pos)
        h = plain.rms_norm(x, wd[p + "post_attention_layernorm.weight"], eps)
        if i % 2:
            x = x + plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
        else:
            scores = h @ wd[p + "moe.router.weight"].T
            top = scores.topk(2, dim=-1).values
            lead = min(lead, float((top[:, 0] - top[:, 1]).min()))
            probs = torch.softmax(scores, dim=-1)
            ys = []
            for t in range(T):
                e = int(probs[t].argmax())
                y = torch.relu(h[t] @ wd[p + f"moe.experts.{e}.up.weight"].T) @ wd[p + f"moe.experts.{e}.down.weight"].T
                ys.append(probs[t, e] * y)
            x = x + torch.stack(ys)
    x = plain.rms_norm(x, wd["model.norm.weight"], eps)
    return (x @ wd["lm_head.weight"].T).float(), lead


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_feed_forward_with_routing_and_another_position_encoding(dtype, device=DEV):
    arch = register_routed_architecture()
    raw = {**TINY_B, "architectures": ["ToyRoutedForCausalLM"], "num_hidden_layers": 4}
    w = routed_weights(raw, seed=42)
    engine = build_engine(arch, raw, w, dtype, device)
    a = torch.randint(0, 1000, (41,), generator=torch.Generator().manual_seed(6)).tolist()
    b = torch.randint(0, 1000, (19,), generator=torch.Generator().manual_seed(7)).tolist()
    (ref_a, lead_a), (ref_b, lead_b) = plain_routed_logits(raw, w, a), plain_routed_logits(raw, w, b)
    assert min(lead_a, lead_b) > 0.5  # of router logits around 10: no choice of an expert hangs on rounding
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    caches = {}
    whole = step_rows(engine, caches, [("a", a, list(range(41)))])
    assert (whole - ref_a).abs().max() <= tol * max(1.0, ref_a.abs().max())
    # cut anywhere and beside another request: routing is per token, angles follow the position
    caches2, got_a, got_b = {}, [], []
    got = step_rows(engine, caches2, [("a2", a[:9], list(range(9))), ("b", b[:2], [0, 1])])
    got_a.append(got[:9]); got_b.append(got[9:])  # noqa: E702
    got = step_rows(engine, caches2, [("b", b[2:18], list(range(16))), ("a2", a[9:10], [0])])
    got_b.append(got[:16]); got_a.append(got[16:])  # noqa: E702
    got = step_rows(engine, caches2, [("a2", a[10:], list(range(31))), ("b", b[18:], [0])])
    got_a.append(got[:31]); got_b.append(got[31:])  # noqa: E702
    assert (torch.cat(got_a) - ref_a).abs().max() <= tol * max(1.0, ref_a.abs().max())
    assert (torch.cat(got_b) - ref_b).abs().max() <= tol * max(1.0, ref_b.abs().max())
    # through the scheduler: decode steps of a model with a part that cannot be captured run eagerly
    assert not engine.runner.model.capturable
    if dtype == torch.float32:
        from atomserve_amd.engine.sequence import SamplingParams

        outs = engine.generate([a[:7], b[:12]], SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))
        for prompt, out in zip((a[:7], b[:12]), outs):
            seq = list(prompt)
            for t in out:
                assert t == int(plain_routed_logits(raw, w, seq)[0][-1].argmax())
                seq.append(t)
    # the test would not pass with the wrong angles: without the slowdown the logits move by 2.4,
    # ten times what the comparison above allows in bfloat16
    assert (plain_routed_logits(raw, w, a, slowdown=1.0)[0] - ref_a).abs().max() > 8 * 3e-2 * ref_a.abs().max()


# ---- each part alone ------------------------------------------------------------------------


def env(dtype):
    from atomserve_amd.parts.base import BuildEnv

    return BuildEnv(dtype=dtype, device=torch.device(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import NormSpec

    norm = build("norm", NormSpec("rmsnorm", 200, 1e-5), env(dtype))
    assert {k: v.shape for k, v in norm.weight_decls().items()} == {"weight": (200,)}
    w = (torch.randn(200, device=DEV) * 0.2 + 1).to(dtype)
    norm.bind({"weight": w})
    x = torch.randn(9, 200, device=DEV)
    delta = torch.randn(9, 200, device=DEV).to(dtype)
    ref, new_x = pk.rmsnorm(x, w, 1e-5, delta)
    x_work = x.clone()
    out = norm.forward(x_work, delta)
    assert out.dtype == dtype and torch.allclose(x_work, new_x, atol=1e-6)
    assert torch.allclose(out.float(), ref, atol=1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import GatedMLPSpec

    ffn = build("feed_forward", GatedMLPSpec("gated_mlp", 96, 160, "silu"), env(dtype))
    assert {k: v.shape for k, v in ffn.weight_decls().items()} == {"gate_up.weight": (320, 96), "down.weight": (96, 160)}
    gate_up = (torch.randn(320, 96, device=DEV) * 0.1).to(dtype)
    down = (torch.randn(96, 160, device=DEV) * 0.1).to(dtype)
    ffn.bind({"gate_up.weight": gate_up, "down.weight": down})
    h = torch.randn(21, 96, device=DEV).to(dtype)
    out = ffn.forward(h, None)
    ref = plain.swiglu(h.double(), gate_up[:160].double(), gate_up[160:].double(), down.double()).float()
    assert (out.float() - ref).abs().max() <= (1e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(ref.abs().max()))
    with pytest.raises(ValueError, match="activation"):
        build("feed_forward", GatedMLPSpec("gated_mlp", 96, 160, "gelu"), env(dtype))


def test_position_part_and_unknown_kinds():
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import NormSpec, RotarySpec

    class Step:
        num_tokens, shared = 4, {}
        positions = torch.tensor([0, 1, 77, 30000], dtype=torch.int32, device=DEV)

    rope = build("position", RotarySpec("rope_half", 32, 1e6), env(torch.float32))
    table = rope.prepare(Step)
    ang = plain.rope_angles(Step.positions.cpu(), 32, 1e6)
    assert torch.allclose(table[..., 0].cpu().double(), ang.cos(), atol=2e-7) and torch.allclose(table[..., 1].cpu().double(), ang.sin(), atol=2e-7)
    assert rope.prepare(Step) is table  # computed once per step, shared by the layers
    with pytest.raises(ValueError, match="no norm part of kind"):
        build("norm", NormSpec("layernorm", 8, 1e-5), env(torch.float32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_alone(dtype):
    """One attention mixer, built from its spec alone, against the plain attention layer: a
    whole prompt, then the same prompt continued token by token from the cache."""
    from atomserve_amd.cache import CacheManager, CachePools
    from atomserve_amd.engine.batch import Row, StepBatch
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import AttentionSpec, NormSpec, RotarySpec

    h, H, KV, D = 80, 5, 1, 32
    spec = AttentionSpec("attention", h, H, KV, D, 1 / math.sqrt(D), NormSpec("rmsnorm", D, 1e-5), RotarySpec("rope_half", D, 5e4))
    mixer = build("mixer", spec, env(dtype))
    torch.manual_seed(7)
    w = {"qkv.weight": torch.randn((H + 2 * KV) * D, h) * 0.2, "o.weight": torch.randn(h, H * D) * 0.2,
         "q_norm.weight": 1 + 0.2 * torch.randn(D), "k_norm.weight": 1 + 0.2 * torch.randn(D)}  # fmt: skip
    w = {k: v.bfloat16().float() for k, v in w.items()}
    mixer.bind({k: v.to(DEV).to(dtype) for k, v in w.items()})
    manager = CacheManager({0: mixer.cache_request()}, 16, 8, 2)
    pools = CachePools(manager, dtype, DEV)
    x = torch.randn(30, h).bfloat16().float()
    named = {"model.layers.0.self_attn.q_proj.weight": w["qkv.weight"][: H * D],
             "model.layers.0.self_attn.k_proj.weight": w["qkv.weight"][H * D : (H + KV) * D],
             "model.layers.0.self_attn.v_proj.weight": w["qkv.weight"][(H + KV) * D :],
             "model.layers.0.self_attn.q_norm.weight": w["q_norm.weight"], "model.layers.0.self_attn.k_norm.weight": w["k_norm.weight"],
             "model.layers.0.self_attn.o_proj.weight": w["o.weight"]}  # fmt: skip
    cfg = {"num_attention_heads": H, "num_key_value_heads": KV, "head_dim": D, "rms_norm_eps": 1e-5, "rope_theta": 5e4}
    ref = plain.attention_layer(x.double(), {k: v.double() for k, v in named.items()}, "model.layers.0.", cfg, torch.arange(30)).float()
    rc = manager.new_request()
    outs, at = [], 0
    for n in (20, 1, 1, 8):
        manager.reserve(rc, at, n)
        batch = StepBatch([Row([0] * n, at, rc.tables, [])], 16, 1, 10, DEV, pools=pools, row_splits=[mixer.row_split()])
        outs.append(mixer.forward(x[at : at + n].to(DEV).to(dtype), batch, batch.cache_view(0, True)).float().cpu())
        at += n
    tol = (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(ref.abs().max()))
    assert (torch.cat(outs) - ref).abs().max() <= tol


# ---- a mixer with state whose decode steps are captured, and a plan with scaled ends -----------


def make_capturable_decay_mixer():
    base = make_decay_mixer()

    class DecayMixerOnDevice(base):
        """The same running sum; a step in which every row brings one token is computed from the
        step's device arrays alone (slots, first positions), so it can be captured and replayed.
        Rows that pad a captured step arrive with the slot that belongs to nobody."""

        capturable = True

        def forward(self, h, step, cache):
            if not step.decode_only:
                return super().forward(h, step, cache)
            slots = step.row_slots.long()
            old = torch.where((step.row_start == 0)[:, None], torch.zeros((), device=h.device), cache.state[slots])
            s = old * self.spec.decay + h.float()
            cache.state.index_copy_(0, slots, s)
            return (s * self.gain.float()).to(h.dtype)

    return DecayMixerOnDevice


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_steps_of_a_mixer_with_state_are_captured_and_replayed(dtype, device=DEV):
    """A model with a state of its own per request decodes through captured steps like any other,
    once its parts say they can be captured: the capture and its warm-up runs work on padding rows
    and the slot that belongs to nobody, so no request's state moves before its step is replayed."""
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.parts.base import register

    arch = register_toy_architecture()
    register("mixer", "toy_decay", make_capturable_decay_mixer(), replace=True)
    raw = {**TINY_B, "architectures": ["ToyDecayForCausalLM"], "num_hidden_layers": 4}
    w = plain_random_weights(raw, seed=5, std=0.2, gain_std=0.2)
    for i in (1, 3):
        for k in [k for k in w if k.startswith(f"model.layers.{i}.self_attn.")]:
            del w[k]
        w[f"model.layers.{i}.decay.gain"] = (1 + 0.2 * torch.randn(raw["hidden_size"])).bfloat16().float()
    engine = build_engine(arch, raw, w, dtype, device)
    assert engine.runner.model.capturable and engine.scheduler.manager.state_groups
    prompts = [torch.randint(0, 1000, (n,), generator=torch.Generator().manual_seed(n)).tolist() for n in (7, 12, 1)]
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True))
    graphs = engine.runner.decode_graphs.graphs
    assert graphs and engine.counters["steps"] >= 9
    assert engine.scheduler.manager.num_free_slots == 4
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for t in out:
            ref = plain_toy_logits(raw, w, seq)[-1]
            if dtype == torch.float32:
                assert t == int(ref.argmax())
            else:
                assert ref[t] >= ref.max() - 6e-2 * max(1.0, float(ref.abs().max()))
            seq.append(t)
    register("mixer", "toy_decay", make_decay_mixer(), replace=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_plan_scales_its_embeddings_and_caps_its_logits(dtype, device=DEV):
    """Embedding multiplier, logit scale and soft cap are fields of the plan that the decoder reads;
    Qwen3 leaves them at 1, 1 and none."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture

    qwen = architecture_for(TINY_A)
    scale_in, scale_out, cap = 3.0, 1.5, 4.0

    def build_plan(c):
        return dataclasses.replace(qwen.build_plan(c), embedding_scale=scale_in, logit_scale=scale_out, logit_softcap=cap)

    arch = register_architecture(
        Architecture("ScaledForCausalLM", qwen.parse_config, build_plan, qwen.checkpoint_map, qwen.checkpoint_shapes), replace=True
    )
    raw = {**TINY_A, "architectures": ["ScaledForCausalLM"]}
    w = plain_random_weights(raw, seed=12, std=0.2, gain_std=0.2)
    engine = build_engine(arch, raw, w, dtype, device)
    ids = torch.randint(0, 256, (30,), generator=torch.Generator().manual_seed(7)).tolist()
    scaled = dict(w)
    scaled["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * scale_in  # tied: the head is the unscaled table
    hidden = plain.hidden_states(raw, scaled, ids)
    hidden = plain.rms_norm(hidden, w["model.norm.weight"].double(), raw["rms_norm_eps"])
    uncapped = hidden @ w["model.embed_tokens.weight"].double().T * scale_out
    ref = (cap * torch.tanh(uncapped / cap)).float()
    caches = {}
    got = torch.cat([step_rows(engine, caches, [("a", ids[:20], list(range(20)))])]
                    + [step_rows(engine, caches, [("a", [ids[i]], [0])]) for i in range(20, 30)])  # fmt: skip
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    # the cap's slope is at most one: an error of the scaled logits passes through no larger
    assert (got - ref).abs().max() <= tol * max(1.0, float(uncapped.abs().max()))
    assert 0.7 * cap < ref.abs().max() < cap  # the cap bites


# ---- two mixers that want a step's rows sorted in different ways ---------------------------------


@dataclasses.dataclass(frozen=True)
class PositionGateSpec:
    kind: str
    hidden_size: int
    period: float


def make_position_gate_mixer():
    from atomserve_amd.parts.base import Mixer, WeightDecl

    class PositionGate(Mixer):
        """y_t = gain * h_t * cos(position_t / period).  It keeps nothing; it asks for every row in work
        items of up to four consecutive tokens, single tokens included, and takes each token's position
        from its work item: another sorting of the step's rows than the attention part asks for."""

        SPLIT = (0, 4)

        def weight_decls(self):
            return {"gain": WeightDecl((self.spec.hidden_size,), role="vector")}

        def row_split(self):
            return self.SPLIT

        def forward(self, h, step, cache):
            out = torch.full_like(h, float("nan"))
            items = step.split(self.SPLIT)
            assert items.num_short_tokens == 0
            for first, count, row, position in items.long_tiles.cpu().tolist():
                assert 1 <= count <= 4 and step.host_rows[row].start <= position
                at = torch.arange(position, position + count, device=h.device, dtype=torch.float32)
                gate = torch.cos(at / self.spec.period)[:, None]
                out[first : first + count] = (h[first : first + count].float() * self.gain.float() * gate).to(h.dtype)
            return out

    return PositionGate


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixers_that_sort_the_rows_differently_share_a_step(dtype):
    """Odd layers gate the stream by position through work items of four tokens, even layers attend:
    the step is packed once for each of the two sortings, and each mixer finds its own."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture
    from atomserve_amd.parts.attention import SHORT_ROW, TILE_Q
    from atomserve_amd.parts.base import register

    register("mixer", "toy_position_gate", make_position_gate_mixer(), replace=True)
    qwen = architecture_for(TINY_A)
    period = 7.0

    def build_plan(c):
        plan = qwen.build_plan(c)
        layers = tuple(dataclasses.replace(layer, mixer=PositionGateSpec("toy_position_gate", c.hidden_size, period)) if i % 2 else layer
                       for i, layer in enumerate(plan.layers))  # fmt: skip
        return dataclasses.replace(plan, layers=layers)

    def checkpoint_map(c):
        names = {k: v for k, v in qwen.checkpoint_map(c).items()
                 if not any(k.startswith(f"layers.{i}.mixer.") for i in range(1, c.num_layers, 2))}  # fmt: skip
        for i in range(1, c.num_layers, 2):
            names[f"layers.{i}.mixer.gain"] = [f"model.layers.{i}.gate.gain"]
        return names

    def checkpoint_shapes(c):
        shapes = {k: v for k, v in qwen.checkpoint_shapes(c).items()
                  if not any(k.startswith(f"model.layers.{i}.self_attn.") for i in range(1, c.num_layers, 2))}  # fmt: skip
        for i in range(1, c.num_layers, 2):
            shapes[f"model.layers.{i}.gate.gain"] = ((c.hidden_size,), "vector")
        return shapes

    arch = register_architecture(
        Architecture("GatedByPositionForCausalLM", qwen.parse_config, build_plan, checkpoint_map, checkpoint_shapes), replace=True
    )
    raw = {**TINY_A, "architectures": ["GatedByPositionForCausalLM"], "num_hidden_layers": 4}
    w = plain_random_weights(raw, seed=12, std=0.2, gain_std=0.2)
    for i in (1, 3):
        for k in [k for k in w if k.startswith(f"model.layers.{i}.self_attn.")]:
            del w[k]
        w[f"model.layers.{i}.gate.gain"] = (1 + 0.2 * torch.randn(raw["hidden_size"])).bfloat16().float()
    engine = build_engine(arch, raw, w, dtype)
    assert engine.runner.row_splits == ((0, 4), (SHORT_ROW, TILE_Q))

    def reference(ids):
        cfg = plain.normalise_config(raw)
        wd = {k: v.double() for k, v in w.items()}
        pos = torch.arange(len(ids))
        x = plain.embed(wd["model.embed_tokens.weight"], torch.as_tensor(ids))
        for i in range(4):
            p = f"model.layers.{i}."
            h = plain.rms_norm(x, wd[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
            if i % 2:
                x = x + h * wd[p + "gate.gain"] * torch.cos(pos.double() / period)[:, None]
            else:
                x = x + plain.attention_layer(h, wd, p, cfg, pos)
            h = plain.rms_norm(x, wd[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
            x = x + plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
        x = plain.rms_norm(x, wd["model.norm.weight"], cfg["rms_norm_eps"])
        return (x @ wd["model.embed_tokens.weight"].T).float()

    a = torch.randint(0, 256, (90,), generator=torch.Generator().manual_seed(21)).tolist()
    b = torch.randint(0, 256, (31,), generator=torch.Generator().manual_seed(22)).tolist()
    ref = {"a": reference(a), "b": reference(b)}
    caches, got = {}, {"a": [], "b": []}
    # a prompt of 70 tokens (tiles of 64 for one mixer, of 4 for the other) beside a short row, then
    # single tokens beside a portion, then decode steps of both
    logits = step_rows(engine, caches, [("a", a[:70], list(range(70))), ("b", b[:3], [0, 1, 2])])
    got["a"].append(logits[:70]); got["b"].append(logits[70:])  # noqa: E702
    logits = step_rows(engine, caches, [("b", b[3:4], [0]), ("a", a[70:83], list(range(13)))])
    got["b"].append(logits[:1]); got["a"].append(logits[1:])  # noqa: E702
    logits = step_rows(engine, caches, [("b", b[4:24], list(range(20)))])
    got["b"].append(logits)
    for i in range(7):
        logits = step_rows(engine, caches, [("a", [a[83 + i]], [0]), ("b", [b[24 + i]], [0])])
        got["a"].append(logits[:1]); got["b"].append(logits[1:])  # noqa: E702
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for name in "ab":
        assert (torch.cat(got[name]) - ref[name]).abs().max() <= tol * max(1.0, ref[name].abs().max()), name
    for rc, _ in caches.values():
        engine.scheduler.manager.release(rc)
    assert engine.scheduler.manager.num_free == engine.scheduler.manager.num_blocks


# ---- another norm and another arrangement of a layer, defined here ---------------------------------


def make_centred_norm():
    from atomserve_amd.parts.base import Norm, SplitSums, WeightDecl

    class CentredNorm(Norm):
        """weight * (x - mean(x)) / sqrt(var(x) + eps): a norm that is not the package's, computed with library
        calls on the fp32 stream.  Like every norm it first adds the pending output of the part before."""

        def weight_decls(self):
            return {"weight": WeightDecl((self.spec.size,), role="vector")}

        def forward(self, x, delta=None, rows=None, update_residual=True):
            assert not isinstance(delta, SplitSums)  # it does not say `takes_split_sums`, so nobody hands it any
            v = x if delta is None else x + delta.float()
            if delta is not None and update_residual:
                x.copy_(v)
            if rows is not None:
                v = v[rows.long()]
            centred = v - v.mean(-1, keepdim=True)
            out = centred / torch.sqrt(centred.pow(2).mean(-1, keepdim=True) + self.spec.eps) * self.weight.float()
            return out.to(self.env.dtype)

    return CentredNorm


def make_parallel_block():
    from atomserve_amd.parts.base import Arrangement, build

    class ParallelBlock(Arrangement):
        """x += mixer(norm(x)) + ffn(norm(x)): one norm feeds both parts, and their outputs are added together
        before they join the stream (in the next norm, as a pending sum)."""

        def __init__(self, spec, env):
            super().__init__(spec, env)
            self.norm = build("norm", spec.mixer_norm, env)
            self.mixer = build("mixer", spec.mixer, env)
            self.ffn = build("feed_forward", spec.ffn, env)

        def parts(self):
            return {"mixer_norm": self.norm, "mixer": self.mixer, "ffn": self.ffn}

        def forward(self, x, delta, step, cache, next_norm=None):
            h = self.norm.forward(x, delta)
            mixed = self.mixer.forward(h, step, cache)
            fed = self.ffn.forward(h, step)
            return (mixed.float() + fed.float()).to(self.env.dtype)

    return ParallelBlock


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_another_norm_and_another_arrangement_of_a_layer(dtype):
    """Every norm of the model is a centred one defined here, and every layer adds its mixer and its feed-forward
    side by side from one norm instead of one after the other: registered from here, built by the plan, loaded by
    name (the second norm's gains are not in the checkpoint and not asked for), stepped whole, in portions and token
    by token beside another request."""
    from atomserve_amd.config.registry import Architecture, architecture_for, register_architecture
    from atomserve_amd.parts.base import register

    register("norm", "toy_centred", make_centred_norm(), replace=True)
    register("arrangement", "toy_parallel", make_parallel_block(), replace=True)
    qwen = architecture_for(TINY_B)

    def build_plan(c):
        plan = qwen.build_plan(c)
        centred = lambda spec: dataclasses.replace(spec, kind="toy_centred")
        layers = tuple(dataclasses.replace(layer, arrangement="toy_parallel", mixer_norm=centred(layer.mixer_norm),
                                           ffn_norm=centred(layer.ffn_norm)) for layer in plan.layers)  # fmt: skip
        return dataclasses.replace(plan, layers=layers, final_norm=centred(plan.final_norm))

    def checkpoint_map(c):
        return {k: v for k, v in qwen.checkpoint_map(c).items() if ".ffn_norm." not in k}

    def checkpoint_shapes(c):
        return {k: v for k, v in qwen.checkpoint_shapes(c).items() if "post_attention_layernorm" not in k}

    arch = register_architecture(
        Architecture("ParallelCentredForCausalLM", qwen.parse_config, build_plan, checkpoint_map, checkpoint_shapes), replace=True
    )
    raw = {**TINY_B, "architectures": ["ParallelCentredForCausalLM"], "num_hidden_layers": 3}
    w = {k: v for k, v in plain_random_weights(raw, seed=14, std=0.2, gain_std=0.2).items() if "post_attention_layernorm" not in k}
    engine = build_engine(arch, raw, w, dtype)
    assert not engine.runner.model.capturable  # the norm defined here does not say it may be captured: steps run one by one

    def centred(x, weight, eps):
        c = x - x.mean(-1, keepdim=True)
        return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * weight

    def reference(ids):
        cfg = plain.normalise_config(raw)
        wd = {k: v.double() for k, v in w.items()}
        pos = torch.arange(len(ids))
        x = plain.embed(wd["model.embed_tokens.weight"], torch.as_tensor(ids))
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            h = centred(x, wd[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
            fed = plain.swiglu(h, wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"], wd[p + "mlp.down_proj.weight"])
            x = x + plain.attention_layer(h, wd, p, cfg, pos) + fed
        x = centred(x, wd["model.norm.weight"], cfg["rms_norm_eps"])
        return (x @ wd["lm_head.weight"].T).float()

    a = torch.randint(0, 1000, (75,), generator=torch.Generator().manual_seed(31)).tolist()
    b = torch.randint(0, 1000, (20,), generator=torch.Generator().manual_seed(32)).tolist()
    ref = {"a": reference(a), "b": reference(b)}
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    caches = {}
    whole = step_rows(engine, caches, [("whole", a, list(range(75)))])
    assert (whole - ref["a"]).abs().max() <= tol * max(1.0, ref["a"].abs().max())
    got = {"a": [], "b": []}
    logits = step_rows(engine, caches, [("a", a[:66], list(range(66))), ("b", b[:2], [0, 1])])
    got["a"].append(logits[:66]); got["b"].append(logits[66:])  # noqa: E702
    for i in range(9):
        logits = step_rows(engine, caches, [("b", b[2 + 2 * i : 4 + 2 * i], [0, 1]), ("a", [a[66 + i]], [0])])
        got["b"].append(logits[:2]); got["a"].append(logits[2:])  # noqa: E702
    for name in "ab":
        assert (torch.cat(got[name]) - ref[name]).abs().max() <= tol * max(1.0, ref[name].abs().max()), name
    for rc, _ in caches.values():
        engine.scheduler.manager.release(rc)
    assert engine.scheduler.manager.num_free == engine.scheduler.manager.num_blocks
    # and through the scheduler: greedy generation equals the plain model's
    if dtype == torch.float32:
        from atomserve_amd.engine.sequence import SamplingParams

        out = engine.generate([a[:9]], SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))[0]
        seq = list(a[:9])
        for t in out:
            assert t == int(reference(seq)[-1].argmax())
            seq.append(t)
