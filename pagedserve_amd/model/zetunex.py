"""Zetunex as data: a decoder whose layers are listed one by one in its configuration.

Each layer norms the stream once (RMS norm with a plain scale) and hands the result to its
mixer and to its feed-forward at the same time; a factor times the sum of the two is added to
the stream.  The mixer is lightning attention (linear attention with a fixed decay per head) or
a sliding-window attention without positions side by side with a selective state-space mixer;
the feed-forward is a gated dense one or a mixture of experts with a group-limited router.  A
run of layers may be passed several times with the same weights; every pass keeps caches and
states of its own and begins by adding a learned vector to the stream.  The head is the token
table.
"""

import math

import torch

from ..config.registry import Architecture, register_architecture
from ..config.spec import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.zetunex import ZetunexConfig
from ..weights.loader import WeightSource


def _mixer_spec(config, layer):
    mixer = layer.mixer
    if layer.type == "lightning":
        return PartSpec.make("lightning_attention", heads=mixer.heads, key_dim=mixer.dim,
                             value_dim=mixer.vdim, decays=tuple(mixer.decay),
                             norm_eps=config.norm_eps)
    left, right = mixer.left, mixer.right
    attention = PartSpec.make(
        "attention", heads=left.heads, kv_heads=left.kv_heads, head_dim=left.dim,
        value_dim=left.vdim, scale=left.scale, window=left.window, bias=True, out_bias=False)
    scan = PartSpec.make("selective_scan", inner=right.inner, states=right.state,
                         dt_rank=right.dt_rank, taps=right.conv)
    return PartSpec.make("side_by_side", left=attention, right=scan, norm_eps=config.norm_eps)


def _feed_forward_spec(mlp):
    if mlp.kind == "dense":
        return PartSpec.make("gated", inner=mlp.ff)
    return PartSpec.make("moe", inner=mlp.ff, experts=mlp.experts, top=mlp.top, groups=mlp.groups,
                         keep=mlp.keep, scale=mlp.scale)


def build_spec(config: ZetunexConfig) -> ModelSpec:
    norm = PartSpec.make("rmsnorm", eps=config.norm_eps)
    blocks = []
    for layer in config.layers:
        parts = {"norm1": norm, "mixer": _mixer_spec(config, layer)}
        arrangement = "parallel_scaled_mixer"
        if layer.mlp is not None:
            parts["feed_forward"] = _feed_forward_spec(layer.mlp)
            arrangement = "parallel_scaled"
        blocks.append(BlockSpec.make(arrangement, params={"factor": config.residual_mult}, **parts))
    # every call of the run order keeps a cache entry of its own: a layer that is passed again
    # shares its weights with the earlier pass, nothing else
    schedule = tuple(LayerCall(block=layer, cache=index, enter=turn)
                     for index, (layer, turn) in enumerate(config.run_order()))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        width=config.width,
        max_positions=config.max_positions,
        position=PartSpec.make("none"),
        blocks=tuple(blocks),
        schedule=schedule,
        final_norm=norm,
        tie_head=True,
        eos_token_id=None,
        embedding=PartSpec.make("lookup"),
        head=PartSpec.make("linear", bias=False),
        pass_rows=config.loop_times,
    )


def _expert_names(prefix, experts, pieces):
    return tuple(f"{prefix}e{e}.{piece}" for e in range(experts) for piece in pieces)


def weight_sources(config: ZetunexConfig, spec: ModelSpec):
    """Parameter path -> checkpoint tensor(s).  Matrices are stored ``[out, in]``; projections
    that read the same input are joined into one packed product, the experts' matrices are
    stacked one behind the other."""
    sources = {
        "embedding.table": WeightSource("embed"),
        "final_norm.gamma": WeightSource("final.norm"),
    }
    if config.loop_times:
        sources["pass_table"] = WeightSource("loop.step")
    for i, layer in enumerate(config.layers):
        b, l = f"blocks.{i}.", f"l{i}."
        sources[b + "norm1.gamma"] = WeightSource(l + "norm1")
        m = l + "mix."
        if layer.type == "lightning":
            sources[b + "mixer.in.weight"] = WeightSource((m + "q", m + "k", m + "v", m + "g"))
            sources[b + "mixer.norm.gamma"] = WeightSource(m + "norm")
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        else:
            a, s = m + "left.", m + "right."
            sources[b + "mixer.left.qkv.weight"] = WeightSource((a + "q", a + "k", a + "v"))
            sources[b + "mixer.left.qkv.bias"] = WeightSource((a + "q.b", a + "k.b", a + "v.b"))
            sources[b + "mixer.left.out.weight"] = WeightSource(a + "o")
            sources[b + "mixer.left_scale"] = WeightSource(a + "out")
            sources[b + "mixer.right.in.weight"] = WeightSource(s + "in")
            sources[b + "mixer.right.conv.weight"] = WeightSource(s + "conv")
            sources[b + "mixer.right.conv.bias"] = WeightSource(s + "conv.b")
            sources[b + "mixer.right.x.weight"] = WeightSource(s + "x")
            sources[b + "mixer.right.dt.weight"] = WeightSource(s + "dt")
            sources[b + "mixer.right.dt.bias"] = WeightSource(s + "dt.b")
            sources[b + "mixer.right.a_log"] = WeightSource(s + "A_log")
            sources[b + "mixer.right.skip"] = WeightSource(s + "D")
            sources[b + "mixer.right.out.weight"] = WeightSource(s + "o")
            sources[b + "mixer.right_scale"] = WeightSource(s + "out")
        if layer.mlp is None:
            continue
        f = l + "mlp."
        if layer.mlp.kind == "dense":
            sources[b + "feed_forward.gate_up.weight"] = WeightSource((f + "gate", f + "up"))
            sources[b + "feed_forward.down.weight"] = WeightSource(f + "down")
        else:
            sources[b + "feed_forward.router.weight"] = WeightSource(f + "router")
            sources[b + "feed_forward.gate_up.weight"] = WeightSource(
                _expert_names(f, layer.mlp.experts, ("gate", "up")))
            sources[b + "feed_forward.down.weight"] = WeightSource(
                _expert_names(f, layer.mlp.experts, ("down",)))
    return sources


def random_tensors(config: ZetunexConfig, seed: int, device="cpu"):
    """Checkpoint tensors of a random model, drawn from one seeded generator in a fixed order.
    Matrices N(0, 1/sqrt(in)); scales, biases, step sizes and decays such that every part
    matters in the output and the recurrences neither die nor blow up."""
    generator = torch.Generator(device=device).manual_seed(int(seed))

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32, device=device) * (high - low) + low

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = config.width
    tensors = {"embed": normal((config.vocab, d))}
    if config.loop_times:
        tensors["loop.step"] = normal((config.loop_times, d), 0.3)
    for i, layer in enumerate(config.layers):
        l, m = f"l{i}.", f"l{i}.mix."
        mixer = layer.mixer
        tensors[l + "norm1"] = 1.0 + normal((d,), 0.1)
        if layer.type == "lightning":
            tensors[m + "q"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "k"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "v"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "g"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim)
            tensors[m + "norm"] = 1.0 + normal((mixer.heads * mixer.vdim,), 0.1)
        else:
            left, right = mixer.left, mixer.right
            a, s = m + "left.", m + "right."
            tensors[a + "q"] = matrix(left.heads * left.dim, d)
            tensors[a + "q.b"] = normal((left.heads * left.dim,), 0.1)
            tensors[a + "k"] = matrix(left.kv_heads * left.dim, d)
            tensors[a + "k.b"] = normal((left.kv_heads * left.dim,), 0.1)
            tensors[a + "v"] = matrix(left.kv_heads * left.vdim, d)
            tensors[a + "v.b"] = normal((left.kv_heads * left.vdim,), 0.1)
            tensors[a + "o"] = matrix(d, left.heads * left.vdim)
            tensors[a + "out"] = 1.0 + normal((d,), 0.1)
            tensors[s + "in"] = matrix(2 * right.inner, d)
            tensors[s + "conv"] = normal((right.inner, right.conv), 1.0 / math.sqrt(right.conv))
            tensors[s + "conv.b"] = normal((right.inner,), 0.1)
            tensors[s + "x"] = matrix(right.dt_rank + 2 * right.state, right.inner)
            tensors[s + "dt"] = matrix(right.inner, right.dt_rank)
            # softplus^-1 of step sizes between 0.001 and 0.1, log-uniform
            steps = torch.exp(uniform((right.inner,), math.log(1e-3), math.log(1e-1)))
            tensors[s + "dt.b"] = steps + torch.log(-torch.expm1(-steps))
            tensors[s + "A_log"] = torch.log(torch.arange(1, right.state + 1, dtype=torch.float32,
                                                          device=device)).repeat(right.inner, 1)
            tensors[s + "D"] = 1.0 + normal((right.inner,), 0.1)
            tensors[s + "o"] = matrix(d, right.inner)
            tensors[s + "out"] = 1.0 + normal((d,), 0.1)
        mlp = layer.mlp
        if mlp is None:
            continue
        f = l + "mlp."
        if mlp.kind == "dense":
            tensors[f + "gate"] = matrix(mlp.ff, d)
            tensors[f + "up"] = matrix(mlp.ff, d)
            tensors[f + "down"] = matrix(d, mlp.ff)
        else:
            tensors[f + "router"] = matrix(mlp.experts, d, 2.0)
            for e in range(mlp.experts):
                tensors[f + f"e{e}.gate"] = matrix(mlp.ff, d)
                tensors[f + f"e{e}.up"] = matrix(mlp.ff, d)
                tensors[f + f"e{e}.down"] = matrix(d, mlp.ff)
    tensors["final.norm"] = 1.0 + normal((d,), 0.1)
    return tensors


ZETUNEX = register_architecture(Architecture(
    name="Zetunex",
    config_class=ZetunexConfig,
    build_spec=build_spec,
    weight_sources=weight_sources,
    random_tensors=random_tensors,
    model_type="zetunex",
))
