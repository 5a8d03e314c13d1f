"""Kosesun as data: a decoder whose layers are listed one by one in its configuration.

Each layer is a pre-norm block (RMS norms whose scale is stored around zero) of a mixer,
causal attention with grouped heads or gated linear attention, and an optional squared-ReLU
feed-forward.  The residual stream may be kept in several copies that every sublayer reads
and writes through learned weights.  The token embedding is scaled, the head is a matrix of
its own, and the logits are capped by a tanh.
"""

import math

import torch

from ..config.kosesun import KosesunConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..weights.loader import WeightSource

RANDOM_DECAY_RANK = 16   # rank of the decay projection of a random model whose configuration names none


def _mixer_spec(config, layer, first_mixing):
    mixer = layer.mixer
    if layer.type == "attention":
        value_mix = "none"
        if mixer.v_mix:
            value_mix = "source" if first_mixing else "mix"
        return PartSpec.make(
            "attention", heads=mixer.heads, kv_heads=mixer.kv_heads, head_dim=mixer.dim,
            value_dim=mixer.vdim, scale=mixer.scale, window=0, bias=False, qk_norm=True,
            norm_eps=config.norm_eps, rotary_dims=mixer.rot_dims, rotary_base=mixer.rot_base,
            sink=True, value_mix=value_mix, head_gate=True)
    rank = mixer.decay_rank if mixer.decay_rank is not None else RANDOM_DECAY_RANK
    return PartSpec.make("gated_linear_attention", heads=mixer.heads, key_dim=mixer.dim,
                         value_dim=mixer.vdim, decay_rank=rank, tau=mixer.tau,
                         norm_eps=config.norm_eps)


def build_spec(config: KosesunConfig) -> ModelSpec:
    norm = PartSpec.make("rmsnorm", eps=config.norm_eps, offset=1.0)
    connection = PartSpec.make("hyper", streams=config.streams) if config.streams else None
    blocks = []
    mixing_seen = False
    for layer in config.layers:
        mixes = layer.type == "attention" and layer.mixer.v_mix
        parts = {"norm1": norm, "mixer": _mixer_spec(config, layer, mixes and not mixing_seen)}
        mixing_seen = mixing_seen or mixes
        if connection is not None:
            parts["connect1"] = connection
        if layer.ff is not None:
            parts["norm2"] = norm
            parts["feed_forward"] = PartSpec.make("dense", inner=layer.ff, activation="relu2", bias=False)
            if connection is not None:
                parts["connect2"] = connection
        arrangement = "hyper_connected" if connection is not None else "pre_norm"
        if layer.ff is None:
            arrangement += "_mixer"
        blocks.append(BlockSpec.make(arrangement, **parts))
    count = len(config.layers)
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        width=config.width,
        max_positions=config.max_positions,
        position=PartSpec.make("none"),
        blocks=tuple(blocks),
        schedule=tuple(LayerCall(block=i, cache=i) for i in range(count)),
        final_norm=norm,
        tie_head=False,
        eos_token_id=None,
        embedding=PartSpec.make("lookup", scale=config.embedding_scale),
        head=PartSpec.make("linear", bias=False, softcap=config.logit_softcap),
        streams=config.streams,
    )


def weight_sources(config: KosesunConfig, spec: ModelSpec):
    """Parameter path -> checkpoint tensor(s).  Matrices are stored ``[out, in]``; the
    projections of a mixer that read the same input are joined into one packed product."""
    sources = {
        "embedding.table": WeightSource("embed"),
        "final_norm.gamma": WeightSource("final.norm"),
        "head.weight": WeightSource("head"),
    }
    mixing_seen = False
    for i, layer in enumerate(config.layers):
        b, l = f"blocks.{i}.", f"l{i}."
        sources[b + "norm1.gamma"] = WeightSource(l + "norm1")
        m = l + "mix."
        if layer.type == "attention":
            sources[b + "mixer.qkv.weight"] = WeightSource((m + "q", m + "k", m + "v", m + "g"))
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
            sources[b + "mixer.q_norm.gamma"] = WeightSource(m + "q.norm")
            sources[b + "mixer.k_norm.gamma"] = WeightSource(m + "k.norm")
            sources[b + "mixer.sink"] = WeightSource(m + "sink")
            if layer.mixer.v_mix and mixing_seen:
                sources[b + "mixer.value_mix.weight"] = WeightSource(m + "vmix")
            mixing_seen = mixing_seen or layer.mixer.v_mix
        else:
            sources[b + "mixer.in.weight"] = WeightSource((m + "q", m + "k", m + "v", m + "g", m + "a1"))
            sources[b + "mixer.decay.weight"] = WeightSource(m + "a2")
            sources[b + "mixer.decay.bias"] = WeightSource(m + "a2.b")
            sources[b + "mixer.norm.gamma"] = WeightSource(m + "norm")
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        if layer.ff is not None:
            sources[b + "norm2.gamma"] = WeightSource(l + "norm2")
            sources[b + "feed_forward.up.weight"] = WeightSource(l + "mlp.up")
            sources[b + "feed_forward.down.weight"] = WeightSource(l + "mlp.down")
        if config.streams:
            for q in (1, 2) if layer.ff is not None else (1,):
                for name in ("in", "out", "mix"):
                    sources[b + f"connect{q}.{name}"] = WeightSource(l + f"hc{q}.{name}")
    return sources


def ignorable(config: KosesunConfig, name: str) -> bool:
    """The value-mixing weight of the first layer that mixes values: stored, never used."""
    for i, layer in enumerate(config.layers):
        if layer.type == "attention" and layer.mixer.v_mix:
            return name == f"l{i}.mix.vmix"
    return False


def complete_config(config: KosesunConfig, shape_of) -> KosesunConfig:
    """Sizes that only the tensors give: the rank of each decay projection."""
    return config.with_decay_ranks(lambda index: shape_of(f"l{index}.mix.a1")[0])


def random_tensors(config: KosesunConfig, seed: int, device="cpu"):
    """Checkpoint tensors of a random model, drawn from one seeded generator in a fixed order.
    Matrices N(0, 1/sqrt(in)), norm scales near zero, sinks, decay biases and the stream
    weights such that every part matters in the output."""
    generator = torch.Generator(device=device).manual_seed(int(seed))

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = config.width
    tensors = {"embed": normal((config.vocab, d), 1.0 / max(config.embedding_scale, 1e-6))}
    streams = config.streams
    mixing_seen = False
    for i, layer in enumerate(config.layers):
        l, m = f"l{i}.", f"l{i}.mix."
        mixer = layer.mixer
        tensors[l + "norm1"] = normal((d,), 0.1)
        if layer.type == "attention":
            tensors[m + "q"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "k"] = matrix(mixer.kv_heads * mixer.dim, d)
            tensors[m + "v"] = matrix(mixer.kv_heads * mixer.vdim, d)
            tensors[m + "g"] = matrix(mixer.heads, d)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim, 0.5)
            tensors[m + "q.norm"] = 1.0 + normal((mixer.heads * mixer.dim,), 0.1)
            tensors[m + "k.norm"] = 1.0 + normal((mixer.kv_heads * mixer.dim,), 0.1)
            tensors[m + "sink"] = normal((mixer.heads,), 1.0)
            if mixer.v_mix:
                tensors[m + "vmix"] = torch.rand((), generator=generator, device=device) * 0.6 + 0.2
        else:
            rank = mixer.decay_rank if mixer.decay_rank is not None else RANDOM_DECAY_RANK
            tensors[m + "q"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "k"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "v"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "g"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "a1"] = matrix(rank, d)
            tensors[m + "a2"] = matrix(mixer.heads * mixer.dim, rank)
            tensors[m + "a2.b"] = 2.0 + normal((mixer.heads * mixer.dim,), 1.0)
            tensors[m + "norm"] = 1.0 + normal((mixer.vdim,), 0.1)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim, 0.5)
        if layer.ff is not None:
            tensors[l + "norm2"] = normal((d,), 0.1)
            tensors[l + "mlp.up"] = matrix(layer.ff, d)
            tensors[l + "mlp.down"] = matrix(d, layer.ff, 0.5)
        if streams:
            for q in (1, 2) if layer.ff is not None else (1,):
                tensors[l + f"hc{q}.in"] = 1.0 / streams + normal((streams,), 0.1)
                tensors[l + f"hc{q}.out"] = 1.0 + normal((streams,), 0.2)
                tensors[l + f"hc{q}.mix"] = (torch.eye(streams, device=device)
                                             + normal((streams, streams), 0.1))
    tensors["final.norm"] = normal((d,), 0.1)
    tensors["head"] = matrix(config.vocab, d)
    return tensors


KOSESUN = register_architecture(Architecture(
    name="Kosesun",
    config_class=KosesunConfig,
    build_spec=build_spec,
    weight_sources=weight_sources,
    random_tensors=random_tensors,
    ignorable=ignorable,
    complete_config=complete_config,
    model_type="kosesun",
))
