"""Small Zetunex configurations for the tests: sizes, head counts, layer orders, windows and
constants that differ from each other in every respect, and folders with random weights."""

import json
import os

import torch

import plain_zetunex


def _lightning(heads, dim, vdim, decay, mlp):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp}


def _parallel(heads, kv_heads, dim, vdim, scale, window, inner, state, dt_rank, conv, mlp):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window}}
    right = {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, count, keep, scale, ff):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


# a recurrent layer first, a run of two layers passed three times, a layer without a feed-forward,
# values wider than keys under two key/value heads, four groups of experts of which two stay open
MODEL_A = {
    "architecture": "Zetunex", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [_lightning(2, 16, 24, [0.9, 0.99], _moe(8, 2, 4, 2, 1.5, 40)),
               _parallel(4, 2, 16, 32, 0.2, 10, 48, 8, 3, 4, _dense(96)),
               _parallel(4, 2, 16, 32, 0.2, 10, 48, 8, 3, 4, None),
               _lightning(2, 16, 24, [0.5, 0.97], _dense(72))],
}
# no loop and no factor on what a layer adds; keys and values of one size that is no multiple of
# 16, as many key/value heads as heads, a window of five, a step size of rank one, a convolution
# of two taps, all experts in one group and one expert per token
MODEL_B = {
    "architecture": "Zetunex", "vocab": 131, "width": 48, "norm": {"eps": 1e-6},
    "layers": [_parallel(2, 2, 24, 24, 0.3, 5, 40, 5, 1, 2, _moe(3, 1, 1, 1, 1.0, 56)),
               _lightning(3, 8, 8, [0.8, 0.95, 0.999], None),
               _parallel(2, 2, 24, 24, 0.3, 5, 40, 5, 1, 2, _dense(64))],
}
# sizes that the matrix-core kernels take as they are; one layer passed twice, then the rest once;
# one key/value head under four heads; a window that ends inside a page; every group stays open
MODEL_C = {
    "architecture": "Zetunex", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "residual_mult": 0.7,
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [_parallel(4, 1, 64, 64, 0.125, 33, 256, 16, 8, 4, _moe(4, 2, 2, 2, 2.0, 128)),
               _lightning(2, 64, 64, [0.96, 0.999], _dense(256)),
               _parallel(4, 1, 64, 64, 0.125, 33, 256, 16, 8, 4, _dense(256))],
}
# a window that no request outgrows, more states per channel than a wave has lanes, a convolution
# of a single tap, keys wider than values, a loop over everything, many experts in many groups
MODEL_D = {
    "architecture": "Zetunex", "vocab": 77, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 1.3,
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [_parallel(3, 1, 40, 8, 0.1, 500, 24, 130, 2, 1, _moe(12, 3, 6, 3, 0.8, 20)),
               _lightning(1, 40, 72, [0.93], _moe(6, 4, 3, 2, 1.0, 24))],
}
# the smallest of everything: a window of one token (a query sees itself only), one state per
# channel, a single head, every expert of the one group chosen, a pass that is made once, sizes
# that are multiples of nothing, a recurrent layer without a feed-forward first
MODEL_E = {
    "architecture": "Zetunex", "vocab": 33, "width": 24, "norm": {"eps": 1e-4}, "residual_mult": 0.25,
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [_lightning(1, 8, 4, [0.75], None),
               _parallel(1, 1, 12, 20, 0.5, 1, 10, 1, 5, 5, _moe(2, 2, 1, 1, 3.0, 7)),
               _parallel(6, 3, 4, 4, 0.7, 2, 18, 3, 2, 3, _dense(9))],
}
# name -> (configuration, page size, seed)
MODELS = {"A": (MODEL_A, 8, 0), "B": (MODEL_B, 16, 1), "C": (MODEL_C, 16, 2), "D": (MODEL_D, 4, 3),
          "E": (MODEL_E, 2, 4)}


def write_folder(folder, raw, tensors):
    """Store a checkpoint as this design's are stored (bfloat16) and return the values as stored."""
    from safetensors.torch import save_file

    stored = {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return {name: tensor.float() for name, tensor in stored.items()}


def folder_of(tmp_path, which):
    """(folder, raw configuration, checkpoint tensors as stored, page size)."""
    raw, page_size, seed = MODELS[which]
    folder = os.path.join(str(tmp_path), f"zetunex_{which}")
    return folder, raw, write_folder(folder, raw, plain_zetunex.random_checkpoint(raw, seed)), page_size


LOUD, ASK = 1, 2      # tokens of the model below


def loud_key_model(tmp_path, window, decay):
    """A model of one windowed layer and one recurrent layer in which one pair of tokens stands
    out: the key of LOUD and the query of ASK point the same way and are long, so that an ASK
    gives nearly all its weight to a LOUD that it can see (the window's edge shows in the logits),
    and the recurrent layer's output at an ASK is dominated by a LOUD however far back it is.
    Returns (folder, raw, tensors)."""
    width = 64
    raw = {
        "architecture": "Zetunex", "vocab": 50, "width": width, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
        "layers": [_parallel(2, 1, 16, 16, 1.0, window, 32, 4, 2, 3, None),
                   _lightning(2, 16, 16, [decay, decay], None)],
    }
    w = plain_zetunex.random_checkpoint(raw, 17)
    # the two tokens' embeddings: long along directions 0 and 1, where no other token has anything
    w["embed"][:, :2] = 0
    w["embed"][LOUD] = 0
    w["embed"][LOUD, 0] = 8.0
    w["embed"][ASK] = 0
    w["embed"][ASK, 1] = 8.0
    for prefix, heads in (("l0.mix.left.", 1), ("l1.mix.", 2)):
        k, q = w[prefix + "k"], w[prefix + "q"]
        k[:, 0] = 0
        k[:, 1] = 0
        q[:, 0] = 0
        q[:, 1] = 0
        # keys of LOUD and queries of ASK: the same direction in every head
        k.view(heads, 16, width)[:, :4, 0] = 1.5
        q.view(-1, 16, width)[:, :4, 1] = 1.5
    for name in ("l0.mix.left.q.b", "l0.mix.left.k.b"):
        w[name] *= 0.1
    folder = os.path.join(str(tmp_path), f"zetunex_loud_{window}")
    return folder, raw, write_folder(folder, raw, w)
