"""Small Kosesun configurations for the tests: sizes, head counts, layer orders and constants
that differ from each other in every respect, and folders with random weights for them."""

import json
import os

import plain_kosesun


def _attention(heads, kv_heads, dim, vdim, rot_dims, base, scale, v_mix, ff):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "v_mix": v_mix, "rot": {"dims": rot_dims, "base": base}}
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _gla(heads, dim, vdim, tau, ff):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# two copies of the stream; a recurrent layer first; values narrower than keys; part of every
# head rotated; three layers that mix values, the last without a feed-forward
MODEL_A = {
    "architecture": "Kosesun", "vocab": 97, "width": 64, "streams": 2, "logit_softcap": 10.0,
    "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
    "layers": [_gla(2, 16, 24, 8.0, 96),
               _attention(4, 2, 16, 32, 8, 10000.0, 0.25, True, 96),
               _attention(4, 2, 16, 32, 16, 500.0, 0.3, True, 80),
               _attention(4, 2, 16, 32, 8, 10000.0, 0.25, True, None)],
}
# one plain stream (no key), as many key/value heads as heads, equal head sizes that are no
# multiple of 16, nothing mixed, no cap, a width that no packed copy is made for
MODEL_B = {
    "architecture": "Kosesun", "vocab": 131, "width": 48,
    "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
    "layers": [_attention(2, 2, 24, 24, 24, 1000.0, 0.2, False, 64),
               _gla(3, 8, 8, 2.0, None),
               _attention(2, 2, 24, 24, 24, 1000.0, 0.2, False, 64)],
}
# a single copy with its own weights, one key/value head under three heads, values wider than
# keys, a recurrent layer whose sizes are no multiples of the kernel's, one layer that mixes alone
MODEL_C = {
    "architecture": "Kosesun", "vocab": 64, "width": 72, "streams": 1, "logit_softcap": 30.0,
    "norm": {"eps": 1e-6}, "embedding": {"scale": 8.5},
    "layers": [_attention(3, 1, 8, 40, 4, 250000.0, 0.35, True, 100),
               _gla(1, 40, 72, 32.0, 100),
               _attention(3, 1, 8, 40, 4, 250000.0, 0.35, False, None)],
}
# three copies, sizes that the matrix-core kernels take as they are (heads of 64 for keys and values)
MODEL_D = {
    "architecture": "Kosesun", "vocab": 256, "width": 128, "streams": 3, "logit_softcap": 20.0,
    "norm": {"eps": 1e-6}, "embedding": {"scale": 11.3},
    "layers": [_attention(4, 2, 64, 64, 32, 10000.0, 0.125, True, 256),
               _gla(2, 64, 64, 16.0, 256),
               _attention(4, 2, 64, 64, 32, 10000.0, 0.125, True, 256)],
}
# recurrent layers only (nothing is paged), two copies, one layer without a feed-forward
MODEL_E = {
    "architecture": "Kosesun", "vocab": 77, "width": 40, "streams": 2,
    "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "layers": [_gla(2, 12, 20, 4.0, 56), _gla(5, 4, 4, 64.0, None), _gla(2, 12, 20, 4.0, 56)],
}
# attention only, sizes that are multiples of nothing (width 100, five heads of 12, a vocabulary of
# 51), eight copies, a single layer
MODEL_F = {
    "architecture": "Kosesun", "vocab": 51, "width": 100, "streams": 8, "logit_softcap": 5.0,
    "norm": {"eps": 1e-6}, "embedding": {"scale": 10.0},
    "layers": [_attention(5, 5, 12, 12, 6, 100.0, 0.4, True, 36)],
}
# name -> (configuration, page size, seed, rank of the decay projection)
MODELS = {"A": (MODEL_A, 8, 0, 4), "B": (MODEL_B, 16, 1, 3), "C": (MODEL_C, 4, 2, 6), "D": (MODEL_D, 16, 3, 16),
          "E": (MODEL_E, 8, 4, 2), "F": (MODEL_F, 16, 5, 1)}


def folder_of(tmp_path, which):
    """(folder, raw configuration, checkpoint tensors as stored, page size)."""
    from safetensors.torch import save_file

    raw, page_size, seed, rank = MODELS[which]
    tensors = plain_kosesun.random_checkpoint(raw, seed, decay_rank=rank)
    # stored as a checkpoint of this design is: matrices in bfloat16 (the plain side reads the same values)
    import torch

    stored = {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}
    folder = os.path.join(str(tmp_path), f"kosesun_{which}")
    os.makedirs(folder, exist_ok=True)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return folder, raw, {name: tensor.float() for name, tensor in stored.items()}, page_size
