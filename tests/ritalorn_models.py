"""Small Ritalorn configurations for the tests, their random weights, and token lists.

The configurations differ from one another in every size and constant: one to four copies of the
stream, grouped and ungrouped heads, value widths above and below the key width, latent ranks above
and below the head widths, convolutions of one to four taps, chunks and windows from one token to
more than any prompt and none at all, a chunk as long as a page, layers that read an earlier layer's
keys and values under a mask and with taps of their own, layers with and without a feed-forward,
with and without a cap on the logits, widths that the few-row product kernels take (multiples of 8)
and ones they do not.  Weights are drawn so that no mechanism hides: queries and the latent's
projections wide enough for peaked attention, convolution taps and biases of both signs, and
connection weights of the stream's copies spread about zero.
"""

from __future__ import annotations

import json
import os

import torch


def attention(heads, kv_heads, dim, vdim, scale, conv, mask=None, kv_from=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "conv": conv}
    if mask is not None:
        mixer["mask"] = {"size": mask}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, dims=None, mask=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
             "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if mask is not None:
        mixer["mask"] = {"size": mask}
    return {"type": "latent_attention", "mixer": mixer}


def layer(mixer, ff=None):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


# A: a latent layer first, a reader of layer 1's keys and values with a mask and taps of its own, a rotation
# over half of the rotated part, three copies of the stream
A = {"architecture": "Ritalorn", "vocab": 301, "width": 64, "norm": {"eps": 2e-6}, "streams": 3, "logit_softcap": 12.0,
     "layers": [
         layer(latent(3, 16, 8, 24, 40, 0.3, base=1000.0, mask=20), ff=96),
         layer(attention(6, 2, 32, 16, 0.4, conv=4, mask=50), ff=80),
         layer(attention(6, 2, 32, 16, 0.25, conv=2, mask=33, kv_from=1)),
         layer(latent(2, 24, 16, 8, 16, 0.2, base=50.0, dims=8, mask=7), ff=40),
     ]}
# B: one copy of the stream, a width the few-row products do not take, one tap, a chunk as long as a page,
# values wider than keys, a window longer than any prompt, no cap on the logits
B = {"architecture": "Ritalorn", "vocab": 211, "width": 100, "norm": {"eps": 1e-5}, "streams": 1, "logit_softcap": None,
     "layers": [
         layer(attention(3, 3, 48, 80, 0.2, conv=1, mask=16), ff=130),
         layer(latent(4, 20, 12, 36, 28, 0.25, base=40000.0, mask=640), ff=60),
         layer(attention(3, 3, 48, 80, 0.3, conv=3, mask=40, kv_from=0), ff=70),
     ]}
# C: heads of 64 and 32 with values as wide (shapes matrix-core kernels may take), two readers of one layer,
# a chunk longer than any prompt, a layer without a mask
C = {"architecture": "Ritalorn", "vocab": 400, "width": 128, "norm": {"eps": 1e-5}, "streams": 2, "logit_softcap": 30.0,
     "layers": [
         layer(attention(8, 2, 64, 64, 0.15, conv=3, mask=48), ff=192),
         layer(latent(5, 32, 32, 48, 128, 0.15, base=3000.0, mask=36)),
         layer(attention(8, 2, 64, 64, 0.2, conv=3, mask=1000, kv_from=0), ff=64),
         layer(attention(4, 4, 32, 32, 0.3, conv=2), ff=64),
         layer(attention(8, 2, 64, 64, 0.1, conv=4, mask=24, kv_from=0)),
     ]}
# D: nothing is a multiple of four, chunks of five and a window of three, four copies
D = {"architecture": "Ritalorn", "vocab": 97, "width": 90, "norm": {"eps": 1e-5}, "streams": 4, "logit_softcap": 8.0,
     "layers": [
         layer(attention(3, 1, 22, 18, 0.3, conv=3, mask=5), ff=70),
         layer(latent(3, 10, 6, 14, 18, 0.4, base=20.0, mask=3), ff=50),
     ]}
# E: windows and chunks of one token (a token sees itself alone), a latent wider than the rows of 64 lanes
E = {"architecture": "Ritalorn", "vocab": 120, "width": 48, "norm": {"eps": 1e-6}, "streams": 2, "logit_softcap": 20.0,
     "layers": [
         layer(latent(2, 8, 4, 12, 72, 0.2, base=100.0, mask=1), ff=32),
         layer(attention(2, 2, 16, 24, 0.5, conv=2, mask=1)),
         layer(latent(1, 40, 24, 72, 8, 0.1, base=7.0), ff=32),
     ]}
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}
SEEDS = {"A": 21, "B": 22, "C": 23, "D": 24, "E": 25}

STD = {"": 0.08, "embed": 0.5, ".conv": 0.4, ".b": 0.3, ".in": 0.6, ".out": 0.6, ".mix": 0.5, ".q": 0.25, ".uk": 0.25,
       ".dkv": 0.2, "head": 0.3}


def make_folder(tmp, name: str, cfg=None) -> str:
    """Write model `name` (or the given config under that name) with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    out = os.path.join(str(tmp), f"ritalorn_{name}")
    pae.write_model_folder(pae.read_config_dict(cfg or CONFIGS[name]), SEEDS.get(name, 5), out, std=STD, norm_std=0.2)
    return out


def read_folder(folder: str):
    """(config dict, tensors by name) read without the product's loader."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as handle:
        for key in handle.keys():
            tensors[key] = handle.get_tensor(key)
    return cfg, tensors


def tokens_for(name: str, length: int, salt: int = 0):
    gen = torch.Generator().manual_seed(1000 * SEEDS.get(name, 5) + length + salt)
    return torch.randint(0, CONFIGS[name]["vocab"], (length,), generator=gen).tolist()
