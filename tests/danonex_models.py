"""Small Danonex configurations for the tests, their random weights, and schedules to replay.

The configurations differ from one another in every size and constant: grouped and ungrouped
heads, value widths above and below the key width, rotations over part of a head and over all of
it, with and without stretched frequencies, with and without a score cap, convolutions of two to
four taps, layers with and without a feed-forward, widths that the few-row product kernels take
(multiples of 8) and one that they do not, residual multipliers and logit scales other than one.
Weights are drawn so that no mechanism hides: sinks about a unit wide, decays and write strengths
spread over (0, 1), convolution taps of both signs, and score scales that make attention peaked.
"""

from __future__ import annotations

import json
import os

import torch


def attention(heads, kv_heads, dim, vdim, scale, softcap=None, rot_dims=None, base=10000.0, scaling=None):
    rot = None if rot_dims is None else {"base": base, "dims": rot_dims, "scaling": scaling}
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale, "softcap": softcap, "rot": rot}}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def layer(mixer, ff=None):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


YARN_A = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
YARN_B = {"factor": 2.5, "original": 512, "fast": 24.0, "slow": 0.5}

# P: both mixers, grouped heads, value widths unlike the key widths, a rotation over half a head
P = {"architecture": "Danonex", "vocab": 300, "width": 64, "norm": {"eps": 2e-6}, "residual_mult": 1.0,
     "logit_scale": 1.0, "layers": [
         layer(delta(4, 2, 16, 24, 3), ff=96),
         layer(attention(6, 2, 32, 16, 0.45, softcap=12.0, rot_dims=16, base=500.0, scaling=YARN_A)),
         layer(attention(2, 2, 64, 64, 0.3, softcap=None, rot_dims=64, base=10000.0, scaling=None), ff=80),
         layer(delta(2, 1, 40, 8, 2)),
     ]}
# Q: a width the few-row product kernels do not take, one key/value head, heads of 48 and values of 80
Q = {"architecture": "Danonex", "vocab": 211, "width": 100, "norm": {"eps": 1e-5}, "residual_mult": 0.4,
     "logit_scale": 3.0, "layers": [
         layer(attention(3, 1, 48, 80, 0.35, softcap=20.0, rot_dims=24, base=2000.0, scaling=YARN_B), ff=130),
         layer(delta(3, 3, 20, 36, 4), ff=60),
         layer(attention(4, 4, 16, 8, 0.6, softcap=5.0, rot_dims=None)),
     ]}
# R: the recurrent mixer alone (a model that keeps no pages at all), and keys wider than a lane group's first share
R = {"architecture": "Danonex", "vocab": 150, "width": 48, "norm": {"eps": 1e-6}, "residual_mult": 1.3,
     "logit_scale": 0.5, "layers": [
         layer(delta(2, 2, 72, 16, 4), ff=64),
         layer(delta(4, 1, 8, 40, 1)),
     ]}
# S: shapes the matrix-core attention kernels take (heads and values of 64 and 32, pages of 16)
S = {"architecture": "Danonex", "vocab": 400, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
     "logit_scale": 0.7, "layers": [
         layer(attention(8, 2, 64, 64, 0.4, softcap=15.0, rot_dims=32, base=3000.0, scaling=YARN_A), ff=192),
         layer(delta(4, 2, 32, 32, 4)),
         layer(attention(3, 3, 32, 32, 0.5, softcap=None, rot_dims=32, base=100.0, scaling=None), ff=64),
     ]}
# T: nothing is a multiple of four: width 90, vocabulary 97, heads of 22 and 10, values of 18 and 14
T = {"architecture": "Danonex", "vocab": 97, "width": 90, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
     "logit_scale": 1.5, "layers": [
         layer(attention(3, 3, 22, 18, 0.5, softcap=9.0, rot_dims=10, base=50.0, scaling=YARN_A), ff=70),
         layer(delta(3, 1, 10, 14, 3), ff=50),
     ]}
CONFIGS = {"P": P, "Q": Q, "R": R, "S": S, "T": T}
SEEDS = {"P": 11, "Q": 12, "R": 13, "S": 14, "T": 15}

STD = {"": 0.08, "embed": 0.5, "sink": 1.5, "A_log": 0.7, "dt_bias": 1.0, ".conv": 0.4, ".b": 0.3, ".a": 0.3}


def make_folder(tmp, name: str, cfg=None) -> str:
    """Write model `name` (or the given config under that name) with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    out = os.path.join(str(tmp), f"danonex_{name}")
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
