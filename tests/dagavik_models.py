"""Small Dagavik configurations for the tests, their random weights, and tokens to replay.

The configurations differ from one another in every size and constant and in the order of their layers:
grouped and ungrouped heads, value widths above and below the key width, rotations over part of a head,
over all of it and none, windows of a few tokens, of more than a page and none, matrix memories with one
head and with several, latent layers that read their own rows and an earlier layer's (two readers of one
layer too), delta rules with grouped keys, one to four taps and narrow products of several widths, experts
in one group and in several with one or more kept, one expert chosen and several, layers without a
feed-forward, no bigram table, widths the few-row product kernels take and widths they do not.
Weights are drawn so that no mechanism hides: sinks about a unit wide, gates' biases and decays spread,
convolution taps of both signs, norm weights (stored around zero) a fifth wide, routers wide enough that
the scores differ between experts.
"""

from __future__ import annotations

import json
import os

import torch


def window(heads, kv_heads, dim, vdim, scale, size=None, rot_dims=None, base=10000.0):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size is not None:
        out["mask"] = {"size": size}
    if rot_dims is not None:
        out["rot"] = {"base": base, "dims": rot_dims}
    return out


def parallel(left, heads, dim, vdim, cap, left_scale, right_scale):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale, "right_scale": right_scale,
                                          "right": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}}


def latent(heads, dim, vdim, rank, scale, kv_from=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": decay_rank, "gate_rank": gate_rank}}


def moe(ff, experts, top, scale, count=None, keep=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if count is not None:
        router["groups"] = {"count": count, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(mixer, mlp=None):
    return dict(mixer, mlp=mlp)


# U: all three mixers, a window shorter than a page, two groups of experts with one kept
U = {"architecture": "Dagavik", "vocab": 300, "width": 64, "norm": {"eps": 2e-6},
     "embedding": {"bigram": {"buckets": 101, "mul_prev": 13, "mul_cur": 5}}, "layers": [
         layer(parallel(window(4, 2, 16, 24, 0.3, size=11, rot_dims=8, base=500.0), 2, 16, 24, 8.0, 0.7, 1.2), moe(24, 6, 2, 1.7, 2, 1)),
         layer(latent(4, 16, 8, 32, 0.3), moe(16, 4, 1, 1.0)),
         layer(delta(4, 2, 16, 24, 3, 8, 16), moe(24, 6, 2, 1.7, 2, 1)),
         layer(latent(2, 24, 16, 32, 0.25, kv_from=1)),
     ]}
# W: a delta layer first, a width the few-row products do not take, one key/value head, three groups with two kept, a
# window longer than a page, a latent layer read by two others
W = {"architecture": "Dagavik", "vocab": 211, "width": 100, "norm": {"eps": 1e-5},
     "embedding": {"bigram": {"buckets": 64, "mul_prev": 1, "mul_cur": 1}}, "layers": [
         layer(delta(3, 3, 20, 36, 4, 12, 5), moe(30, 9, 3, 0.8, 3, 2)),
         layer(latent(3, 20, 28, 48, 0.2), moe(20, 5, 5, 2.0)),
         layer(parallel(window(3, 1, 48, 80, 0.2, size=37, rot_dims=48, base=2000.0), 1, 40, 12, 15.0, 1.0, 0.5)),
         layer(latent(5, 12, 12, 48, 0.3, kv_from=1), moe(30, 9, 3, 0.8, 3, 2)),
         layer(latent(2, 32, 8, 48, 0.2, kv_from=1), moe(12, 2, 1, 1.0, 2, 1)),
     ]}
# X: recurrent mixers with a full causal attention beside the memory (no window, no rotation), no bigram table, one tap
X = {"architecture": "Dagavik", "vocab": 150, "width": 48, "norm": {"eps": 1e-6}, "layers": [
         layer(parallel(window(2, 2, 24, 8, 0.35), 3, 8, 40, 4.0, 0.4, 1.0), moe(32, 8, 2, 2.5, 4, 2)),
         layer(delta(2, 1, 72, 16, 1, 4, 4), moe(16, 3, 2, 1.0)),
         layer(delta(4, 4, 8, 40, 2, 16, 8)),
     ]}
# Y: shapes the matrix-core kernels take (heads and values of 64 and 32, pages of 16, a latent row of 64), a
# window of exactly two pages
Y = {"architecture": "Dagavik", "vocab": 400, "width": 128, "norm": {"eps": 1e-5},
     "embedding": {"bigram": {"buckets": 257, "mul_prev": 31, "mul_cur": 7}}, "layers": [
         layer(latent(4, 32, 32, 64, 0.25), moe(64, 8, 2, 2.0, 2, 1)),
         layer(parallel(window(8, 2, 64, 64, 0.18, size=32, rot_dims=32, base=3000.0), 4, 32, 32, 10.0, 0.9, 0.6), moe(64, 8, 2, 2.0, 2, 1)),
         layer(delta(4, 2, 32, 32, 4, 24, 24), moe(32, 4, 2, 1.5)),
         layer(parallel(window(4, 4, 32, 32, 0.25, size=16, rot_dims=16, base=100.0), 2, 64, 64, 12.0, 0.5, 1.5)),
         layer(latent(8, 16, 16, 64, 0.3, kv_from=0), moe(64, 8, 2, 2.0, 2, 1)),
     ]}
# Z: nothing is a multiple of four; values as wide as keys at a width the first attention path does not take; a window
# of one token (a token sees itself alone)
Z = {"architecture": "Dagavik", "vocab": 97, "width": 90, "norm": {"eps": 1e-5},
     "embedding": {"bigram": {"buckets": 7, "mul_prev": 1000003, "mul_cur": 999983}}, "layers": [
         layer(parallel(window(3, 3, 22, 22, 0.3, size=1, rot_dims=10, base=50.0), 3, 10, 14, 6.0, 1.1, 0.9), moe(14, 6, 1, 3.0, 3, 1)),
         layer(delta(3, 1, 10, 14, 3, 6, 10), moe(10, 7, 3, 0.5)),
         layer(latent(3, 10, 14, 22, 0.35), moe(14, 6, 1, 3.0, 3, 1)),
     ]}
CONFIGS = {"U": U, "W": W, "X": X, "Y": Y, "Z": Z}
SEEDS = {"U": 21, "W": 22, "X": 23, "Y": 24, "Z": 25}

STD = {"": 0.08, "embed": 0.5, "bigram": 0.3, "sink": 1.5, "A_log": 0.7, "dt_bias": 1.0, ".conv": 0.4, ".b": 0.5,
       "router": 0.6, "norm1": 0.2, "norm2": 0.2, "final.norm": 0.2, "mix.i": 0.3, "mix.f": 0.3}


def make_folder(tmp, name: str, cfg=None, std=None) -> str:
    """Write model `name` (or the given config under that name) with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    out = os.path.join(str(tmp), f"dagavik_{name}")
    pae.write_model_folder(pae.read_config_dict(cfg or CONFIGS[name]), SEEDS.get(name, 5), out, std=std or STD, norm_std=0.2)
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
