"""Small Zikezen configurations for the tests, their random weights, and tokens to replay.

The configurations differ from one another in every size and constant and in the order of their layers: grouped,
ungrouped and single key/value heads, value widths above and below the key width, rotations over part of a head, over
all of it and none, with stretched frequencies and without, windows of one token, of less than a page, of exactly two
pages, of more than a page and none, linear attention with one head and with several and key widths that take each of
the recurrence's lane groupings, narrow products that are and are not multiples of eight, dense and routed
feed-forwards and layers without one, one expert chosen, several and all, layers run once, twice and three times from
the first layer on or from a later one, a second token table and none, a logit cap and none, widths the few-row product
kernels take and widths they do not.  Weights are drawn so that no mechanism hides: biases half a unit wide, decays'
biases spread, norm weights a fifth wide, routers wide enough that the scores differ between experts (and no wider: a
router whose logits are many units wide turns a rounding of the stream into another choice) and corrections
large enough to change the choice, positions and the second token table as large as the embedding.
"""

from __future__ import annotations

import json
import os

import torch


def left(heads, kv_heads, dim, vdim, scale, size=None, rot_dims=None, base=10000.0, scaling=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size is not None:
        out["mask"] = {"size": size}
    if rot_dims is not None:
        out["rot"] = {"base": base, "dims": rot_dims}
        if scaling is not None:
            out["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def right(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank}


def layer(left_mixer, right_mixer, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left_mixer, "right": right_mixer, "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


# P: the middle layers twice; dense, routed and no feed-forward; a window shorter than a page; stretched frequencies
# of which one pair is kept, one blended and two divided
P = {"architecture": "Zikezen", "vocab": 300, "width": 64, "max_positions": 256, "embedding": {"scale": 0.7},
     "norm": {"eps": 2e-6}, "loop": {"start": 1, "stop": 3, "times": 2}, "token_side": {"dim": 8}, "logit_softcap": 20.0,
     "layers": [
         layer(left(4, 2, 16, 24, 0.3, size=11, rot_dims=8, base=500.0, scaling=(8.0, 1.0, 4.0, 64)), right(2, 16, 24, 4.0, 8), 0.7, 1.2, dense(40)),
         layer(left(4, 4, 16, 8, 0.25, size=20, rot_dims=16, base=100.0), right(3, 8, 40, 16.0, 4), 1.1, 0.6, moe(24, 6, 2)),
         layer(left(2, 1, 24, 16, 0.2, size=5, rot_dims=12, base=1000.0, scaling=(2.0, 1.0, 2.0, 32)), right(1, 24, 16, 2.0, 5), 0.5, 1.5),
         layer(left(4, 2, 16, 24, 0.3, size=11, rot_dims=8, base=500.0, scaling=(8.0, 1.0, 4.0, 64)), right(2, 16, 24, 4.0, 8), 1.0, 1.0, moe(16, 4, 1)),
     ]}
# Q: a width the few-row products do not take, one key/value head, a window longer than a page, the first two layers
# three times, every expert chosen, no second token table, no logit cap, the embedding as it is
Q = {"architecture": "Zikezen", "vocab": 211, "width": 100, "max_positions": 200, "norm": {"eps": 1e-5},
     "loop": {"start": 0, "stop": 2, "times": 3}, "layers": [
         layer(left(3, 1, 48, 80, 0.2, size=37, rot_dims=48, base=2000.0), right(3, 20, 36, 8.0, 12), 1.0, 0.5, moe(20, 5, 5)),
         layer(left(6, 3, 20, 12, 0.3, size=17, rot_dims=4, base=50.0, scaling=(4.0, 1.0, 4.0, 16)), right(1, 40, 12, 32.0, 7), 0.8, 0.8, dense(30)),
         layer(left(2, 2, 28, 28, 0.25), right(2, 72, 16, 3.0, 16), 1.3, 0.4, moe(30, 9, 3)),
     ]}
# R: shapes the matrix-core kernels take (heads and values of 64 and 32, pages of 16, expert widths in multiples of 32),
# a window of exactly two pages and one of exactly one; the only layer with experts runs twice
R = {"architecture": "Zikezen", "vocab": 400, "width": 128, "max_positions": 512, "embedding": {"scale": 1.5},
     "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 2, "times": 2}, "token_side": {"dim": 16}, "logit_softcap": 12.0,
     "layers": [
         layer(left(8, 2, 64, 64, 0.18, size=32, rot_dims=32, base=3000.0, scaling=(4.0, 1.0, 4.0, 128)), right(4, 32, 32, 16.0, 16), 0.9, 0.6, dense(256)),
         layer(left(4, 4, 32, 32, 0.25, size=16, rot_dims=16, base=100.0), right(2, 64, 64, 6.0, 24), 0.5, 1.5, moe(64, 8, 2)),
         layer(left(4, 1, 32, 32, 0.2, rot_dims=32, base=10000.0), right(1, 128, 32, 10.0, 8), 1.0, 1.0),
     ]}
# S: nothing is a multiple of four; a window of one token (a token sees itself and the sink); attention without a
# window and without a rotation; a temperature of one; no loop
S = {"architecture": "Zikezen", "vocab": 97, "width": 90, "max_positions": 160, "embedding": {"scale": 0.9},
     "norm": {"eps": 1e-5}, "token_side": {"dim": 5}, "layers": [
         layer(left(3, 3, 22, 22, 0.3, size=1, rot_dims=10, base=50.0), right(3, 10, 14, 1.0, 3), 1.1, 0.9, moe(14, 7, 3)),
         layer(left(5, 1, 18, 10, 0.35), right(2, 6, 26, 5.0, 9), 0.6, 1.4, dense(50)),
     ]}
CONFIGS = {"P": P, "Q": Q, "R": R, "S": S}
SEEDS = {"P": 31, "Q": 32, "R": 33, "S": 34}

STD = {"": 0.08, "embed": 0.5, "pos": 0.3, "a2.b": 1.0, ".b": 0.5, "a1": 0.3, "a2": 0.4, "router": 0.2, "correction": 0.1,
       "left.q": 0.2, "left.k": 0.2}


def make_folder(tmp, name: str, cfg=None, std=None) -> str:
    """Write model `name` (or the given config under that name) with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    out = os.path.join(str(tmp), f"zikezen_{name}")
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
