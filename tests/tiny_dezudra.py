"""Tiny Dezudra configurations that differ from each other in every size and option, and a folder of random weights
for each (norm weights drawn at random too, so that a norm taken for another one shows)."""
import json
import os

import numpy as np
import torch


def delta(heads, kv, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def attention(heads, kv, dim, vdim, conv, scale, diff, rot, mask, mlp):
    mixer = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale, "diff": diff}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
    if mask is not None:
        mixer["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def experts(ff, n, top, groups=None):
    router = {"experts": n, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def config(vocab, width, eps, logit_scale, layers):
    return {"architecture": "Dezudra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers, "initializer_range": 0.08}


# A: attention first, then the recurrent mixer; matrix-core sizes; three groups of which two are kept; windows of
# two sizes, one that keeps no first tokens
A = config(320, 96, 1e-5, 0.5, [
    attention(6, 2, 32, 32, 4, 0.2, 0.3, (32, 10000.0), (24, 3), experts(64, 6, 2, (3, 2))),
    delta(4, 4, 16, 48, 2, experts(64, 6, 2, (3, 2))),
    attention(2, 2, 16, 48, 2, 0.3, 0.8, (8, 500.0), (9, 0), experts(40, 4, 4, (2, 2))),
])
# B: sizes that are no multiple of 4 or 16; one key/value head; a layer without feed-forward; one expert per token;
# a convolution of one tap (no state at all) and one of five; every token seen (no mask); no rotation in one layer
B = config(131, 72, 1e-6, 1.0, [
    delta(3, 1, 20, 12, 5, experts(36, 5, 1)),
    attention(3, 1, 12, 20, 1, 0.25, 0.5, None, None, None),
    attention(6, 3, 20, 12, 3, 0.22, 0.1, (10, 100.0), (17, 5), experts(52, 9, 3, (3, 1))),
    delta(2, 2, 24, 40, 1, None),
])
# C: one head everywhere, a window of one token plus kept first tokens, a keep_first larger than a page
C = config(97, 40, 1e-5, 2.0, [
    attention(1, 1, 16, 16, 2, 0.25, 0.6, (16, 10000.0), (1, 2), experts(24, 2, 1, (2, 1))),
    delta(1, 1, 16, 16, 3, experts(24, 2, 2, (1, 1))),
    attention(1, 1, 16, 16, 2, 0.25, 0.2, (4, 10000.0), (6, 20), experts(24, 3, 2)),
])
# D: wider heads (the recurrent state's rows spread over more registers), values wider than 64, many experts
D = config(256, 128, 1e-5, 0.25, [
    delta(2, 1, 128, 80, 4, experts(32, 16, 4, (4, 2))),
    attention(4, 1, 64, 96, 4, 0.125, 0.4, (32, 1000.0), (33, 1), experts(32, 16, 4, (8, 3))),
])
# E: recurrent layers only (nothing is kept in pages), a width and a vocabulary that are no multiple of 8, groups of one
# expert, the logits' scale left to its default
E = config(77, 90, 1e-5, 1.0, [
    delta(2, 1, 24, 20, 3, experts(28, 6, 2, (6, 3))),
    delta(3, 3, 10, 14, 2, experts(28, 3, 1, (1, 1))),
])
del E["logit_scale"]
# F: attention layers only, key/value heads omitted (as many as heads), values as wide as keys by omission, more
# query heads per key/value head than a tile has columns
F = config(203, 104, 1e-6, 0.125, [
    attention(5, 5, 16, 16, 2, 0.3, 0.25, (6, 77.0), (11, 1), experts(44, 8, 3, (4, 2))),
    attention(34, 1, 16, 8, 3, 0.2, 0.7, None, (5, 6), experts(44, 8, 8, (2, 2))),
])
for _name in ("kv_heads", "vdim"):
    del F["layers"][0]["mixer"][_name]
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F}


def make_folder(raw_config: dict, seed: int, out_dir: str, dtype: str = "bfloat16") -> str:
    from safetensors.torch import load_file, save_file
    from inferx_amd.config import config_from_dict
    from inferx_amd.weights import write_model_folder
    write_model_folder(config_from_dict(json.loads(json.dumps(raw_config))), seed, out_dir, dtype)
    path = os.path.join(out_dir, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed + 1)
    for name, t in tensors.items():
        last = name.split(".")[-1]
        if last.startswith("norm") and t.dim() == 1:  # l<i>.norm1, .norm1b, ..., final.norm, l<i>.mix.norm
            tensors[name] = (1.0 + 0.3 * torch.randn(t.shape, generator=g)).to(t.dtype)
    save_file(tensors, path)
    return out_dir


def read_folder(model_dir: str):
    """config dict and tensors as float64 arrays, through the safetensors library (not the framework's reader)."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    tensors = load_file(os.path.join(model_dir, "model.safetensors"))
    return cfg, {k: v.to(torch.float64).numpy() for k, v in tensors.items()}


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
