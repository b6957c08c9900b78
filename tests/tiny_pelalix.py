"""Tiny Pelalix configurations that differ from each other in every size and option, and a folder of random
weights for each."""
import json
import os

import torch


def _layer(heads, kv, dim, vdim, scale, v_mix, ff):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _config(vocab, width, scale, eps, layers):
    return {"architecture": "Pelalix", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "layers": layers, "initializer_range": 0.08}


# P: the matrix-core sizes (heads of 32 and 16 numbers), three layers that all mix their values
P = _config(320, 96, 4.0, 1e-5, [_layer(6, 3, 32, 16, 0.2, True, 160) for _ in range(3)])
# Q: one key/value head, values wider than keys, a layer without feed-forward, the first layer does not mix its
# values (so the source of the mixing is layer 1), sizes that are no multiple of 16
Q = _config(131, 72, 1.0, 1e-6, [_layer(4, 1, 24, 40, 0.3, False, 100), _layer(4, 1, 24, 40, 0.25, True, None),
                                 _layer(2, 2, 48, 40, 0.15, False, 52), _layer(8, 1, 16, 40, 0.2, True, 88)])
# R: as many key/value heads as heads, one layer, one head size of 64 and values of 64
R = _config(256, 128, 8.0, 1e-5, [_layer(2, 2, 64, 64, 0.125, True, 256)])
# S: a single head
S = _config(97, 40, 2.0, 1e-5, [_layer(1, 1, 16, 16, 0.25, True, 64), _layer(1, 1, 16, 16, 0.25, True, 64)])
# U: nothing is a multiple of 4 where the design allows it; the embedding's scale is left to its default
U = _config(77, 90, 1.0, 1e-5, [_layer(3, 1, 20, 12, 0.22, True, 50), _layer(6, 1, 20, 12, 0.3, True, 70)])
del U["embedding"]
CONFIGS = {"P": P, "Q": Q, "R": R, "S": S, "U": U}


def make_folder(raw_config: dict, seed: int, out_dir: str, dtype: str = "bfloat16") -> str:
    from inferx_amd.config import config_from_dict
    from inferx_amd.weights import write_model_folder
    write_model_folder(config_from_dict(dict(raw_config)), seed, out_dir, dtype)
    return out_dir


def read_folder(model_dir: str):
    """config dict and tensors, through the safetensors library (not the framework's reader)."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, load_file(os.path.join(model_dir, "model.safetensors"))


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
