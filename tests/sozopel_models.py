"""Small Sozopel configurations for the tests, and model folders with random weights for them.

The configurations differ from each other in every size and option: heads that share key/value heads and heads that
do not, one head, values wider and narrower than keys, windows shorter than a cache block and longer than one,
convolutions of one to five taps, layers with and without a feed-forward in every order.
"""
import os

import torch

MIXED = {
    "architecture": "Sozopel", "vocab": 101, "width": 40, "max_positions": 320, "norm": {"eps": 1e-5}, "canon": {"taps": 3},
    "layers": [
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 72},
         "mixer": {"left": {"heads": 6, "kv_heads": 3, "dim": 24, "vdim": 40, "conv": 2, "mask": {"size": 17}, "scale": 0.3},
                   "right": {"heads": 3, "dim": 16, "vdim": 24, "tau": 7.0, "rank": 5}}},
        {"type": "retention", "mlp": {"kind": "dense", "ff": 56},
         "mixer": {"heads": 3, "dim": 20, "vdim": 36, "decay": [0.9, 0.99609375, 0.5]}},
        {"type": "wkv", "mlp": None, "mixer": {"heads": 2, "dim": 24, "rank": 6}},
    ],
}
WIDE = {
    "architecture": "Sozopel", "vocab": 128, "width": 64, "max_positions": 256, "norm": {"eps": 1e-6}, "canon": {"taps": 5},
    "layers": [
        {"type": "wkv", "mlp": {"kind": "dense", "ff": 96}, "mixer": {"heads": 1, "dim": 64, "rank": 8}},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "conv": 4, "mask": {"size": 70}, "scale": 0.2},
                   "right": {"heads": 1, "dim": 32, "vdim": 136, "tau": 1.0, "rank": 4}}},
        {"type": "retention", "mlp": None, "mixer": {"heads": 1, "dim": 8, "vdim": 72, "decay": [0.953125]}},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 40},
         "mixer": {"left": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 8, "conv": 1, "mask": {"size": 3}, "scale": 1.0},
                   "right": {"heads": 2, "dim": 136, "vdim": 16, "tau": 30.0, "rank": 16}}},
    ],
}
ONE_TAP = {
    "architecture": "Sozopel", "vocab": 64, "width": 32, "max_positions": 192, "norm": {"eps": 1e-3}, "canon": {"taps": 1},
    "layers": [
        {"type": "retention", "mlp": {"kind": "dense", "ff": 32}, "mixer": {"heads": 2, "dim": 32, "vdim": 16, "decay": [1.0, 0.75]}},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 1, "kv_heads": 1, "dim": 64, "vdim": 64, "conv": 5, "mask": {"size": 1000}, "scale": 0.125},
                   "right": {"heads": 2, "dim": 16, "vdim": 16, "tau": 4.0, "rank": 8}}},
    ],
}
CONFIGS = {"mixed": MIXED, "wide": WIDE, "one_tap": ONE_TAP}


def make_sozopel_folder(raw_config, folder, seed, std=0.2, keep_rank=True):
    """A model folder for `raw_config` with the library's random weights, where the small tensors are then given values that
    make them matter: gains near one, mixes between 0 and 1, decays that neither forget at once nor keep everything, a bonus
    and activation numbers away from zero. With keep_rank False, config.json leaves the inner widths of the decay
    projections to the tensors' shapes."""
    import json

    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.weights import SafetensorsFile, write_random_model, write_safetensors

    folder = str(folder)
    write_random_model(parse_config(raw_config), folder, seed=seed, std=std)
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as file:
        tensors = {name: file.read(name) for name in file.names()}
    generator = torch.Generator().manual_seed(seed + 1)

    def normal(shape, mean, deviation):
        return mean + deviation * torch.randn(shape, generator=generator)

    for name, tensor in tensors.items():
        last = name.split(".")[-1]
        if tensor.dim() == 0 or last in ("norm", "out"):
            new = normal(tensor.shape, 1.0, 0.3)
        elif ".mu." in name:
            new = torch.rand(tensor.shape, generator=generator)
        elif last == "w0":
            new = normal(tensor.shape, -2.0, 1.0)
        elif name.endswith("a2.b"):
            new = normal(tensor.shape, 2.0, 1.0)
        elif last in ("u", "act"):
            new = normal(tensor.shape, 0.0, 0.5)
        elif last == "conv" or "canon" in last:
            new = normal(tensor.shape, 0.0, 0.5)
        elif last == "pos":
            new = normal(tensor.shape, 0.0, 0.5)
        else:
            continue
        tensors[name] = new.to(tensor.dtype)
    write_safetensors(path, tensors)
    if not keep_rank:
        with open(os.path.join(folder, "config.json")) as handle:
            raw = json.load(handle)
        for layer in raw["layers"]:
            (layer["mixer"] if layer["type"] != "parallel" else layer["mixer"]["right"]).pop("rank", None)
        with open(os.path.join(folder, "config.json"), "w") as handle:
            json.dump(raw, handle)
    return folder
