"""Small Ledudra configurations for the tests, and model folders with random weights for them.

The configurations differ from each other in every size and option: heads that share key/value heads and heads that
do not, groups of more than four heads, one head, values wider and narrower than keys, head sizes that are no
multiples of eight, windows shorter than a cache block and longer than one and no window at all, rotations over a part
of a head, over the whole head and none, with and without stretched frequencies, tables of an even and an odd number of
distance buckets that end inside and beyond the window, layers with and without a feed-forward and with and without
shared values in either order of the two mixers, and a number on the residual that is one and that is not.
"""
import json
import os

import torch

MIXED = {
    "architecture": "Ledudra", "vocab": 97, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 56},
         "mixer": {"heads": 6, "kv_heads": 3, "dim": 20, "vdim": 12, "mask": {"size": 17}, "scale": 0.3, "v_mix": True,
                   "rot": {"dims": 8, "base": 10000.0, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}}},
        {"type": "attention_2", "mlp": None,
         "mixer": {"heads": 4, "kv_heads": 1, "dim": 24, "vdim": 36, "mask": {"size": 70}, "scale": 0.2, "v_mix": True,
                   "bias_max": 50, "bias_rows": 10}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": 72},
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 18, "scale": 0.15, "v_mix": True,
                   "rot": {"dims": 32, "base": 500.0}}},
    ],
}
WIDE = {
    "architecture": "Ledudra", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "layers": [
        {"type": "attention_2", "mlp": {"kind": "dense", "ff": 96},
         "mixer": {"heads": 8, "kv_heads": 8, "dim": 16, "vdim": 8, "mask": {"size": 3}, "scale": 0.25, "v_mix": True,
                   "bias_max": 20, "bias_rows": 7}},
        {"type": "attention", "mlp": None,
         "mixer": {"heads": 8, "kv_heads": 1, "dim": 64, "vdim": 64, "mask": {"size": 129}, "scale": 0.125, "v_mix": True,
                   "rot": {"dims": 2, "base": 100.0, "scaling": {"factor": 2.0, "original": 32, "fast": 4.0, "slow": 1.0}}}},
        {"type": "attention_2", "mlp": {"kind": "dense", "ff": 40},
         "mixer": {"heads": 1, "kv_heads": 1, "dim": 136, "vdim": 64, "mask": {"size": 64}, "scale": 0.08, "v_mix": False,
                   "bias_max": 300, "bias_rows": 32}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": 24},
         "mixer": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 72, "mask": {"size": 1000}, "scale": 0.35, "v_mix": False}},
    ],
}
NARROW = {
    "architecture": "Ledudra", "vocab": 64, "width": 32, "norm": {"eps": 1e-3}, "residual_mult": 1.5,
    "layers": [
        {"type": "attention", "mlp": None,
         "mixer": {"heads": 1, "kv_heads": 1, "dim": 64, "vdim": 64, "mask": {"size": 1}, "scale": 0.125, "v_mix": False,
                   "rot": {"dims": 16, "base": 250.0}}},
        {"type": "attention_2", "mlp": {"kind": "dense", "ff": 32},
         "mixer": {"heads": 5, "kv_heads": 5, "dim": 10, "vdim": 6, "mask": {"size": 2}, "scale": 0.3, "v_mix": True,
                   "bias_max": 9, "bias_rows": 4}},
        {"type": "attention_2", "mlp": {"kind": "dense", "ff": 48},
         "mixer": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 30, "scale": 0.18, "v_mix": True, "bias_max": 64, "bias_rows": 16}},
    ],
}
CONFIGS = {"mixed": MIXED, "wide": WIDE, "narrow": NARROW}


def make_ledudra_folder(raw_config, folder, seed, std=0.2, keep_rows=True):
    """A model folder for `raw_config` with the library's random weights, where the small tensors are then given values that
    make them matter: norm weights near one and biases away from zero, shifts and value shares between 0 and 1, a mix of
    the heads that is no identity, numbers per head that leave some weights small and some large, a table of biases with
    rows that differ. With keep_rows False, config.json leaves the rows of the bias tables to the tensors' shapes."""
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
        parts = name.split(".")
        last = parts[-1]
        if last == "b":
            new = normal(tensor.shape, 0.0, 0.3)
        elif last == "norm" or last.startswith("norm"):
            new = normal(tensor.shape, 1.0, 0.3)
        elif last in ("shift", "vmix"):
            new = 0.1 + 0.8 * torch.rand(tensor.shape, generator=generator)
        elif last == "talk":
            new = torch.eye(tensor.shape[0]) + normal(tensor.shape, 0.0, 0.3)
        elif last == "pb":
            new = normal(tensor.shape, -1.0, 1.0)
        elif last == "rel":
            new = normal(tensor.shape, 0.0, 1.0)
        else:
            continue
        tensors[name] = new.to(tensor.dtype)
    write_safetensors(path, tensors)
    if not keep_rows:
        with open(os.path.join(folder, "config.json")) as handle:
            raw = json.load(handle)
        for layer in raw["layers"]:
            layer["mixer"].pop("bias_rows", None)
        with open(os.path.join(folder, "config.json"), "w") as handle:
            json.dump(raw, handle)
    return folder
