"""The Ledudra decoder in plain arithmetic: whole sequences, no cache, one function per mechanism.

Slow on purpose (loops over tokens and heads, float64 throughout) and written from the design's equations alone; it
shares no code with the package. A model is a dict of tensors by checkpoint name plus the raw configuration.

Notation: x is the residual stream [T, W]; h what a sublayer reads; i a query's position and j a key's, both counted
from 0 in one sequence; H query heads, G key/value heads, d the key size and e the value size of a head.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

F = torch.float64


# ---- reading a folder ----------------------------------------------------------------------------------------

def read_folder(folder):
    """(raw configuration, {name: float64 tensor}) of a folder with config.json and model.safetensors."""
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    with open(os.path.join(folder, "model.safetensors"), "rb") as handle:
        size = struct.unpack("<Q", handle.read(8))[0]
        header = json.loads(handle.read(size))
        data = handle.read()
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32}
    tensors = {}
    for name, entry in header.items():
        if name == "__metadata__":
            continue
        lo, hi = entry["data_offsets"]
        flat = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[entry["dtype"]])
        tensors[name] = flat.reshape(entry["shape"]).to(F)
    return raw, tensors


# ---- small pieces --------------------------------------------------------------------------------------------

def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * w + b over the last dimension."""
    mean = x.mean(-1, keepdim=True)
    var = (x - mean).pow(2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def sigmoid(z):
    return 1 / (1 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def towards_the_token_before(h, mu):
    """h_t + (h_(t-1) - h_t) * mu, with zeros before the first token; the h on the right are the rows as given."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (before - h) * mu


# ---- positions -----------------------------------------------------------------------------------------------

def rotary_frequencies(dims, base, scaling=None):
    """(frequency of pair n for n < dims / 2, the number that multiplies cosines and sines).
    Without scaling f_n = base^(-2n / dims) and 1. With {factor, original, fast, slow}: the pair index at which a
    wave of t turns over the original length, c(t) = dims ln(original / (2 pi t)) / (2 ln base); lo = max(floor(c(fast)), 0),
    hi = min(ceil(c(slow)), dims - 1); r_n = clamp((n - lo) / max(hi - lo, 0.001), 0, 1); the frequency becomes
    f_n / factor * r_n + f_n (1 - r_n), and the multiplier 0.1 ln(factor) + 1."""
    freqs = [base ** (-2.0 * n / dims) for n in range(dims // 2)]
    if not scaling:
        return torch.tensor(freqs, dtype=F), 1.0

    def turns_at(t):
        return dims * math.log(scaling["original"] / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(turns_at(scaling["fast"])), 0)
    hi = min(math.ceil(turns_at(scaling["slow"])), dims - 1)
    out = []
    for n, f in enumerate(freqs):
        r = min(max((n - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / scaling["factor"] * r + f * (1 - r))
    return torch.tensor(out, dtype=F), 0.1 * math.log(scaling["factor"]) + 1.0


def rotate_neighbours(u, positions, freqs, magnitude):
    """u [T, heads, d]: dims (2n, 2n + 1) for n < len(freqs) turn by the angle position * freqs[n]; the rest stay."""
    out = u.clone()
    for t, p in enumerate(positions):
        for n, f in enumerate(freqs.tolist()):
            c, s = math.cos(p * f) * magnitude, math.sin(p * f) * magnitude
            a, b = u[t, :, 2 * n], u[t, :, 2 * n + 1]
            out[t, :, 2 * n] = a * c - b * s
            out[t, :, 2 * n + 1] = b * c + a * s
    return out


def distance_bucket(n, rows, far):
    """Row of a table of `rows` rows for a distance n >= 0: the distance itself below half the rows, then steps that grow
    logarithmically and reach the last row at distance `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


# ---- the two mixers ------------------------------------------------------------------------------------------

def visible(i, j, window):
    """Whether the query at position i sees the key at position j: itself and the window - 1 tokens before it."""
    return 0 <= i - j and (window is None or i - j < window)


def gated_sigmoid_attention(h, positions, m, t, p, v_first):
    """Mixer 'attention'. Returns (output [T, W], the values [T, G, e] that were used)."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).reshape(T, H, d)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).reshape(T, G, d)
    v = (h @ t[p + "v"].T + t[p + "v.b"]).reshape(T, G, e)
    rot = m.get("rot")
    if rot:
        freqs, magnitude = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_neighbours(q, positions, freqs, magnitude), rotate_neighbours(k, positions, freqs, magnitude)
    if m.get("v_mix") and v_first is not None:
        lam = t[p + "vmix"]
        v = (1 - lam) * v + lam * v_first.reshape(T, G, e)       # (a token's values side by side, however the heads cut them)
    window = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, e, dtype=F)
    for a in range(T):
        seen = [b for b in range(T) if visible(positions[a], positions[b], window)]
        raw = torch.stack([k[seen, head // (H // G)] @ q[a, head] for head in range(H)]) * m["scale"]      # [H, keys]
        mixed = t[p + "talk"] @ raw                                    # every head's score is a mix of all heads' scores
        weight = sigmoid(mixed + t[p + "pb"][:, None])                 # no normalisation over the keys
        for head in range(H):
            out[a, head] = weight[head] @ v[seen, head // (H // G)]
    gate = sigmoid(h @ t[p + "g"].T)                                   # [T, H]
    out = out * gate[:, :, None]
    return out.reshape(T, H * e) @ t[p + "o"].T + t[p + "o.b"], v


def biased_softmax_attention(h, positions, m, t, p, v_first, eps):
    """Mixer 'attention_2'. Returns (output [T, W], the values [T, G, e] that were used)."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ t[p + "q"].T).reshape(T, H, d), t[p + "q.norm"], eps)
    k = rms_norm((h @ t[p + "k"].T).reshape(T, G, d), t[p + "k.norm"], eps)
    v = (h @ t[p + "v"].T).reshape(T, G, e)
    if m.get("v_mix") and v_first is not None:
        lam = t[p + "vmix"]
        v = (1 - lam) * v + lam * v_first.reshape(T, G, e)       # (a token's values side by side, however the heads cut them)
    window = (m.get("mask") or {}).get("size")
    rel = t[p + "rel"]
    out = torch.zeros(T, H, e, dtype=F)
    for head in range(H):
        for a in range(T):
            seen = [b for b in range(T) if visible(positions[a], positions[b], window)]
            bias = torch.stack([rel[distance_bucket(positions[a] - positions[b], rel.shape[0], m["bias_max"]), head] for b in seen])
            scores = k[seen, head // (H // G)] @ q[a, head] * m["scale"] + bias
            out[a, head] = torch.softmax(scores, 0) @ v[seen, head // (H // G)]
    return out.reshape(T, H * e) @ t[p + "o"].T, v


def gated_feed_forward(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


# ---- the model -----------------------------------------------------------------------------------------------

def forward(raw, t, tokens, keep_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer, if asked)."""
    eps, mult = raw["norm"]["eps"], raw["residual_mult"]
    positions = list(range(len(tokens)))
    x = t["embed"][torch.tensor(tokens, dtype=torch.long)]
    v_first, after = None, []
    for index, layer in enumerate(raw["layers"]):
        p = f"l{index}."
        h = layer_norm(x, t[p + "norm1"], t[p + "norm1.b"], eps)
        h = towards_the_token_before(h, t[p + "shift"])
        if layer["type"] == "attention":
            y, v = gated_sigmoid_attention(h, positions, layer["mixer"], t, p + "mix.", v_first)
        else:
            y, v = biased_softmax_attention(h, positions, layer["mixer"], t, p + "mix.", v_first, eps)
        if layer["mixer"].get("v_mix") and v_first is None:
            v_first = v
        x = x + mult * layer_norm(y, t[p + "norm1b"], t[p + "norm1b.b"], eps)
        if layer.get("mlp"):
            y = gated_feed_forward(layer_norm(x, t[p + "norm2"], t[p + "norm2.b"], eps), t, p + "mlp.")
            x = x + mult * layer_norm(y, t[p + "norm2b"], t[p + "norm2b.b"], eps)
        after.append(x)
    logits = layer_norm(x, t["final.norm"], t["final.norm.b"], eps) @ t["head"].T
    return (logits, torch.stack(after)) if keep_layers else logits


class PlainModel:
    def __init__(self, folder):
        self.raw, self.tensors = read_folder(folder)

    def logits(self, tokens):
        return forward(self.raw, self.tensors, list(tokens))
