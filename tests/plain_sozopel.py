"""The Sozopel decoder in plain arithmetic: whole sequences, no cache, one function per mechanism.

Slow on purpose (loops over tokens, float64 throughout) and written from the design's equations alone; it shares
no code with the package. A model is a dict of tensors by checkpoint name plus the raw configuration.

Notation: x is the residual stream [T, W]; h what a sublayer reads; t counts tokens of one sequence from 0.
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

def rms_divide(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def silu(z):
    return z / (1 + torch.exp(-z))


def causal_conv(u, w):
    """y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the sequence. u [T, C], w [C, taps]."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def xielu(z, p, q):
    ap, an = softplus(p), 0.5 + softplus(q)
    pos = ap * z * z + z / 2
    neg = an * (torch.expm1(torch.clamp(z, max=0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def recurrence(q, k, v, decay, bonus=None):
    """Per head a matrix state S [dim, vdim], zero at the start.
    Without bonus: S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.
    With bonus u [H, dim]: o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, then the same update.
    q, k, decay [T, H, dim]; v [T, H, vdim]; returns o [T, H, vdim]."""
    T, H, dim = q.shape
    vdim = v.shape[2]
    out = torch.zeros(T, H, vdim, dtype=F)
    for h in range(H):
        S = torch.zeros(dim, vdim, dtype=F)
        for t in range(T):
            kv = torch.outer(k[t, h], v[t, h])
            if bonus is None:
                S = decay[t, h][:, None] * S + kv
                out[t, h] = S.T @ q[t, h]
            else:
                out[t, h] = (S + bonus[h][:, None] * kv).T @ q[t, h]
                S = decay[t, h][:, None] * S + kv
    return out


# ---- mixers --------------------------------------------------------------------------------------------------

def retention(h, m, W, p, eps):
    H, dim, vdim = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).reshape(T, H, dim)
    k = (h @ W[p + "k"].T).reshape(T, H, dim) * dim ** -0.5
    v = (h @ W[p + "v"].T).reshape(T, H, vdim)
    decay = torch.tensor(m["decay"], dtype=F)[None, :, None].expand(T, H, dim)
    o = rms_divide(recurrence(q, k, v, decay), eps).reshape(T, H * vdim)
    return (o * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def wkv(h, m, W, p, eps):
    H, dim = m["heads"], m["dim"]
    T = h.shape[0]
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=F), h[:-1]])
    mix = {s: h + (before - h) * W[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ W[p + "r"].T).reshape(T, H, dim)
    k = (mix["k"] @ W[p + "k"].T).reshape(T, H, dim)
    v = (mix["v"] @ W[p + "v"].T).reshape(T, H, dim)
    gate = silu(mix["g"] @ W[p + "g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mix["w"] @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).reshape(T, H, dim)
    o = rms_divide(recurrence(r, k, v, w, bonus=W[p + "u"]), eps).reshape(T, H * dim)
    return (o * W[p + "norm"] * gate) @ W[p + "o"].T


def biased_window_attention(h, m, W, p):
    """The left half of the parallel mixer: grouped heads, short convolutions after the projections, a distance bias,
    a sliding window, and a softmax whose denominator has one more."""
    H, G, dim, vdim, window = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"]
    T = h.shape[0]
    q = causal_conv(h @ W[p + "q"].T, W[p + "q.conv"]).reshape(T, H, dim)
    k = causal_conv(h @ W[p + "k"].T, W[p + "k.conv"]).reshape(T, G, dim)
    v = causal_conv(h @ W[p + "v"].T, W[p + "v.conv"]).reshape(T, G, vdim)
    out = torch.zeros(T, H, vdim, dtype=F)
    for head in range(H):
        slope = 2.0 ** (-8.0 * (head + 1) / H)
        g = head // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, head]) * m["scale"]
            s = s - slope * (i - torch.arange(lo, i + 1, dtype=F))
            e = torch.exp(s)
            out[i, head] = (e / (1 + e.sum())) @ v[lo:i + 1, g]
    return out.reshape(T, H * vdim) @ W[p + "o"].T


def gated_linear_attention(h, m, W, p, eps):
    H, dim, vdim = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).reshape(T, H, dim) * dim ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, dim)
    v = (h @ W[p + "v"].T).reshape(T, H, vdim)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).reshape(T, H, dim)
    o = rms_divide(recurrence(q, k, v, alpha), eps) * W[p + "norm"]
    return (o.reshape(T, H * vdim) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel(h, m, W, p, eps):
    left = biased_window_attention(h, m["left"], W, p + "left.")
    right = gated_linear_attention(h, m["right"], W, p + "right.", eps)
    return 0.5 * (rms_divide(left, eps) * W[p + "left.out"] + rms_divide(right, eps) * W[p + "right.out"])


MIXERS = {"retention": lambda h, m, W, p, eps: retention(h, m, W, p, eps),
          "wkv": lambda h, m, W, p, eps: wkv(h, m, W, p, eps),
          "parallel": lambda h, m, W, p, eps: parallel(h, m, W, p, eps)}


# ---- the model -----------------------------------------------------------------------------------------------

def dense_ff(h, W, p):
    act = W[p + "act"]
    return xielu(h @ W[p + "up"].T, act[0], act[1]) @ W[p + "down"].T


def sublayer_input(x, gain, conv_w, eps):
    h = rms_divide(x, eps) * gain
    return h + causal_conv(h, conv_w)


def forward(raw, W, tokens, layers_out=None):
    """Logits [T, vocab] (float64) of one whole sequence; layers_out, a list, receives x after every layer."""
    eps = raw["norm"]["eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    x = W["embed"][ids] + W["pos"][:len(tokens)]
    for index, layer in enumerate(raw["layers"]):
        p = f"l{index}."
        h = sublayer_input(x, W[p + "norm1"], W[p + "canon1"], eps)
        x = x + MIXERS[layer["type"]](h, layer["mixer"], W, p + "mix.", eps)
        if layer.get("mlp") is not None:
            h = sublayer_input(x, W[p + "norm2"], W[p + "canon2"], eps)
            x = x + dense_ff(h, W, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms_divide(x, eps) * W["final.norm"]) @ W["head"].T


class PlainModel:
    def __init__(self, folder):
        self.raw, self.W = read_folder(folder)

    def logits(self, tokens):
        return forward(self.raw, self.W, list(tokens)).to(torch.float32)


def generate_greedy(model, prompt, count):
    ids, out = list(prompt), []
    for _ in range(count):
        token = int(model.logits(ids)[-1].argmax())
        out.append(token)
        ids.append(token)
    return out
