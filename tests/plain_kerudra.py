"""Kerudra, plainly: one function per mechanism, written from the design's equations, whole sequences at once (no
cache, no pages, no state carried between calls), float64 by default.  Nothing here is shared with the package: the
tests hold the engine's results against these.

``r`` is a rounding function (identity by default): with ``rounding_to(torch.bfloat16)`` the functions round where
16-bit kernels round (products' results, rows that products read, cached rows), which shows what such a run may lose.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def same(x):
    return x


def rounding_to(dtype):
    return lambda x: x.to(dtype).to(x.dtype)


def read_folder(folder, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as handle:
        for name in handle.keys():
            tensor = handle.get_tensor(name)
            tensors[name] = tensor.to(dtype) if tensor.is_floating_point() else tensor
    return config, tensors


def unit_root_mean_square(x, eps):
    """x / sqrt(mean(x^2) + eps), eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def norm(x, weight, eps):
    return unit_root_mean_square(x, eps) * weight


def frequencies(dims, base, dtype):
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=dtype)


def rotate_halves(x, positions, base, dims):
    """x [T, heads, d]: dimension i turns with dimension i + dims/2 by the angle position * base^(-2i/dims); the rest passes."""
    if not dims:
        return x
    half = dims // 2
    angle = positions.to(x.dtype)[:, None] * frequencies(dims, base, x.dtype)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def rotate_neighbours(x, positions, base, dims):
    """x [T, heads, d]: dimension 2i turns with dimension 2i + 1."""
    if not dims:
        return x
    angle = positions.to(x.dtype)[:, None] * frequencies(dims, base, x.dtype)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(length, window):
    """[query, key]: key j is seen from position i if j <= i and, with a window, i - j < window."""
    i, j = torch.arange(length)[:, None], torch.arange(length)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & (i - j < window)
    return seen


def softmax_attention(q, k, v, scale, window, r=same):
    """q, k [T, heads, d], v [T, heads, dv] -> [T, heads * dv]."""
    scores = torch.einsum("ihd,jhd->hij", q, k) * scale
    scores = scores.masked_fill(~visible(q.shape[0], window), float("-inf"))
    weights = r(torch.softmax(scores, dim=-1))
    return r(torch.einsum("hij,jhd->ihd", weights, v)).reshape(q.shape[0], -1)


def window_of(sizes):
    return sizes["mask"]["size"] if sizes.get("mask") else None


def rotation_of(sizes):
    rot = sizes.get("rot")
    return (rot["dims"], rot["base"]) if rot else (0, 1.0)


def shared_value_attention(h, t, p, sizes, r=same):
    """Grouped heads; value rows are the key product's rows (bias included), not rotated."""
    n, heads, dim = h.shape[0], sizes["heads"], sizes["dim"]
    groups = sizes.get("kv_heads", heads)
    q = r(h @ t[p + "q"].T + t[p + "q.b"]).view(n, heads, dim)
    k = r(h @ t[p + "k"].T + t[p + "k.b"]).view(n, groups, dim)
    v = k
    dims, base = rotation_of(sizes)
    positions = torch.arange(n)
    q, k = r(rotate_halves(q, positions, base, dims)), r(rotate_halves(k, positions, base, dims))
    each = heads // groups
    mixed = softmax_attention(q, k.repeat_interleave(each, dim=1), v.repeat_interleave(each, dim=1), sizes["scale"], window_of(sizes), r)
    return r(mixed @ t[p + "o"].T)


def latent_attention(h, t, p, sizes, eps, r=same):
    """Keys and values from one normed latent a token, one rotated key part shared by the heads, a gate per channel."""
    n, heads, dim, rot_dim, vdim, rank = h.shape[0], sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    q = r(h @ t[p + "q"].T).view(n, heads, dim + rot_dim)
    down = r(h @ t[p + "dkv"].T)
    latent = r(norm(down[:, :rank], t[p + "dkv.norm"], eps))
    dims, base = rotation_of(sizes)
    positions = torch.arange(n)
    key_part = r(rotate_neighbours(down[:, rank:].view(n, 1, rot_dim), positions, base, dims))
    q_turned = r(rotate_neighbours(q[..., dim:], positions, base, dims))
    keys = (latent @ t[p + "uk"].T).view(n, heads, dim)
    values = (latent @ t[p + "uv"].T).view(n, heads, vdim)
    queries = torch.cat([q[..., :dim], q_turned], dim=-1)
    full_keys = torch.cat([keys, key_part.expand(n, heads, rot_dim)], dim=-1)
    mixed = softmax_attention(queries, full_keys, values, sizes["scale"], window_of(sizes), r)
    gated = r(mixed * torch.sigmoid(r(h @ t[p + "g"].T)))
    return r(gated @ t[p + "o"].T)


def capped(z, cap):
    return cap * torch.tanh(z / cap)


def matrix_memory(h, t, p, sizes, eps, r=same, floor=1e-6):
    """mLSTM: S and n per head, kept in range by a stabiliser m (the largest log weight so far; 0 in front of the first token)."""
    n_tokens, heads, dim, vdim, cap = h.shape[0], sizes["heads"], sizes["dim"], sizes["vdim"], sizes["gate_cap"]
    q = r(h @ t[p + "q"].T).view(n_tokens, heads, dim) * dim ** -0.5
    k = r(h @ t[p + "k"].T).view(n_tokens, heads, dim)
    v = r(h @ t[p + "v"].T).view(n_tokens, heads, vdim)
    log_in = capped(h @ t[p + "i"].T + t[p + "i.b"], cap)
    log_forget = torch.nn.functional.logsigmoid(capped(h @ t[p + "f"].T + t[p + "f.b"], cap))
    S = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    n = torch.zeros(heads, dim, dtype=h.dtype)
    m = torch.zeros(heads, dtype=h.dtype)
    out = torch.zeros(n_tokens, heads, vdim, dtype=h.dtype)
    for step in range(n_tokens):
        m_new = torch.maximum(log_forget[step] + m, log_in[step])
        keep, take = torch.exp(log_forget[step] + m - m_new), torch.exp(log_in[step] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[step][:, :, None] * v[step][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[step]
        m = m_new
        below = torch.maximum((n * q[step]).sum(dim=-1).abs(), torch.exp(-m)) + floor
        out[step] = torch.einsum("hdv,hd->hv", S, q[step]) / below[:, None]
    out = unit_root_mean_square(out, eps).reshape(n_tokens, heads * vdim) * t[p + "norm"]
    gated = r(out * torch.sigmoid(r(h @ t[p + "g"].T)))
    return r(gated @ t[p + "o"].T)


def feed_forward(h, t, p, r=same):
    return r(r(torch.relu(r(h @ t[p + "up"].T)) ** 2) @ t[p + "down"].T)


def mixer(kind, h, t, p, sizes, eps, r=same):
    if kind == "attention":
        return shared_value_attention(h, t, p, sizes, r)
    if kind == "latent_attention":
        return latent_attention(h, t, p, sizes, eps, r)
    if kind == "mlstm":
        return matrix_memory(h, t, p, sizes, eps, r)
    raise ValueError(kind)


def layer_runs(config):
    count, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return list(range(count))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], count))


def connect(x, y, t, p, mult):
    """Hyper-connection: each new stream is a mix of the streams as they stood before, plus its share of the sublayer's result."""
    return torch.einsum("st,snw->tnw", t[p + "mix"], x) + mult * t[p + "out"][:, None, None] * y[None]


def forward(config, t, tokens, r=same, keep=None):
    """Logits [T, vocab] of a whole sequence.  ``keep``: a list that gets the (summed) stream behind every layer run."""
    eps, mult = config["norm"]["eps"], config.get("residual_mult", 1.0)
    streams = config.get("streams", 0)
    x = t["embed"][torch.tensor(tokens)] * (config.get("embedding") or {}).get("scale", 1.0)
    if streams:
        x = x[None].repeat(streams, 1, 1)
    for index in layer_runs(config):
        layer, p = config["layers"][index], f"l{index}."
        sublayers = [(1, lambda h, layer=layer, p=p: mixer(layer["type"], h, t, p + "mix.", layer["mixer"], eps, r))]
        if layer.get("mlp") is not None:
            sublayers.append((2, lambda h, p=p: feed_forward(h, t, p + "mlp.", r)))
        for number, sublayer in sublayers:
            weight = t[p + f"norm{number}"]
            if streams:
                read = torch.einsum("s,snw->nw", t[p + f"hc{number}.in"], x)
                x = connect(x, sublayer(r(norm(read, weight, eps))), t, p + f"hc{number}.", mult)
            else:
                x = x + mult * sublayer(r(norm(x, weight, eps)))
        if keep is not None:
            keep.append(x.sum(dim=0) if streams else x)
    if streams:
        x = x.sum(dim=0)
    return r(norm(x, t["final.norm"], eps)) @ t["embed"].T * config.get("logit_scale", 1.0)


def greedy_generate(config, t, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(config, t, tokens)[-1].argmax()))
    return tokens[len(prompt):]
