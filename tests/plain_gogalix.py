"""Gogalix, plainly: one function per mechanism, written from the design's equations, whole sequences at once (no
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


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return unit_root_mean_square(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_convolution(x, taps):
    """x [T, C], taps [C, K]: out_t = sum_j taps[:, j] * x_(t - K + 1 + j), zeros in front of the sequence."""
    count = taps.shape[1]
    padded = torch.cat([x.new_zeros((count - 1, x.shape[1])), x], dim=0)
    out = torch.zeros_like(x)
    for j in range(count):
        out = out + padded[j:j + x.shape[0]] * taps[:, j]
    return out


def unit_vectors(x):
    return x / torch.sqrt(x.pow(2).sum(dim=-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, D], v [T, H, V], beta [T, H], decay [T, H] or [T, H, D] (per key channel: rows of the state).
    Per head: S <- decay * S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    count, heads, dim = q.shape
    state = q.new_zeros((heads, dim, v.shape[-1]))
    out = []
    for t in range(count):
        g = decay[t]
        state = state * (g[:, None, None] if g.dim() == 1 else g[:, :, None])
        seen = torch.einsum("hdv,hd->hv", state, k[t])
        u = beta[t][:, None] * (v[t] - seen)
        state = state + torch.einsum("hd,hv->hdv", k[t], u)
        out.append(torch.einsum("hdv,hd->hv", state, q[t]))
    return torch.stack(out)


def delta_inputs(h, tensors, prefix, sizes, r):
    """What both delta mixers share: projections, convolutions with silu, unit vectors, the write strength."""
    heads, kv_heads, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    count = h.shape[0]

    def path(name):
        return r(silu(r(causal_convolution(r(h @ tensors[f"{prefix}.{name}"].T), tensors[f"{prefix}.{name}.conv"]))))

    q = unit_vectors(path("q").view(count, kv_heads, dim)) * dim ** -0.5
    k = unit_vectors(path("k").view(count, kv_heads, dim))
    v = path("v").view(count, heads, vdim)
    repeat = heads // kv_heads
    q, k = q.repeat_interleave(repeat, dim=1), k.repeat_interleave(repeat, dim=1)
    beta = torch.sigmoid(r(h @ tensors[f"{prefix}.b"].T))
    return q, k, v, beta


def delta_output(o, gate, tensors, prefix, eps, r):
    """Per head: o / rms(o) * weight (shared by the heads) * gate; then the output projection."""
    count = o.shape[0]
    normed = unit_root_mean_square(o, eps) * tensors[f"{prefix}.norm"]
    return r(r((normed * gate).reshape(count, -1)) @ tensors[f"{prefix}.o"].T)


def delta_mixer(h, tensors, prefix, sizes, eps, r=same):
    """One decay per head: exp(-exp(A_log) * softplus(W_a h + dt_bias)); the gate is silu(W_g h)."""
    count = h.shape[0]
    q, k, v, beta = delta_inputs(h, tensors, prefix, sizes, r)
    step = softplus(r(h @ tensors[f"{prefix}.a"].T) + tensors[f"{prefix}.dt_bias"])
    decay = torch.exp(-torch.exp(tensors[f"{prefix}.A_log"]) * step)
    o = delta_rule(q, k, v, beta, decay)
    gate = silu(r(h @ tensors[f"{prefix}.g"].T)).view(count, sizes["heads"], sizes["vdim"])
    return delta_output(o, gate, tensors, prefix, eps, r)


def channel_delta_mixer(h, tensors, prefix, sizes, eps, r=same):
    """One decay per head and key channel through a low-rank map; the gate is sigmoid of a low-rank map."""
    count, heads, dim, vdim = h.shape[0], sizes["heads"], sizes["dim"], sizes["vdim"]
    q, k, v, beta = delta_inputs(h, tensors, prefix, sizes, r)
    inner = r(r(h @ tensors[f"{prefix}.a1"].T) @ tensors[f"{prefix}.a2"].T)
    step = softplus(inner + tensors[f"{prefix}.dt_bias"]).view(count, heads, dim)
    decay = torch.exp(-torch.exp(tensors[f"{prefix}.A_log"])[None, :, None] * step)
    o = delta_rule(q, k, v, beta, decay)
    gate = torch.sigmoid(r(r(h @ tensors[f"{prefix}.g1"].T) @ tensors[f"{prefix}.g2"].T)).view(count, heads, vdim)
    return delta_output(o, gate, tensors, prefix, eps, r)


def windowed_softmax(scores, window):
    """scores [H, T, T] (query, key): key j is visible to query i if 0 <= i - j < window (window None: all before)."""
    count = scores.shape[-1]
    i, j = torch.arange(count)[:, None], torch.arange(count)[None, :]
    visible = (j <= i) if window is None else ((j <= i) & (i - j < window))
    return torch.softmax(scores.masked_fill(~visible, -math.inf), dim=-1)


def differential_attention(h, tensors, prefix, sizes, eps, keys_values=None, r=same):
    """Two softmax maps per head over the same values, ``a1 - lambda a2``, normed per head without a weight, times
    ``1 - diff``.  ``keys_values``: another layer's keys and values (this layer has none of its own).  Returns
    (result, (keys, values))."""
    heads, kv_heads, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    count = h.shape[0]
    q = r(h @ tensors[f"{prefix}.q"].T).view(count, heads, 2, dim)
    if keys_values is None:
        k = r(h @ tensors[f"{prefix}.k"].T).view(count, kv_heads, 2, dim)
        v = r(h @ tensors[f"{prefix}.v"].T).view(count, kv_heads, vdim)
    else:
        k, v = keys_values
    repeat = heads // kv_heads
    ke, ve = k.repeat_interleave(repeat, dim=1), v.repeat_interleave(repeat, dim=1)
    window = sizes["mask"]["size"] if sizes.get("mask") else None
    maps = []
    for m in range(2):
        scores = torch.einsum("ihd,jhd->hij", q[:, :, m], ke[:, :, m]) * sizes["scale"]
        maps.append(torch.einsum("hij,jhv->ihv", r(windowed_softmax(scores, window)), ve))
    lam = math.exp(float((tensors[f"{prefix}.lq1"] * tensors[f"{prefix}.lk1"]).sum())) \
        - math.exp(float((tensors[f"{prefix}.lq2"] * tensors[f"{prefix}.lk2"]).sum())) + sizes["diff"]
    o = unit_root_mean_square(maps[0] - lam * maps[1], eps) * (1.0 - sizes["diff"])
    return r(r(o.reshape(count, -1)) @ tensors[f"{prefix}.o"].T), (k, v)


def dense_feed_forward(h, tensors, prefix, r=same):
    gate = r(h @ tensors[f"{prefix}.gate"].T + tensors[f"{prefix}.gate.b"])
    up = r(h @ tensors[f"{prefix}.up"].T + tensors[f"{prefix}.up.b"])
    return r(r(silu(gate) * up) @ tensors[f"{prefix}.down"].T + tensors[f"{prefix}.down.b"])


def routed_feed_forward(h, tensors, prefix, sizes, r=same):
    experts, top = sizes["router"]["experts"], sizes["router"]["top"]
    logits = h @ tensors[f"{prefix}.router"].T + tensors[f"{prefix}.router.b"]
    best, where = torch.topk(logits, top, dim=-1)
    weights = torch.softmax(best, dim=-1)
    out = torch.zeros_like(h)
    for e in range(experts):
        gate, up, down = (tensors[f"{prefix}.e{e}.{name}"] for name in ("gate", "up", "down"))
        for slot in range(top):
            rows = (where[:, slot] == e).nonzero().flatten()
            if len(rows):
                x = h[rows]
                y = r(silu(r(x @ gate.T)) * r(x @ up.T)) @ down.T
                out[rows] += weights[rows, slot][:, None] * y
    return out


def forward(config, tensors, tokens, r=same, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence.  ``layer_outputs``: a list that receives the stream behind every layer."""
    eps = config["norm"]["eps"]
    dtype = tensors["embed"].dtype
    x = tensors["embed"][torch.tensor(tokens)] * config.get("embedding", {}).get("scale", 1.0)
    kept = {}
    for index, layer in enumerate(config["layers"]):
        prefix, sizes = f"l{index}", layer["mixer"]
        h = r(scalar_norm(x, tensors[f"{prefix}.norm1"], eps))
        if layer["type"] == "delta":
            mixed = delta_mixer(h, tensors, f"{prefix}.mix", sizes, eps, r)
        elif layer["type"] == "channel_delta":
            mixed = channel_delta_mixer(h, tensors, f"{prefix}.mix", sizes, eps, r)
        elif layer["type"] == "attention":
            source = kept[sizes["kv_from"]] if sizes.get("kv_from") is not None else None
            mixed, kept[index] = differential_attention(h, tensors, f"{prefix}.mix", sizes, eps, source, r)
        else:
            raise ValueError(layer["type"])
        update = tensors[f"{prefix}.ls1"] * torch.sigmoid(r(h @ tensors[f"{prefix}.rg1"].T + tensors[f"{prefix}.rg1.b"])) * mixed
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] == "dense":
                fed = dense_feed_forward(h, tensors, f"{prefix}.mlp", r)
            else:
                fed = routed_feed_forward(h, tensors, f"{prefix}.mlp", layer["mlp"], r)
            update = update + tensors[f"{prefix}.ls2"] * torch.sigmoid(r(h @ tensors[f"{prefix}.rg2"].T + tensors[f"{prefix}.rg2.b"])) * fed
        x = x + update
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    final = r(scalar_norm(x, tensors["final.norm"], eps))
    return (final @ tensors["head"].T).to(dtype)


def greedy_generate(config, tensors, prompt, count):
    """The prompt's ``count`` most likely continuations, one token at a time, the first of equal logits."""
    tokens, made = list(prompt), []
    for _ in range(count):
        made.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
        tokens.append(made[-1])
    return made
