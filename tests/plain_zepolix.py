"""A plain, slow implementation of the Zepolix decoder: whole sequences, no cache, one function for
each mechanism, written from the design's equations.  It shares no code with the engine (it reads
config.json and the safetensors file itself) and is the oracle of the tests.  Arithmetic is float64
by default, so that the oracle's own rounding lies far below the tolerances used against it.

Notation: ``T`` tokens of one sequence, positions 0 .. T-1, ``W`` the model's width.

The design in short.  Token rows are normalised once after the embedding.  A layer reads the stream ``x``
itself (no norm in front of a sublayer) and normalises what the sublayer returns:
``x <- x + s1 * n1(mixer(x + conv(x)))`` and ``x <- x + s2 * n2(experts(x))``, where ``n`` is an RMS norm whose
stored weight lies around zero (``1 + w`` multiplies), ``s`` a per-channel scale and ``conv`` a short causal
convolution over time on every channel.  What a layer hands to the next one is a weighted sum of the
embedding's output and the results of all layers so far.  The mixer is attention over a shared low-rank
latent: keys and values of every head are linear maps of one normalised vector per token, plus one small
rotated key part that all heads share; the softmax has one extra term per head that carries no value, and
every head's output passes a sigmoid gate computed from the mixer's input.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def exact(x):
    return x


def rounding_to(dtype):
    """``x -> x`` rounded to ``dtype`` and widened back: stands where kernels of that type round their results.  With
    it the same equations say how far a faultless run in that type lies from the exact result on given tokens."""
    return lambda x: x.to(dtype).to(x.dtype)


def read_folder(folder, dtype=torch.float64):
    """config.json as a dict and every tensor of model.safetensors (floats widened to ``dtype``)."""
    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as handle:
        for name in handle.keys():
            tensor = handle.get_tensor(name)
            tensors[name] = tensor.to(dtype) if tensor.is_floating_point() else tensor
    return config, tensors


def root_mean_square_norm(x, eps):
    """x / sqrt(mean(x^2) + eps), eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    """The layers' and the model's norm: the stored weight lies around zero, 1 + w multiplies."""
    return root_mean_square_norm(x, eps) * (1.0 + weight)


def norm_plain_weight(x, weight, eps):
    """The latent's norm: the stored weight multiplies as it is."""
    return root_mean_square_norm(x, eps) * weight


def short_convolution(h, weight):
    """conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start; ``h [T, W]``, ``weight [W, taps]``."""
    taps = weight.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j                     # tap j looks this many tokens back
        if back < h.shape[0]:
            out[back:] += weight[:, j] * h[:h.shape[0] - back]
    return out


def rotate_pairs(x, positions, base, dims, angle_dtype=torch.float32):
    """Rotation of neighbouring pairs (2i, 2i+1) of the first ``dims`` dimensions of the last axis by the angle
    ``position * base^(-2i/dims)``; the rest passes.  ``x [T, ..., d]``, ``positions [T]``.  Angles are formed in
    ``angle_dtype`` (the design's precision for them is 32-bit)."""
    half = dims // 2
    frequencies = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=angle_dtype)
    angles = positions.to(angle_dtype)[:, None] * frequencies[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angles).to(x.dtype).view(shape), torch.sin(angles).to(x.dtype).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rotated = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
    return torch.cat([rotated, x[..., dims:]], dim=-1)


def softmax_with_sink(scores, sink):
    """Weights of the keys when the denominator holds one more term exp(sink) that has no key; ``scores [..., keys]``
    with -inf where a key is hidden, ``sink`` broadcastable to ``scores[..., 0]``."""
    top = torch.maximum(scores.max(dim=-1).values, sink)
    weights = torch.exp(scores - top[..., None])
    return weights / (weights.sum(dim=-1) + torch.exp(sink - top))[..., None]


def causal_mask(n_tokens):
    """True where key j is hidden from query i (j > i)."""
    index = torch.arange(n_tokens)
    return index[None, :] > index[:, None]


def latent_attention(h, tensors, prefix, sizes, eps, angle_dtype=torch.float32, r=exact):
    """The mixer.  ``sizes``: the layer's ``mixer`` entry of config.json.  ``r`` rounds what 16-bit kernels would round:
    the projections' results, the normed latent, rotated parts, keys and values, the heads' outputs."""
    n = h.shape[0]
    heads, dim, rot_dim, vdim, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    positions = torch.arange(n)
    q = r(h @ tensors[prefix + "q"].T).view(n, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], q[..., dim:]
    down = r(h @ tensors[prefix + "dkv"].T)
    latent = r(norm_plain_weight(down[:, :rank], tensors[prefix + "dkv.norm"], eps))
    k_rot = down[:, rank:]                                                          # one for all heads, not normed
    k_plain = r(latent @ tensors[prefix + "uk"].T).view(n, heads, dim)
    values = r(latent @ tensors[prefix + "uv"].T).view(n, heads, vdim)
    rot = sizes["rot"]
    q_rot = r(rotate_pairs(q_rot, positions, rot["base"], rot["dims"], angle_dtype))
    k_rot = r(rotate_pairs(k_rot, positions, rot["base"], rot["dims"], angle_dtype))
    scores = (torch.einsum("qhd,khd->hqk", q_plain, k_plain) + torch.einsum("qhd,kd->hqk", q_rot, k_rot)) * sizes["scale"]
    scores = scores.masked_fill(causal_mask(n)[None], float("-inf"))
    weights = softmax_with_sink(scores, tensors[prefix + "sink"][:, None])
    mixed = r(torch.einsum("hqk,khd->qhd", r(weights), values))
    gate = torch.sigmoid(r(h @ tensors[prefix + "g"].T))                            # [T, heads]
    return r(r(mixed * gate[..., None]).reshape(n, heads * vdim) @ tensors[prefix + "o"].T)


def route(h, router_weight, top):
    """Chosen experts ``[T, top]`` and their weights: softmax over the chosen logits only."""
    logits = h @ router_weight.T
    chosen = torch.topk(logits, top, dim=-1)
    return chosen.indices, torch.softmax(chosen.values, dim=-1)


def expert(h, tensors, prefix, r=exact):
    gate, up = r(h @ tensors[prefix + "gate"].T), r(h @ tensors[prefix + "up"].T)
    return r(r((gate * torch.sigmoid(gate)) * up) @ tensors[prefix + "down"].T)


def routed_experts(h, tensors, prefix, sizes, r=exact):
    """Every token's weighted sum of its chosen experts' outputs."""
    indices, weights = route(h, tensors[prefix + "router"], sizes["router"]["top"])
    out = torch.zeros_like(h)
    for token in range(h.shape[0]):
        for index, weight in zip(indices[token].tolist(), weights[token]):
            out[token] += weight * expert(h[token:token + 1], tensors, f"{prefix}e{index}.", r)[0]
    return out


def depth_average(states, weights):
    """sum_j weights[j] * states[j]."""
    return sum(weight * state for weight, state in zip(weights, states))


def layer(x, tensors, index, entry, config, angle_dtype=torch.float32, r=exact):
    """One layer's result (before the average over depth).  The stream itself is never rounded; what the sublayers
    read of it is (``r``)."""
    eps = config["norm"]["eps"]
    prefix = f"l{index}."
    h = x
    if "canon" in config and prefix + "canon1" in tensors:
        h = h + short_convolution(h, tensors[prefix + "canon1"])
    if entry["type"] != "latent_attention":
        raise ValueError(f"no mixer {entry['type']!r} in this design")
    mixed = latent_attention(r(h), tensors, prefix + "mix.", entry["mixer"], eps, angle_dtype, r)
    x = x + norm_around_zero(mixed, tensors[prefix + "norm1"], eps) * tensors[prefix + "ls1"]
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "moe":
            raise ValueError(f"no feed-forward {entry['mlp']['kind']!r} in this design")
        fed = routed_experts(r(x), tensors, prefix + "mlp.", entry["mlp"], r)
        x = x + norm_around_zero(fed, tensors[prefix + "norm2"], eps) * tensors[prefix + "ls2"]
    return x


def forward(config, tensors, tokens, angle_dtype=torch.float32, streams=False, r=exact):
    """Logits ``[T, vocab]`` of one sequence; with ``streams`` also every layer's result ``[layers, T, W]``."""
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = norm_around_zero(tensors["embed"][ids], tensors["embed.norm"], eps)
    states, results = [x], []
    for index, entry in enumerate(config["layers"]):
        result = layer(x, tensors, index, entry, config, angle_dtype, r)
        results.append(result)
        states.append(result)
        x = depth_average(states, tensors[f"l{index}.dwa"])
    logits = r(norm_around_zero(x, tensors["final.norm"], eps)) @ tensors["head"].T
    return (logits, torch.stack(results)) if streams else logits


def head_scale(config):
    """The design's usual score scale, 1 / sqrt(dimensions of a head's key), for configurations made by tests."""
    sizes = config["layers"][0]["mixer"]
    return 1.0 / math.sqrt(sizes["dim"] + sizes["rot_dim"])


def greedy_generate(config, tensors, prompt, count):
    """``count`` tokens, each the first largest logit behind everything before it (the whole sequence again every time)."""
    tokens, made = list(prompt), []
    for _ in range(count):
        made.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
        tokens.append(made[-1])
    return made
