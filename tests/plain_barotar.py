"""A plain, slow implementation of the Barotar decoder: whole sequences, no cache, one function for each
mechanism, written from the design's equations.  It shares no code with the engine (it reads config.json and
the safetensors file itself) and is the oracle of the tests.  Arithmetic is float64 by default, so that the
oracle's own rounding lies far below the tolerances used against it.

Notation: ``T`` tokens of one sequence, positions 0 .. T-1, ``W`` the model's width.

The design in short.  The stream ``x`` starts as the embedding row.  A layer is two sublayers with a norm in front
and a norm behind: ``x <- x + n1b(mixer(n1(x)))``, ``x <- x + n2b(ff(n2(x)))`` (a layer may have no feed-forward),
all norms RMS norms with a plain weight.  Mixers: ``gla``, a linear recurrence per head with a decay per key channel;
``parallel``, the weighted sum of a sliding-window softmax attention (grouped heads, q/k norm, rotation of
neighbouring pairs on part of a head, capped scores, one sink term per head) and an RWKV-style time mixing (inputs
mixed with the token before, a decay per channel from a low-rank map, a bonus for the current token).  Feed-forward:
dense gated (tanh form of gelu) or routed experts (sigmoid scores, groups of experts of which the best are kept,
clamped activations).  The head is the embedding table.
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
    """``x -> x`` rounded to ``dtype`` and widened back: stands where kernels of that type round their results."""
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


def unit_root_mean_square(x, eps):
    """x / sqrt(mean(x^2) + eps), eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def norm(x, weight, eps):
    return unit_root_mean_square(x, eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, positions, base, dims, angle_dtype=torch.float32):
    """Dimensions (2i, 2i+1), i < dims/2, of the last axis turn by ``position * base^(-2i/dims)``; the rest passes.
    ``x [T, heads, d]``.  Angles are formed in ``angle_dtype`` (the design's precision for them is 32-bit)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64).to(angle_dtype)
    angle = positions.to(angle_dtype)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# -- mixers ----------------------------------------------------------------------------------------------------------
def gated_linear_attention(h, t, prefix, sizes, eps, r=exact):
    """``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head, ``alpha = sigmoid(z)^(1/tau)``."""
    heads, dim, vdim, tau = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["tau"]
    n = h.shape[0]
    q = r(h @ t[prefix + "q"].T).view(n, heads, dim) * dim ** -0.5
    k = r(h @ t[prefix + "k"].T).view(n, heads, dim)
    v = r(h @ t[prefix + "v"].T).view(n, heads, vdim)
    z = r(r(h @ t[prefix + "a1"].T) @ t[prefix + "a2"].T) + t[prefix + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(n, heads, dim)
    state = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for i in range(n):
        state = alpha[i][:, :, None] * state + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hdv,hd->hv", state, q[i])
    out = norm(out, t[prefix + "norm"], eps).reshape(n, heads * vdim)
    gate = silu(r(h @ t[prefix + "g"].T))
    return r(r(out * gate) @ t[prefix + "o"].T)


def window_attention(h, t, prefix, sizes, eps, r=exact):
    """Softmax attention over the last ``mask.size`` positions, scores capped by tanh, one sink term per head."""
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    n = h.shape[0]
    positions = torch.arange(n)
    q = r(h @ t[prefix + "q"].T).view(n, heads, dim)
    k = r(h @ t[prefix + "k"].T).view(n, groups, dim)
    v = r(h @ t[prefix + "v"].T).view(n, groups, vdim)
    q = norm(q, t[prefix + "q.norm"], eps)
    k = norm(k, t[prefix + "k.norm"], eps)
    q = r(rotate_pairs(q, positions, sizes["rot"]["base"], sizes["rot"]["dims"]))
    k = r(rotate_pairs(k, positions, sizes["rot"]["base"], sizes["rot"]["dims"]))
    per = heads // groups
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    distance = positions[:, None] - positions[None, :]
    seen = (distance >= 0) & (distance < sizes["mask"]["size"])
    cap = sizes["softcap"]
    for head in range(heads):
        score = (q[:, head] @ k[:, head // per].T) * sizes["scale"]
        score = cap * torch.tanh(score / cap)
        score = score.masked_fill(~seen, -math.inf)
        sink = t[prefix + "sink"][head]
        top = torch.maximum(score.max(dim=-1, keepdim=True).values, sink)
        weight = torch.exp(score - top)
        weight = weight / (weight.sum(dim=-1, keepdim=True) + torch.exp(sink - top))
        out[:, head] = r(weight) @ v[:, head // per]
    return r(r(out).reshape(n, heads * vdim) @ t[prefix + "o"].T)


def time_mixing(h, t, prefix, sizes, eps, r=exact):
    """RWKV-style: every projection reads its own mix of the token and the one before; ``o_t = (S_(t-1) + diag(u) k_t
    v_t^T)^T r_t``, then ``S_t = diag(w_t) S_(t-1) + k_t v_t^T`` with ``w = exp(-exp(.))``."""
    heads, dim = sizes["heads"], sizes["dim"]
    n = h.shape[0]
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)

    def mixed(which):
        return r(h + (before - h) * t[prefix + "mu." + which])

    rr = r(mixed("r") @ t[prefix + "r"].T).view(n, heads, dim)
    k = r(mixed("k") @ t[prefix + "k"].T).view(n, heads, dim)
    v = r(mixed("v") @ t[prefix + "v"].T).view(n, heads, dim)
    gate = silu(r(mixed("g") @ t[prefix + "g"].T))
    low = torch.tanh(r(mixed("w") @ t[prefix + "w1"].T))
    w = torch.exp(-torch.exp(r(r(low) @ t[prefix + "w2"].T) + t[prefix + "w0"])).view(n, heads, dim)
    u = t[prefix + "u"]
    state = torch.zeros(heads, dim, dim, dtype=h.dtype)
    out = torch.zeros(n, heads, dim, dtype=h.dtype)
    for i in range(n):
        kv = k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hdv,hd->hv", state + u[:, :, None] * kv, rr[i])
        state = w[i][:, :, None] * state + kv
    out = unit_root_mean_square(out, eps).reshape(n, heads * dim) * t[prefix + "norm"]
    return r(r(out * gate) @ t[prefix + "o"].T)


def parallel_mixer(h, t, prefix, sizes, eps, r=exact):
    left = window_attention(h, t, prefix + "left.", sizes["left"], eps, r)
    right = time_mixing(h, t, prefix + "right.", sizes["right"], eps, r)
    return sizes["left_scale"] * left + sizes["right_scale"] * right


# -- feed-forwards ---------------------------------------------------------------------------------------------------
def dense_feed_forward(h, t, prefix, r=exact):
    return r(r(gelu_tanh(r(h @ t[prefix + "gate"].T)) * r(h @ t[prefix + "up"].T)) @ t[prefix + "down"].T)


def route(h, router, sizes):
    """Chosen experts ``[T, top]`` and their weights: sigmoid scores, the best ``keep`` of ``count`` groups of
    neighbours by the sum of each group's two largest scores, the ``top`` largest scores among those groups."""
    experts, top = sizes["experts"], sizes["top"]
    count, keep = sizes["groups"]["count"], sizes["groups"]["keep"]
    score = torch.sigmoid(h.to(torch.float32) @ router.to(torch.float32).T)            # 32-bit, as the design says
    per = experts // count
    grouped = score.view(-1, count, per)
    group_score = grouped.topk(min(2, per), dim=-1).values.sum(dim=-1)
    kept = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros_like(group_score, dtype=torch.bool).scatter_(1, kept, True)
    masked = score.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(-1, experts), -math.inf)
    chosen = masked.topk(top, dim=-1).indices
    return chosen, score.gather(1, chosen).to(h.dtype)


def expert(h, t, prefix, limit, r=exact):
    g = r(h @ t[prefix + "gate"].T).clamp(max=limit)
    u = r(h @ t[prefix + "up"].T).clamp(min=-limit, max=limit)
    return r(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[prefix + "down"].T


def routed_experts(h, t, prefix, sizes, r=exact):
    chosen, weights = route(h, t[prefix + "router"], sizes["router"])
    out = torch.zeros_like(h)
    for token in range(h.shape[0]):
        for slot in range(chosen.shape[1]):
            index = int(chosen[token, slot])
            out[token] += weights[token, slot] * expert(h[token:token + 1], t, f"{prefix}e{index}.", sizes["expert"]["limit"], r)[0]
    return out


# -- the model -------------------------------------------------------------------------------------------------------
MIXERS = {"gla": gated_linear_attention, "parallel": parallel_mixer}


def forward(config, t, tokens, r=exact, streams=False):
    """Logits ``[T, vocab]`` of one sequence; with ``streams`` also the stream after every layer."""
    eps = config["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kept = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        mixed = MIXERS[layer["type"]](r(norm(x, t[p + "norm1"], eps)), t, p + "mix.", layer["mixer"], eps, r)
        x = x + norm(mixed, t[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = r(norm(x, t[p + "norm2"], eps))
            if layer["mlp"]["kind"] == "dense":
                fed = dense_feed_forward(h, t, p + "mlp.", r)
            else:
                fed = routed_experts(h, t, p + "mlp.", layer["mlp"], r)
            x = x + norm(fed, t[p + "norm2b"], eps)
        kept.append(x)
    logits = r(norm(x, t["final.norm"], eps)) @ t["embed"].T
    return (logits, kept) if streams else logits


def greedy_generate(config, t, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(config, t, tokens)[-1].argmax()))
    return tokens[len(prompt):]
