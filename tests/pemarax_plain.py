"""A plain, slow Pemarax: whole sequences, no cache, float64, one function per mechanism.

It shares no code with the package; it reads the design's own configuration keys and the stored tensor names.
``forward(config, tensors, tokens)`` returns the logits [tokens, vocab] and, with ``streams=True``, the residual
stream behind every layer.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(u, taps_weight, bias=None):
    """u [T, C], taps_weight [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = taps_weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u])
    y = torch.zeros(T, C, dtype=u.dtype)
    for j in range(taps):
        y = y + padded[j:j + T] * taps_weight[:, j]
    if bias is not None:
        y = y + bias
    return y


def rotary_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i / dims); with YaRN scaling blended with f_i / factor by a ramp over i, and the magnitude
    that cos and sin are multiplied by."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def where(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, positions, frequencies, dims, interleaved, magnitude=1.0):
    """x [T, heads, width]: the first ``dims`` dimensions of every head turned by position * frequency."""
    angles = positions.to(F64)[:, None] * torch.tensor(frequencies, dtype=F64)[None, :]
    cos, sin = (torch.cos(angles) * magnitude)[:, None, :], (torch.sin(angles) * magnitude)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


def visible(T, window, keep_first=0):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) & ((i - j < window) | (j < keep_first)) if window else (j <= i)
    return seen


def weighted_values(scores, seen, values, sink):
    """scores [H, T, T], values [T, H, dv]: softmax over the visible keys, with one more in the denominator when
    ``sink`` (a key of score 0 that brings no value)."""
    scores = scores.masked_fill(~seen[None], float("-inf"))
    top = scores.max(dim=-1, keepdim=True).values
    if sink:
        top = torch.clamp(top, min=0.0)
    e = torch.exp(scores - top)
    denominator = e.sum(dim=-1, keepdim=True)
    if sink:
        denominator = denominator + torch.exp(-top)
    return torch.einsum("hts,shd->thd", e / denominator, values)


def attention_mixer(h, m, w, eps):
    """The mixer ``attention``: short convolutions behind the projections, interleaved rotation with YaRN, unit
    norms of q and k, a window that keeps the first tokens, a sink in the softmax."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    if m.get("conv"):
        q, k, v = causal_conv(q, w["q.conv"]), causal_conv(k, w["k.conv"]), causal_conv(v, w["v.conv"])
    q, k, v = q.view(T, H, dim), k.view(T, G, dim), v.view(T, G, vdim)
    positions = torch.arange(T)
    if m.get("rot"):
        f, magnitude = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"], m["rot"].get("scaling"))
        q = rotate(q, positions, f, m["rot"]["dims"], True, magnitude)
        k = rotate(k, positions, f, m["rot"]["dims"], True, magnitude)
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * m["scale"]
    seen = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    return weighted_values(scores, seen, v, sink=True).reshape(T, H * vdim) @ w["o"].T


def latent_attention_mixer(h, m, w, eps):
    T = h.shape[0]
    H, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).view(T, H, dim + rot_dim)
    down = h @ w["dkv"].T
    c = rms_unit(down[:, :rank], eps) * w["dkv.norm"]
    shared = down[:, rank:].view(T, 1, rot_dim)
    positions = torch.arange(T)
    q_plain, q_turned = q[..., :dim], q[..., dim:]
    if rot_dim:
        f, _ = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"])
        q_turned = rotate(q_turned, positions, f, m["rot"]["dims"], False)
        shared = rotate(shared, positions, f, m["rot"]["dims"], False)
    keys = (c @ w["uk"].T).view(T, H, dim)
    values = (c @ w["uv"].T).view(T, H, vdim)
    scores = torch.einsum("thd,shd->hts", q_plain, keys) + torch.einsum("thd,sd->hts", q_turned, shared[:, 0])
    seen = visible(T, m["mask"]["size"])
    return weighted_values(scores * m["scale"], seen, values, sink=False).reshape(T, H * vdim) @ w["o"].T


def windowed_attention(h, m, w, eps):
    """The left half of ``parallel``: normed queries and keys (one weight for all heads), no rotation."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit((h @ w["q"].T).view(T, H, dim), eps) * w["q.norm"]
    k = rms_unit((h @ w["k"].T).view(T, G, dim), eps) * w["k.norm"]
    v = (h @ w["v"].T).view(T, G, vdim)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * m["scale"]
    return weighted_values(scores, visible(T, m["mask"]["size"]), v, sink=False).reshape(T, H * vdim) @ w["o"].T


def state_space(h, m, w, eps):
    """The right half of ``parallel``: the recurrence S <- exp(-exp(A_log) dt) S + dt B x^T token by token."""
    T = h.shape[0]
    heads, P, N, groups = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * P
    u = h @ w["in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * groups * N], u[:, 2 * inner + 2 * groups * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].view(T, heads, P)
    B = xbc[:, inner:inner + groups * N].view(T, groups, N)
    C = xbc[:, inner + groups * N:].view(T, groups, N)
    dt = softplus(dt + w["dt_bias"])
    decay = torch.exp(-torch.exp(w["A_log"])[None, :] * dt)
    S = torch.zeros(heads, N, P, dtype=F64)
    y = torch.zeros(T, heads, P, dtype=F64)
    per_group = heads // groups
    for t in range(T):
        for head in range(heads):
            g = head // per_group
            S[head] = decay[t, head] * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + w["D"][head] * x[t, head]
    gated = y.reshape(T, inner) * silu(z)
    parts = m.get("norm_groups", 1)
    normed = rms_unit(gated.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return normed @ w["o"].T


def parallel_mixer(h, m, w, eps):
    left = {k[len("left."):]: v for k, v in w.items() if k.startswith("left.")}
    right = {k[len("right."):]: v for k, v in w.items() if k.startswith("right.")}
    a = rms_unit(windowed_attention(h, m["left"], left, eps), eps) * w["left.out"]
    b = rms_unit(state_space(h, m["right"], right, eps), eps) * w["right.out"]
    return 0.5 * (a + b)


def router_choice(h, mlp, w):
    """(experts [T, top], weights [T, top], margin [T]): the ``top`` largest logits, the softmax over them, and
    by how much the last chosen logit beats the first that was not chosen."""
    logits = h @ w["router"].T + w["router.b"]
    top = mlp["router"]["top"]
    ordered, experts = torch.sort(logits, dim=-1, descending=True, stable=True)
    margin = ordered[:, top - 1] - ordered[:, top] if logits.shape[1] > top else torch.full((h.shape[0],), float("inf"), dtype=F64)
    return experts[:, :top], torch.softmax(ordered[:, :top], dim=-1), margin


def mixture(h, mlp, w):
    experts, weights, _ = router_choice(h, mlp, w)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, weight in zip(experts[t].tolist(), weights[t]):
            inner = torch.relu(w[f"e{e}.up"] @ h[t]) ** 2
            out[t] = out[t] + weight * (w[f"e{e}.down"] @ inner)
    return out


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "parallel": parallel_mixer}


def layer_tensors(tensors, prefix):
    return {name[len(prefix):]: value.to(F64) for name, value in tensors.items() if name.startswith(prefix)}


def forward(config, tensors, tokens, streams=False):
    eps = float(config["norm"]["eps"])
    mult = float(config.get("residual_mult", 1.0))
    x = tensors["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    behind = []
    for index, layer in enumerate(config["layers"]):
        w = layer_tensors(tensors, f"l{index}.")
        mix = layer_tensors(tensors, f"l{index}.mix.")
        normed = rms_unit(x, eps) * (1.0 + w["norm1"])
        x = x + mult * MIXERS[layer["type"]](normed, layer["mixer"], mix, eps)
        if layer.get("mlp") is not None:
            normed = rms_unit(x, eps) * (1.0 + w["norm2"])
            x = x + mult * mixture(normed, layer["mlp"], layer_tensors(tensors, f"l{index}.mlp."))
        behind.append(x.clone())
    final = rms_unit(x, eps) * (1.0 + tensors["final.norm"].to(F64))
    logits = final @ tensors["head"].to(F64).T
    return (logits, behind) if streams else logits


def choice_margins(config, tensors, tokens):
    """Per token, the smallest margin of any layer's router: positions where 16-bit rounding may turn a choice."""
    eps = float(config["norm"]["eps"])
    mult = float(config.get("residual_mult", 1.0))
    x = tensors["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    least = torch.full((x.shape[0],), float("inf"), dtype=F64)
    for index, layer in enumerate(config["layers"]):
        w = layer_tensors(tensors, f"l{index}.")
        normed = rms_unit(x, eps) * (1.0 + w["norm1"])
        x = x + mult * MIXERS[layer["type"]](normed, layer["mixer"], layer_tensors(tensors, f"l{index}.mix."), eps)
        if layer.get("mlp") is not None:
            normed = rms_unit(x, eps) * (1.0 + w["norm2"])
            mlp = layer_tensors(tensors, f"l{index}.mlp.")
            least = torch.minimum(least, router_choice(normed, layer["mlp"], mlp)[2])
            x = x + mult * mixture(normed, layer["mlp"], mlp)
    return least
