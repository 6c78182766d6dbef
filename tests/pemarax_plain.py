"""A plain, slow Pemarax: whole sequences, no cache, float64, one function per mechanism.

It shares no code with the package; it reads the design's own configuration keys and the stored tensor names.
``forward(config, tensors, tokens)`` returns the logits [tokens, vocab] and, with ``streams=True``, the residual
stream behind every layer.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64

# Rounding of activations, for measuring what 16-bit rounding alone does to a model: None (exact), or a function
# that rounds a float64 tensor the way a 16-bit engine rounds its activations (see ``activations_rounded``).
_ROUND = None


def rnd(x):
    return x if _ROUND is None else _ROUND(x)


class activations_rounded:
    """Within the block the plain model rounds its activations to bfloat16 where a 16-bit engine holds them in 16
    bits (projections' outputs, normed rows, convolutions, attended heads, expert rows).  With a generator the
    rounding is dithered (up or down at random, in proportion), so that several runs are several samples."""

    def __init__(self, generator=None):
        self.generator = generator

    def _round(self, x):
        if self.generator is None:
            return x.to(torch.bfloat16).to(F64)
        low = (x.to(torch.float32).view(torch.int32) & -65536).view(torch.float32).to(F64)      # toward zero
        step = (low.abs() * 2.0 ** -7).clamp(min=1e-30)
        share = ((x - low).abs() / step).clamp(0.0, 1.0)
        up = torch.rand(x.shape, generator=self.generator, dtype=F64) < share
        return torch.where(up, (low + torch.sign(x) * step), low).to(torch.bfloat16).to(F64)

    def __enter__(self):
        global _ROUND
        self.before, _ROUND = _ROUND, self._round

    def __exit__(self, *exc):
        global _ROUND
        _ROUND = self.before


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
    q, k, v = rnd(h @ w["q"].T), rnd(h @ w["k"].T), rnd(h @ w["v"].T)
    if m.get("conv"):
        q, k, v = rnd(causal_conv(q, w["q.conv"])), rnd(causal_conv(k, w["k.conv"])), rnd(causal_conv(v, w["v.conv"]))
    q, k, v = q.view(T, H, dim), k.view(T, G, dim), v.view(T, G, vdim)
    positions = torch.arange(T)
    if m.get("rot"):
        f, magnitude = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"], m["rot"].get("scaling"))
        q = rotate(q, positions, f, m["rot"]["dims"], True, magnitude)
        k = rotate(k, positions, f, m["rot"]["dims"], True, magnitude)
    q, k = rnd(rms_unit(q, eps)), rnd(rms_unit(k, eps))
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * m["scale"]
    seen = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    return rnd(rnd(weighted_values(scores, seen, v, sink=True).reshape(T, H * vdim)) @ w["o"].T)


def latent_attention_mixer(h, m, w, eps):
    T = h.shape[0]
    H, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = rnd(h @ w["q"].T).view(T, H, dim + rot_dim)
    down = rnd(h @ w["dkv"].T)
    c = rnd(rms_unit(down[:, :rank], eps) * w["dkv.norm"])
    shared = down[:, rank:].view(T, 1, rot_dim)
    positions = torch.arange(T)
    q_plain, q_turned = q[..., :dim], q[..., dim:]
    if rot_dim:
        f, _ = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"])
        q_turned = rnd(rotate(q_turned, positions, f, m["rot"]["dims"], False))
        shared = rnd(rotate(shared, positions, f, m["rot"]["dims"], False))
    keys = (c @ w["uk"].T).view(T, H, dim)
    values = (c @ w["uv"].T).view(T, H, vdim)
    scores = torch.einsum("thd,shd->hts", q_plain, keys) + torch.einsum("thd,sd->hts", q_turned, shared[:, 0])
    seen = visible(T, m["mask"]["size"])
    return rnd(rnd(weighted_values(scores * m["scale"], seen, values, sink=False).reshape(T, H * vdim)) @ w["o"].T)


def windowed_attention(h, m, w, eps):
    """The left half of ``parallel``: normed queries and keys (one weight for all heads), no rotation."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(rms_unit(rnd(h @ w["q"].T).view(T, H, dim), eps) * w["q.norm"])
    k = rnd(rms_unit(rnd(h @ w["k"].T).view(T, G, dim), eps) * w["k.norm"])
    v = rnd(h @ w["v"].T).view(T, G, vdim)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * m["scale"]
    return rnd(rnd(weighted_values(scores, visible(T, m["mask"]["size"]), v, sink=False).reshape(T, H * vdim)) @ w["o"].T)


def state_space(h, m, w, eps):
    """The right half of ``parallel``: the recurrence S <- exp(-exp(A_log) dt) S + dt B x^T token by token."""
    T = h.shape[0]
    heads, P, N, groups = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * P
    u = rnd(h @ w["in"].T)
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * groups * N], u[:, 2 * inner + 2 * groups * N:]
    xbc = rnd(silu(causal_conv(xbc, w["conv"], w["conv.b"])))
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
    return rnd(rnd(normed) @ w["o"].T)


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
            inner = rnd(torch.relu(w[f"e{e}.up"] @ h[t]) ** 2)
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
        normed = rnd(rms_unit(x, eps) * (1.0 + w["norm1"]))
        x = x + mult * MIXERS[layer["type"]](normed, layer["mixer"], mix, eps)
        if layer.get("mlp") is not None:
            normed = rnd(rms_unit(x, eps) * (1.0 + w["norm2"]))
            x = x + mult * mixture(normed, layer["mlp"], layer_tensors(tensors, f"l{index}.mlp."))
        behind.append(x.clone())
    final = rnd(rms_unit(x, eps) * (1.0 + tensors["final.norm"].to(F64)))
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
        normed = rnd(rms_unit(x, eps) * (1.0 + w["norm1"]))
        x = x + mult * MIXERS[layer["type"]](normed, layer["mixer"], layer_tensors(tensors, f"l{index}.mix."), eps)
        if layer.get("mlp") is not None:
            normed = rnd(rms_unit(x, eps) * (1.0 + w["norm2"]))
            mlp = layer_tensors(tensors, f"l{index}.mlp.")
            least = torch.minimum(least, router_choice(normed, layer["mlp"], mlp)[2])
            x = x + mult * mixture(normed, layer["mlp"], mlp)
    return least


def rounding_noise(config, tensors, tokens, samples=4, seed=1):
    """Per position, how far 16-bit rounding of the activations alone moves the plain model's logits (max-abs over
    the vocabulary, the largest of ``samples`` dithered runs and one that rounds to nearest)."""
    exact = forward(config, tensors, tokens)
    generator = torch.Generator().manual_seed(seed)
    worst = torch.zeros(exact.shape[0], dtype=F64)
    for sample in range(samples + 1):
        with activations_rounded(generator if sample else None):
            moved = forward(config, tensors, tokens)
        worst = torch.maximum(worst, (moved - exact).abs().max(dim=-1).values)
    return worst
