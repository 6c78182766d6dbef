"""A plain, slow Motolix: whole sequences in float64, one function per mechanism, the checkpoint's own tensor names.
It shares no code with the package and is what the tests compare the engine with.

Notation: x [T, d] rows of one sequence, positions 0 .. T - 1 (or ``positions``), W tensors by stored name.
"""
import contextlib
import math

import torch

F64 = torch.float64

# Inside ``activations_rounded_to(torch.bfloat16)`` every activation that a 16-bit engine keeps in 16 bits between
# two kernels (normed rows, projected rows, turned queries, keys and values, attended rows, gated rows, the
# feed-forward's activations, each branch's output, the rows that enter the mix before a pass) is rounded to that
# dtype and widened again; sums, weights of keys, norm statistics, decays, the recurrence and the residual stream
# stay exact.  How far that moves the logits is what 16-bit activations cost on a given set of weights: the model's
# conditioning, not a kernel's doing.  With ``dither`` (a torch.Generator) every value is first moved by a random
# fraction of its last kept bit, so that several runs give several samples of the rounding noise.
_ROUND_TO = None
_DITHER = None


@contextlib.contextmanager
def activations_rounded_to(dtype, dither=None):
    global _ROUND_TO, _DITHER
    before = (_ROUND_TO, _DITHER)
    _ROUND_TO, _DITHER = dtype, dither
    try:
        yield
    finally:
        _ROUND_TO, _DITHER = before


def _r(x):
    if _ROUND_TO is None:
        return x
    if _DITHER is not None:
        x = x * (1.0 + (torch.rand(x.shape, generator=_DITHER).to(F64) - 0.5) * 2.0 ** -8)
    return x.to(_ROUND_TO).to(F64)


def layer_norm(x, weight, bias, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight + bias."""
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt((centred * centred).mean(dim=-1, keepdim=True) + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def frequencies(base, dims, scaling=None):
    """f_i = base^(-2i / dims); with ``scaling`` stretched by wavelength."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            length = 2.0 * math.pi / f
            if length > scaling["original"] / scaling["low"]:
                f = f / scaling["factor"]
            elif length >= scaling["original"] / scaling["high"]:
                s = (scaling["original"] / length - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def turn(x, positions, freq, dims, backwards=False):
    """x [T, heads, width]: the first ``dims`` of every head turned in pairs (i, i + dims / 2) by position * freq[i]."""
    angle = positions.to(F64)[:, None] * freq[None, :] * (-1.0 if backwards else 1.0)
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def sigmoid_attention(h, prefix, W, mixer, positions=None):
    """Values are the keys as projected; every visible key weighs sigmoid(score * temp + pb) on its own."""
    T = h.shape[0]
    positions = torch.arange(T) if positions is None else positions
    heads, groups, dim = mixer["heads"], mixer["kv_heads"], mixer["dim"]
    q = _r(h @ W[f"{prefix}.q"].T + W[f"{prefix}.q.b"]).reshape(T, heads, dim)
    k = _r(h @ W[f"{prefix}.k"].T + W[f"{prefix}.k.b"]).reshape(T, groups, dim)
    v = k
    if mixer.get("rot") is not None:
        freq = frequencies(mixer["rot"]["base"], mixer["rot"]["dims"], mixer["rot"].get("scaling"))
        q, k = _r(turn(q, positions, freq, mixer["rot"]["dims"])), _r(turn(k, positions, freq, mixer["rot"]["dims"]))
    seen = positions[None, :] <= positions[:, None]
    out = torch.zeros(T, heads, dim, dtype=F64)
    for head in range(heads):
        group = head // (heads // groups)
        score = (q[:, head] @ k[:, group].T) * mixer["scale"] * W[f"{prefix}.temp"][head]
        weight = torch.sigmoid(score + W[f"{prefix}.pb"][head]) * seen
        out[:, head] = weight @ v[:, group]
    return _r(_r(out).reshape(T, heads * dim) @ W[f"{prefix}.o"].T + W[f"{prefix}.o.b"])


def softmax_attention(h, prefix, W, mixer, eps, positions=None):
    """q and k normed over their whole projections, turned; values turned by their position, outputs turned back."""
    T = h.shape[0]
    positions = torch.arange(T) if positions is None else positions
    heads, groups, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    rot = mixer["rot"]
    q = rms_norm(_r(h @ W[f"{prefix}.q"].T), W[f"{prefix}.q.norm"], eps).reshape(T, heads, dim)
    k = rms_norm(_r(h @ W[f"{prefix}.k"].T), W[f"{prefix}.k.norm"], eps).reshape(T, groups, dim)
    v = _r(h @ W[f"{prefix}.v"].T).reshape(T, groups, vdim)
    freq = frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    q, k = _r(turn(q, positions, freq, rot["dims"])), _r(turn(k, positions, freq, rot["dims"]))
    value_freq = frequencies(rot["base"], vdim)
    v = _r(turn(v, positions, value_freq, vdim))
    seen = positions[None, :] <= positions[:, None]
    out = torch.zeros(T, heads, vdim, dtype=F64)
    for head in range(heads):
        group = head // (heads // groups)
        score = ((q[:, head] @ k[:, group].T) * mixer["scale"]).masked_fill(~seen, -math.inf)
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, group]
    out = _r(turn(_r(out), positions, value_freq, vdim, backwards=True))
    return _r(out.reshape(T, heads * vdim) @ W[f"{prefix}.o"].T)


def gated_linear(h, prefix, W, mixer, eps, state=None):
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; returns (rows, final state [H, dk, dv])."""
    T = h.shape[0]
    heads, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = (_r(h @ W[f"{prefix}.q"].T) * dim ** -0.5).reshape(T, heads, dim)
    k = _r(h @ W[f"{prefix}.k"].T).reshape(T, heads, dim)
    v = _r(h @ W[f"{prefix}.v"].T).reshape(T, heads, vdim)
    z = _r(h @ W[f"{prefix}.a1"].T) @ W[f"{prefix}.a2"].T + W[f"{prefix}.a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / mixer["tau"])).reshape(T, heads, dim)
    S = torch.zeros(heads, dim, vdim, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, heads, vdim, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms_norm(o, W[f"{prefix}.norm"], eps)
    gate = _r(h @ W[f"{prefix}.g"].T)
    return _r(_r(o.reshape(T, heads * vdim) * (gate * torch.sigmoid(gate))) @ W[f"{prefix}.o"].T), S


def feed_forward(h, prefix, W):
    return _r(_r(gelu_tanh(_r(h @ W[f"{prefix}.gate"].T)) * _r(h @ W[f"{prefix}.up"].T)) @ W[f"{prefix}.down"].T)


def layer(x, index, W, entry, eps):
    prefix = f"l{index}"
    norm = lambda rows, name: layer_norm(rows, W[f"{prefix}.{name}"], W[f"{prefix}.{name}.b"], eps)
    h = _r(norm(x, "norm1"))
    mixer = entry["mixer"]
    if entry["type"] == "attention":
        mixed = sigmoid_attention(h, f"{prefix}.mix", W, mixer)
    else:
        left = softmax_attention(h, f"{prefix}.mix.left", W, mixer["left"], eps)
        right, _ = gated_linear(h, f"{prefix}.mix.right", W, mixer["right"], eps)
        mixed = mixer.get("left_scale", 1.0) * left + mixer.get("right_scale", 1.0) * right
    x = x + norm(mixed, "norm1b")
    if entry.get("mlp") is not None:
        x = x + norm(feed_forward(_r(norm(x, "norm2")), f"{prefix}.mlp", W), "norm2b")
    return x


def run_order(raw):
    """[(layer, pass number or None)]: a number where a pass begins."""
    count, loop = len(raw["layers"]), raw.get("loop")
    if loop is None:
        return [(index, None) for index in range(count)]
    order = [(index, None) for index in range(loop["start"])]
    for turn_number in range(loop["times"]):
        order += [(index, turn_number if index == loop["start"] else None) for index in range(loop["start"], loop["stop"])]
    return order + [(index, None) for index in range(loop["stop"], count)]


def forward(tokens, tensors, raw, stream_after=None):
    """Logits [T, vocab] of one sequence; ``stream_after`` (a list) receives the stream behind every run of a layer."""
    W = {name: tensor.to(F64) for name, tensor in tensors.items()}
    eps = raw["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * raw.get("embedding", {}).get("scale", 1.0)
    embedded = x
    for index, begins in run_order(raw):
        if begins is not None:
            x = _r(torch.cat([x, embedded], dim=-1)) @ W["loop.in"].T + W["loop.step"][begins]
        x = layer(x, index, W, raw["layers"][index], eps)
        if stream_after is not None:
            stream_after.append(x)
    x = _r(layer_norm(x, W["final.norm"], W["final.norm.b"], eps))
    return x @ W["head"].T * raw.get("logit_scale", 1.0)


def greedy(tokens, tensors, raw, count):
    """``count`` tokens, each the most likely one after everything before it."""
    tokens, out = list(tokens), []
    for _ in range(count):
        out.append(int(forward(tokens, tensors, raw)[-1].argmax()))
        tokens.append(out[-1])
    return out


def rounding_noise(tokens, tensors, raw, want, samples=8):
    """Per position, the largest departure (max over the vocabulary) from ``want`` (the exact logits) among
    ``samples`` runs with bfloat16-rounded activations: the first rounds to nearest, the others dither."""
    generator = torch.Generator().manual_seed(1)
    worst = torch.zeros(len(tokens), dtype=F64)
    for sample in range(samples):
        with activations_rounded_to(torch.bfloat16, generator if sample else None):
            noisy = forward(tokens, tensors, raw)
        worst = torch.maximum(worst, (noisy - want).abs().max(dim=-1).values)
    return worst
