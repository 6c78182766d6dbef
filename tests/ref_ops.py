"""Plain PyTorch float32 versions of the HIP operations, with the same signatures and the
same effects on the same (paged, slotted) buffers.

Two uses: GPU tests run a kernel and its reference here on copies of the same inputs and
compare; CPU tests install these in place of the kernels (``install``) to exercise the
cache manager, the step function and the scheduler where there is no GPU.  They are test
doubles only: the package itself has no CPU path.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _f(t):
    return t.float()


def embed(token_ids, table, multiplier, out):
    out.copy_(_f(table)[token_ids.long()] * multiplier)


def feed_tokens(token_ids, source, dst, src):
    for place, row in zip(dst, src):
        token_ids[int(place)] = source[int(row)]


def add_rmsnorm(h, deltas, weight, eps, out, rows=None, factors=None):
    total = h.clone()
    for index, delta in enumerate(deltas):
        total += _f(delta) * (1.0 if factors is None else float(factors[index]))
    if rows is None:
        if deltas:
            h.copy_(total)
        picked = total
    else:
        picked = total[rows.long()]
    if out is not None:
        normed = picked / torch.sqrt(picked.pow(2).mean(-1, keepdim=True) + eps) * weight
        out.copy_(normed.to(out.dtype))


def cast_rows(source, out):
    out.copy_(source.to(out.dtype))


def attention_prepare(qkv, num_heads, num_kv_heads, head_dim, value_dim, positions, inv_freq, rotary_dim, slot_mapping,
                      k_cache, v_cache, *, values_from_keys=False, q_norm=None, k_norm=None, norm_eps=0.0,
                      value_inv_freq=None, interleaved=False, turn_scale=1.0, head_norm=None, q_head_weight=None,
                      k_head_weight=None, head_eps=0.0):
    T = qkv.shape[0]
    q_cols, k_cols = num_heads * head_dim, num_kv_heads * head_dim
    q = _f(qkv[:, :q_cols]).clone()
    k = _f(qkv[:, q_cols:q_cols + k_cols]).clone()
    if values_from_keys:
        v = k.clone().reshape(T, num_kv_heads, head_dim)
    else:
        v = _f(qkv[:, q_cols + k_cols:q_cols + k_cols + num_kv_heads * value_dim]).reshape(T, num_kv_heads, value_dim).clone()
    if q_norm is not None:
        q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + norm_eps) * q_norm
        k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + norm_eps) * k_norm
    q = q.reshape(T, num_heads, head_dim)
    k = k.reshape(T, num_kv_heads, head_dim)
    spots = positions.to(torch.float32)

    def rotate(x, frequencies, width, neighbours=False, magnitude=1.0):
        half = width // 2
        angle = spots[:, None] * frequencies[None, :]
        cos, sin = angle.cos()[:, None, :] * magnitude, angle.sin()[:, None, :] * magnitude
        if neighbours:
            out = x.clone()
            a, b = x[..., 0:width:2], x[..., 1:width:2]
            out[..., 0:width:2] = a * cos - b * sin
            out[..., 1:width:2] = b * cos + a * sin
            return out
        a, b = x[..., :half], x[..., half:width]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., width:]], dim=-1)

    def norm_heads(x, weight):
        x = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + head_eps)
        return x if weight is None else x * weight
    if head_norm == "before_rotation":
        q, k = norm_heads(q, q_head_weight), norm_heads(k, k_head_weight)
    if inv_freq is not None and rotary_dim > 0:
        q = rotate(q, inv_freq, rotary_dim, interleaved, turn_scale)
        k = rotate(k, inv_freq, rotary_dim, interleaved, turn_scale)
    if head_norm == "after_rotation":
        q, k = norm_heads(q, q_head_weight), norm_heads(k, k_head_weight)
    if value_inv_freq is not None:
        v = rotate(v, value_inv_freq, value_dim)
    qkv[:, :q_cols] = q.reshape(T, q_cols).to(qkv.dtype)
    if slot_mapping is not None:
        page_size = k_cache.shape[2]
        pages = (slot_mapping // page_size).long()
        offsets = (slot_mapping % page_size).long()
        k_cache[pages, :, offsets, :] = k.to(k_cache.dtype)
        v_cache[pages, :, :, offsets] = v.to(v_cache.dtype)


def swiglu(gate_up, out, tile=0, activation="silu"):
    inner = gate_up.shape[1] // 2
    if tile:
        tiles = gate_up.reshape(gate_up.shape[0], inner // tile, 2, tile)
        gate, up = tiles[:, :, 0].reshape(-1, inner), tiles[:, :, 1].reshape(-1, inner)
    else:
        gate, up = gate_up[:, :inner], gate_up[:, inner:]
    if activation == "gelu_tanh":
        z = _f(gate)
        bent = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
    else:
        bent = F.silu(_f(gate))
    out.copy_((bent * _f(up)).to(out.dtype))


def scale_to_f32(values, multiplier, out):
    out.copy_(_f(values).reshape(out.shape) * multiplier)


def tanh_softcap(logits, cap):
    logits.copy_(cap * torch.tanh(logits / cap))


def fused_gemm_split(weight, bias, x, partial, feature_tiles=1, fragments=None):
    """Slab s: the sums over the s-th run of K (in chunks of 32), the bias in slab 0."""
    S = partial.shape[0]
    chunks = weight.shape[1] // 32
    per_split = -(-chunks // S)
    for s in range(S):
        lo, hi = min(s * per_split, chunks) * 32, min((s + 1) * per_split, chunks) * 32
        partial[s] = _f(x[:, lo:hi]) @ _f(weight[:, lo:hi]).T
    if bias is not None:
        partial[0] += bias


def add_partials_rmsnorm(h, partial, weight, eps, out):
    for s in range(partial.shape[0]):
        h += partial[s]
    if out is not None:
        out.copy_((h / torch.sqrt(h.pow(2).mean(dim=-1, keepdim=True) + eps) * weight).to(out.dtype))


def linear(x, weight, bias, keep_float32=False):
    y = _f(x) @ _f(weight).T
    if bias is not None:
        y = y + bias
    return y if keep_float32 else y.to(x.dtype)


def rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, positions, inv_freq, rotary_dim, slot_mapping,
                  k_cache, v_cache, value_dim=None):
    T = qkv.shape[0]
    value_dim = head_dim if value_dim is None else value_dim
    q_cols = num_heads * head_dim
    k_cols = num_kv_heads * head_dim
    q = _f(qkv[:, :q_cols]).reshape(T, num_heads, head_dim).clone()
    k = _f(qkv[:, q_cols:q_cols + k_cols]).reshape(T, num_kv_heads, head_dim).clone()
    v = qkv[:, q_cols + k_cols:q_cols + k_cols + num_kv_heads * value_dim].reshape(T, num_kv_heads, value_dim)
    if inv_freq is not None and rotary_dim > 0:
        half = rotary_dim // 2
        angle = positions.to(torch.float32)[:, None] * inv_freq[None, :]
        cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]

        def rotate(x):
            a, b = x[..., :half], x[..., half:rotary_dim]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., rotary_dim:]], dim=-1)
        q, k = rotate(q), rotate(k)
    qkv[:, :q_cols] = q.reshape(T, q_cols).to(qkv.dtype)
    if slot_mapping is not None:
        page_size = k_cache.shape[2]
        pages = (slot_mapping // page_size).long()
        offsets = (slot_mapping % page_size).long()
        k_cache[pages, :, offsets, :] = k.to(k_cache.dtype)
        v_cache[pages, :, :, offsets] = v.to(v_cache.dtype)        # V pages are [Hkv, dh, token]


def paged_attention(q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lane_of_token,
                    positions, scale, window, out, max_seq_len=None, slopes=None, query_tiles=None, tile_tokens=0,
                    cu_seqlens=None, log_bias=None, sinks=None, value_dim=None, head_scales=None, score_bias=None,
                    sigmoid=False, keep_first=0, fixed_sink=None):
    """``max_seq_len`` sizes the kernel's launch and nothing else: not used here, and neither is the table of
    runs that picks the kernel for lanes of several tokens.  ``slopes``: a bias on the scores,
    ``-slopes[head] * (query position - key position)``; ``log_bias`` [Hq, 2] = (r1, r2): the scores lose
    r1 * ln(1 + r2 * distance); ``sinks`` [Hq]: exp(sink) is one more term of the denominator."""
    T = q.shape[0]
    value_dim = head_dim if value_dim is None else value_dim
    page_size = k_cache.shape[2]
    group = num_heads // num_kv_heads
    for token in range(T):
        lane = int(lane_of_token[token])
        position = int(positions[token])
        first = 0 if not window else max(0, position - window + 1)
        keys = torch.arange(first, position + 1)
        if keep_first and first > 0:
            keys = torch.cat([torch.arange(0, min(keep_first, first)), keys])
        pages = block_tables[lane][(keys // page_size).long()].long()
        offsets = (keys % page_size).long()
        k = _f(k_cache[pages, :, offsets, :])        # [keys, Hkv, dh]
        v = _f(v_cache[pages, :, :, offsets])
        for head in range(num_heads):
            query = _f(q[token, head * head_dim:(head + 1) * head_dim])
            scores = (k[:, head // group, :] @ query) * scale
            if head_scales is not None:
                scores = scores * head_scales[head]
            if sigmoid:
                weights = torch.sigmoid(scores + (score_bias[head] if score_bias is not None else 0.0))
                out[token, head * value_dim:(head + 1) * value_dim] = (weights @ v[:, head // group, :]).to(out.dtype)
                continue
            if slopes is not None:
                scores = scores - slopes[head] * (position - keys).float()
            if log_bias is not None:
                scores = scores - log_bias[head, 0] * torch.log1p(log_bias[head, 1] * (position - keys).float())
            if fixed_sink is not None:
                weights = torch.softmax(torch.cat([scores, torch.tensor([float(fixed_sink)])]), dim=0)[:-1]
            elif sinks is not None:
                weights = torch.softmax(torch.cat([scores, sinks[head].reshape(1)]), dim=0)[:-1]
            else:
                weights = torch.softmax(scores, dim=0)
            out[token, head * value_dim:(head + 1) * value_dim] = (weights @ v[:, head // group, :]).to(out.dtype)


def decode_attention_supported(dtype, num_heads, num_kv_heads, head_dim, page_size, value_dim=None, keep_first=0):
    return False


def prefill_attention_supported(dtype, num_heads, num_kv_heads, head_dim, page_size):
    return False


def decode_attention(q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lane_of_token, positions,
                     scale, window, max_seq_len, out, value_dim=None, head_scales=None, score_bias=None, sigmoid=False,
                     keep_first=0, sinks=None):
    paged_attention(q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lane_of_token, positions,
                    scale, window, out, value_dim=value_dim, head_scales=head_scales, score_bias=score_bias,
                    sigmoid=sigmoid, keep_first=keep_first, sinks=sinks)


def conv1d_silu(u, col_offset, width, weight, bias, conv_state, lane_of_token, cu_seqlens, slot_ids, out, activation=True):
    K = weight.shape[1]
    for lane in range(slot_ids.numel()):
        begin, end = int(cu_seqlens[lane]), int(cu_seqlens[lane + 1])
        rows = _f(u[begin:end, col_offset:col_offset + width])
        window = torch.cat([_f(conv_state[int(slot_ids[lane])]), rows], dim=0)
        total = torch.zeros(end - begin, width)
        for tap in range(K):
            total += window[tap:tap + end - begin] * weight[:, tap][None, :]
        if bias is not None:
            total += bias[None, :]
        out[begin:end] = (F.silu(total) if activation else total).to(out.dtype)


def conv_state_update(u, col_offset, width, kernel, conv_state, cu_seqlens, slot_ids):
    if kernel <= 1:
        return
    for lane in range(slot_ids.numel()):
        begin, end = int(cu_seqlens[lane]), int(cu_seqlens[lane + 1])
        slot = int(slot_ids[lane])
        window = torch.cat([conv_state[slot], u[begin:end, col_offset:col_offset + width]], dim=0)
        conv_state[slot] = window[-(kernel - 1):]


def conv_step(u, col_offset, width, weight, bias, conv_state, slot_ids, activation=True):
    M = u.shape[0]
    lanes = torch.arange(M + 1, dtype=torch.int32)
    out = torch.empty((M, width), dtype=u.dtype)
    conv1d_silu(u, col_offset, width, weight, bias, conv_state, lanes[:M], lanes, slot_ids[:M], out, activation)
    conv_state_update(u, col_offset, width, weight.shape[1], conv_state, lanes, slot_ids[:M])
    u[:, col_offset:col_offset + width] = out


def ssm_scan(xbc, dt, dt_bias, A, D, ssm_state, cu_seqlens, slot_ids, num_groups, y, longest=0):
    _, H, P, N = ssm_state.shape
    E = H * P
    GN = num_groups * N
    group_of_head = torch.arange(H) // (H // num_groups)
    for lane in range(slot_ids.numel()):
        begin, end = int(cu_seqlens[lane]), int(cu_seqlens[lane + 1])
        slot = int(slot_ids[lane])
        state = ssm_state[slot].clone()
        for t in range(begin, end):
            row = _f(xbc[t])
            x = row[:E].reshape(H, P)
            B = row[E:E + GN].reshape(num_groups, N)[group_of_head]
            C = row[E + GN:].reshape(num_groups, N)[group_of_head]
            raw = _f(dt[t]) + dt_bias
            delta = torch.clamp(raw, min=0) + torch.log1p(torch.exp(-raw.abs()))
            decay = torch.exp(delta * A)
            state = state * decay[:, None, None] + (delta[:, None] * x)[:, :, None] * B[:, None, :]
            y[t] = ((state * C[:, None, :]).sum(-1) + D[:, None] * x).reshape(E)
        ssm_state[slot] = state


def gate_norm(y, z, weight, num_groups, eps, out):
    T, E = y.shape
    v = y * F.silu(_f(z))
    if weight is not None:
        grouped = v.reshape(T, num_groups, E // num_groups)
        grouped = grouped / torch.sqrt(grouped.pow(2).mean(-1, keepdim=True) + eps)
        v = grouped.reshape(T, E) * weight[None, :]
    out.copy_(v.to(out.dtype))


def add_scaled_rmsnorm(h, delta, scale, weight, eps, out, rows=None):
    total = h + _f(delta) * scale
    if rows is None:
        h.copy_(total)
        picked = total
    else:
        picked = total[rows.long()]
    if out is not None:
        out.copy_((picked / torch.sqrt(picked.pow(2).mean(-1, keepdim=True) + eps) * weight).to(out.dtype))


def polynorm(z, coefficients, eps, out):
    x = _f(z)
    unit = lambda values: values / torch.sqrt(values.pow(2).mean(-1, keepdim=True) + eps)
    c = coefficients
    out.copy_((c[0] * unit(x) + c[1] * unit(x * x) + c[2] * unit(x * x * x) + c[3]).to(out.dtype))


def tanh_rows(x, out):
    out.copy_(torch.tanh(_f(x)).to(out.dtype))


def head_norm_gate(raw, gate, weight, num_heads, eps, activation, out):
    T, width = raw.shape
    heads = raw.reshape(T, num_heads, width // num_heads)
    normed = (heads / torch.sqrt(heads.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, width)
    if weight is not None:
        normed = normed * weight
    g = _f(gate)
    out.copy_((normed * (F.silu(g) if activation == "silu" else torch.sigmoid(g))).to(out.dtype))


def linear_state_scan(u, *, q_col, k_col, v_col, num_heads, key_dim, value_dim, state, cu_seqlens, slot_ids, out,
                      max_query_len=0, head_decay=None, key_scale=1.0, positions=None, inv_freq=None, rotary_dim=0,
                      removal_col=-1, decay_logits=None, decay_bias=None, decay_floor=0.0, key_eps=0.0, chunks=None,
                      gate_power=0.0, query_scale=1.0):
    """``state`` [slots, H, value dim, key dim] holds the transposed state of every head."""
    H, K, V = num_heads, key_dim, value_dim
    T = u.shape[0]
    q = _f(u[:, q_col:q_col + H * K]).reshape(T, H, K).clone()
    k = _f(u[:, k_col:k_col + H * K]).reshape(T, H, K).clone()
    v = _f(u[:, v_col:v_col + H * V]).reshape(T, H, V)
    delta = removal_col >= 0
    gated = not delta and gate_power > 0
    if inv_freq is not None and rotary_dim > 0:
        half = rotary_dim // 2
        angle = positions.to(torch.float32)[:, None] * inv_freq[None, :]
        cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]

        def rotate(x):
            a, b = x[..., :half], x[..., half:rotary_dim]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., rotary_dim:]], dim=-1)
        q, k = rotate(q), rotate(k)
    q = q * query_scale
    if gated:
        decay = torch.exp(F.logsigmoid(decay_logits + decay_bias) * gate_power).reshape(T, H, K)
    if delta:
        unit = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + key_eps)
        removal = torch.sigmoid(_f(u[:, removal_col:removal_col + H * K])).reshape(T, H, K)
        decay = torch.exp(-decay_floor * torch.sigmoid(decay_logits + decay_bias)).reshape(T, H, K)
    else:
        k = k * key_scale
    for lane in range(cu_seqlens.numel() - 1):
        slot = int(slot_ids[lane])
        S = state[slot].transpose(-1, -2).clone()                   # [H, K, V]
        for t in range(int(cu_seqlens[lane]), int(cu_seqlens[lane + 1])):
            if delta:
                along = torch.einsum("hk,hkv->hv", unit[t], S)
                S = decay[t][:, :, None] * S - (removal[t] * unit[t])[:, :, None] * along[:, None, :] \
                    + k[t][:, :, None] * v[t][:, None, :]
            elif gated:
                S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            else:
                S = head_decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S, q[t]).reshape(H * V)
        state[slot] = S.transpose(-1, -2)


def argmax(logits, out):
    out.copy_(torch.argmax(logits, dim=-1).to(torch.int32))


# --------------------------------------------------------------------------- bigram embedding, layer norm
def embed_bigram(token_ids, table, multiplier, bigram, buckets, mul_prev, mul_cur, positions, lane_of_token,
                 cu_seqlens, slot_ids, previous, out):
    """out[t] = table[token] * multiplier + bigram[row], row = (token before * mul_prev + token * mul_cur) mod
    buckets, the last row (``buckets``) at position 0; the token before a lane's first one is
    ``previous[slot of the lane]``, which then takes the lane's last token."""
    ids = token_ids.long()
    rows = torch.empty_like(ids)
    for token in range(ids.numel()):
        lane = int(lane_of_token[token])
        if int(positions[token]) == 0:
            rows[token] = buckets
            continue
        before = int(previous[int(slot_ids[lane]), 0]) if token == int(cu_seqlens[lane]) else int(ids[token - 1])
        rows[token] = (before * mul_prev + int(ids[token]) * mul_cur) % buckets
    out.copy_(_f(table)[ids] * multiplier + _f(bigram)[rows])
    for lane in range(slot_ids.numel()):
        if int(cu_seqlens[lane + 1]) > int(cu_seqlens[lane]):
            previous[int(slot_ids[lane]), 0] = token_ids[int(cu_seqlens[lane + 1]) - 1]


def stream_add(h, rows, factor, vector):
    if rows is not None:
        h += float(factor) * _f(rows)
    if vector is not None:
        h += vector


def add_layernorm(h, branches, vector, weight, bias, eps, out, rows=None, branch_norm=None):
    total = h.clone()
    if branch_norm is not None:
        summed = torch.zeros_like(h)
        for tensor, factor in branches:
            summed = summed + float(factor) * _f(tensor)
        centred = summed - summed.mean(dim=-1, keepdim=True)
        variance = (centred * centred).mean(dim=-1, keepdim=True)
        total = total + centred / torch.sqrt(variance + branch_norm[2]) * branch_norm[0] + branch_norm[1]
        branches = []
    for tensor, factor in branches:
        total = total + float(factor) * _f(tensor)
    if vector is not None:
        total = total + vector
    if rows is None:
        h.copy_(total)
        picked = total
    else:
        picked = total[rows.long()]
    if out is not None:
        mean = picked.mean(dim=-1, keepdim=True)
        centred = picked - mean
        variance = (centred * centred).mean(dim=-1, keepdim=True)
        out.copy_((centred / torch.sqrt(variance + eps) * weight + bias).to(out.dtype))


def clamped_glu(gate_up, limit, alpha, up_offset, out):
    inner = out.shape[1]
    gate = _f(gate_up[:, :inner]).clamp(max=limit)
    up = _f(gate_up[:, inner:2 * inner]).clamp(min=-limit, max=limit)
    out.copy_((gate * torch.sigmoid(alpha * gate) * (up + up_offset)).to(out.dtype))


# --------------------------------------------------------------------------- latent attention
def _turn(x, positions, inv_freq, rotary_dim, interleaved):
    """x float32 [T, ..., width]: its first ``rotary_dim`` dimensions turned in pairs."""
    if inv_freq is None or rotary_dim == 0:
        return x
    half = rotary_dim // 2
    angle = positions.to(torch.float32).reshape(-1, *([1] * (x.dim() - 1))) * inv_freq
    cos, sin = angle.cos(), angle.sin()
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2] = a * cos - b * sin
        out[..., 1:rotary_dim:2] = b * cos + a * sin
    else:
        a, b = x[..., :half], x[..., half:rotary_dim]
        out[..., :half] = a * cos - b * sin
        out[..., half:rotary_dim] = b * cos + a * sin
    return out


def latent_prepare(down, q_rank, kv_rank, rope_dim, q_norm, kv_norm, eps, positions, inv_freq, rotary_dim,
                   interleaved, slot_mapping, k_cache, v_cache, query_latent):
    rows = _f(down)
    def rms(x, weight):
        return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight
    if q_rank > 0:
        query_latent.copy_(rms(rows[:, :q_rank], q_norm).to(query_latent.dtype))
    if slot_mapping is None:
        return
    latent = rms(rows[:, q_rank:q_rank + kv_rank], kv_norm)
    turned = _turn(rows[:, q_rank + kv_rank:q_rank + kv_rank + rope_dim], positions, inv_freq, rotary_dim, interleaved)
    page_size = k_cache.shape[2]
    pages = (slot_mapping // page_size).long()
    offsets = (slot_mapping % page_size).long()
    k_cache[pages, 0, offsets, :] = torch.cat([latent, turned], dim=1).to(k_cache.dtype)
    v_cache[pages, 0, :, offsets] = latent.to(v_cache.dtype)


def head_linear(x, x_col, x_head_stride, weight, out, out_col, out_head_stride):
    heads, features, inner = weight.shape
    for head in range(heads):
        rows = _f(x[:, x_col + head * x_head_stride:x_col + head * x_head_stride + inner])
        first = out_col + head * out_head_stride
        out[:, first:first + features] = (rows @ _f(weight[head]).T).to(out.dtype)


def rotate_heads(x, col, head_stride, num_heads, width, positions, inv_freq, rotary_dim, interleaved, out, out_col,
                 out_head_stride):
    for head in range(num_heads):
        rows = _f(x[:, col + head * head_stride:col + head * head_stride + width])
        first = out_col + head * out_head_stride
        out[:, first:first + width] = _turn(rows, positions, inv_freq, rotary_dim, interleaved).to(out.dtype)


def latent_attention_supported(dtype, num_heads, kv_rank, rope_dim, page_size):
    return False


# --------------------------------------------------------------------------- routed experts
def moe_route(logits, num_experts, top_k, correction, scale, eps, shared_gate, routing="softmax_then_top"):
    if routing == "top_then_softmax":
        biased = _f(logits[:, :num_experts]) + correction
        picked, chosen = torch.topk(biased, top_k, dim=-1)
        gate = torch.sigmoid(_f(logits[:, num_experts])) if shared_gate else None
        return chosen.to(torch.int32), torch.softmax(picked, dim=-1) * scale, gate
    scores = torch.softmax(_f(logits[:, :num_experts]), dim=-1)
    chosen = torch.topk(scores + correction, top_k, dim=-1).indices
    picked = torch.gather(scores, 1, chosen)
    weights = picked / (picked.sum(dim=-1, keepdim=True) + eps) * scale
    gate = torch.sigmoid(_f(logits[:, num_experts])) if shared_gate else None
    return chosen.to(torch.int32), weights, gate


class MoePlan:
    def __init__(self, chosen, num_experts, pad=16):
        tokens, top_k = chosen.shape
        self.pad, self.tokens, self.top_k = pad, tokens, top_k
        self.capacity = -(-(tokens * top_k + num_experts * (pad - 1)) // pad) * pad
        self.source = torch.full((self.capacity,), -1, dtype=torch.int32)
        self.place = torch.zeros((tokens * top_k,), dtype=torch.int32)
        self.tile_expert = torch.full((self.capacity // pad,), -1, dtype=torch.int32)
        cursor = 0
        flat = chosen.reshape(-1)
        for expert in range(num_experts):
            entries = torch.nonzero(flat == expert).reshape(-1)
            for index, entry in enumerate(entries.tolist()):
                self.source[cursor + index] = entry // top_k
                self.place[entry] = cursor + index
            tiles = -(-len(entries) // pad)
            self.tile_expert[cursor // pad:cursor // pad + tiles] = expert
            cursor += tiles * pad


def moe_plan(chosen, num_experts, pad=None):
    return MoePlan(chosen, num_experts, pad or 16)


def moe_expert_gemm(x, plan, weight, out, gather, glu, squared_relu=False):
    out.zero_()
    for tile in range(plan.tile_expert.numel()):
        expert = int(plan.tile_expert[tile])
        if expert < 0:
            continue
        for place in range(tile * plan.pad, (tile + 1) * plan.pad):
            source = int(plan.source[place])
            if source < 0:
                continue
            row = _f(x[source if gather else place])
            sums = _f(weight[expert]) @ row
            if glu is not None:
                inner = sums.numel() // 2
                gate = sums[:inner].clamp(max=glu.limit)
                up = sums[inner:].clamp(min=-glu.limit, max=glu.limit)
                sums = gate * torch.sigmoid(glu.alpha * gate) * (up + glu.up_offset)
            elif squared_relu:
                sums = torch.relu(sums) ** 2
            out[place] = sums.to(out.dtype)


def normed_sum(branches, out):
    total = torch.zeros(out.shape, dtype=torch.float32)
    for rows, factor, weight, eps in branches:
        x = _f(rows)
        total += factor * (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight)
    out.copy_(total)


def moe_combine(down, plan, weights, shared_rows, shared_gate, out):
    places = plan.place.long().reshape(plan.tokens, plan.top_k)
    total = (down[places] * weights[:, :, None]).sum(dim=1)
    if shared_rows is not None:
        total = total + shared_gate[:, None] * _f(shared_rows)
    out.copy_(total)


NAMES = ["fused_gemm_split", "add_partials_rmsnorm", "prefill_attention_supported", "decode_attention_supported", "decode_attention", "embed", "add_rmsnorm", "swiglu", "scale_to_f32", "tanh_softcap", "linear", "rope_kv_store", "paged_attention",
         "conv1d_silu", "conv_state_update", "conv_step", "ssm_scan", "gate_norm", "argmax", "feed_tokens", "keep_allowed",
         "add_scaled_rmsnorm", "polynorm", "tanh_rows", "head_norm_gate", "linear_state_scan",
         "embed_bigram", "stream_add", "add_layernorm", "clamped_glu", "latent_prepare", "head_linear", "rotate_heads",
         "latent_attention_supported", "moe_route", "moe_plan", "moe_expert_gemm", "moe_combine", "cast_rows",
         "attention_prepare", "normed_sum"]


def install(monkeypatch):
    """Replace the package's kernels with the functions above for one test."""
    from macllm_infer_amd.kernels import ops
    for name in NAMES:
        monkeypatch.setattr(ops, name, globals()[name])


def apply_penalties(logits, tokens, offsets, prompt_lens, repetition, presence, frequency, count_all, count_gen,
                    extra_source=None, extra_rows=None):
    for row in range(logits.shape[0]):
        history = tokens[int(offsets[row]):int(offsets[row + 1])].tolist()
        if extra_rows is not None and int(extra_rows[row]) >= 0:
            history.append(int(extra_source[int(extra_rows[row])]))          # the newest token, still on the device
        generated = history[int(prompt_lens[row]):]
        rep, pres, freq = float(repetition[row]), float(presence[row]), float(frequency[row])
        if rep > 0 and abs(rep - 1.0) >= 1.1920929e-07:
            for token in set(history):
                value = logits[row, token]
                logits[row, token] = value * rep if value < 0 else value / rep
        if pres != 0.0 or freq != 0.0:
            for token in set(generated):
                logits[row, token] -= freq * generated.count(token) + pres


def keep_allowed(logits, ids, offsets, keep):
    for row in range(logits.shape[0]):
        allowed = ids[int(offsets[row]):int(offsets[row + 1])].long()
        if allowed.numel():
            kept = torch.full_like(logits[row], float("-inf"))
            kept[allowed] = logits[row, allowed]
            logits[row] = kept


def sample(logits, temperature, top_k, top_p, seeds, draw_index, keys, out, done=None):
    import plain_impl
    for row in range(logits.shape[0]):
        out[row] = plain_impl.sample_token(
            logits[row], temperature=float(temperature[row]), top_k=int(top_k[row]), top_p=float(top_p[row]),
            seed=int(seeds[row]) & ((1 << 64) - 1), draw_index=int(draw_index[row]))


NAMES += ["apply_penalties", "sample"]


# ---------------------------------------------------------------- fused decode kernels, as compositions
PRO_NORM, PRO_PLAIN = 0, 1
EPI_PLAIN, EPI_SWIGLU, EPI_CONV = 0, 1, 2


def fused_gemm_supported(normed, rows, in_features):
    return False


def mixer_decode_supported(num_heads, num_kv_heads, head_dim, page_size, state_size, max_seq_len=1, window=None,
                           rotary_dim=0):
    return False


def fused_gemm_residual(weight, bias, x, h, hb, next_weight, ssq, fragments=None):
    """h += x . W^T + bias; hb = bfloat16(h * next_weight); ssq[b, m] = the sum of h[m]^2 over features 16 b .. 16 b + 15."""
    y = _f(x) @ _f(weight).T
    if bias is not None:
        y = y + bias
    h += y
    hb.copy_((h * next_weight).to(hb.dtype))
    M, N = h.shape
    squares = torch.zeros(M, ssq.shape[0] * 16)
    squares[:, :N] = h.pow(2)
    ssq.zero_()
    ssq[:, :M] = squares.reshape(M, -1, 16).sum(-1).T


def fused_gemm(weight, bias, out, *, out_scale=1.0, x=None, h_in=None, deltas=(), h_out=None, norm_weight=None,
               eps=0.0, epilogue=EPI_PLAIN, conv=None, feature_tiles=1, fragments=None, row_scale=None):
    if x is None:
        total = h_in.clone()
        for delta in deltas:
            total += _f(delta)
        if h_out is not None:
            h_out.copy_(total)
        normed = total / torch.sqrt(total.pow(2).mean(-1, keepdim=True) + eps) * norm_weight
        rows = _f(normed.to(torch.bfloat16))
    else:
        rows = _f(x)
    y = rows @ _f(weight).T
    if row_scale is not None:                  # the norm's division, on the float32 sums
        squares = row_scale.ssq[:, :y.shape[0]].sum(0)
        y = y * (1.0 / torch.sqrt(squares / row_scale.width + row_scale.eps))[:, None]
    if bias is not None:
        y = y + bias
    M, N = y.shape
    if epilogue == EPI_PLAIN:
        out.copy_((y * out_scale).to(out.dtype))
    elif epilogue == EPI_SWIGLU:
        tiles = _f(y.to(torch.bfloat16)).reshape(M, N // 16, 16)
        out.copy_((F.silu(tiles[..., :8]) * tiles[..., 8:]).reshape(M, N // 2).to(out.dtype))
    else:
        lo, hi, taps = conv["lo"], conv["hi"], conv["taps"]
        result = y.to(torch.bfloat16)
        sample = result[:, lo:hi].clone()
        for m in range(M):
            slot = int(conv["slot_ids"][m])
            window = torch.cat([conv["state"][slot], sample[m:m + 1]], dim=0)        # [taps, C]
            total = (_f(window) * conv["weight"].T).sum(0)
            if conv.get("bias") is not None:
                total = total + conv["bias"]
            result[m, lo:hi] = F.silu(total).to(torch.bfloat16)
            if taps > 1:
                conv["state"][slot] = window[1:]
        out.copy_(result)


def mixer_decode(u, *, num_heads, num_kv_heads, head_dim, q_col, k_col, v_col, inv_freq, rotary_dim, k_cache, v_cache,
                 block_tables, positions, slot_mapping, scale, window, max_seq_len, ssm_heads, ssm_head_dim,
                 state_size, num_groups, z_col, x_col, dt_col, dt_bias, A, D, ssm_state, slot_ids, out, ssm_y):
    M = u.shape[0]
    q_width, kv_width = num_heads * head_dim, num_kv_heads * head_dim
    qkv = torch.cat([u[:, q_col:q_col + q_width], u[:, k_col:k_col + kv_width], u[:, v_col:v_col + kv_width]], dim=1).clone()
    rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, positions, inv_freq, rotary_dim, slot_mapping, k_cache, v_cache)
    lanes = torch.arange(M, dtype=torch.int32)
    paged_attention(qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lanes, positions, scale,
                    window, out[:, :q_width])
    E = ssm_heads * ssm_head_dim
    width = E + 2 * num_groups * state_size
    y = torch.empty(M, E)
    cu = torch.arange(M + 1, dtype=torch.int32)
    ssm_scan(u[:, x_col:x_col + width], u[:, dt_col:dt_col + ssm_heads], dt_bias, A, D, ssm_state, cu, slot_ids,
             num_groups, y)
    if ssm_y is not None:
        ssm_y.copy_(y)
    else:
        gate_norm(y, u[:, z_col:z_col + E], None, num_groups, 0.0, out[:, q_width:])


NAMES += ["fused_gemm_supported", "mixer_decode_supported", "fused_gemm", "mixer_decode"]


def ssd_supported(chunk_size, head_dim, state_size, num_groups, inner_size):
    return False          # the host engine scans token by token


NAMES += ["ssd_supported"]
