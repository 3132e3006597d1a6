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


def add_rmsnorm(h, deltas, weight, eps, out, rows=None):
    total = h.clone()
    for delta in deltas:
        total += _f(delta)
    if rows is None:
        if deltas:
            h.copy_(total)
        picked = total
    else:
        picked = total[rows.long()]
    if out is not None:
        normed = picked / torch.sqrt(picked.pow(2).mean(-1, keepdim=True) + eps) * weight
        out.copy_(normed.to(out.dtype))


def swiglu(gate_up, out, tile=0):
    inner = gate_up.shape[1] // 2
    if tile:
        tiles = gate_up.reshape(gate_up.shape[0], inner // tile, 2, tile)
        gate, up = tiles[:, :, 0].reshape(-1, inner), tiles[:, :, 1].reshape(-1, inner)
    else:
        gate, up = gate_up[:, :inner], gate_up[:, inner:]
    out.copy_((F.silu(_f(gate)) * _f(up)).to(out.dtype))


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
                  k_cache, v_cache):
    T = qkv.shape[0]
    q_cols = num_heads * head_dim
    k_cols = num_kv_heads * head_dim
    q = _f(qkv[:, :q_cols]).reshape(T, num_heads, head_dim).clone()
    k = _f(qkv[:, q_cols:q_cols + k_cols]).reshape(T, num_kv_heads, head_dim).clone()
    v = qkv[:, q_cols + k_cols:q_cols + 2 * k_cols].reshape(T, num_kv_heads, head_dim)
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
                    cu_seqlens=None):
    """``max_seq_len`` sizes the kernel's launch and nothing else: not used here, and neither is the table of
    runs that picks the kernel for lanes of several tokens.  ``slopes``: a bias on the scores,
    ``-slopes[head] * (query position - key position)``."""
    T = q.shape[0]
    page_size = k_cache.shape[2]
    group = num_heads // num_kv_heads
    for token in range(T):
        lane = int(lane_of_token[token])
        position = int(positions[token])
        first = 0 if not window else max(0, position - window + 1)
        keys = torch.arange(first, position + 1)
        pages = block_tables[lane][(keys // page_size).long()].long()
        offsets = (keys % page_size).long()
        k = _f(k_cache[pages, :, offsets, :])        # [keys, Hkv, dh]
        v = _f(v_cache[pages, :, :, offsets])
        for head in range(num_heads):
            query = _f(q[token, head * head_dim:(head + 1) * head_dim])
            scores = (k[:, head // group, :] @ query) * scale
            if slopes is not None:
                scores = scores - slopes[head] * (position - keys).float()
            weights = torch.softmax(scores, dim=0)
            out[token, head * head_dim:(head + 1) * head_dim] = (weights @ v[:, head // group, :]).to(out.dtype)


def decode_attention_supported(dtype, num_heads, num_kv_heads, head_dim, page_size):
    return False


def prefill_attention_supported(dtype, num_heads, num_kv_heads, head_dim, page_size):
    return False


def decode_attention(q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lane_of_token, positions,
                     scale, window, max_seq_len, out):
    paged_attention(q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_tables, lane_of_token, positions,
                    scale, window, out)


def conv1d_silu(u, col_offset, width, weight, bias, conv_state, lane_of_token, cu_seqlens, slot_ids, out):
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
        out[begin:end] = F.silu(total).to(out.dtype)


def conv_state_update(u, col_offset, width, kernel, conv_state, cu_seqlens, slot_ids):
    if kernel <= 1:
        return
    for lane in range(slot_ids.numel()):
        begin, end = int(cu_seqlens[lane]), int(cu_seqlens[lane + 1])
        slot = int(slot_ids[lane])
        window = torch.cat([conv_state[slot], u[begin:end, col_offset:col_offset + width]], dim=0)
        conv_state[slot] = window[-(kernel - 1):]


def conv_step(u, col_offset, width, weight, bias, conv_state, slot_ids):
    M = u.shape[0]
    lanes = torch.arange(M + 1, dtype=torch.int32)
    out = torch.empty((M, width), dtype=u.dtype)
    conv1d_silu(u, col_offset, width, weight, bias, conv_state, lanes[:M], lanes, slot_ids[:M], out)
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


def argmax(logits, out):
    out.copy_(torch.argmax(logits, dim=-1).to(torch.int32))


NAMES = ["fused_gemm_split", "add_partials_rmsnorm", "prefill_attention_supported", "decode_attention_supported", "decode_attention", "embed", "add_rmsnorm", "swiglu", "scale_to_f32", "tanh_softcap", "linear", "rope_kv_store", "paged_attention",
         "conv1d_silu", "conv_state_update", "conv_step", "ssm_scan", "gate_norm", "argmax", "feed_tokens", "keep_allowed"]


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
