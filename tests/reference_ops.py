"""Plain torch versions of every kernel in ``lucciola_amd.kernels.ops``, with the same
signatures and memory layouts (paged caches, block tables, slot lists).  They compute in
float64 and round once to the output dtype.  Two uses: each GPU kernel is tested alone against
its function here, and CPU tests put these in place of the kernels to exercise the step
function, the cache and the scheduler without a GPU.  Nothing under ``lucciola_amd`` imports
this file.
"""
import math

import torch

F64 = torch.float64


def embedding(ids, table, scale=1.0):
    return table[ids.long()].to(torch.float32) * scale


def rmsnorm(h, delta, weight, eps, out_dtype, rows=None, scaled=False):   # never hands out scaled rows
    if rows is None:
        if delta is not None:
            h += delta.to(torch.float32)
        v = h.to(F64)
    else:
        v = h[rows.long()].to(F64)
        if delta is not None:
            v = (h[rows.long()] + delta[rows.long()].to(torch.float32)).to(F64)
    inv = torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return (v * inv * weight.to(F64)).to(out_dtype)


def rmsnorm_act(x, weight, eps, column=None):
    v = x.to(F64) if column is None else x[:, column:column + weight.shape[0]].to(F64)
    inv = torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return (v * inv * weight.to(F64)).to(x.dtype)


def gemm(x, w, out_dtype=None, defer=False, shares=False):   # never defers, never hands out shares
    return (x.to(F64) @ w.to(F64).T).to(out_dtype or x.dtype)


def qk_norm_rope_write(qkv, nh, nkv, d, q_weight, k_weight, eps, positions, rope_table,
                       k_cache, v_cache, slots, page_size):
    T = qkv.shape[0]
    x = qkv.view(T, nh + 2 * nkv, d)
    q, k, v = x[:, :nh].to(F64), x[:, nh:nh + nkv].to(F64), x[:, nh + nkv:]
    if q_weight is not None:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.to(F64)
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.to(F64)
    if rope_table is not None:
        rot = rope_table.shape[1]
        half = rot // 2
        cs = rope_table[positions.long()].to(F64)
        cos, sin = cs[:, None, :half], cs[:, None, half:]

        def rotate(t):
            a, b = t[..., :half], t[..., half:rot]
            return torch.cat([a * cos - b * sin, a * sin + b * cos, t[..., rot:]], dim=-1)
        q, k = rotate(q), rotate(k)
    x[:, :nh] = q.to(qkv.dtype)
    x[:, nh:nh + nkv] = k.to(qkv.dtype)
    if k_cache is not None and slots is not None:
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            page, off = divmod(s, page_size)
            k_cache[page, :, off, :] = x[t, nh:nh + nkv]
            v_cache[page, :, :, off] = v[t]


def attention(qkv, batch, k_cache, v_cache, nh, nkv, d, page_size, scale, window=0, prologue=None):
    if prologue is not None:
        qk_norm_rope_write(qkv, nh, nkv, d, prologue.q_weight, prologue.k_weight, prologue.eps,
                           batch.positions, prologue.rope_table, k_cache, v_cache, prologue.slots,
                           page_size)
    T = qkv.shape[0]
    q = qkv[:, :nh * d].reshape(T, nh, d).to(F64)     # the q heads come first (alone, or with k and v behind)
    out = torch.zeros(T, nh, d, dtype=F64, device=qkv.device)
    group = nh // nkv
    tok_req = batch.tok_req.tolist()
    positions = batch.positions.tolist()
    tables = batch.block_table.tolist()
    for t in range(T):
        p = positions[t]
        lo = max(0, p - window + 1) if window else 0
        table = tables[tok_req[t]]
        js = list(range(lo, p + 1))
        pages = torch.tensor([table[j // page_size] for j in js], dtype=torch.long)
        assert (pages >= 0).all(), "attention reads a page that was given back"
        offs = torch.tensor([j % page_size for j in js], dtype=torch.long)
        keys = k_cache[pages, :, offs, :].to(F64)      # [n, nkv, d]
        vals = v_cache[pages, :, :, offs].to(F64)
        for h in range(nh):
            s = (keys[:, h // group, :] @ q[t, h]) * scale
            w = torch.softmax(s, dim=0)
            out[t, h] = w @ vals[:, h // group, :]
    return out.reshape(T, nh * d).to(qkv.dtype)


def swiglu(gu):
    I = gu.shape[1] // 2
    g, u = gu[:, :I].to(F64), gu[:, I:].to(F64)
    return (g / (1 + torch.exp(-g)) * u).to(gu.dtype)


def sample(logits, temperature=None, uniform=None):
    R = logits.shape[0]
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    for r in range(R):
        t = float(temperature[r]) if temperature is not None else 0.0
        if t <= 0:
            out[r] = int(torch.argmax(logits[r]))
            continue
        z = logits[r].to(F64) / t
        p = torch.exp(z - z.max())
        cdf = torch.cumsum(p, 0)
        target = float(uniform[r]) * float(cdf[-1])
        out[r] = int(min(int(torch.searchsorted(cdf, torch.tensor(target, dtype=F64), right=True)),
                         logits.shape[1] - 1))
    return out


# ------------------------------------------------------------------ the kernels of later parts
def dynamic_tanh(h, delta, weight, bias, alpha, out_dtype, rows=None):
    if rows is None:
        if delta is not None:
            h += delta.to(torch.float32)
        v = h.to(F64)
    else:
        v = h[rows.long()].to(F64)
        if delta is not None:
            v = (h[rows.long()] + delta[rows.long()].to(torch.float32)).to(F64)
    return (torch.tanh(alpha * v) * weight.to(F64) + bias.to(F64)).to(out_dtype)


def stream_add(h, delta, vector, more=None):
    if delta is not None:
        h += delta.to(torch.float32)
    if more is not None:
        h += more
    h += vector


def scale_(x, factor):
    x *= factor
    return x


def _shift_rows(u, mix, state, q_offsets, slot_ids):
    """u [T, n] float64 normed rows -> shifted rows; the state takes every request's last row."""
    y = torch.empty_like(u)
    starts, slots = q_offsets.tolist(), slot_ids.tolist()
    for r, slot in enumerate(slots):
        a, b = starts[r], starts[r + 1]
        if b <= a:
            continue
        before = torch.cat([state[slot].to(F64)[None], u[a:b - 1]], dim=0)
        y[a:b] = u[a:b] + (before - u[a:b]) * mix.to(F64)
        state[slot] = u[b - 1].to(torch.float32)
    return y


def token_shift(x, mix, state, tok_req, q_offsets, slot_ids):
    return _shift_rows(x.to(F64), mix, state, q_offsets, slot_ids).to(x.dtype)


def rms_shift(h, delta, gain, eps, mix, state, tok_req, q_offsets, slot_ids, out_dtype):
    v = h.clone()
    if delta is not None:
        v += delta.to(torch.float32)
    v64 = v.to(F64)
    u = v64 * torch.rsqrt((v64 * v64).mean(dim=-1, keepdim=True) + eps) * gain
    return v, _shift_rows(u, mix, state, q_offsets, slot_ids).to(out_dtype)


def _act(z, kind, params=(0.0, 0.0)):
    if kind == "xielu":
        neg = torch.clamp(z, max=0)
        return torch.where(z > 0, params[0] * z * z + 0.5 * z, params[1] * (torch.expm1(neg) - neg) + 0.5 * z)
    if kind == "gelu_tanh":
        return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))
    if kind == "relu_squared":
        return torch.clamp(z, min=0) ** 2
    raise ValueError(kind)


def activation(x, kind, params=(0.0, 0.0)):
    x.copy_(_act(x.to(F64), kind, params).to(x.dtype))
    return x


def gemm_act(x, w, kind, out_dtype, params=(0.0, 0.0)):
    return _act(x.to(F64) @ w.to(F64).T, kind, params).to(out_dtype)


def grouped_gemm(x, w, out, rows, gate=None, activation=None, gate_per_group=False):
    G, N, K = w.shape
    for g in range(G):
        xs = x.tensor[:rows, x.column + g * x.group: x.column + g * x.group + K].to(F64)
        y = xs @ w[g].to(F64).T
        if activation:
            y = _act(y, activation)
        if gate is not None:
            width = 1 if gate_per_group else N
            y = y * torch.sigmoid(gate.tensor[:rows, gate.column + g * gate.group: gate.column + g * gate.group + width].to(F64))
        out.tensor[:rows, out.column + g * out.group: out.column + g * out.group + N] = y.to(out.tensor.dtype)


def _turn(part, cs, rd, pairing):
    """part [T, ..., n] (float64), cs [T, rd] cosines then sines"""
    if cs is None or rd == 0:
        return part
    half = rd // 2
    shape = [part.shape[0]] + [1] * (part.dim() - 2) + [half]
    cos, sin = cs[:, :half].view(shape), cs[:, half:].view(shape)
    out = part.clone()
    if pairing == "interleaved":
        u, v = part[..., 0:rd:2], part[..., 1:rd:2]
        out[..., 0:rd:2] = u * cos - v * sin
        out[..., 1:rd:2] = v * cos + u * sin
    else:
        u, v = part[..., :half], part[..., half:rd]
        out[..., :half] = u * cos - v * sin
        out[..., half:rd] = v * cos + u * sin
    return out


def latent_prepare(proj, heads, dim, rot, rank, norm_weight, eps, positions, rope_table, pairing, cache, slots, qa,
                   q=None, kv_column=None):
    T = proj.shape[0]
    if q is None:
        q, kv_column = proj, heads * (dim + rot)
    kv_column = int(kv_column or 0)
    q = q[:, :heads * (dim + rot)].reshape(T, heads, dim + rot).to(F64)
    down = proj[:, kv_column: kv_column + rank + rot].to(F64)
    c = down[:, :rank]
    c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * norm_weight.to(F64)
    cs = rope_table[positions.long()].to(F64) if rope_table is not None and rot else None
    rd = rope_table.shape[1] if cs is not None else 0
    kr = _turn(down[:, rank:], cs, rd, pairing)
    qr = _turn(q[..., dim:], cs, rd, pairing)
    qa.view(T, heads, rank + rot)[..., rank:] = qr.to(qa.dtype)
    if slots is not None:
        page = cache.shape[1]
        row = torch.cat([c, kr], dim=-1).to(cache.dtype)
        for t in range(T):
            s = int(slots[t])
            if s >= 0:
                cache[s // page, s % page] = row[t]


def latent_attention(qa, heads, rank, rot, tok_req, positions, block_table, cache, page_size, scale, window=0,
                     plan=None, max_ctx=0, sink=None):
    T = qa.shape[0]
    q = qa.view(T, heads, rank + rot).to(F64)
    out = torch.zeros(T, heads, rank, dtype=F64, device=qa.device)
    reqs, pos, tables = tok_req.tolist(), positions.tolist(), block_table.tolist()
    for t in range(T):
        p = pos[t]
        lo = max(0, p - window + 1) if window else 0
        table = tables[reqs[t]]
        js = list(range(lo, p + 1))
        pages = torch.tensor([table[j // page_size] for j in js], dtype=torch.long)
        assert (pages >= 0).all(), "latent attention reads a page that was given back"
        offs = torch.tensor([j % page_size for j in js], dtype=torch.long)
        rows = cache[pages, offs].to(F64)                  # [n, rank + rot]
        s = (q[t] @ rows.T) * scale                         # [heads, n]
        if sink is not None:                                # one more term in the denominator, no row
            s = torch.cat([s, sink.to(F64)[:, None]], dim=-1)
        w = torch.softmax(s, dim=-1)[:, :len(js)]
        out[t] = w @ rows[:, :rank]
    return out.reshape(T, heads * rank).to(qa.dtype)


class _Routing:
    pass


def moe_route(logits, top, renormalise=True, eps=1e-20, large_tiles=False):
    s = torch.softmax(logits.to(F64), dim=-1)
    picked, ids = torch.topk(s, top, dim=-1)
    if renormalise:
        picked = picked / (picked.sum(-1, keepdim=True) + eps)
    r = _Routing()
    r.ids, r.weights = ids.to(torch.int32), picked.to(torch.float32)
    return r


def moe_route_sigmoid(logits, top, correction=None, groups=1, keep=1, scale=1.0, large_tiles=False):
    T, E = logits.shape
    s = torch.sigmoid(logits.to(F64))
    choice = s + correction.to(F64) if correction is not None else s.clone()
    if groups > 1:
        per = E // groups
        ranks = torch.topk(choice.view(T, groups, per), min(2, per), dim=-1).values.sum(-1)
        kept = torch.zeros(T, groups, dtype=torch.bool)
        kept.scatter_(1, torch.topk(ranks, keep, dim=-1).indices, True)
        choice = choice.masked_fill(~kept.repeat_interleave(per, dim=1), float("-inf"))
    ids = torch.topk(choice, top, dim=-1).indices
    r = _Routing()
    r.ids, r.weights = ids.to(torch.int32), (torch.gather(s, 1, ids) * scale).to(torch.float32)
    return r


def lightning_prepare(proj, heads, key_dim, value_dim, decay):
    T = proj.shape[0]
    nk, nv = heads * key_dim, heads * value_dim

    def silu(z):
        return z * torch.sigmoid(z)
    p = proj.to(F64)
    coef = torch.zeros(3, T, nk, dtype=F64)       # decay, write, read: the recurrence without removal
    coef[0] = decay.to(F64).repeat_interleave(key_dim)[None, :]
    coef[1] = silu(p[:, nk:2 * nk])
    coef[2] = silu(p[:, :nk])
    return coef.to(torch.float32), silu(p[:, 2 * nk:2 * nk + nv]).to(torch.float32)


def lightning_readout(o, gates, gate_column, weight, eps, out_dtype):
    x = o.to(F64)
    n = x.shape[1]
    inv = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return (x * inv * weight.to(F64) * torch.sigmoid(gates[:, gate_column:gate_column + n].to(F64))).to(out_dtype)


def moe_experts(x, w, routing, out_dtype, activation=None, gather=False):
    """Rows in (token, choice) order here: the order of the sorted rows is the kernels' own matter."""
    T, top = routing.ids.shape
    out = torch.zeros(T * top, w.shape[1], dtype=F64, device=x.device)
    for t in range(T):
        for k in range(top):
            row = x[t] if gather else x[t * top + k]
            y = w[int(routing.ids[t, k])].to(F64) @ row.to(F64)
            out[t * top + k] = _act(y, activation) if activation else y
    return out.to(out_dtype)


def moe_combine(y, routing, out_dtype):
    T, top = routing.ids.shape
    return (y.to(F64).view(T, top, -1) * routing.weights.to(F64)[:, :, None]).sum(1).to(out_dtype)


def attention_takes_shares(*args, **kwargs):
    return False


def feed_tokens(ids, source, sampled):
    take = source >= 0
    ids[take] = sampled[source[take].long()]


# ------------------------------------------------------------------ layer norm, position vector, heads in slots
def _layer_norm64(v, weight, bias, eps):
    mean = v.mean(-1, keepdim=True)
    dev = v - mean
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * weight.to(F64) + bias.to(F64)


def layer_norm_act(x, weight, bias, eps):
    return _layer_norm64(x.to(F64), weight, bias, eps).to(x.dtype)


def layer_norm(h, delta, weight, bias, eps, out_dtype, rows=None, branch_scale=1.0):
    from lucciola_amd.kernels import ops
    if isinstance(delta, ops.NormedBranch):
        delta = _layer_norm64(delta.x.to(F64), delta.weight, delta.bias, delta.eps).to(torch.float32)
    elif delta is not None and not isinstance(delta, torch.Tensor):
        delta = delta.value()
    if rows is None:
        if delta is not None:
            h += (branch_scale * delta.to(F64)).to(torch.float32)
        v = h.to(F64)
    else:
        v = h[rows.long()].to(F64)
        if delta is not None:
            v = (h[rows.long()] + (branch_scale * delta[rows.long()].to(F64)).to(torch.float32)).to(F64)
    return _layer_norm64(v, weight, bias, eps).to(out_dtype)


def embedding_sinusoid(ids, table, positions, frequencies, scale=1.0):
    H = table.shape[1]
    angle = positions.to(torch.float32)[:, None] * frequencies[None, :]
    out = table[ids.long()].to(torch.float32) * scale
    out[:, 0::2] += torch.sin(angle)
    out[:, 1::2] += torch.cos(angle)[:, :H // 2]
    return out


def gated_activation(gu, kind):
    I = gu.shape[1] // 2
    g, u = gu[:, :I].to(F64), gu[:, I:].to(F64)
    a = g / (1 + torch.exp(-g)) if kind == "silu" else _act(g, kind)
    return (a * u).to(gu.dtype)


def attention_head_slot(size):
    for slot in (32, 64, 96, 128):
        if size <= slot:
            return slot
    return -(-size // 16) * 16


def head_norm_write(proj, nh, nkv, d, dv, slot, q_weight, k_weight, eps, head_scale, k_cache, v_cache, slots,
                    page_size):
    T = proj.shape[0]
    q = proj[:, :nh * d].view(T, nh, d).to(F64)
    if q_weight is not None:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.to(F64)
    if head_scale is not None:
        q = q * head_scale.to(F64)[None, :, None]
    out = torch.zeros(T, nh, slot, dtype=proj.dtype, device=proj.device)
    out[:, :, :d] = q.to(proj.dtype)
    if nkv and slots is not None and k_cache is not None:
        k = proj[:, nh * d: (nh + nkv) * d].view(T, nkv, d).to(F64)
        if k_weight is not None:
            k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.to(F64)
        v = proj[:, (nh + nkv) * d:].view(T, nkv, dv)
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            page, off = divmod(s, page_size)
            k_cache[page, :, off, :] = 0
            k_cache[page, :, off, :d] = k[t].to(k_cache.dtype)
            v_cache[page, :, :, off] = 0
            v_cache[page, :, :dv, off] = v[t].to(v_cache.dtype)
    return out.view(T, nh * slot)


# ------------------------------------------------------------------ delta rules
def check_delta_sizes(what, key_dim, value_dim, taps=1):
    pass


def general_delta_prepare(proj, heads, dim, inner, decay_out, decay_bias, removal_bias, unit_eps, decay_scale):
    T, n = proj.shape[0], heads * dim
    p = proj.to(F64)
    r, k, v, removal, decay_in = p[:, :n], p[:, n:2 * n], p[:, 2 * n:3 * n], p[:, 4 * n:5 * n], p[:, 5 * n:]
    w = torch.exp(-decay_scale * torch.sigmoid(torch.tanh(decay_in) @ decay_out.to(F64).T + decay_bias.to(F64)))
    a = torch.sigmoid(removal + removal_bias.to(F64))
    kh = k.view(T, heads, dim)
    u = (kh / torch.sqrt((kh * kh).sum(-1, keepdim=True) + unit_eps)).view(T, n)
    coef = torch.stack([w, u, a * u, k, r]).to(torch.float32)
    return coef, v.to(torch.float32).contiguous()


def _conv_inputs(proj, tail, C, K, tok_req, q_offsets, slot_ids):
    """[K, T, C]: input j steps back of every token and channel."""
    T = proj.shape[0]
    x = torch.zeros(K, T, C, dtype=F64)
    starts = q_offsets.tolist()
    for t in range(T):
        r = int(tok_req[t])
        n = t - starts[r]
        for j in range(K):
            if j <= n:
                x[j, t] = proj[t - j, :C].to(F64)
            else:
                x[j, t] = tail[int(slot_ids[r]), (K - 1) - (j - n)].to(F64)
    return x


def gated_delta_prepare(proj, tail, taps, rate_log, rate_bias, heads, kv_heads, key_dim, value_dim, num_taps,
                        unit_eps, tok_req, q_offsets, slot_ids):
    T = proj.shape[0]
    nk, nv = kv_heads * key_dim, heads * value_dim
    C = 2 * nk + nv
    x = _conv_inputs(proj, tail, C, num_taps, tok_req, q_offsets, slot_ids)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(num_taps):
        y += x[j] * taps.to(F64)[:, num_taps - 1 - j][None, :]
    y = y / (1 + torch.exp(-y))
    q, k, v = y[:, :nk].view(T, kv_heads, key_dim), y[:, nk:2 * nk].view(T, kv_heads, key_dim), y[:, 2 * nk:]
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * key_dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
    rep = heads // kv_heads
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)        # [T, heads, key_dim]
    beta = torch.sigmoid(proj[:, C + nv: C + nv + heads].to(F64))[:, :, None]
    rate = proj[:, C + nv + heads:].to(F64) + rate_bias.to(F64)
    g = torch.exp(-torch.exp(rate_log.to(F64)) * torch.nn.functional.softplus(rate))[:, :, None]
    coef = torch.stack([g.expand_as(k), g * k, beta * k, beta * k, q]).reshape(5, T, heads * key_dim)
    return coef.to(torch.float32).contiguous(), v.to(torch.float32).contiguous()


def conv_tail_update(proj, tail, channels, num_taps, q_offsets, slot_ids, num_requests):
    if num_taps <= 1:
        return
    starts = q_offsets.tolist()
    for r in range(num_requests):
        s = int(slot_ids[r])
        rows = torch.cat([tail[s], proj[starts[r]:starts[r + 1], :channels].to(tail.dtype)], dim=0)
        tail[s] = rows[-(num_taps - 1):]


def delta_scan(coef, v, state, q_offsets, slot_ids, num_requests, heads, key_dim, value_dim):
    T = v.shape[0]
    if coef.shape[0] == 3:      # decay, write, read: no removal term
        zero = torch.zeros_like(coef[0])
        coef = torch.stack([coef[0], zero, zero, coef[1], coef[2]])
    c = coef.to(F64).view(5, T, heads, key_dim)
    vv = v.to(F64).view(T, heads, value_dim)
    out = torch.zeros(T, heads, value_dim, dtype=F64)
    starts = q_offsets.tolist()
    for r in range(num_requests):
        S = state[int(slot_ids[r])].to(F64).transpose(1, 2)    # kept as [heads, value, key]; here [heads, key, value]
        for t in range(starts[r], starts[r + 1]):
            taken = torch.einsum("hk,hkv->hv", c[1, t], S)
            S = c[0, t][:, :, None] * S - c[2, t][:, :, None] * taken[:, None, :] + c[3, t][:, :, None] * vv[t][:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S, c[4, t])
        state[int(slot_ids[r])] = S.transpose(1, 2).to(state.dtype)
    return out.view(T, heads * value_dim).to(torch.float32)


def head_gate_norm(o, gates, gate_column, weight, weight_per_head, eps, gate, heads, dim, out_dtype):
    T = o.shape[0]
    x = o.to(F64).view(T, heads, dim)
    x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    w = weight.to(F64).view(heads, dim) if weight_per_head else weight.to(F64)[None, :]
    g = gates[:, gate_column:gate_column + heads * dim].to(F64).view(T, heads, dim)
    g = torch.sigmoid(g) if gate == "sigmoid" else g * torch.sigmoid(g)
    return (x * w * g).view(T, heads * dim).to(out_dtype)


def moe_route_logits(logits, experts, top, bias=None, large_tiles=False):
    z = logits[:, :experts].to(F64)
    if bias is not None:
        z = z + bias.to(F64)
    picked, ids = torch.topk(z, top, dim=-1)
    r = _Routing()
    r.ids, r.weights = ids.to(torch.int32), torch.softmax(picked, dim=-1).to(torch.float32)
    return r


def moe_combine_shared(y, routing, shared, gates, gate_column, out_dtype, weighted=True):
    T, top = routing.ids.shape
    total = y.to(F64).view(T, top, -1)
    if weighted:
        total = total * routing.weights.to(F64)[:, :, None]
    total = total.sum(1)
    if shared is not None:
        gate = torch.sigmoid(gates[:, gate_column].to(F64))[:, None] if gates is not None else 1.0
        total = total + gate * shared.to(F64)
    return total.to(out_dtype)


def gated_activation_weighted(gu, kind, routing):
    """Rows in (token, choice) order, as :func:`moe_experts` leaves them here."""
    I = gu.shape[1] // 2
    w = routing.weights.to(F64).reshape(-1, 1)
    g, u = w * gu[:, :I].to(F64), w * gu[:, I:].to(F64)
    a = g / (1 + torch.exp(-g)) if kind == "silu" else _act(g, kind)
    return (a * u).to(gu.dtype)


MASKED_ATTENTION_MAX = 256
SHORT_CONV_MAX_TAPS = 16


def _convolved(proj, C, taps, tail, tok_req, q_offsets, slot_ids, bias=None):
    """The first C columns of proj through their causal convolutions, float64 [T, C]."""
    K = taps.shape[1]
    x = _conv_inputs(proj, tail, C, K, tok_req, q_offsets, slot_ids)
    y = torch.zeros(proj.shape[0], C, dtype=F64)
    for j in range(K):
        y += x[j] * taps.to(F64)[:, K - 1 - j][None, :]
    return y if bias is None else y + bias.to(F64)


def attention_prepare(proj, nq, nk, nv, d, dv, out_dtype, k_cache, v_cache, rows, taps=None, tail=None, tok_req=None,
                      q_offsets=None, slot_ids=None, table=None, rot=0, positions=None, unit_eps=None):
    T = proj.shape[0]
    C = (nq + nk) * d + nv * dv
    y = proj[:, :C].to(F64) if taps is None else _convolved(proj, C, taps, tail, tok_req, q_offsets, slot_ids)
    qk = y[:, :(nq + nk) * d].reshape(T, nq + nk, d).clone()
    if table is not None:
        cs = table[positions.long()].to(F64)
        cos, sin = cs[:, None, :rot // 2], cs[:, None, rot // 2:]
        a, b = qk[..., 0:rot:2].clone(), qk[..., 1:rot:2].clone()
        qk[..., 0:rot:2] = a * cos - b * sin
        qk[..., 1:rot:2] = b * cos + a * sin
    if unit_eps is not None:
        qk = qk / torch.sqrt((qk * qk).mean(-1, keepdim=True) + unit_eps)
    if rows is not None:
        page = k_cache.shape[1]
        keep = rows >= 0
        at = rows[keep].long()
        k_cache[at // page, at % page] = qk[keep, nq:].reshape(-1, nk * d).to(k_cache.dtype)
        v_cache[at // page, :, at % page] = y[keep, (nq + nk) * d:C].to(v_cache.dtype)      # transposed inside a page
    return qk[:, :nq].reshape(T, nq * d).to(out_dtype)


def masked_attention(q, k_cache, v_cache, tok_req, positions, block_table, page_size, heads, kv_heads, maps, d, dv,
                     scale, chunk=0, window=0, r1=None, r2=None, sink=None, subtract=0.0, unit_eps=None,
                     out_scale=1.0, gate=None, gate_column=0, plan=None, max_ctx=0):
    T = q.shape[0]
    kc = k_cache.reshape(-1, kv_heads, maps, d).to(F64)
    vc = v_cache.transpose(1, 2).reshape(-1, kv_heads, dv).to(F64)
    qq = q.to(F64).view(T, heads, maps, d)
    out = torch.zeros(T, heads, dv, dtype=F64)
    for t in range(T):
        p, r = int(positions[t]), int(tok_req[t])
        lo = 0
        if chunk > 0:
            lo = p - p % chunk
        if window > 0:
            lo = max(lo, p - window + 1)
        js = torch.arange(lo, p + 1)
        rows = block_table[r].long()[js // page_size] * page_size + js % page_size
        for h in range(heads):
            g = h // (heads // kv_heads)
            a = []
            for m in range(maps):
                s = (kc[rows, g, m] @ qq[t, h, m]) * scale
                if r1 is not None:
                    s = s - float(r1[h]) * torch.log1p(float(r2[h]) * (p - js).to(F64))
                top = s.max() if sink is None else torch.maximum(s.max(), sink[h].to(F64))
                e = torch.exp(s - top)
                total = e.sum() + (torch.exp(sink[h].to(F64) - top) if sink is not None else 0.0)
                a.append((e / total) @ vc[rows, g])
            o = a[0] if maps == 1 else a[0] - subtract * a[1]
            if unit_eps is not None:
                o = o / torch.sqrt((o * o).mean() + unit_eps) * out_scale
            out[t, h] = o
    out = out.view(T, heads * dv)
    if gate is not None:
        out = out * torch.sigmoid(gate[:, gate_column:gate_column + heads * dv].to(F64))
    return out.to(q.dtype)


def state_space_prepare(proj, heads, groups, state, value_dim, taps, bias, tail, dt_bias, a_log, tok_req, q_offsets,
                        slot_ids):
    T = proj.shape[0]
    inner = heads * value_dim
    C = inner + 2 * groups * state
    y = _convolved(proj, C, taps, tail, tok_req, q_offsets, slot_ids, bias)
    y = y * torch.sigmoid(y)
    rep = heads // groups
    B = y[:, inner:inner + groups * state].view(T, groups, state).repeat_interleave(rep, dim=1)
    Cm = y[:, inner + groups * state:].view(T, groups, state).repeat_interleave(rep, dim=1)
    step = torch.nn.functional.softplus(proj[:, C + inner:].to(F64) + dt_bias.to(F64))        # [T, heads]
    decay = torch.exp(-torch.exp(a_log.to(F64)) * step)
    coef = torch.stack([decay[:, :, None].expand(T, heads, state), step[:, :, None] * B, Cm])
    return coef.reshape(3, T, heads * state).to(torch.float32).contiguous(), y[:, :inner].to(torch.float32).contiguous()


def state_space_readout(o, x, gates, z_column, skip, heads, value_dim, weight, parts, eps, out_dtype):
    T, n = o.shape
    z = gates[:, z_column:z_column + n].to(F64)
    y = (o.to(F64) + skip.to(F64).repeat_interleave(value_dim)[None, :] * x.to(F64)) * (z * torch.sigmoid(z))
    y = y.view(T, parts, n // parts)
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, n) * weight.to(F64)).to(out_dtype)


def scaled_sum(a, a_scale, b, b_scale):
    a = a if isinstance(a, torch.Tensor) else a.value()
    b = b if isinstance(b, torch.Tensor) else b.value()
    return (a_scale * a.to(F64) + b_scale * b.to(F64)).to(torch.float32)


def moe_large_tiles(x_dtype, up, down):
    return False


ALL = ("layer_norm", "layer_norm_act", "embedding_sinusoid", "gated_activation", "attention_head_slot", "head_norm_write",
       "check_delta_sizes", "general_delta_prepare", "gated_delta_prepare", "conv_tail_update", "delta_scan",
       "head_gate_norm", "moe_route_logits", "moe_combine_shared", "feed_tokens", "attention_takes_shares", "embedding", "rmsnorm", "rmsnorm_act", "gemm", "qk_norm_rope_write", "attention",
       "swiglu", "sample", "dynamic_tanh", "stream_add", "activation", "gemm_act", "grouped_gemm",
       "latent_prepare", "latent_attention", "moe_route", "moe_experts", "moe_combine",
       "scale_", "token_shift", "rms_shift", "moe_route_sigmoid", "lightning_prepare", "lightning_readout",
       "gated_activation_weighted", "attention_prepare", "masked_attention", "state_space_prepare",
       "state_space_readout", "scaled_sum")


def install(monkeypatch):
    """Put these functions in place of the kernels (CPU tests of the engine's host logic)."""
    from lucciola_amd.kernels import ops
    for name in ALL:
        monkeypatch.setattr(ops, name, globals()[name])
