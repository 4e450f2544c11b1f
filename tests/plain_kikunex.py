"""A plain, slow implementation of the Kikunex decoder: whole sequences, no cache, one function
for each mechanism, float64 on the CPU.  It shares no code with the engine under
``lucciola_amd`` and is what the engine is compared with.

Notation: x is the residual stream [T, width]; a linear weight is stored [out, in] and applied
as W x; positions count from 0.
"""
import math

import torch

F64 = torch.float64


def linear(x, weight):
    """y[t, n] = sum_k x[t, k] W[n, k]"""
    return x.to(F64) @ weight.to(F64).T


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension (eps inside the root)."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return unit_rms(x, eps) * float(g)


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def silu(z):
    z = z.to(F64)
    return z * torch.sigmoid(z)


def relu_squared(z):
    return torch.clamp(z.to(F64), min=0.0) ** 2


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    z = z.to(F64)
    a, b = softplus(float(p)), 0.5 + softplus(float(q))
    neg = torch.clamp(z, max=0.0)
    return torch.where(z > 0, a * z * z + 0.5 * z, b * (torch.expm1(neg) - neg) + 0.5 * z)


def token_shift(h, mix):
    """Row t becomes h_t + (h_(t-1) - h_t) * mix, with the rows as they were before; a row of
    zeros stands before the first."""
    h = h.to(F64)
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * mix.to(F64)


def rotate_half(x, positions, dims, base):
    """x: [T, ..., n].  Of the last dimension's first ``dims`` entries, entry i pairs with entry
    i + dims/2: (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * base^(-2i/dims);
    the rest pass unchanged."""
    x = x.to(F64).clone()
    half = dims // 2
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * torch.arange(half, dtype=F64) / dims)
    angle = torch.as_tensor(positions, dtype=F64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    u, v = x[..., :half].clone(), x[..., half:dims].clone()
    x[..., :half] = u * cos - v * sin
    x[..., half:dims] = v * cos + u * sin
    return x


def sink_softmax(scores, positions, window, sink):
    """scores [T, T] of one head; row i sees column j where 0 <= p_i - p_j (< window).  The
    denominator holds one more term, exp(sink), which has no column."""
    pos = torch.as_tensor(positions, dtype=torch.long)
    diff = pos[:, None] - pos[None, :]
    seen = diff >= 0
    if window:
        seen &= diff < window
    s = scores.masked_fill(~seen, float("-inf"))
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=float(sink))
    p = torch.exp(s - top)
    return p / (p.sum(dim=-1, keepdim=True) + torch.exp(float(sink) - top))


def latent_attention(h, w, m, positions, eps):
    """The attention mixer.  ``w``: its tensors by short name; ``m``: its sizes and constants."""
    H, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    rot = m.get("rot") or {}
    query_latent = unit_rms(linear(h, w["dq"]), eps) * w["dq.norm"].to(F64)
    q = linear(query_latent, w["uq"]).view(T, H, dim + rot_dim)
    q_plain, q_turn = q[..., :dim], q[..., dim:]
    down = linear(h, w["dkv"])
    latent = unit_rms(down[:, :rank], eps) * w["dkv.norm"].to(F64)
    k_turn = down[:, rank:].view(T, 1, rot_dim)
    if rot and rot_dim:
        q_turn = rotate_half(q_turn, positions, rot["dims"], rot["base"])
        k_turn = rotate_half(k_turn, positions, rot["dims"], rot["base"])
    k_plain = linear(latent, w["uk"]).view(T, H, dim)
    value = linear(latent, w["uv"]).view(T, H, vdim)
    window = (m.get("mask") or {}).get("size")
    gate = torch.sigmoid(linear(h, w["g"]))                 # one number per head
    out = torch.zeros(T, H, vdim, dtype=F64)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_turn[:, head] @ k_turn[:, 0].T) * float(m["scale"])
        p = sink_softmax(s, positions, window, float(w["sink"][head]))
        out[:, head] = (p @ value[:, head]) * gate[:, head:head + 1]
    return linear(out.reshape(T, H * vdim), w["o"])


def lightning(h, w, m, eps):
    """The recurrent mixer: per head S <- decay S + k v^T, o = S^T q, from a state of zeros."""
    H, dim, vdim = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(linear(h, w["q"])).view(T, H, dim)
    k = silu(linear(h, w["k"])).view(T, H, dim)
    v = silu(linear(h, w["v"])).view(T, H, vdim)
    out = torch.zeros(T, H, vdim, dtype=F64)
    for head in range(H):
        state = torch.zeros(dim, vdim, dtype=F64)
        decay = float(m["decay"][head])
        for t in range(T):
            state = decay * state + torch.outer(k[t, head], v[t, head])
            out[t, head] = state.T @ q[t, head]
    y = unit_rms(out.reshape(T, H * vdim), eps) * w["norm"].to(F64)
    return linear(y * torch.sigmoid(linear(h, w["g"])), w["o"])


def dense_feed_forward(h, w):
    return linear(xielu(linear(h, w["up"]), w["act"][0], w["act"][1]), w["down"])


def route(logits, correction, router):
    """The chosen experts [T, top] and their weights.  Scores are sigmoids; the choice goes by
    score + correction, among the experts of the ``keep`` groups whose two largest choice scores
    sum highest; the weights are the plain scores times ``scale``."""
    T, E = logits.shape
    top = router["top"]
    scores = torch.sigmoid(logits.to(F64))
    choice = scores + correction.to(F64)
    groups = router.get("groups")
    if groups and groups["count"] > 1:
        count, keep = groups["count"], groups["keep"]
        per = choice.view(T, count, E // count)
        rank = torch.topk(per, min(2, E // count), dim=-1).values.sum(dim=-1)
        kept = torch.topk(rank, keep, dim=-1).indices
        allowed = torch.zeros(T, count, dtype=torch.bool)
        allowed.scatter_(1, kept, True)
        choice = choice.masked_fill(~allowed[:, :, None].expand(T, count, E // count).reshape(T, E), float("-inf"))
    chosen = torch.topk(choice, top, dim=-1).indices
    return chosen, torch.gather(scores, 1, chosen) * float(router.get("scale", 1.0))


def routed_feed_forward(h, w, router):
    T = h.shape[0]
    chosen, weights = route(linear(h, w["router"]), w["correction"], router)
    out = torch.zeros(T, h.shape[1], dtype=F64)
    for t in range(T):
        for k in range(chosen.shape[1]):
            e = int(chosen[t, k])
            y = linear(relu_squared(linear(h[t:t + 1], w[f"e{e}.up"])), w[f"e{e}.down"])
            out[t] += weights[t, k] * y[0]
    return out


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer(x, cfg, weights, index, positions):
    entry = cfg["layers"][index]
    eps = cfg["norm"]["eps"]
    p = f"l{index}."
    h = token_shift(scalar_norm(x, weights[p + "norm1"], eps), weights[p + "shift"])
    if entry["type"] == "latent_attention":
        x = x + latent_attention(h, _sub(weights, p + "mix."), entry["mixer"], positions, eps)
    elif entry["type"] == "lightning":
        x = x + lightning(h, _sub(weights, p + "mix."), entry["mixer"], eps)
    else:
        raise ValueError(entry["type"])
    mlp = entry.get("mlp")
    if mlp:
        h = scalar_norm(x, weights[p + "norm2"], eps)
        if mlp["kind"] == "dense":
            x = x + dense_feed_forward(h, _sub(weights, p + "mlp."))
        else:
            x = x + routed_feed_forward(h, _sub(weights, p + "mlp."), mlp["router"])
    return x


def run_order(cfg):
    """(layer, pass number or None) in the order they run: the layers of the loop ``times``
    times in a row, the others once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, weights, ids, positions=None, trace=None):
    """Logits [T, vocab] of one sequence.  ``trace``: a list that receives the stream after every
    layer run."""
    T = len(ids)
    positions = list(range(T)) if positions is None else positions
    eps = cfg["norm"]["eps"]
    x = scalar_norm(weights["embed"][torch.as_tensor(ids, dtype=torch.long)], weights["embed.norm"], eps)
    start = x.clone()
    loop = cfg.get("loop")
    for index, turn in run_order(cfg):
        if turn is not None and index == loop["start"]:
            if turn > 0:
                x = x + start
            x = x + weights["loop.step"][turn].to(F64)
        x = layer(x, cfg, weights, index, positions)
        if trace is not None:
            trace.append(x.clone())
    return linear(scalar_norm(x, weights["final.norm"], eps), weights["head"]) * float(cfg.get("logit_scale", 1.0))


def greedy(cfg, weights, prompt, new_tokens):
    """Greedy generation by running the whole sequence again for every token; ties go to the
    lowest index."""
    ids, out = list(prompt), []
    for _ in range(new_tokens):
        tok = int(torch.argmax(forward(cfg, weights, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
