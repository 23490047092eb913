"""A plain, slow statement of the Nidasun decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations and sharing no code with the product package: model folders are read with the
`safetensors` package, every tensor stays on the CPU, and every call recomputes the whole sequence in float64.

The design, in this file's notation.  X is the list of residual streams, each [T, W]; rms(z) = z / sqrt(mean(z^2) + eps).
  embedding    x_t = E[id_t]; every stream starts as x
  sublayer q   u = sum_s in_q[s] X_s;  y = f(rms(u) * g_q);  X_t <- sum_s mix_q[s, t] X_s + out_q[t] * y   (all t at once)
               (q = 1: the mixer, q = 2: the feed-forward, absent in a layer without one); without streams: x <- x + y
  loop         layers [start, stop) run `times` times with the same weights, every pass from a state of its own
  attention    q = Wq h + bq, k = Wk h + bk, v = Wv h + bv; q and k turned by position on their first `dims` coordinates
               (coordinate i pairs with i + dims/2, angle p * f_i, f_i = base^(-2i/dims) / factor); token i sees the
               tokens j <= i of its own chunk (i // size == j // size); p_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij)),
               s_ij = scale * q_i . k_j; out = Wo concat_h sum_j p_ij v_j + bo
  lightning    q = silu(Wq h), k = silu(Wk h), v = silu(Wv h); per head S_t = d_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t;
               out = Wo (rms(concat_h o) * w * sigmoid(Wg h))
  parallel     left_scale * left(h) + right_scale * right(h)
    left       q = rms(Wq h) * wq, k = rms(Wk h) * wk over the whole projection, then turned by position; token i sees
               the tokens j with 0 <= i - j < size; plain softmax; out = Wo concat_h sum_j p_ij v_j
    right      y = gelu_tanh(Wy h + by); u = conv(Wx h + bx) + bc (causal over time, per channel); per block b of the
               channels r = sigmoid(Ra[b] u_b + ra[b]), i = sigmoid(Ri[b] u_b + ri[b]); a = exp(-8 r softplus(lam));
               S_t = a S_(t-1) + sqrt(1 - a^2) i u; out = Wo (S * y)
  ff dense     Wdown relu(Wup h)^2
  ff routed    s = sigmoid(Wr h); c = s + correction; groups of neighbouring experts are scored by their two largest c,
               the best `keep` groups stay; among them the `top` largest c are chosen; weights = s / (sum of the chosen s
               + 1e-20) * scale; y = sum_e weight_e * expert_e(h); expert(h) = Wdown (silu(Wgate h) * (Wup h))
  output       logits = Whead (rms(sum_s X_s) * g)
"""
import json
import math
import os

import torch

F64 = torch.float64
DECAY_RATE = 8.0
WEIGHT_FLOOR = 1e-20


def read_config(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder, dtype=F64):
    from safetensors import safe_open
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return tensors


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def turn(x, positions, base, dims, factor=1.0):
    """x [T, heads, dim]: the first `dims` coordinates of every head turned by the token's position."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def visible(pos, kind, size):
    """[T, T] booleans: whether the token at position pos[i] sees the one at pos[j]."""
    i, j = pos[:, None], pos[None, :]
    seen = j <= i
    if kind == "chunk":
        seen = seen & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))
    elif kind == "window":
        seen = seen & (i - j < size)
    return seen


def softmax_attention(q, k, v, scale, kind, size, sink=None, positions=None):
    """q [T, H, D], k [T, G, D], v [T, G, V] -> [T, H * V].  sink [H] or None: a score without a value."""
    T, H, _ = q.shape
    G = k.shape[1]
    pos = torch.arange(T) if positions is None else torch.as_tensor(positions, dtype=torch.long)
    seen = visible(pos, kind, size)
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = ((q[:, h] @ k[:, g].T) * scale).masked_fill(~seen, float("-inf"))
        m = s.max(dim=1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h])
        e = torch.exp(s - m)
        den = e.sum(dim=1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out.reshape(T, -1)


def rotation_of(m):
    rot = m.get("rot")
    if rot is None:
        return None
    return dict(base=float(rot["base"]), dims=int(rot["dims"]), factor=float((rot.get("scaling") or {}).get("factor", 1.0)))


def attention_mixer(h, w, p, m):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    pos = torch.arange(T)
    r = rotation_of(m)
    if r is not None:
        q, k = turn(q, pos, **r), turn(k, pos, **r)
    mask = m.get("mask")
    o = softmax_attention(q, k, v, m["scale"], "chunk" if mask else "all", mask["size"] if mask else 0, sink=w[p + "sink"])
    return o @ w[p + "o"].T + w[p + "o.b"]


def decayed_outer_products(q, k, v, decay):
    """q, k [T, H, D], v [T, H, V], decay [H] -> o [T, H, V]: S_t = d S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, D = q.shape
    S = torch.zeros((H, D, v.shape[2]), dtype=q.dtype)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def lightning_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, V)
    o = decayed_outer_products(q, k, v, torch.tensor(m["decay"], dtype=h.dtype)).reshape(T, H * V)
    o = rms(o, eps) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def window_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (rms(h @ w[p + "q"].T, eps) * w[p + "q.norm"]).reshape(T, H, D)
    k = (rms(h @ w[p + "k"].T, eps) * w[p + "k.norm"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, V)
    pos = torch.arange(T)
    r = rotation_of(m)
    if r is not None:
        q, k = turn(q, pos, **r), turn(k, pos, **r)
    mask = m.get("mask")
    o = softmax_attention(q, k, v, m["scale"], "window" if mask else "all", mask["size"] if mask else 0)
    return o @ w[p + "o"].T


def causal_convolution(x, taps_w, bias):
    """x [T, C], taps_w [C, taps] (the last column is the current token's), bias [C]."""
    T, taps = x.shape[0], taps_w.shape[1]
    out = torch.zeros_like(x) + bias
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += taps_w[:, j] * x[:T - back]
    return out


def gated_linear_recurrence(u, w, p, blocks):
    """u [T, C] -> S [T, C]: the real-gated linear recurrent unit over time."""
    T, C = u.shape
    ub = u.reshape(T, blocks, C // blocks)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + "ra"], ub) + w[p + "ra.b"]).reshape(T, C)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + "ri"], ub) + w[p + "ri.b"]).reshape(T, C)
    log_a = -DECAY_RATE * r * torch.nn.functional.softplus(w[p + "lam"])
    a = torch.exp(log_a)
    b = torch.sqrt(1.0 - a * a) * i * u
    S = torch.zeros(C, dtype=u.dtype)
    out = []
    for t in range(T):
        S = a[t] * S + b[t]
        out.append(S)
    return torch.stack(out)


def recurrent_mixer(h, w, p, m):
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_convolution(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    return (gated_linear_recurrence(u, w, p, m["blocks"]) * y) @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    return (m["left_scale"] * window_mixer(h, w, p + "left.", m["left"], eps)
            + m["right_scale"] * recurrent_mixer(h, w, p + "right.", m["right"]))


def dense_feed_forward(h, w, p):
    return torch.relu(h @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def route(h, w, p, router):
    """-> (ids [T, top], weights [T, top])."""
    E, top = router["experts"], router["top"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    c = s + w[p + "correction"]
    groups = router.get("groups")
    ids, weights = [], []
    for t in range(h.shape[0]):
        allowed = list(range(E))
        if groups is not None:
            n = E // groups["count"]
            score = []
            for g in range(groups["count"]):
                best = sorted((float(c[t, e]) for e in range(g * n, (g + 1) * n)), reverse=True)
                score.append(sum(best[:2]))
            kept = sorted(range(groups["count"]), key=lambda g: (-score[g], g))[:groups["keep"]]
            allowed = [e for e in range(E) if e // n in kept]
        chosen = sorted(allowed, key=lambda e: (-float(c[t, e]), e))[:top]
        total = sum(s[t, e] for e in chosen) + WEIGHT_FLOOR
        ids.append(chosen)
        weights.append([s[t, e] / total * router["scale"] for e in chosen])
    return ids, weights


def routed_feed_forward(h, w, p, mlp):
    ids, weights = route(h, w, p, mlp["router"])
    out = torch.zeros((h.shape[0], w[p + "e0.down"].shape[0]), dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], weights[t]):
            q = p + "e%d." % e
            out[t] += wt * ((silu(w[q + "gate"] @ h[t]) * (w[q + "up"] @ h[t])) @ w[q + "down"].T)
    return out


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    return (list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"]
            + list(range(loop["stop"], n)))


def sublayer(X, f, w, prefix, q, eps, streams):
    """One sublayer around the streams (or around the one stream, without hyper-connections)."""
    g = w[prefix + "norm%d" % q]
    if streams is None:
        return [X[0] + f(rms(X[0], eps) * g)]
    hc = prefix + "hc%d." % q
    u = sum(w[hc + "in"][s] * X[s] for s in range(streams))
    y = f(rms(u, eps) * g)
    return [sum(w[hc + "mix"][s, t] * X[s] for s in range(streams)) + w[hc + "out"][t] * y for t in range(streams)]


def forward(cfg, w, ids, streams_after_runs=None):
    """Logits [T, vocab] of one whole sequence.  streams_after_runs: a list that receives the sum of the streams after
    every run of a layer."""
    eps = cfg["norm"]["eps"]
    streams = cfg.get("streams")
    x = w["embed"][torch.tensor(ids, dtype=torch.long)]
    X = [x.clone() for _ in range(streams or 1)]
    for i in run_order(cfg):
        layer = cfg["layers"][i]
        p, m = "l%d." % i, layer["mixer"]
        if layer["type"] == "attention":
            mixer = lambda h: attention_mixer(h, w, p + "mix.", m)
        elif layer["type"] == "lightning":
            mixer = lambda h: lightning_mixer(h, w, p + "mix.", m, eps)
        elif layer["type"] == "parallel":
            mixer = lambda h: parallel_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError("unknown mixer %r" % layer["type"])
        X = sublayer(X, mixer, w, p, 1, eps, streams)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                ff = lambda h: dense_feed_forward(h, w, p + "mlp.")
            else:
                ff = lambda h: routed_feed_forward(h, w, p + "mlp.", mlp)
            X = sublayer(X, ff, w, p, 2, eps, streams)
        if streams_after_runs is not None:
            streams_after_runs.append(sum(X))
    return (rms(sum(X), eps) * w["final.norm"]) @ w["head"].T
