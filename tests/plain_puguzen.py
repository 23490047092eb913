"""A plain, slow statement of the Puguzen decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations and sharing no code with the product package: model folders are read with the
`safetensors` package, every tensor stays on the CPU, and every call recomputes the whole sequence in float64.

The design, in this file's notation.  x is the residual stream [T, W].
  embedding   x_t = E[id_t]
  norm_c      y = x / sqrt(mean(x^2) + eps) * (1 + g): the gain is stored around zero
  layer       n = norm_c(x);  x <- x + sigmoid(R1 n + r1) * mixer(n) + sigmoid(R2 n + r2) * ff(n)   (ff may be absent):
              one norm, both sublayers read it, each result passes a gate of its own that reads n too
  gla         q = Wq n / sqrt(dim), k = Wk n, v = Wv n;  a = sigmoid(Wa2 (Wa1 n) + b)^(1/tau), one decay per key channel;
              per head S_t = diag(a_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  o_t / rms(o_t) * w (w shared by the heads);
              out = Wo (concat_h o * silu(Wg n))
  retention   q = Wq n, k = Wk n, both turned by position on their first `dims` coordinates (coordinate i pairs with
              i + dims/2), then k / sqrt(dim);  per head S_t = d_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  o_t / rms(o_t);
              out = Wo (concat_h o * silu(Wg n))
  attention   q = Wq n, k = Wk n, v = Wv n; q and k turned by position on their first `dims` coordinates (coordinate 2i
              pairs with 2i + 1), then each head's q and k divided by its root mean square;  s_ij = scale * q_i . k_j;
              token i sees the tokens j with 0 <= i - j < size, and for every block of `pool` tokens that lies wholly
              before them (its last token <= i - size) one key and one value, the means of the block's keys and values;
              weight = sigmoid(s + b_h), not normalised;  out = Wo (concat_h sum_j weight_ij v_j * sigmoid(Wg n))
  ff          Wdown (relu(Wgate n) * (Wup n))
  output      logits = E norm_c(x)
"""
import json
import math
import os

import torch

F64 = torch.float64


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


def centered_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * (1.0 + g)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def angles(rot, positions):
    """[T, dims / 2]: position times frequency, both 32-bit numbers, multiplied in 32-bit as the design computes."""
    dims = rot["dims"]
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64).to(torch.float32)
    p = torch.tensor(list(positions), dtype=torch.float32)
    return (p[:, None] * f[None, :]).to(F64)


def turn_halves(u, rot, first_position=0):
    """u [T, heads, dim]: coordinate i < dims/2 pairs with i + dims/2."""
    half = rot["dims"] // 2
    a = angles(rot, range(first_position, first_position + u.shape[0]))
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = u.clone()
    lo, hi = u[..., :half], u[..., half:2 * half]
    out[..., :half] = lo * c - hi * s
    out[..., half:2 * half] = hi * c + lo * s
    return out


def turn_neighbours(u, rot, first_position=0):
    """u [T, heads, dim]: coordinate 2i pairs with 2i + 1, for i < dims/2."""
    dims = rot["dims"]
    a = angles(rot, range(first_position, first_position + u.shape[0]))
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = u.clone()
    even, odd = u[..., 0:dims:2], u[..., 1:dims:2]
    out[..., 0:dims:2] = even * c - odd * s
    out[..., 1:dims:2] = odd * c + even * s
    return out


def decayed_outer_recurrence(q, k, v, decay):
    """q, k [T, heads, dim], v [T, heads, vdim], decay [T, heads, dim] (what multiplies the rows of S before token t is
    written).  S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token."""
    T, H, D = q.shape
    S = torch.zeros((H, D, v.shape[2]), dtype=q.dtype)
    out = []
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def gla(n, w, p, m, eps):
    T = n.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (n @ w[p + "q"].T).view(T, H, D) / math.sqrt(D)
    k = (n @ w[p + "k"].T).view(T, H, D)
    v = (n @ w[p + "v"].T).view(T, H, V)
    z = (n @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / float(m["tau"])).view(T, H, D)
    o = decayed_outer_recurrence(q, k, v, decay)
    o = unit_rms(o, eps) * w[p + "norm"]
    g = n @ w[p + "g"].T
    return (o.reshape(T, H * V) * (g * torch.sigmoid(g))) @ w[p + "o"].T


def retention(n, w, p, m, eps):
    T = n.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (n @ w[p + "q"].T).view(T, H, D)
    k = (n @ w[p + "k"].T).view(T, H, D)
    v = (n @ w[p + "v"].T).view(T, H, V)
    if m.get("rot"):
        q, k = turn_halves(q, m["rot"]), turn_halves(k, m["rot"])
    k = k / math.sqrt(D)
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=n.dtype)[None, :, None].expand(T, H, D)
    o = unit_rms(decayed_outer_recurrence(q, k, v, decay), eps)
    g = n @ w[p + "g"].T
    return (o.reshape(T, H * V) * (g * torch.sigmoid(g))) @ w[p + "o"].T


def visible(i, T_keys, size, pool):
    """What token i sees: (the blocks b whose pooled key it sees, the tokens j it sees)."""
    blocks = [b for b in range(0, T_keys // pool + 1) if b * pool + pool - 1 <= i - size]
    tokens = [j for j in range(max(0, i - size + 1), i + 1)]
    return blocks, tokens


def sigmoid_attention(q, k, v, bias, scale, size, pool):
    """q [T, H, D], k [T, G, D], v [T, G, V] as the cache holds them, bias [H]: every token over its window and the means
    of the blocks before it, weights sigmoid(scale q . k + bias), not normalised.  Returns [T, H, V]."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    nblocks = T // pool
    kp = torch.stack([k[b * pool:(b + 1) * pool].mean(dim=0) for b in range(nblocks)]) if nblocks else k[:0]
    vp = torch.stack([v[b * pool:(b + 1) * pool].mean(dim=0) for b in range(nblocks)]) if nblocks else v[:0]
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    per = H // G
    for i in range(T):
        blocks, tokens = visible(i, T, size, pool)
        blocks = [b for b in blocks if b < nblocks]
        keys = torch.cat([kp[blocks], k[tokens]]) if blocks else k[tokens]
        vals = torch.cat([vp[blocks], v[tokens]]) if blocks else v[tokens]
        group = [h // per for h in range(H)]             # query head h reads kv head h // (H / G)
        s = torch.einsum("nhd,hd->nh", keys[:, group], q[i]) * float(scale) + bias
        out[i] = torch.einsum("nh,nhv->hv", torch.sigmoid(s), vals[:, group])
    return out


def attention_inputs(n, w, p, m, eps, first_position=0):
    """(q [T, H, D], k [T, G, D], v [T, G, V]) behind projection, rotation and the unit norm."""
    T = n.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (n @ w[p + "q"].T).view(T, H, D)
    k = (n @ w[p + "k"].T).view(T, G, D)
    v = (n @ w[p + "v"].T).view(T, G, V)
    if m.get("rot"):
        q, k = turn_neighbours(q, m["rot"], first_position), turn_neighbours(k, m["rot"], first_position)
    return unit_rms(q, eps), unit_rms(k, eps), v


def pooled_window_attention(n, w, p, m, eps, round_cache=None):
    """round_cache: a function applied to keys and values before they are pooled and attended to (what a cache of
    fewer bits does to them); None: nothing."""
    T = n.shape[0]
    q, k, v = attention_inputs(n, w, p, m, eps)
    if round_cache is not None:
        k, v = round_cache(k), round_cache(v)
    out = sigmoid_attention(q, k, v, w[p + "pb"], m["scale"], m["mask"]["size"], m["mask"]["pool"])
    gate = torch.sigmoid(n @ w[p + "g"].T)
    return (out.reshape(T, -1) * gate) @ w[p + "o"].T


def relu_glu(n, w, p):
    return (torch.relu(n @ w[p + "gate"].T) * (n @ w[p + "up"].T)) @ w[p + "down"].T


MIXERS = {"gla": gla, "retention": retention, "attention": pooled_window_attention}


def layer(x, w, i, spec, eps, **kw):
    p = "l%d." % i
    n = centered_norm(x, w[p + "norm1"], eps)
    mixed = MIXERS[spec["type"]](n, w, p + "mix.", spec["mixer"], eps, **(kw if spec["type"] == "attention" else {}))
    x = x + torch.sigmoid(n @ w[p + "rg1"].T + w[p + "rg1.b"]) * mixed
    if spec.get("mlp") is not None:
        x = x + torch.sigmoid(n @ w[p + "rg2"].T + w[p + "rg2.b"]) * relu_glu(n, w, p + "mlp.")
    return x


def forward(cfg, w, ids, streams=None, **kw):
    """Logits [T, vocab] of the whole sequence.  streams: a list that receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(list(ids), dtype=torch.long)]
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, w, i, spec, eps, **kw)
        if streams is not None:
            streams.append(x.clone())
    return centered_norm(x, w["final.norm"], eps) @ w["embed"].T


def logits(ids, w, cfg):
    return forward(cfg, w, ids)


def residual_streams(ids, w, cfg):
    streams = []
    forward(cfg, w, ids, streams)
    return torch.stack(streams)
