"""A plain, slow implementation of the Surasun decoder, one function per mechanism, in float64 and
token by token wherever a recurrence is involved. It takes a config.json's dict and a dict of
tensors (name -> torch tensor) and shares no code with the engine: it is what the engine's
results are compared with.

Notation: h is a mixer's or feed-forward's input (tokens, width); `w` is the tensor dict; `p` a
tensor name prefix ending in "."; positions count from 0.
"""

import math

import torch

F = torch.float64


def _t(w, name):
    return w[name].to(F)


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * weight, var = mean of squared deviations; no bias."""
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * weight


def rms_unit(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x, taps, bias):
    """out[t, c] = bias[c] + sum_j taps[c, K - 1 - j] * x[t - j, c], zeros before the first token."""
    T, C = x.shape
    K = taps.shape[1]
    out = bias.expand(T, C).clone()
    for j in range(K):
        if j < T:
            out[j:] += taps[:, K - 1 - j] * x[:T - j]
    return out


def turn_neighbours(v, positions, dims, base):
    """Pairs (2i, 2i + 1) of the first `dims` numbers of the last axis turn by position * base^(-2i/dims)."""
    out = v.clone()
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq[None, :]
    shape = (v.shape[0],) + (1,) * (v.dim() - 2) + (half,)
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def turn_halves(v, positions, dims, base):
    """Pairs (i, i + dims/2) of the first `dims` numbers of the last axis turn by position * base^(-2i/dims)."""
    out = v.clone()
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq[None, :]
    shape = (v.shape[0],) + (1,) * (v.dim() - 2) + (half,)
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    a, b = v[..., :half], v[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def mamba2(h, w, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ _t(w, p + "in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, _t(w, p + "conv"), _t(w, p + "conv.b")))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + _t(w, p + "dt_bias"))
    rate = torch.exp(_t(w, p + "A_log"))
    D = _t(w, p + "D")
    y = torch.zeros(T, H, P, dtype=F)
    S = torch.zeros(H, N, P, dtype=F)
    for t in range(T):
        for k in range(H):
            g = k // (H // G)
            S[k] = math.exp(-float(rate[k]) * float(dt[t, k])) * S[k] + float(dt[t, k]) * torch.outer(B[t, g], x[t, k])
            y[t, k] = S[k].T @ C[t, g] + D[k] * x[t, k]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_unit(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * _t(w, p + "norm")
    return y @ _t(w, p + "o").T


def rglru(h, w, p, m):
    T = h.shape[0]
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(h @ _t(w, p + "y").T + _t(w, p + "y.b"))
    u = causal_conv(h @ _t(w, p + "x").T + _t(w, p + "x.b"), _t(w, p + "conv"), _t(w, p + "conv.b"))
    ub = u.reshape(T, blocks, width // blocks)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, _t(w, p + "ra")) + _t(w, p + "ra.b")).reshape(T, width)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, _t(w, p + "ri")) + _t(w, p + "ri.b")).reshape(T, width)
    a = torch.exp(-8.0 * r * softplus(_t(w, p + "lam")))
    S = torch.zeros(width, dtype=F)
    out = torch.zeros(T, width, dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] * a[t]) * i[t] * u[t]
        out[t] = S
    return (out * y) @ _t(w, p + "o").T


def softcap_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = h @ _t(w, p + "q").T + _t(w, p + "q.b")
    k = h @ _t(w, p + "k").T + _t(w, p + "k.b")
    v = (h @ _t(w, p + "v").T + _t(w, p + "v.b")).reshape(T, G, dv)
    q = (rms_unit(q, eps) * _t(w, p + "q.norm")).reshape(T, H, d)
    k = (rms_unit(k, eps) * _t(w, p + "k.norm")).reshape(T, G, d)
    if m.get("rot"):
        q = turn_neighbours(q, pos, m["rot"]["dims"], m["rot"]["base"])
        k = turn_neighbours(k, pos, m["rot"]["dims"], m["rot"]["base"])
    gate = torch.sigmoid(h @ _t(w, p + "g").T)
    cap = m.get("softcap")
    out = torch.zeros(T, H, dv, dtype=F)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g] * gate[:, a:a + 1]
    return out.reshape(T, H * dv) @ _t(w, p + "o").T


def retention(h, w, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q, k = (h @ _t(w, p + "q").T).reshape(T, H, d), (h @ _t(w, p + "k").T).reshape(T, H, d)
    if m.get("rot"):
        q = turn_halves(q, pos, m["rot"]["dims"], m["rot"]["base"])
        k = turn_halves(k, pos, m["rot"]["dims"], m["rot"]["base"])
    k = k * d ** -0.5
    v = (h @ _t(w, p + "v").T).reshape(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F)
    S = torch.zeros(H, d, dv, dtype=F)
    for t in range(T):
        for a in range(H):
            S[a] = float(m["decay"][a]) * S[a] + torch.outer(k[t, a], v[t, a])
            o[t, a] = S[a].T @ q[t, a]
    o = rms_unit(o, eps).reshape(T, H * dv) * silu(h @ _t(w, p + "g").T)
    return o @ _t(w, p + "o").T


def parallel(h, w, p, m, eps):
    return (m["left_scale"] * softcap_attention(h, w, p + "left.", m["left"], eps)
            + m["right_scale"] * retention(h, w, p + "right.", m["right"], eps))


def dense_ff(h, w, p):
    return (silu(h @ _t(w, p + "gate").T) * (h @ _t(w, p + "up").T)) @ _t(w, p + "down").T


def mixer(kind, h, w, p, m, eps):
    if kind == "mamba2":
        return mamba2(h, w, p, m, eps)
    if kind == "rglru":
        return rglru(h, w, p, m)
    if kind == "parallel":
        return parallel(h, w, p, m, eps)
    raise ValueError(kind)


def forward(config, w, tokens, streams_behind_layers=None):
    """Logits (tokens, vocab) float64 of one sequence. `streams_behind_layers`: a list that receives
    the residual stream (the sum of the streams) behind every layer."""
    eps = config["norm"]["eps"]
    mult = config.get("residual_mult", 1.0)
    n = config.get("streams")
    x = _t(w, "embed")[torch.as_tensor(tokens)]
    xs = [x.clone() for _ in range(n)] if n else None
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % i
        subs = [(1, lambda h: mixer(layer["type"], h, w, p + "mix.", layer["mixer"], eps))]
        if layer.get("mlp") is not None:
            subs.append((2, lambda h: dense_ff(h, w, p + "mlp.")))
        for number, sub in subs:
            weight = _t(w, p + "norm%d" % number)
            if xs is None:
                x = x + mult * sub(layer_norm(x, weight, eps))
                continue
            hc = p + "hc%d." % number
            read, write, mix = _t(w, hc + "in"), _t(w, hc + "out"), _t(w, hc + "mix")
            y = sub(layer_norm(sum(read[s] * xs[s] for s in range(n)), weight, eps))
            xs = [sum(mix[s, t] * xs[s] for s in range(n)) + mult * write[t] * y for t in range(n)]
        if streams_behind_layers is not None:
            streams_behind_layers.append(x.clone() if xs is None else sum(xs))
    if xs is not None:
        x = sum(xs)
    return layer_norm(x, _t(w, "final.norm"), eps) @ _t(w, "embed").T


def greedy(config, w, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(config, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
