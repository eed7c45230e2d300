"""The Kodisun decoder on one whole sequence with elementary tensor operations, one function per
mechanism, in the dtype of the weights it is given (float64 for a truth, float32 to see what
rounding does). It shares no code with the package: the tests compare the engine with this.

`config` is config.json as a dict, `w` maps tensor names to tensors.
"""

import math

import torch


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def rotation_frequencies(rot):
    """(frequency per pair, factor on cos and sin) of a `rot` entry: base^(-2i/dims), and with a
    `scaling` entry the long-context blend: pairs that turn fewer than `slow` times within
    `original` positions are slowed by `factor`, pairs that turn more than `fast` times stay,
    those between are blended linearly in the pair's index."""
    dims, base = int(rot["dims"]), float(rot["base"])
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    scaling = rot.get("scaling")
    if not scaling:
        return freqs, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, rot):
    """x (T, heads, n): the first rot.dims numbers of every head turn, (2i, 2i + 1) together, by
    position * frequency_i; the rest pass."""
    dims = int(rot["dims"])
    freqs, factor = rotation_frequencies(rot)
    f = torch.tensor(freqs, dtype=torch.float32)
    angle = positions.to(torch.float32)[:, None] * f[None, :]          # 32-bit angles, as the engine forms them
    cos = (angle.to(torch.float64).cos() * factor).to(x.dtype)[:, None, :]
    sin = (angle.to(torch.float64).sin() * factor).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack((u * cos - v * sin, v * cos + u * sin), dim=-1).flatten(-2)
    return torch.cat((turned, x[..., dims:]), dim=-1)


def latent_attention(h, w, p, m, eps):
    """h (T, width) -> (T, width). Queries and keys/values each pass a narrow vector that is
    normalised; per head a key is [part made from the latent | one rotated part shared by all
    heads], a value is made from the latent; a query sees itself and mask.size - 1 before."""
    T = h.shape[0]
    H, dn, dr, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T)
    cq = rms_norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps)
    q = (cq @ w[p + ".uq"].T).view(T, H, dn + dr)
    down = h @ w[p + ".dkv"].T
    c = rms_norm(down[:, :rank], w[p + ".dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, None, rank:], pos, m["rot"])           # (T, 1, dr)
    q_rot = rotate_pairs(q[..., dn:], pos, m["rot"])
    k_flat = (c @ w[p + ".uk"].T).view(T, H, dn)
    v = (c @ w[p + ".uv"].T).view(T, H, dv)
    scores = torch.einsum("thd,shd->hts", q[..., :dn], k_flat) + torch.einsum("thd,sd->hts", q_rot, k_rot[:, 0])
    scores = scores * float(m["scale"])
    back = pos[:, None] - pos[None, :]
    hidden = back < 0
    if m.get("mask") and m["mask"].get("size"):
        hidden = hidden | (back >= int(m["mask"]["size"]))
    scores = scores.masked_fill(hidden[None], float("-inf"))
    o = torch.einsum("hts,shd->thd", torch.softmax(scores, dim=-1), v)
    return o.reshape(T, H * dv) @ w[p + ".o"].T


def expert(h, w, p):
    return gelu_erf(h @ w[p + ".up"].T) @ w[p + ".down"].T


def routed_feed_forward(h, w, p, f):
    """Each token's `top` experts by softmax score over all experts, weighted by their scores
    divided by the scores' sum, plus an expert that every token passes."""
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    s = torch.softmax(h @ w[p + ".router"].T, dim=-1)
    best, chosen = torch.topk(s, top, dim=-1)
    share = best / (best.sum(dim=-1, keepdim=True) + 1e-20)
    out = torch.zeros_like(h)
    for e in range(E):
        for k in range(top):
            rows = (chosen[:, k] == e).nonzero()[:, 0]
            if rows.numel():
                out[rows] += share[rows, k, None] * expert(h[rows], w, "%s.e%d" % (p, e))
    if f.get("shared"):
        out = out + expert(h, w, p + ".shared")
    return out


def run_order(config):
    """[(layer, number of the pass that starts here or None)]"""
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if b <= a:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def logits_of_sequence(config, w, tokens, layers_out=None):
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    for i, enters in run_order(config):
        layer, p = config["layers"][i], "l%d" % i
        if enters is not None:
            x = x + w["loop.step"][enters]
        assert layer["type"] == "latent_attention"
        mixed = latent_attention(rms_norm(x, w[p + ".norm1"], eps), w, p + ".mix", layer["mixer"], eps)
        x = x + rms_norm(mixed, w[p + ".norm1b"], eps)
        if layer.get("mlp"):
            assert layer["mlp"]["kind"] == "moe"
            fed = routed_feed_forward(rms_norm(x, w[p + ".norm2"], eps), w, p + ".mlp", layer["mlp"])
            x = x + rms_norm(fed, w[p + ".norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
