"""Plain float64 oracle for the Sudevik decoder, one function per mechanism.

Everything here works on one whole sequence at a time with dense
O(T^2) attention and a token-by-token recurrence: no cache, no paging,
no batching, no kernels. It shares no code with gllm_amd.
``weights`` maps tensor names to torch tensors; ``cfg`` is the parsed
config.json dictionary.
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def rotary_table(rot):
    """Per-pair frequencies and the cos/sin magnitude."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = sc["factor"], sc["original"]

    def corr(t):
        return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(corr(sc["fast"])), 0)
    hi = min(math.ceil(corr(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    f = f / factor * ramp + f * (1 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot):
    """x [T, heads, dim]; pairs (2i, 2i+1) of the first rot.dims rotate."""
    f, mag = rotary_table(rot)
    dims = rot["dims"]
    a = pos.to(F64)[:, None] * f[None, :]
    c, s = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def attention_keys(h, w, pre, m, eps):
    """Keys (normed, rotated) and values of an attention layer that owns
    them: [T, G, dim], [T, G, vdim]."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = (h @ w[pre + "v"].T).view(T, G, Dv)
    k = rms_unit(k, eps) * w[pre + "k.norm"]
    pos = torch.arange(T)
    if m.get("rot"):
        k = rotate(k, pos, m["rot"])
    return k, v


def attention_mixer(h, w, pre, m, eps, kv):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    k, v = kv
    q = (h @ w[pre + "q"].T).view(T, H, D)
    q = rms_unit(q, eps) * w[pre + "q.norm"]
    pos = torch.arange(T)
    if m.get("rot"):
        q = rotate(q, pos, m["rot"])
    i = pos[:, None]
    j = pos[None, :]
    see = j <= i
    mask = m.get("mask")
    if mask:
        see = see & ((i - j < mask["size"]) | (j < mask.get("keep_first", 0)))
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        e = torch.where(see, torch.exp(s), torch.zeros_like(s))
        p = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, hh] = p @ v[:, g]
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    return (out.reshape(T, H * Dv) * gate) @ w[pre + "o"].T


def short_conv(x, cw):
    """x [T, C], cw [C, taps]; the last tap is the current token's."""
    T, C = x.shape
    taps = cw.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x])
    y = torch.zeros_like(x)
    for t in range(taps):
        y = y + xp[t:t + T] * cw[:, t]
    return y


def delta_mixer(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    decay = torch.exp(-torch.exp(w[pre + "A_log"]) * torch.nn.functional.softplus(
        h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hh] = S.T @ q[t, g]
    o = rms_unit(o, eps) * w[pre + "norm"]
    o = o.reshape(T, H * Dv) * silu(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def moe(h, w, pre, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[pre + "router"].T + w[pre + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    p = torch.softmax(val, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(idx[t, c])
            ep = "%se%d." % (pre, e)
            x = h[t]
            y = w[ep + "down"] @ (silu(w[ep + "gate"] @ x) * (w[ep + "up"] @ x))
            out[t] += p[t, c] * y
    return out


def forward(cfg, weights, tokens, with_layers=False):
    """Logits [T, vocab] (float64) of one whole sequence from position 0."""
    w = {k: v.to(F64) for k, v in weights.items() if v.is_floating_point()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens)]
    kvs = {}
    trail = []

    def ln(name, t):
        return layer_norm(t, w[name], w[name + ".b"], eps)

    for li, layer in enumerate(cfg["layers"]):
        p = "l%d." % li
        m = layer["mixer"]
        h = ln(p + "norm1", x)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[li] = attention_keys(h, w, p + "mix.", m, eps)
                src = li
            y = attention_mixer(h, w, p + "mix.", m, eps, kvs[src])
        elif layer["type"] == "delta":
            y = delta_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + ln(p + "norm1b", y)
        if layer.get("mlp"):
            h = ln(p + "norm2", x)
            x = x + ln(p + "norm2b", moe(h, w, p + "mlp.", layer["mlp"]))
        trail.append(x)
    logits = ln("final.norm", x) @ w["head"].T
    if with_layers:
        return logits, torch.stack(trail)
    return logits
