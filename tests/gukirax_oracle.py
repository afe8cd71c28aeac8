"""Plain float64 oracle for the Gukirax decoder, one function per mechanism.

One whole sequence at a time, dense O(T^2) attention, no cache, no paging,
no batching, no kernels; it shares no code with gllm_amd. ``weights`` maps
tensor names to torch tensors, ``cfg`` is the parsed config.json dictionary.

The design in short: token embedding followed by a weight-only layer norm;
a span of layers that is run several times with the same weights (each pass
starts by mixing the stream with the embedding output through one linear
map); every sublayer wrapped in layer norms with a sigmoid gate on its
result; attention whose values are the un-normalised, un-rotated keys, whose
per-head scores are mixed across heads before the softmax and whose softmax
carries a learned sink; dense xIELU or routed relu^2 feed-forwards; scaled,
tanh-capped logits tied to the embedding table.
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def rotate_half(x, pos, rot):
    """x [T, heads, dim]; dimension i pairs with i + dims/2 on the first
    rot.dims dimensions, the rest pass through."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def talking_attention(h, w, pre, m, eps):
    """Keys double as values (before rotation and norm); the H score
    planes are mixed by ``talk`` before the causal sink softmax."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = k
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        q, k = rotate_half(q, pos, rot), rotate_half(k, pos, rot)
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    s = torch.stack([(q[:, hh] @ k[:, hh // (H // G)].T) * m["scale"]
                     for hh in range(H)])                     # [H, T, T]
    s = torch.einsum("hg,gij->hij", w[pre + "talk"], s)
    see = pos[None, :] <= pos[:, None]
    sink = w[pre + "sink"]
    out = torch.zeros(T, H, D, dtype=F64)
    for hh in range(H):
        # subtract a common offset: the sink enters like one more score
        top = torch.maximum(
            torch.where(see, s[hh], torch.full_like(s[hh], -math.inf))
            .max(-1, keepdim=True).values, sink[hh])
        e = torch.where(see, torch.exp(s[hh] - top), torch.zeros_like(s[hh]))
        p = e / (e.sum(-1, keepdim=True) + torch.exp(sink[hh] - top))
        out[:, hh] = p @ v[:, hh // (H // G)]
    return out.reshape(T, H * D) @ w[pre + "o"].T


def xielu(z, p, q):
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.expm1(z.clamp(max=0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff(h, w, pre):
    act = w[pre + "act"]
    return xielu(h @ w[pre + "up"].T, act[0], act[1]) @ w[pre + "down"].T


def relu2_expert(h, w, pre):
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def moe_ff(h, w, pre, mlp):
    top = mlp["router"]["top"]
    s = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(top):
            out[t] += val[t, c] * relu2_expert(
                h[t:t + 1], w, "%se%d." % (pre, int(idx[t, c])))[0]
    if mlp.get("shared"):
        out = out + relu2_expert(h, w, pre + "shared.")
    return out


def gated(y, h, w, name):
    return y * torch.sigmoid(h @ w[name].T + w[name + ".b"])


def run_layer(x, w, li, layer, eps):
    p = "l%d." % li
    h = layer_norm(x, w[p + "norm1"], eps)
    if layer["type"] != "attention":
        raise ValueError(layer["type"])
    y = gated(talking_attention(h, w, p + "mix.", layer["mixer"], eps),
              h, w, p + "rg1")
    x = x + layer_norm(y, w[p + "norm1b"], eps)
    mlp = layer.get("mlp")
    if mlp:
        h = layer_norm(x, w[p + "norm2"], eps)
        if mlp["kind"] == "dense":
            y = dense_ff(h, w, p + "mlp.")
        elif mlp["kind"] == "moe":
            y = moe_ff(h, w, p + "mlp.", mlp)
        else:
            raise ValueError(mlp["kind"])
        x = x + layer_norm(gated(y, h, w, p + "rg2"), w[p + "norm2b"], eps)
    return x


def layer_schedule(cfg):
    """Layer indices in the order they run; True marks a pass start."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg, weights, tokens, with_layers=False):
    """Logits [T, vocab] (float64) of one whole sequence from position 0."""
    w = {k: v.to(F64) for k, v in weights.items() if v.is_floating_point()}
    eps = cfg["norm"]["eps"]
    x0 = layer_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    x = x0
    trail = []
    for li, starts_pass in layer_schedule(cfg):
        if starts_pass:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        x = run_layer(x, w, li, cfg["layers"][li], eps)
        trail.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["embed"].T
    logits = logits * cfg["logit_scale"]
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    if with_layers:
        return logits, torch.stack(trail)
    return logits
