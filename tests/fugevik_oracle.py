"""Plain float64 statement of the Fugevik design, whole sequences only, one
function per mechanism.  Shares no code with the package: it reads the
config.json dictionary and checkpoint-named tensors directly.

Notation: T tokens, S streams, W width; x [T, S, W] the streams; positions
count from 0.
"""
import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------- pieces
def unit_rms(v, eps):
    return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)


def centred_norm(v, weight, eps):
    """RMS norm whose stored weight is the offset from one."""
    return unit_rms(v, eps) * (1.0 + weight)


def stream_read(x, read_w):
    return (x * read_w[None, :, None]).sum(1)


def stream_write(x, y, mix, write_w):
    """All streams at once from the old ones; mix is indexed [from, to]."""
    new = torch.zeros_like(x)
    S = x.shape[1]
    for to in range(S):
        for frm in range(S):
            new[:, to] += mix[frm, to] * x[:, frm]
        new[:, to] += write_w[to] * y
    return new


def input_conv(h, w):
    """h + causal depthwise convolution of h; w [W, taps], the last tap
    weighs the current token, zeros before the sequence."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def rotate_interleaved(v, positions, dims, base):
    """Pairs (2i, 2i+1) of the leading `dims` elements turn by position *
    base^(-2i/dims); v [T, ..., d]."""
    out = v.clone()
    for i in range(dims // 2):
        ang = positions.to(F64) * base ** (-2.0 * i / dims)
        shape = [-1] + [1] * (v.dim() - 2)
        c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def visible(T, size):
    """[i, j] true where 0 <= i - j (< size when size > 0)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None]
    ok = (i - j) >= 0
    if size > 0:
        ok &= (i - j) < size
    return ok


def latent_attention(h, m, w, pre, eps):
    T = h.shape[0]
    H, dim, rd, vd, R = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                         m["kv_rank"])
    pos = torch.arange(T)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = (h @ w[pre + "q"].T).view(T, H, dim + rd)
    down = h @ w[pre + "dkv"].T
    c = unit_rms(down[:, :R], eps) * w[pre + "dkv.norm"]
    k_rot = rotate_interleaved(down[:, R:], pos, rot["dims"], rot["base"])
    q_rot = rotate_interleaved(q[..., dim:], pos, rot["dims"], rot["base"])
    k_up = (c @ w[pre + "uk"].T).view(T, H, dim)
    v = (c @ w[pre + "uv"].T).view(T, H, vd)
    ok = visible(T, (m.get("mask") or {}).get("size", 0))
    heads = []
    for hd in range(H):
        s = (q[:, hd, :dim] @ k_up[:, hd].T + q_rot[:, hd] @ k_rot.T) \
            * m["scale"]
        s = s.masked_fill(~ok, -math.inf)
        sink = w[pre + "sink"][hd]
        top = torch.maximum(s.max(-1, keepdim=True)[0], sink)
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True) + torch.exp(sink - top)
        heads.append((e / den) @ v[:, hd])
    o = torch.cat(heads, -1) * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def biased_attention(h, m, w, pre, shared_kv=None):
    """Returns (output, (k, v)); shared_kv = another layer's (k, v)."""
    T = h.shape[0]
    H, G = m["heads"], m.get("kv_heads", m["heads"])
    dim, vd = m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, dim)
    if shared_kv is None:
        k = (h @ w[pre + "k"].T).view(T, G, dim)
        v = (h @ w[pre + "v"].T).view(T, G, vd)
    else:
        k, v = shared_kv
    ok = visible(T, (m.get("mask") or {}).get("size", 0))
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None]).clamp(min=0)
    cap = m.get("softcap") or 0.0
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        s = q[:, hd] @ k[:, g].T * m["scale"]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s - w[pre + "r1"][hd] * torch.log(
            1.0 + w[pre + "r2"][hd] * dist.to(F64))
        s = s.masked_fill(~ok, -math.inf)
        heads.append(torch.softmax(s, -1) @ v[:, g])
    return torch.cat(heads, -1) @ w[pre + "o"].T, (k, v)


def squared_relu_ff(h, w, pre):
    return torch.relu(h @ w[pre + "up"].T).pow(2) @ w[pre + "down"].T


# ------------------------------------------------------------ whole model
def forward(tokens, cfg, w, keep_layers=False):
    """tokens -> logits [T, V] (and the sum of the streams after each
    layer)."""
    w = {k: v.to(F64) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams", 1)
    x = w["embed"][torch.tensor(tokens)][:, None, :].repeat(1, S, 1)
    kv, layers = {}, []
    for i, lc in enumerate(cfg["layers"]):
        pre = f"l{i}."
        for q in (1, 2):
            if q == 2 and lc.get("mlp") is None:
                continue
            port = pre + f"hc{q}."
            u = stream_read(x, w[port + "in"])
            h = input_conv(centred_norm(u, w[pre + f"norm{q}"], eps),
                           w[pre + f"canon{q}"])
            if q == 2:
                y = squared_relu_ff(h, w, pre + "mlp.")
            elif lc["type"] == "latent_attention":
                y = latent_attention(h, lc["mixer"], w, pre + "mix.", eps)
            else:
                src = lc["mixer"].get("kv_from")
                y, kv[i] = biased_attention(
                    h, lc["mixer"], w, pre + "mix.",
                    kv[src] if src is not None else None)
            x = stream_write(x, y, w[port + "mix"], w[port + "out"])
        layers.append(x.sum(1))
    logits = centred_norm(x.sum(1), w["final.norm"], eps) @ w["embed"].T
    return (logits, layers) if keep_layers else logits


# --------------------------------------------------------- random weights
def random_weights(cfg, seed, dtype=torch.bfloat16, gain=1.0):
    """Checkpoint-named random tensors for a config dictionary, rounded to
    `dtype` (the oracle and the framework then start from equal numbers)."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 1)
    taps = (cfg.get("canon") or {}).get("taps", 1)
    out = {}

    def rnd(name, *shape, std=1.0, mean=0.0):
        out[name] = (mean + std * torch.randn(*shape, generator=g)).to(dtype)

    def lin(name, o, i):
        rnd(name, o, i, std=gain * i ** -0.5)
    rnd("embed", cfg["vocab"], W)
    rnd("final.norm", W, std=0.2)
    for i, lc in enumerate(cfg["layers"]):
        pre, mp = f"l{i}.", f"l{i}.mix."
        m = lc["mixer"]
        for q in (1, 2):
            if q == 2 and lc.get("mlp") is None:
                continue
            rnd(pre + f"norm{q}", W, std=0.2)
            rnd(pre + f"canon{q}", W, taps, std=0.3)
            rnd(pre + f"hc{q}.in", S, std=0.2, mean=1.0 / S)
            rnd(pre + f"hc{q}.out", S, std=0.3, mean=0.7)
            out[pre + f"hc{q}.mix"] = (
                torch.eye(S) + 0.2 * torch.randn(S, S, generator=g)).to(dtype)
        H = m["heads"]
        if lc["type"] == "latent_attention":
            R, rd = m["kv_rank"], m["rot_dim"]
            lin(mp + "q", H * (m["dim"] + rd), W)
            lin(mp + "dkv", R + rd, W)
            rnd(mp + "dkv.norm", R, std=0.2, mean=1.0)
            lin(mp + "uk", H * m["dim"], R)
            lin(mp + "uv", H * m["vdim"], R)
            rnd(mp + "sink", H, std=1.5)
            lin(mp + "g", H * m["vdim"], W)
            lin(mp + "o", W, H * m["vdim"])
        else:
            G = m.get("kv_heads", H)
            lin(mp + "q", H * m["dim"], W)
            if m.get("kv_from") is None:
                lin(mp + "k", G * m["dim"], W)
                lin(mp + "v", G * m["vdim"], W)
            out[mp + "r1"] = (0.2 + 0.8 * torch.rand(H, generator=g)).to(dtype)
            out[mp + "r2"] = (0.1 + 1.9 * torch.rand(H, generator=g)).to(dtype)
            lin(mp + "o", W, H * m["vdim"])
        if lc.get("mlp") is not None:
            lin(pre + "mlp.up", lc["mlp"]["ff"], W)
            lin(pre + "mlp.down", W, lc["mlp"]["ff"])
    return out
