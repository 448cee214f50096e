"""Plain float64 statement of the Vabedra decoder, one function per mechanism.

Whole sequences only, no cache, no batching, no kernels: every function takes
the full [T, ...] input of one sequence and loops where the definition loops.
It shares no code with the package and is the yardstick of test_vabedra.py.

Tensors are looked up by checkpoint name in a dict `P` (values are cast to
float64 on use); `cfg` is the parsed config.json.
"""
import math

import torch

F64 = torch.float64


def _f(t):
    return t.to(F64)


def lin(h, P, name, bias=False):
    y = h @ _f(P[name]).t()
    return y + _f(P[name + ".b"]) if bias else y


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * _f(w)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30.0, z,
                       torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------- gated delta rule
def short_conv(x, w):
    """out[t, c] = sum_j w[c, j] x[t - (taps-1-j), c]: the last column weighs
    the current token, inputs before the start are zero, no bias."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] += _f(w)[:, j] * x[s]
    return out


def unit(x):
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, g):
    """Per head, from a zero state S [dim, vdim]:
        S <- g_t * S           (g_t a number, or one value per row of S)
        u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
    q, k [T, H, dim], v [T, H, vdim], beta [T, H], g [T, H] or [T, H, dim]."""
    T, H, dk = q.shape
    dv = v.shape[2]
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            gt = g[t, h]
            S = (gt[:, None] if gt.dim() == 1 else gt) * S
            u = beta[t, h] * (v[t, h] - S.t() @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.t() @ q[t, h]
    return out


def delta_mixer(h, P, pre, m, eps, low_rank):
    """The gated-delta-rule mixer.  low_rank False: one decay per head from
    '.a' and a SiLU output gate from '.g'; True: one decay per head and key
    channel from '.a2' ('.a1' h) and a sigmoid output gate from '.g2'
    ('.g1' h)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(lin(h, P, pre + "q"), P[pre + "q.conv"]))
    k = silu(short_conv(lin(h, P, pre + "k"), P[pre + "k.conv"]))
    v = silu(short_conv(lin(h, P, pre + "v"), P[pre + "v.conv"]))
    q = unit(q.view(T, G, dk)) * dk ** -0.5
    k = unit(k.view(T, G, dk))
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    v = v.view(T, H, dv)
    beta = torch.sigmoid(lin(h, P, pre + "b"))
    rate = torch.exp(_f(P[pre + "A_log"]))
    if low_rank:
        z = lin(lin(h, P, pre + "a1"), P, pre + "a2") + _f(P[pre + "dt_bias"])
        g = torch.exp(-rate[None, :, None] * softplus(z.view(T, H, dk)))
        gate = torch.sigmoid(lin(lin(h, P, pre + "g1"), P, pre + "g2"))
    else:
        z = lin(h, P, pre + "a") + _f(P[pre + "dt_bias"])
        g = torch.exp(-rate[None, :] * softplus(z))
        gate = silu(lin(h, P, pre + "g"))
    o = delta_rule(q, k, v, beta, g)
    o = rms_norm(o, P[pre + "norm"], eps)
    return lin(o.reshape(T, H * dv) * gate, P, pre + "o")


# ------------------------------------------------- windowed sink attention
def scaled_frequencies(rot):
    """f_i = base^(-2i/dims); with 'scaling' {factor, low, high, original}:
    wavelength l = 2 pi / f; l < original/high keeps f, l > original/low
    gives f / factor, in between a linear blend in s = (original / l - low)
    / (high - low)."""
    dims = rot["dims"]
    out = []
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        sc = rot.get("scaling")
        if sc:
            orig, fac = float(sc["original"]), float(sc["factor"])
            lo, hi = float(sc["low"]), float(sc["high"])
            l = 2.0 * math.pi / f
            if l < orig / hi:
                pass
            elif l > orig / lo:
                f = f / fac
            else:
                s = (orig / l - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_half(x, rot, positions=None):
    """Rotary positions on the first rot.dims elements of each head of
    x [T, H, d]: element i pairs with i + dims/2 (positions 0..T-1 unless
    given)."""
    if not rot or rot["dims"] == 0:
        return x
    T = x.shape[0]
    half = rot["dims"] // 2
    pos = torch.arange(T, dtype=F64) if positions is None else \
        torch.as_tensor(positions, dtype=F64)
    ang = pos[:, None] * scaled_frequencies(rot)[None]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    u, w = x[..., :half], x[..., half:2 * half]
    out = x.clone()
    out[..., :half] = u * c - w * s
    out[..., half:2 * half] = w * c + u * s
    return out


def attend(q, k, v, m):
    """Softmax attention of q [T, H, d] over k [T, G, d], v [T, G, dv], query
    i seeing key j iff j <= i and (i - j < mask.size or j < mask.keep_first);
    score q.k * scale, soft-capped; one added to the softmax denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    mask = m.get("mask") or {}
    size, first = mask.get("size", 0), mask.get("keep_first", 0)
    cap = m.get("softcap") or 0.0
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1)
                  if size <= 0 or i - j < size or j < first]
            s = (k[js, g] @ q[i, hh]) * m["scale"]
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            e = torch.exp(s)
            out[i, hh] = (e @ v[js, g]) / (1.0 + e.sum())
    return out


def sink_attention(h, P, pre, m, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = lin(h, P, pre + "q", True).view(T, H, dk)
    k = lin(h, P, pre + "k", True).view(T, G, dk)
    v = lin(h, P, pre + "v", True).view(T, G, dv)
    q = rotate_half(rms_norm(q, P[pre + "q.norm"], eps), m.get("rot"))
    k = rotate_half(rms_norm(k, P[pre + "k.norm"], eps), m.get("rot"))
    return lin(attend(q, k, v, m).reshape(T, H * dv), P, pre + "o")


def parallel_mixer(h, P, pre, m, eps):
    a = sink_attention(h, P, pre + "left.", m["left"], eps)
    b = delta_mixer(h, P, pre + "right.", m["right"], eps, True)
    return 0.5 * (rms_norm(a, P[pre + "left.out"], eps)
                  + rms_norm(b, P[pre + "right.out"], eps))


# ------------------------------------------------------------ feed-forward
def expert(h, P, pre, limit):
    g = torch.clamp(lin(h, P, pre + "gate"), max=limit)
    u = torch.clamp(lin(h, P, pre + "up"), -limit, limit)
    return lin(g * torch.sigmoid(1.702 * g) * (u + 1.0), P, pre + "down")


def route(h, P, pre, top):
    """(chosen experts [T, top], their softmax scores [T, top])."""
    s = torch.softmax(lin(h, P, pre + "router"), -1)
    choice = s + _f(P[pre + "correction"])
    idx = torch.topk(choice, top, dim=-1).indices
    return idx, s.gather(1, idx)


def moe(h, P, pre, m):
    top, limit = m["router"]["top"], m["expert"]["limit"]
    idx, w = route(h, P, pre, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for r in range(top):
            e = int(idx[t, r])
            out[t] += w[t, r] * expert(h[t:t + 1], P, f"{pre}e{e}.", limit)[0]
    return out


# ------------------------------------------------------------------- model
def token_side(x, tokens, P, i, dim, eps):
    pre = f"l{i}.side."
    e = _f(P["side.embed"])[tokens][:, i * dim:(i + 1) * dim]
    y = lin(gelu_tanh(lin(x, P, pre + "gate")) * e, P, pre + "proj")
    return x + rms_norm(y, P[pre + "norm"], eps)


def forward(tokens, P, cfg, layers_out=None):
    """tokens [T] -> logits [T, vocab] (float64).  layers_out: a list that
    receives the residual after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = _f(P["embed"])[tokens] * cfg["embedding"]["scale"]
    side = (cfg.get("token_side") or {}).get("dim", 0)
    for i, lc in enumerate(cfg["layers"]):
        pre = f"l{i}."
        if lc["type"] == "delta":
            y = delta_mixer(x, P, pre + "mix.", lc["mixer"], eps, False)
        else:
            y = parallel_mixer(x, P, pre + "mix.", lc["mixer"], eps)
        x = rms_norm(alpha * x + y, P[pre + "norm1"], eps)
        if lc.get("mlp") is not None:
            x = rms_norm(alpha * x + moe(x, P, pre + "mlp.", lc["mlp"]),
                         P[pre + "norm2"], eps)
        if side:
            x = token_side(x, tokens, P, i, side, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return lin(rms_norm(x, P["final.norm"], eps), P, "head")


# ---------------------------------------------------------- random weights
def random_weights(cfg, seed=0):
    """Checkpoint-named random tensors (bf16-representable float32) for any
    config, at scales that keep every branch alive."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    P = {}

    def rnd(name, *shape, std=None, mean=0.0):
        std = std if std is not None else shape[-1] ** -0.5
        t = torch.randn(*shape, generator=g) * std + mean
        P[name] = t.to(torch.bfloat16).float()

    def delta(pre, m, low_rank, rank=6):
        H, G, dk, dv, taps = (m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                              m["conv"])
        rnd(pre + "q", G * dk, W)
        rnd(pre + "k", G * dk, W)
        rnd(pre + "v", H * dv, W)
        for n, c in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
            rnd(pre + n + ".conv", c, taps, std=0.7)
        rnd(pre + "b", H, W)
        rnd(pre + "A_log", H, std=0.5, mean=-1.0)
        rnd(pre + "norm", dv, std=0.1, mean=1.0)
        if low_rank:
            rnd(pre + "a1", rank, W)
            rnd(pre + "a2", H * dk, rank)
            rnd(pre + "dt_bias", H * dk, std=1.0)
            rnd(pre + "g1", rank, W)
            rnd(pre + "g2", H * dv, rank)
        else:
            rnd(pre + "a", H, W)
            rnd(pre + "dt_bias", H, std=1.0)
            rnd(pre + "g", H * dv, W)
        rnd(pre + "o", W, H * dv)

    rnd("embed", V, W, std=1.0)
    rnd("head", V, W)
    rnd("final.norm", W, std=0.1, mean=1.0)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        rnd("side.embed", V, side * len(cfg["layers"]), std=1.0)
    for i, lc in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", lc["mixer"]
        rnd(pre + "norm1", W, std=0.1, mean=1.0)
        if lc["type"] == "delta":
            delta(pre + "mix.", m, False)
        else:
            le = m["left"]
            H, G, dk, dv = le["heads"], le["kv_heads"], le["dim"], le["vdim"]
            for n, c in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                rnd(pre + "mix.left." + n, c, W)
                rnd(pre + "mix.left." + n + ".b", c, std=0.3)
            rnd(pre + "mix.left.q.norm", dk, std=0.1, mean=1.0)
            rnd(pre + "mix.left.k.norm", dk, std=0.1, mean=1.0)
            rnd(pre + "mix.left.o", W, H * dv)
            delta(pre + "mix.right.", m["right"], True)
            rnd(pre + "mix.left.out", W, std=0.1, mean=1.0)
            rnd(pre + "mix.right.out", W, std=0.1, mean=1.0)
        f = lc.get("mlp")
        if f is not None:
            rnd(pre + "norm2", W, std=0.1, mean=1.0)
            E, F = f["router"]["experts"], f["expert"]["ff"]
            for e in range(E):
                rnd(f"{pre}mlp.e{e}.gate", F, W, std=2.0 * W ** -0.5)
                rnd(f"{pre}mlp.e{e}.up", F, W, std=2.0 * W ** -0.5)
                rnd(f"{pre}mlp.e{e}.down", W, F)
            rnd(pre + "mlp.router", E, W, std=4.0 * W ** -0.5)
            rnd(pre + "mlp.correction", E, std=0.05)
        if side:
            rnd(pre + "side.gate", side, W)
            rnd(pre + "side.proj", W, side)
            rnd(pre + "side.norm", W, std=0.1, mean=1.0)
    return P
