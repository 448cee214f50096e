"""Fugevik (hyper-connected streams, input convolutions, latent attention,
soft-capped attention with a logarithmic distance bias and shared K/V,
squared-ReLU feed-forward) against the plain float64 oracle in
fugevik_oracle.py: every mechanism alone, then whole models through the
engine's cache, state slots, batching, scheduler and generation.

Each test runs on the CPU op path and, marked gpu, on the gfx950 kernels.
fp32 runs are held to rounding-level agreement; bf16 runs to bf16 rounding.
"""
import json
import math
import subprocess
import sys
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))

import fugevik_oracle as orc  # noqa: E402
from agentfield_amd.engine import LLMEngine, SamplingParams  # noqa: E402
from agentfield_amd.models import load_model  # noqa: E402
from agentfield_amd.models.fugevik import (BiasedAttention,  # noqa: E402
                                           FugevikConfig, FugevikForCausalLM,
                                           LatentAttention, save_fugevik)
from agentfield_amd.models.hybrid import HybridCache  # noqa: E402
from agentfield_amd.ops import seqmix as sm  # noqa: E402

REPO = Path(__file__).resolve().parent.parent
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


# ------------------------------------------------------------ model zoo
def _lat(heads, dim, rot_dim, vdim, rank, window=None, dims=None, base=1e4):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
         "kv_rank": rank, "scale": (dim + rot_dim) ** -0.5,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def _att(heads, kv_heads, dim, vdim, window=None, cap=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if cap:
        m["softcap"] = cap
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def _with_ff(layer, ff):
    layer["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return layer


def cfg_mixed():
    """Unequal sizes everywhere; attention first; sharing layers that are not
    neighbours; a layer without feed-forward; windows that differ and end
    inside pages; rotation on part of the rotary slice."""
    layers = [
        _with_ff(_att(6, 3, 12, 20, window=21, cap=4.0), 40),
        _with_ff(_lat(4, 16, 8, 12, 24, window=19, dims=4, base=50.0), 56),
        _with_ff(_att(6, 3, 12, 20, window=13, cap=2.5, kv_from=0), None),
        _with_ff(_lat(2, 8, 16, 24, 40, window=37), 24),
        _with_ff(_att(6, 3, 12, 20, window=30, kv_from=0), 32),
    ]
    return {"architecture": "Fugevik", "vocab": 61, "width": 36,
            "streams": 3, "canon": {"taps": 3}, "layers": layers,
            "norm": {"eps": 1e-5}}


def cfg_degenerate():
    """Everything equal or 1: one stream, one tap, one head, one K/V head,
    no windows, no soft cap."""
    layers = [
        _with_ff(_lat(1, 8, 8, 8, 8), 16),
        _with_ff(_att(1, 1, 8, 8), 16),
    ]
    return {"architecture": "Fugevik", "vocab": 40, "width": 16,
            "streams": 1, "canon": {"taps": 1}, "layers": layers,
            "norm": {"eps": 1e-6}}


def cfg_odd():
    """Nothing divisible by 4 or 8: odd width and head sizes, seven streams,
    five taps (longer than two-token portions), latent wider than the heads,
    as many K/V heads as query heads."""
    layers = [
        _with_ff(_lat(3, 10, 6, 14, 50, window=33, dims=6, base=123.0), 30),
        _with_ff(_att(5, 5, 6, 10, window=9, cap=20.0), 26),
        _with_ff(_att(5, 5, 6, 10, window=64, cap=1.5, kv_from=1), 18),
        _with_ff(_lat(5, 6, 2, 6, 10), None),
    ]
    return {"architecture": "Fugevik", "vocab": 33, "width": 30,
            "streams": 7, "canon": {"taps": 5}, "layers": layers,
            "norm": {"eps": 1e-4}}


ZOO = {"mixed": cfg_mixed, "degenerate": cfg_degenerate, "odd": cfg_odd}


def build(cfg_json, device, dtype, seed=0, page=8, pages=64, live=4,
          paced=True, graphs=False):
    w = orc.random_weights(cfg_json, seed, dtype)
    cfg = FugevikConfig.from_json(cfg_json)
    cfg.max_position = 512
    model = FugevikForCausalLM(cfg, device=device, dtype=dtype)
    model.load_tensors(w.__getitem__)
    eng = LLMEngine(cfg, device=device, dtype=dtype, page_size=page,
                    num_pages=pages, max_num_seqs=live, model=model,
                    enable_graphs=graphs, caller_paced=paced, eos_id=-1)
    return eng, w


def tokens_for(cfg_json, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg_json["vocab"], (n,), generator=g).tolist()


def rel_err(got, want):
    """Row-wise: rms of the mean-free difference over rms of the oracle."""
    d = got.to(F64).cpu() - want
    d = d - d.mean(-1, keepdim=True)
    scale = want.pow(2).mean().sqrt()
    return float((d.pow(2).mean(-1).sqrt() / scale).max())


def tol(dtype):
    return 2e-4 if dtype == torch.float32 else 8e-2


def close(got, want, dtype, factor=1.0):
    return rel_err(got, want) < tol(dtype) * factor


def run_schedule(eng, requests, schedule):
    """requests: name -> tokens.  schedule: list of steps, each a list of
    (name, count).  Every fed position's logits are collected; a request is
    closed when its last token went in.  Returns name -> [T, V]."""
    at = {n: 0 for n in requests}
    seqs, out = {}, {n: [] for n in requests}
    for step in schedule:
        entries, names = [], []
        for name, count in step:
            if name not in seqs:
                seqs[name] = eng.open_request()
            lo = at[name]
            entries.append((seqs[name], requests[name][lo:lo + count],
                            list(range(count))))
            names.append((name, count))
            at[name] = lo + count
        logits = eng.feed_step(entries)
        r = 0
        for name, count in names:
            out[name].append(logits[r:r + count].cpu())
            r += count
            if at[name] == len(requests[name]):
                eng.close_request(seqs.pop(name))
    return {n: torch.cat(v) for n, v in out.items()}


def md_for(chunks, starts, slots, device, page=8, pages_per_seq=16,
           decode=False):
    """Batch description for op-level tests: sequence i runs chunks[i] rows
    from position starts[i], owns pages 1 + i*pages_per_seq .."""
    cu, rowseq, pos, kvslots = [0], [], [], []
    bt = torch.zeros(len(chunks), pages_per_seq, dtype=torch.int32)
    for i, (n, s0) in enumerate(zip(chunks, starts)):
        cu.append(cu[-1] + n)
        rowseq += [i] * n
        bt[i] = torch.arange(pages_per_seq) + 1 + i * pages_per_seq
        for p in range(s0, s0 + n):
            pos.append(p)
            kvslots.append(int(bt[i, p // page]) * page + p % page)
    t = lambda v, d: torch.tensor(v, dtype=d, device=device)  # noqa: E731
    md = SimpleNamespace(cu_seqlens=t(cu, torch.int32),
                         q_start=t(starts, torch.int32),
                         state_slots=t(slots, torch.int32),
                         row_seq=t(rowseq, torch.int32),
                         block_table=bt.to(device),
                         slots=t(kvslots, torch.int64),
                         seq_lens=None if decode else list(chunks),
                         is_prefill=not decode)
    return md, t(pos, torch.int32)


PORTIONS = ((0, 11), (11, 13), (13, 14), (14, 31), (31, 33), (33, 90))


# ====================================================== mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
def test_kernel_groups_present(device):
    if device == "cuda":
        from agentfield_amd.ops import _lib
        for group in ("glue", "seq", "hyper"):
            assert _lib.mixgroup(group) is not None


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 16), (3, 30), (4, 64), (7, 33),
                                   (16, 8), (4, 2048), (2, 1030), (3, 5001)])
def test_stream_step_alone(device, dtype, shape):
    """Write a sublayer output into the streams and read the next input out:
    both halves apart and fused, against the oracle's loops."""
    S, W = shape
    T = 9
    g = torch.Generator().manual_seed(S * 100 + W)
    x0 = torch.randn(T, S, W, generator=g)
    y = torch.randn(T, W, generator=g).to(dtype)
    mix = torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)
    outw, inw = torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = (0.2 * torch.randn(W, generator=g)).to(dtype)
    eps = 1e-5
    want_x = orc.stream_write(x0.to(F64), y.to(F64), mix.to(F64),
                              outw.to(F64))
    want_u = orc.stream_read(want_x, inw.to(F64))
    want_n = orc.centred_norm(want_u, nw.to(F64), eps)
    d = lambda t: t.to(device)  # noqa: E731
    x = d(x0.clone())
    n = sm.hyper_step(x, d(y), d(mix), d(outw), d(inw), d(nw), eps)
    assert (x.cpu().to(F64) - want_x).abs().max() < 1e-4
    assert (n.cpu().to(F64) - want_n).abs().max() < 1e-4
    # halves apart: write only, then read without a norm
    x = d(x0.clone())
    assert sm.hyper_step(x, d(y), d(mix), d(outw), None, None, eps) is None
    u = sm.hyper_step(x, None, None, None, d(inw), None, eps)
    assert (x.cpu().to(F64) - want_x).abs().max() < 1e-4
    assert (u.cpu().to(F64) - want_u).abs().max() < 1e-4
    xs = sm.embed_streams(d(torch.tensor([2, 0, 1], dtype=torch.int32)),
                          d(torch.randn(3, W, generator=g).to(dtype)), S)
    assert xs.shape == (3, S, W) and (xs[:, 0] == xs[:, S - 1]).all()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4, 6])
def test_input_conv_alone(device, dtype, taps):
    """Portions down to one and two tokens (shorter than the taps) through a
    slot that holds another sequence's leftovers; two sequences per step."""
    W, T = 21, 40
    g = torch.Generator().manual_seed(taps)
    w = (0.5 * torch.randn(W, taps, generator=g)).to(dtype)
    seqs = [torch.randn(T, W, generator=g), torch.randn(T, W, generator=g)]
    want = [orc.input_conv(s.to(F64), w.to(F64)) for s in seqs]
    state = torch.full((4, max(taps - 1, 1), W), 7.0, device=device)
    cuts = [0, 1, 3, 5, 6, 8, 17, 19, 40]
    got = [[], []]
    for lo, hi in zip(cuts, cuts[1:]):
        md, _ = md_for([hi - lo, hi - lo], [lo, lo], [3, 1], device)
        n = torch.cat([seqs[0][lo:hi], seqs[1][lo:hi]]).to(device)
        h = sm.canon_conv(n, w.to(device), state, md, dtype)
        got[0].append(h[:hi - lo].cpu())
        got[1].append(h[hi - lo:].cpu())
    lim = 1e-5 if dtype == torch.float32 else 3e-2
    for b in range(2):
        assert (torch.cat(got[b]).to(F64) - want[b]).abs().max() < lim
    if taps > 1:   # the slot now holds the last taps-1 inputs, oldest first
        assert torch.equal(state[3].cpu(), seqs[0][T - taps + 1:])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(3, 30, 3), (4, 64, 4), (1, 16, 1),
                                   (7, 33, 5), (2, 8, 2), (4, 2048, 4),
                                   (2, 1030, 3), (2, 4500, 2)])
def test_decode_step_fuses_input_conv(device, dtype, shape):
    """Steps of one row per sequence (write, read, norm, convolution, slot
    moved on in one kernel) against the separate ops, from position 0 on."""
    S, W, taps = shape
    B, steps = 3, 7
    g = torch.Generator().manual_seed(S + W + taps)
    d = lambda t: t.to(device)  # noqa: E731
    mix = d(torch.eye(S) + 0.3 * torch.randn(S, S, generator=g))
    outw, inw = d(torch.randn(S, generator=g)), d(torch.randn(S, generator=g))
    nw = d((0.2 * torch.randn(W, generator=g)).to(dtype))
    cw = d((0.5 * torch.randn(W, taps, generator=g)).to(dtype))
    hist = max(taps - 1, 1)
    st_a = torch.full((5, hist, W), 7.0, device=device)
    st_b = st_a.clone()
    starts = [0, 0, 0]
    for step in range(steps):
        x0 = torch.randn(B, S, W, generator=g)
        y = d(torch.randn(B, W, generator=g).to(dtype))
        md_a, pos = md_for([1] * B, [step] * B, [4, 1, 2], device)
        md_b, _ = md_for([1] * B, [step] * B, [4, 1, 2], device, decode=True)
        xa, xb = d(x0.clone()), d(x0.clone())
        ha = sm.hyper_conv_step(xa, y, mix, outw, inw, nw, 1e-5, cw, st_a,
                                md_a, pos, dtype)
        hb = sm.hyper_conv_step(xb, y, mix, outw, inw, nw, 1e-5, cw, st_b,
                                md_b, pos, dtype)
        assert torch.equal(xa, xb)
        assert (ha.float() - hb.float()).abs().max() < \
            (1e-5 if dtype == torch.float32 else 5e-2)
        if taps > 1:
            keep = min(step + 1, taps - 1)      # places of real positions
            assert (st_a[[4, 1, 2], hist - keep:] -
                    st_b[[4, 1, 2], hist - keep:]).abs().max() < 1e-5


def _attn_close(got, want, dtype):
    d = (got.to(F64).cpu() - want).pow(2).mean().sqrt()
    return float(d / want.pow(2).mean().sqrt()) < \
        (1e-5 if dtype == torch.float32 else 2e-2)


def _run_mixer(mod, layout, h, device, dtype, portions, page=8, decode_from=None):
    """Feed rows of h through a mixer module in portions via a fresh cache
    whose slot 2 / pages hold garbage; returns the stacked outputs."""
    cache = HybridCache(layout, 40, page, 4, device, dtype)
    for t in list(cache.k.values()) + list(cache.v.values()):
        t.fill_(3.0)
    outs = []
    for lo, hi in portions:
        dec = decode_from is not None and lo >= decode_from and hi - lo == 1
        md, pos = md_for([hi - lo], [lo], [2], device, page=page, decode=dec)
        outs.append(mod(h[lo:hi].to(device), cache, 0, md, pos).cpu())
    return torch.cat(outs), cache


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [
    # heads, dim, rot_dim, vdim, rank, window, rotated dims
    (4, 16, 8, 12, 24, 19, 8),
    (1, 8, 8, 8, 8, 0, 8),
    (3, 10, 6, 14, 50, 33, 4),
    (2, 32, 16, 32, 144, 50, 16),     # wide rows: latent + key part = 160
    (2, 8, 8, 8, 328, 70, 8),         # wider than 320
    (2, 8, 16, 8, 600, 50, 16),       # wider than any tile kernel
    (5, 6, 2, 6, 10, 7, 0),           # nothing rotates
    (9, 8, 8, 8, 24, 19, 8),          # many heads on the one latent row
    (20, 16, 8, 12, 40, 0, 8),
    (70, 4, 4, 4, 12, 30, 4)])        # more heads than one 64-row block
def test_latent_attention_alone(device, dtype, shape):
    H, dim, rd, vd, R, window, dims = shape
    W, T = 28, 90
    m = _lat(H, dim, rd, vd, R, window=window, dims=dims, base=77.0)["mixer"]
    cj = {"architecture": "Fugevik", "vocab": 8, "width": W, "streams": 1,
          "layers": [{"type": "latent_attention", "mixer": m, "mlp": None}],
          "norm": {"eps": 1e-5}}
    w = orc.random_weights(cj, 5, dtype, gain=1.5)
    cfg = FugevikConfig.from_json(cj)
    model = FugevikForCausalLM(cfg, device=device, dtype=dtype)
    model.load_tensors(w.__getitem__)
    mod = model.layers[0].mixer
    assert isinstance(mod, LatentAttention)
    g = torch.Generator().manual_seed(3)
    h = torch.randn(T, W, generator=g).to(dtype)
    w64 = {k: v.to(F64) for k, v in w.items()}
    want = orc.latent_attention(h.to(F64), m, w64, "l0.mix.", 1e-5)
    layout = [{"kv": (1, R + rd, 0), "state": {}}]
    got, cache = _run_mixer(mod, layout, h, device, dtype, PORTIONS)
    assert _attn_close(got, want, dtype)
    assert not cache.v                      # one row per token, no V pages
    one, _ = _run_mixer(mod, layout, h, device, dtype,
                        [(0, 40)] + [(i, i + 1) for i in range(40, T)],
                        decode_from=40)
    assert _attn_close(one, want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [
    # heads, kv_heads, dim, vdim, window, cap
    (6, 3, 12, 20, 21, 4.0),
    (1, 1, 8, 8, 0, 0.0),
    (5, 5, 6, 10, 9, 20.0),
    (8, 1, 64, 64, 40, 1.5),
    (24, 2, 8, 8, 21, 3.0),            # twelve heads per K/V head
    (4, 2, 40, 136, 64, 2.0)])         # values wider than 128
def test_biased_attention_alone(device, dtype, shape):
    H, G, dim, vd, window, cap = shape
    W, T = 28, 90
    a0 = _att(H, G, dim, vd, window=window, cap=cap)
    a1 = _att(H, G, dim, vd, window=max(window // 2, 0), cap=cap, kv_from=0)
    cj = {"architecture": "Fugevik", "vocab": 8, "width": W, "streams": 1,
          "layers": [_with_ff(a0, None), _with_ff(a1, None)],
          "norm": {"eps": 1e-5}}
    w = orc.random_weights(cj, 6, dtype, gain=2.0)
    cfg = FugevikConfig.from_json(cj)
    model = FugevikForCausalLM(cfg, device=device, dtype=dtype)
    model.load_tensors(w.__getitem__)
    own, shared = model.layers[0].mixer, model.layers[1].mixer
    assert isinstance(own, BiasedAttention)
    assert shared.w_in.shape[0] < own.w_in.shape[0]   # queries only
    g = torch.Generator().manual_seed(4)
    h = torch.randn(T, W, generator=g).to(dtype)
    h2 = torch.randn(T, W, generator=g).to(dtype)
    w64 = {k: v.to(F64) for k, v in w.items()}
    want, kv = orc.biased_attention(h.to(F64), a0["mixer"], w64, "l0.mix.")
    want2, _ = orc.biased_attention(h2.to(F64), a1["mixer"], w64, "l1.mix.",
                                    kv)
    layout = [{"kv": (G, dim, vd), "state": {}}]
    for portions, dec in ((PORTIONS, None),
                          ([(0, 40)] + [(i, i + 1) for i in range(40, T)],
                           40)):
        got, cache = _run_mixer(own, layout, h, device, dtype, portions,
                                decode_from=dec)
        assert _attn_close(got, want, dtype)
        # the sharing layer: its own queries over the first layer's pages
        md, pos = md_for([T], [0], [2], device)
        got2 = shared(h2.to(device), cache, 1, md, pos)
        assert _attn_close(got2, want2, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_alone(device, dtype):
    g = torch.Generator().manual_seed(8)
    z = torch.randn(7, 50, generator=g).to(dtype)
    got = sm.relu2(z.to(device)[:, 3:36])             # a strided view
    want = torch.relu(z[:, 3:36].to(F64)).pow(2)
    assert (got.cpu().to(F64) - want).abs().max() < \
        (1e-6 if dtype == torch.float32 else 5e-2)


# ================================== edges made visible by chosen inputs
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H", [2, 16])
def test_window_edge_and_far_key(device, dtype, decode, H):
    """One loud key among hundreds: it is heard exactly while it is inside
    the window (distances window-1 and window apart), at a page's last and
    first place and far from the query; prompt rows and single rows."""
    page, T, window = 16, 400, 129
    G, dk, dv = 1, 8, 8
    for loud in (0, 15, 16, 255, 270):
        pages = T // page
        kc = torch.zeros(pages + 2, G, page, dk, dtype=dtype, device=device)
        vc = torch.zeros_like(kc)
        bt = torch.arange(1, pages + 2, dtype=torch.int32)
        pg, off = int(bt[loud // page]), loud % page
        kc[pg, 0, off, 0] = 30.0
        vc[pg, 0, off, :] = 1.0
        rows = [loud, loud + 1, loud + window - 2, loud + window - 1,
                loud + window, loud + window + 1]
        rows = [r for r in rows if r < T]
        q = torch.zeros(len(rows), H * dk, dtype=dtype, device=device)
        q[:, 0::dk] = 1.0
        if decode:
            md = SimpleNamespace(
                block_table=bt[None].repeat(len(rows), 1).to(device),
                row_seq=torch.arange(len(rows), dtype=torch.int32,
                                     device=device),
                seq_lens=None)
            pos = torch.tensor(rows, dtype=torch.int32, device=device)
            out = sm.masked_attention(q, kc, vc, md, pos, 1.0, H,
                                      window=window)
        else:
            # the rows as the tails of prompt portions that end at each row
            out = []
            for i, r in enumerate(rows):
                n = min(r + 1, 40)
                md, pos = md_for([n], [r + 1 - n], [1], device, page=page,
                                 pages_per_seq=pages + 1)
                qq = torch.zeros(n, H * dk, dtype=dtype, device=device)
                qq[-1] = q[i]
                out.append(sm.masked_attention(qq, kc, vc, md, pos, 1.0, H,
                                               window=window)[-1])
            out = torch.stack(out)
        for r, o in zip(rows, out.float().cpu()):
            heard = r - loud < window
            assert (o > 0.99).all() if heard else (o.abs() < 1e-6).all(), \
                (loud, r)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [3, 9])
def test_sink_takes_weight_without_value(device, dtype, H):
    """Equal scores everywhere: n keys share 1 - e^sink / (n + e^sink) of the
    weight; a huge sink silences the head, a tiny one changes nothing; the
    sink is not multiplied by the score scale."""
    page, T, dk, dv = 8, 70, 8, 6
    kc = torch.zeros(12, 1, page, dk, dtype=dtype, device=device)
    vc = torch.ones(12, 1, page, dv, dtype=dtype, device=device)
    sink = torch.tensor([math.log(5.0), 40.0, -40.0] + [0.0] * (H - 3),
                        device=device)
    q = torch.zeros(T, H * dk, dtype=dtype, device=device)
    for decode in (False, True):
        md, pos = md_for([T], [0], [1], device, page=page, decode=decode)
        o = sm.masked_attention(q, kc, vc, md, pos, 0.01, H, window=32,
                                sink=sink).float().cpu().view(T, H, dv)
        n = torch.arange(1, T + 1).clamp(max=32).float()
        assert (o[:, 0, 0] - n / (n + 5.0)).abs().max() < 1e-2
        assert o[:, 1].abs().max() < 1e-6
        assert (o[:, 2] - 1.0).abs().max() < 1e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_distance_bias_and_cap_formulas(device, dtype):
    """Two keys only, scores set by hand: the weights follow
    cap*tanh(s/cap) - r1 ln(1 + r2 d) exactly, per head."""
    page, H, dk, dv = 8, 2, 4, 2
    cap = 2.0
    r1 = torch.tensor([0.5, 1.25], device=device)
    r2 = torch.tensor([2.0, 0.25], device=device)
    for d in (1, 7, 8, 9, 30):
        T = d + 1
        kc = torch.zeros(8, 1, page, dk, dtype=dtype, device=device)
        vc = torch.zeros(8, 1, page, dv, dtype=dtype, device=device)
        md, pos = md_for([T], [0], [1], device, page=page)
        bt = md.block_table[0]
        kc[int(bt[0]), 0, 0, 0] = 3.0          # key 0: raw score 3
        kc[int(bt[d // page]), 0, d % page, 0] = 1.0
        vc[int(bt[0]), 0, 0, 0] = 1.0          # value marks key 0
        vc[int(bt[d // page]), 0, d % page, 1] = 1.0
        q = torch.zeros(T, H * dk, dtype=dtype, device=device)
        q[:, 0] = q[:, dk] = 1.0
        for decode in (False, True):
            md.seq_lens = None if decode else [T]
            o = sm.masked_attention(q, kc, vc, md, pos, 1.0, H, window=d + 1,
                                    softcap=cap, log_bias=(r1, r2))
            o = o.float().cpu().view(T, H, dv)[d]
            for h in range(H):
                s0 = cap * math.tanh(3.0 / cap) - float(r1[h]) * math.log(
                    1.0 + float(r2[h]) * d)
                s1 = cap * math.tanh(1.0 / cap)
                # the keys between score 0 at their own distances
                mid = [-float(r1[h]) * math.log(1.0 + float(r2[h]) * k)
                       for k in range(1, d)]
                den = math.exp(s0) + math.exp(s1) + sum(map(math.exp, mid))
                assert abs(float(o[h, 0]) - math.exp(s0) / den) < 6e-3
                assert abs(float(o[h, 1]) - math.exp(s1) / den) < 6e-3


@pytest.mark.parametrize("device", DEVICES)
def test_rotation_pairs_neighbours(device):
    """Interleaved layout: (0,1), (2,3) turn together; the tail passes."""
    T, R, rd, H, dim = 5, 4, 6, 1, 2
    inv = sm.rotary_inv_freq(4, 100.0, device)
    pos = torch.tensor([0, 1, 2, 50, 51], dtype=torch.int32, device=device)
    dkv = torch.zeros(T, R + rd, device=device)
    dkv[:, :R] = 1.0
    dkv[:, R + 0] = 1.0     # pair 0: (1, 0)
    dkv[:, R + 3] = 2.0     # pair 1: (0, 2)
    dkv[:, R + 5] = 9.0     # not rotated
    q = torch.zeros(T, H * (dim + rd), device=device)
    q[:, dim + 1] = 1.0
    kc = torch.zeros(10, 1, 8, R + rd, device=device)
    slots = torch.arange(8, 8 + T, dtype=torch.int64, device=device)
    qf = torch.full((T, H * (R + rd)), 5.0, device=device)
    qf = sm.latent_prep(q, dkv, qf, torch.ones(R, device=device), 0.0, inv,
                        pos, kc, slots, H, dim).cpu()
    assert (qf[:, :R] == 5.0).all()         # the caller's slice is left alone
    rows = kc.view(-1, R + rd)[8:8 + T].cpu()
    for i, p in enumerate(pos.tolist()):
        a0, a1 = p * 1.0, p * 100.0 ** -0.5
        want = [math.cos(a0), math.sin(a0), -2 * math.sin(a1),
                2 * math.cos(a1), 0.0, 9.0]
        assert (rows[i, R:] - torch.tensor(want)).abs().max() < 1e-5
        assert (rows[i, :R] - 1.0).abs().max() < 1e-6
        assert abs(float(qf[i, R + 0]) + math.sin(a0)) < 1e-5
        assert abs(float(qf[i, R + 1]) - math.cos(a0)) < 1e-5


# ================================================ models through the engine
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(ZOO))
def test_whole_prompt_and_layers(device, dtype, name):
    cj = ZOO[name]()
    eng, w = build(cj, device, dtype)
    toks = tokens_for(cj, 70, 1)
    want, layers = orc.forward(toks, cj, w, keep_layers=True)
    eng.model.record_runs = []
    got = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    assert close(got, want, dtype)
    assert len(eng.model.record_runs) == len(layers)
    for g, r in zip(eng.model.record_runs, layers):
        assert close(g, r, dtype)
    # recording splits the fused stream steps; the logits do not move
    eng.model.record_runs = None
    again = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    assert rel_err(again, got.to(F64)) < (1e-5 if dtype == torch.float32
                                          else 4e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(ZOO))
def test_prefill_then_token_by_token(device, dtype, name):
    """The first tokens of a sequence one by one, a prompt portion, then long
    decoding: past every window, tap count and page border."""
    cj = ZOO[name]()
    eng, w = build(cj, device, dtype, pages=40)
    toks = tokens_for(cj, 200, 2)
    want = orc.forward(toks, cj, w)
    sched = [[("a", 1)]] * 6 + [[("a", 44)]] + [[("a", 1)]] * 150
    got = run_schedule(eng, {"a": toks}, sched)["a"]
    assert close(got, want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_portions_down_to_two_tokens(device, dtype, name):
    cj = ZOO[name]()
    eng, w = build(cj, device, dtype)
    toks = tokens_for(cj, 120, 3)
    want = orc.forward(toks, cj, w)
    cuts = [2, 2, 3, 2, 17, 2, 40, 5, 2, 16, 1, 2, 26]
    assert sum(cuts) == len(toks)
    got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert close(got, want, dtype)
    whole = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    # how a prompt is cut changes nothing beyond rounding
    assert close(got, whole.to(F64), dtype)
    if dtype == torch.float32:
        assert rel_err(got, whole.to(F64)) < 5e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_mixed_batches_reuse_pages_and_slots(device, dtype, name):
    """Eight unequal requests through two state slots and a pool of nine
    pages: portions beside single tokens, requests paused and resumed, pages
    and slots handed to the next request as soon as one ends."""
    cj = ZOO[name]()
    eng, w = build(cj, device, dtype, page=8, pages=10, live=2)
    lens = [30, 9, 33, 2, 17, 25, 1, 12]
    reqs = {f"r{i}": tokens_for(cj, n, 10 + i) for i, n in enumerate(lens)}
    sched = [
        [("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7)],          # r1 ends
        [("r2", 3)], [("r0", 20), ("r2", 1)], [("r0", 4), ("r2", 2)],
        [("r2", 27)],                                            # r0, r2 end
        [("r3", 2), ("r4", 16)], [("r4", 1), ("r5", 2)],         # r3, r4 end
        [("r5", 23), ("r6", 1)],                                 # both end
        [("r7", 2)], [("r7", 1)], [("r7", 9)]]
    got = run_schedule(eng, reqs, sched)
    want = {n: orc.forward(toks, cj, w) for n, toks in reqs.items()}
    assert close(torch.cat([got[n] for n in reqs]),
                 torch.cat([want[n] for n in reqs]), dtype)
    assert eng.sched.alloc.num_free == 9
    assert eng.state_slots.num_free == 2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_scheduler(device, dtype):
    """engine.generate: the scheduler's batched prefill, (on GPU) the
    graph-captured decode step and the sampler reproduce the oracle's greedy
    continuation of unequal prompts."""
    cj = cfg_mixed()
    eng, w = build(cj, device, dtype, paced=False,
                   graphs=(device == "cuda"), pages=48)
    prompts = [tokens_for(cj, n, 20 + n) for n in (5, 23, 1, 14)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12,
                                                temperature=0.0,
                                                ignore_eos=True))
    # the GPU sampler reads logits rounded to bf16, so near-ties may fall
    # either way: every emitted token must be (all but) the oracle's best
    # given the tokens emitted before it
    slack = 0.5 if dtype == torch.bfloat16 else \
        (0.05 if device == "cuda" else 1e-3)
    for p, o in zip(prompts, outs):
        assert len(o) == 12
        want = orc.forward(p + o, cj, w)
        for i, tok in enumerate(o):
            row = want[len(p) + i - 1]
            assert row[tok] >= row.max() - slack, (len(p), i)
    assert eng.state_slots.num_free == 4   # all slots given back


def test_scheduler_preemption_restarts_state():
    """Running out of pages preempts a sequence; on re-admission it
    recomputes from position 0 in whatever slot is free and still produces
    the oracle's greedy tokens."""
    cj = cfg_odd()
    eng, w = build(cj, "cpu", torch.float32, seed=17, page=4, pages=9,
                   live=3, paced=False)
    prompts = [tokens_for(cj, 6, 40 + i) for i in range(3)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10,
                                                ignore_eos=True))
    assert eng.sched.n_preempted > 0
    for p, o in zip(prompts, outs):
        want = orc.forward(p + o, cj, w)
        for i, tok in enumerate(o):
            row = want[len(p) + i - 1]
            assert row[tok] >= row.max() - 1e-3


def test_config_round_trip_and_registry(tmp_path):
    cj = cfg_mixed()
    w = orc.random_weights(cj, 4, torch.bfloat16)
    cfg = FugevikConfig.from_json(cj)
    again = FugevikConfig.from_json(cfg.to_json())
    assert again.layers == cfg.layers and again.eps == cfg.eps
    assert (again.streams, again.taps) == (3, 3)
    save_fugevik(w, cfg, str(tmp_path / "ckpt"))
    model = load_model(str(tmp_path / "ckpt"), device="cpu",
                       dtype=torch.float32)
    assert isinstance(model, FugevikForCausalLM)
    assert model.cfg.layers == cfg.layers
    bad = cfg_mixed()
    bad["layers"][2]["mixer"]["kv_from"] = 1      # a latent layer
    with pytest.raises(ValueError):
        FugevikConfig.from_json(bad)


def test_trace_runner_subprocess(tmp_path):
    """bin/trace_run on a checkpoint directory: a mixed schedule with reuse,
    logits compared with the oracle."""
    cj = cfg_odd()
    w = orc.random_weights(cj, 6, torch.bfloat16)
    save_fugevik(w, FugevikConfig.from_json(cj), str(tmp_path / "m"))
    a, b = tokens_for(cj, 70, 30), tokens_for(cj, 9, 31)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [49]},
                                {"id": "b", "tokens": b[:2], "want": []}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:51], "want": [0]},
                                {"id": "b", "tokens": b[2:], "want": [0, 6]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[51:], "want": [18]}],
         "end": ["a"]}]
    r = subprocess.run(
        [sys.executable, str(REPO / "bin" / "trace_run"), "--model",
         str(tmp_path / "m"), "--dtype", "float32", "--out",
         str(tmp_path / "o"), "--max-tokens", "128", "--device", "cpu"],
        input="\n".join(json.dumps(s) for s in steps) + "\n",
        capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    import numpy as np
    wa, wb = orc.forward(a, cj, w), orc.forward(b, cj, w)
    V = cj["vocab"]
    for step, rows in ((0, [wa[49]]), (1, [wa[50], wb[2], wb[8]]),
                       (2, [wa[69]])):
        got = torch.from_numpy(np.fromfile(str(tmp_path / "o" / f"{step}.f32"),
                                           dtype="<f4").reshape(-1, V))
        assert rel_err(got, torch.stack(rows)) < 2e-4
