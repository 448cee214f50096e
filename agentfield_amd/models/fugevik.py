"""Hyper-connected decoders with latent attention: the Fugevik design.

A Fugevik model keeps `streams` fp32 copies of the residual per token instead
of one.  Each sublayer (mixer, then feed-forward) reads a learned combination
of the streams, u = sum_s in[s] x_s, through a zero-centred RMSNorm and an
input convolution (a short depthwise causal convolution over time, added to
its own input), and its output y goes back into all streams at once:
x_r <- sum_s mix[s, r] x_s + out[r] y.  The logits come from the sum of the
streams through the final norm and the embedding table.

config.json lists the layers; each names one of two mixers and a
feed-forward (or none):

  * ``latent_attention`` — keys and values are up-projections of one normed
    latent per token plus one rotary key part shared by the heads; only
    [latent | rotated key part] is cached.  Interleaved rotary positions,
    sliding window, a learned per-head sink in the softmax denominator, an
    element-wise sigmoid output gate.  Runs in absorbed form: the unrotated
    query is carried into latent space (q W_uk), attention is one K/V head
    over the cached rows whose values are the latents themselves, and the
    result is carried to value space (W_uv) afterwards.
  * ``attention`` — grouped-query softmax attention without rotation: scores
    are tanh-soft-capped and a per-head logarithmic distance bias is taken
    off; sliding window.  A layer may use the keys and values of an earlier
    layer (`kv_from`) with its own queries.
  * feed-forward — W_down relu(W_up h)^2.

Every mechanism is a module parameterised by its spec on the sequence-mixer
op set (ops/seqmix.py): gfx950 kernels on GPU, vendor GEMMs for projections.
Pages and convolution inputs live in `HybridCache`; the engine's scheduler
hands out pages and state slots.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable

import torch
from torch import nn

from ..ops import seqmix as sm
from .hybrid import HybridCache


# ------------------------------------------------------------------ specs
@dataclass
class LatentAttnSpec:
    heads: int
    dim: int                    # unrotated query/key size per head
    rot_dim: int                # rotary query/key size per head
    vdim: int
    kv_rank: int                # latent size
    scale: float
    window: int = 0             # 0: every earlier key
    rot_dims: int = 0           # leading dims of the rotary part that turn
    rot_base: float = 10000.0


@dataclass
class BiasedAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    softcap: float = 0.0        # 0: scores are not capped
    kv_from: int | None = None  # layer whose keys and values are used


@dataclass
class FLayerSpec:
    kind: str                                   # "latent_attention" | "attention"
    mixer: LatentAttnSpec | BiasedAttnSpec
    ff: int | None = None                       # None: no feed-forward


@dataclass
class FugevikConfig:
    name: str = "fugevik"
    vocab_size: int = 512
    width: int = 256
    layers: list = field(default_factory=list)
    streams: int = 1
    taps: int = 1               # input-convolution taps (1: current token only)
    eps: float = 1e-6
    max_position: int = 8192    # serving limit (block-table width)

    architecture = "Fugevik"
    # engine-facing traits
    stateful = True
    num_kv_heads = 1
    num_experts = 1
    sliding_window = 0

    def __post_init__(self):
        for i, ls in enumerate(self.layers):
            m = ls.mixer
            if ls.kind != "attention" or m.kv_from is None:
                continue
            j = m.kv_from
            if not 0 <= j < i or self.layers[j].kind != "attention" or \
                    self.layers[j].mixer.kv_from is not None:
                raise ValueError(f"layer {i}: kv_from must name an earlier "
                                 "attention layer with projections of its own")
            o = self.layers[j].mixer
            if (o.kv_heads, o.dim, o.vdim) != (m.kv_heads, m.dim, m.vdim):
                raise ValueError(f"layer {i}: key/value geometry differs "
                                 f"from layer {j}'s")

    def build_model(self, device="cpu", dtype=torch.bfloat16):
        return FugevikForCausalLM(self, device=device, dtype=dtype)

    def cache_layout(self) -> list:
        """What every layer keeps between steps (HybridCache): key pages
        holding [latent | rotary key part] (no value pages), K/V pages, or
        nothing for a layer that reads another layer's; plus the inputs of
        both input convolutions."""
        hist = (max(self.taps - 1, 1), self.width)
        out = []
        for ls in self.layers:
            m = ls.mixer
            if ls.kind == "latent_attention":
                kv = (1, m.kv_rank + m.rot_dim, 0)
            elif m.kv_from is None:
                kv = (m.kv_heads, m.dim, m.vdim)
            else:
                kv = None
            state = {"canon1": (hist, "f32")}
            if ls.ff is not None:
                state["canon2"] = (hist, "f32")
            out.append({"kv": kv, "state": state})
        return out

    @staticmethod
    def from_json(c: dict, name: str = "fugevik") -> "FugevikConfig":
        """Read a checkpoint's config.json."""
        layers = []
        for i, lc in enumerate(c["layers"]):
            m = lc["mixer"]
            window = int((m.get("mask") or {}).get("size", 0))
            if lc["type"] == "latent_attention":
                rot = m.get("rot") or {}
                mixer = LatentAttnSpec(
                    heads=int(m["heads"]), dim=int(m["dim"]),
                    rot_dim=int(m.get("rot_dim", 0)),
                    vdim=int(m.get("vdim", m["dim"])),
                    kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                    window=window,
                    rot_dims=int(rot.get("dims", m.get("rot_dim", 0))),
                    rot_base=float(rot.get("base", 10000.0)))
            elif lc["type"] == "attention":
                src = m.get("kv_from")
                mixer = BiasedAttnSpec(
                    heads=int(m["heads"]),
                    kv_heads=int(m.get("kv_heads", m["heads"])),
                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                    scale=float(m["scale"]), window=window,
                    softcap=float(m.get("softcap") or 0.0),
                    kv_from=int(src) if src is not None else None)
            else:
                raise ValueError(f"layer {i}: unknown type {lc['type']}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown mlp kind {mlp['kind']}")
            layers.append(FLayerSpec(
                kind=lc["type"], mixer=mixer,
                ff=int(mlp["ff"]) if mlp is not None else None))
        return FugevikConfig(
            name=name, vocab_size=int(c["vocab"]), width=int(c["width"]),
            layers=layers, streams=int(c.get("streams", 1)),
            taps=int((c.get("canon") or {}).get("taps", 1)),
            eps=float(c["norm"]["eps"]))

    def to_json(self) -> dict:
        layers = []
        for ls in self.layers:
            m = ls.mixer
            if ls.kind == "latent_attention":
                mixer = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank,
                         "rot": {"base": m.rot_base, "dims": m.rot_dims},
                         "rot_dim": m.rot_dim, "scale": m.scale,
                         "vdim": m.vdim}
            else:
                mixer = {"dim": m.dim, "heads": m.heads,
                         "kv_heads": m.kv_heads, "scale": m.scale,
                         "vdim": m.vdim}
                if m.softcap > 0:
                    mixer["softcap"] = m.softcap
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            if m.window > 0:
                mixer["mask"] = {"size": m.window}
            layers.append({
                "mixer": mixer, "type": ls.kind,
                "mlp": ({"ff": ls.ff, "kind": "dense"}
                        if ls.ff is not None else None)})
        return {"architecture": self.architecture,
                "canon": {"taps": self.taps}, "layers": layers,
                "norm": {"eps": self.eps}, "streams": self.streams,
                "vocab": self.vocab_size, "width": self.width}


def _f32(*shape):
    return torch.zeros(*shape, dtype=torch.float32)


def _pad8(n: int) -> int:
    return n + (-n) % 8


# ----------------------------------------------------------------- mixers
class LatentAttention(nn.Module):
    """[q | latent, rotary key part | gate logits] = W h (one GEMM).  The
    latent c is RMS-normed; key_h = [W_uk,h c | rot(key part)], value_h =
    W_uv,h c.  Since q_u . (W_uk,h c) = (q_u W_uk,h) . c and sum_j w_j
    W_uv,h c_j = W_uv,h sum_j w_j c_j, attention runs over the cached rows
    [c | rot(key part)] directly (ops.masked_attention, one K/V head, values
    inside the key rows) between two per-head batched GEMMs."""

    def __init__(self, spec: LatentAttnSpec, width: int, eps: float):
        super().__init__()
        s = self.spec = spec
        self.eps = eps
        self.nq = s.heads * (s.dim + s.rot_dim)
        self.nc = s.kv_rank + s.rot_dim
        self.ng = s.heads * s.vdim
        # blocks start at multiples of 8 rows so every view is 16-byte aligned
        self.c0 = _pad8(self.nq)
        self.g0 = self.c0 + _pad8(self.nc)
        self.w_in = nn.Parameter(torch.empty(self.g0 + _pad8(self.ng), width))
        self.c_norm = nn.Parameter(torch.empty(s.kv_rank))
        self.uk = nn.Parameter(torch.empty(s.heads, s.dim, s.kv_rank))
        self.uv = nn.Parameter(torch.empty(s.heads, s.kv_rank, s.vdim))
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))
        self.register_buffer("sink", _f32(s.heads))
        self.register_buffer(
            "inv_freq", sm.rotary_inv_freq(s.rot_dims, s.rot_base, "cpu")
            if s.rot_dims > 0 else None)

    def forward(self, h, cache: HybridCache, run: int, md, positions):
        s = self.spec
        T = h.shape[0]
        p = sm.matmul(h, self.w_in)
        q = p[:, :self.nq]
        dkv = p[:, self.c0:self.c0 + self.nc]
        g = p[:, self.g0:self.g0 + self.ng]
        qu = q.view(T, s.heads, s.dim + s.rot_dim)[:, :, :s.dim]
        # attention queries per head [q in latent space | rotated part]: the
        # batched GEMM writes the first slices in place, latent_prep the rest
        qf = torch.empty(T, s.heads * self.nc, dtype=h.dtype, device=h.device)
        torch.bmm(qu.transpose(0, 1), self.uk,
                  out=qf.view(T, s.heads, self.nc)[:, :, :s.kv_rank]
                  .transpose(0, 1))
        sm.latent_prep(q, dkv, qf, self.c_norm, self.eps, self.inv_freq,
                       positions, cache.k[run], md.slots, s.heads, s.dim)
        ol = sm.masked_attention(qf, cache.k[run], None, md, positions,
                                 s.scale, s.heads, window=s.window,
                                 sink=self.sink, v_width=s.kv_rank)
        ov = torch.bmm(ol.view(T, s.heads, s.kv_rank).transpose(0, 1),
                       self.uv)                              # [H, T, vdim]
        return sm.matmul(sm.gate_heads(ov, g), self.o)


class BiasedAttention(nn.Module):
    """Grouped-query softmax attention without rotation; scores soft-capped
    with tanh, minus r1_h ln(1 + r2_h distance); sliding window.  A layer
    with `kv_from` projects queries only and reads that layer's pages."""

    def __init__(self, spec: BiasedAttnSpec, width: int, eps: float):
        super().__init__()
        s = self.spec = spec
        self.eps = eps
        self.nq = s.heads * s.dim
        self.nk, self.nv = s.kv_heads * s.dim, s.kv_heads * s.vdim
        self.k0 = _pad8(self.nq)
        self.v0 = self.k0 + _pad8(self.nk)
        rows = self.k0 if s.kv_from is not None else self.v0 + _pad8(self.nv)
        self.w_in = nn.Parameter(torch.empty(rows, width))
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))
        self.register_buffer("r1", _f32(s.heads))
        self.register_buffer("r2", _f32(s.heads))

    def forward(self, h, cache: HybridCache, run: int, md, positions):
        s = self.spec
        p = sm.matmul(h, self.w_in)
        q = p[:, :self.nq]
        src = run
        if s.kv_from is None:
            q = sm.qk_norm_cache(q, p[:, self.k0:self.k0 + self.nk],
                                 p[:, self.v0:self.v0 + self.nv], None, None,
                                 self.eps, cache.k[run], cache.v[run],
                                 md.slots)
        else:
            src = s.kv_from
        o = sm.masked_attention(q, cache.k[src], cache.v[src], md, positions,
                                s.scale, s.heads, window=s.window,
                                softcap=s.softcap, log_bias=(self.r1, self.r2))
        return sm.matmul(o, self.o)


class SquaredReluMLP(nn.Module):
    """W_down relu(W_up h)^2."""

    def __init__(self, ff: int, width: int):
        super().__init__()
        self.up = nn.Parameter(torch.empty(ff, width))
        self.down = nn.Parameter(torch.empty(width, ff))

    def forward(self, h):
        return sm.matmul(sm.relu2(sm.matmul(h, self.up)), self.down)


# ------------------------------------------------------------------- layer
class StreamPort(nn.Module):
    """How one sublayer is wired to the streams: read weights `inw` [S], the
    norm and the input convolution on the way in; write weights `outw` [S]
    and the stream mixing matrix `mix` [S, S] (indexed [from, to]) on the way
    back."""

    def __init__(self, streams: int, width: int, taps: int):
        super().__init__()
        self.norm = nn.Parameter(torch.empty(width))
        self.canon = nn.Parameter(torch.empty(width, taps))
        self.register_buffer("inw", _f32(streams))
        self.register_buffer("outw", _f32(streams))
        self.register_buffer("mix", _f32(streams, streams))


class FugevikLayer(nn.Module):
    def __init__(self, cfg: FugevikConfig, spec: FLayerSpec):
        super().__init__()
        W = cfg.width
        self.spec = spec
        self.port1 = StreamPort(cfg.streams, W, cfg.taps)
        if spec.kind == "latent_attention":
            self.mixer = LatentAttention(spec.mixer, W, cfg.eps)
        else:
            self.mixer = BiasedAttention(spec.mixer, W, cfg.eps)
        if spec.ff is None:
            self.port2 = self.mlp = None
        else:
            self.port2 = StreamPort(cfg.streams, W, cfg.taps)
            self.mlp = SquaredReluMLP(spec.ff, W)


class FugevikForCausalLM(nn.Module):
    # the engine asks these before wiring a model in
    needs_state_slots = True
    supports_speculation = False    # rejected drafts would need the
    supports_prefix_cache = False   # convolution inputs rolled back / restored

    def __init__(self, cfg: FugevikConfig, device="cpu",
                 dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        with torch.device(device):
            self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
            self.layers = nn.ModuleList(
                [FugevikLayer(cfg, ls) for ls in cfg.layers])
            self.final_norm = nn.Parameter(torch.empty(cfg.width))
            self.register_buffer("ones", torch.ones(cfg.streams,
                                                    dtype=torch.float32))
        for p in self.parameters():
            p.data = p.data.to(dtype)
            p.requires_grad_(False)
        self.to(device)
        self.record_runs: list | None = None  # set to [] to keep x per layer

    # -- engine interface ---------------------------------------------------
    def make_cache(self, num_pages: int, page_size: int, num_slots: int,
                   device, dtype):
        return HybridCache(self.cfg.cache_layout(), num_pages, page_size,
                           num_slots, device, dtype)

    def cache_bytes_per_page(self, page_size: int) -> int:
        return HybridCache.bytes_per_page(self.cfg.cache_layout(), page_size,
                                          self.embed.element_size())

    def forward(self, ids, positions, cache: HybridCache, md,
                logit_rows: torch.Tensor | None = None):
        """ids/positions [T] i32 -> fp32 logits [T or len(logit_rows), V]."""
        cfg = self.cfg
        dt = self.embed.dtype
        eps = cfg.eps
        x = sm.embed_streams(ids, self.embed, cfg.streams)
        # a sublayer's output enters the streams in the same kernel that
        # reads the next sublayer's input out of them
        back = (None, None, None)
        for run, L in enumerate(self.layers):
            port = L.port1
            h = sm.hyper_conv_step(x, *back, port.inw, port.norm, eps,
                                   port.canon, cache.state["canon1"][run], md,
                                   positions, dt)
            y = L.mixer(h, cache, run, md, positions)
            back = (y, port.mix, port.outw)
            if L.mlp is not None:
                port = L.port2
                h = sm.hyper_conv_step(x, *back, port.inw, port.norm, eps,
                                       port.canon,
                                       cache.state["canon2"][run], md,
                                       positions, dt)
                back = (L.mlp(h), port.mix, port.outw)
            if self.record_runs is not None:
                self.record_runs.append(
                    sm.hyper_step(x, *back, self.ones, None, eps))
                back = (None, None, None)
        xs = sm.hyper_step(x, *back, self.ones, None, eps)
        hn = sm.norm_rows(xs, self.final_norm, eps, logit_rows, dt)
        # vocabulary-sized N: the vendor GEMM wins there at every row count
        return sm.matmul(hn, self.embed, skinny=False).float()

    # -- weights ------------------------------------------------------------
    @torch.no_grad()
    def load_tensors(self, get: Callable[[str], torch.Tensor]):
        """Fill parameters from checkpoint tensors by name: 'embed',
        'final.norm', and per layer i 'l<i>.norm1|norm2', 'l<i>.canon1|
        canon2', 'l<i>.hc1|hc2.in|out|mix', 'l<i>.mix.<...>',
        'l<i>.mlp.up|down'.  Linear weights are [out, in]."""
        def put(dst, src):
            dst.copy_(src.to(dst.device, dst.dtype))

        def blocks(dst, parts):
            """Stack row blocks, each padded to a multiple of 8 rows."""
            rows = []
            for t in parts:
                rows.append(t)
                if t.shape[0] % 8:
                    rows.append(t.new_zeros(8 - t.shape[0] % 8, t.shape[1]))
            put(dst, torch.cat(rows, 0))

        def port(pt, pre, q):
            put(pt.norm, get(f"{pre}norm{q}"))
            put(pt.canon, get(f"{pre}canon{q}"))
            put(pt.inw, get(f"{pre}hc{q}.in"))
            put(pt.outw, get(f"{pre}hc{q}.out"))
            put(pt.mix, get(f"{pre}hc{q}.mix"))
        put(self.embed, get("embed"))
        put(self.final_norm, get("final.norm"))
        for i, L in enumerate(self.layers):
            pre, mp = f"l{i}.", f"l{i}.mix."
            port(L.port1, pre, 1)
            m, s = L.mixer, L.mixer.spec
            if isinstance(m, LatentAttention):
                blocks(m.w_in, [get(mp + "q"), get(mp + "dkv"), get(mp + "g")])
                put(m.c_norm, get(mp + "dkv.norm"))
                put(m.uk, get(mp + "uk").view(s.heads, s.dim, s.kv_rank))
                put(m.uv, get(mp + "uv").view(s.heads, s.vdim, s.kv_rank)
                    .transpose(1, 2))
                put(m.sink, get(mp + "sink"))
            else:
                parts = [get(mp + "q")]
                if s.kv_from is None:
                    parts += [get(mp + "k"), get(mp + "v")]
                blocks(m.w_in, parts)
                put(m.r1, get(mp + "r1"))
                put(m.r2, get(mp + "r2"))
            put(m.o, get(mp + "o"))
            if L.mlp is not None:
                port(L.port2, pre, 2)
                put(L.mlp.up, get(pre + "mlp.up"))
                put(L.mlp.down, get(pre + "mlp.down"))
        return self

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        """Random weights at scales that keep activations O(1) through depth
        (benchmarks and smoke runs; not a trained model)."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(t, std, mean=0.0):
            t.copy_((mean + torch.randn(t.shape, generator=g) * std)
                    .to(t.dtype))
        S = self.cfg.streams
        for name, p in list(self.named_parameters()) + \
                list(self.named_buffers()):
            leaf = name.rsplit(".", 1)[-1]
            if p is None or leaf in ("inv_freq", "ones"):
                continue
            if leaf == "mix":
                p.copy_(torch.eye(S) + 0.05 * torch.randn(S, S, generator=g))
            elif leaf == "inw":
                rnd(p, 0.05, 1.0 / S)
            elif leaf == "outw":
                rnd(p, 0.05, 0.5)
            elif leaf == "r2":
                p.copy_(0.1 + torch.rand(p.shape, generator=g))
            elif leaf in ("r1", "sink"):
                rnd(p, 0.3)
            elif leaf == "canon":
                rnd(p, 0.2)
            elif leaf in ("norm", "final_norm"):
                rnd(p, 0.1)
            elif leaf == "c_norm":
                rnd(p, 0.1, 1.0)
            elif leaf == "embed":
                rnd(p, 1.0)
            elif leaf == "uk":
                rnd(p, p.shape[2] ** -0.5)
            else:
                rnd(p, p.shape[1] ** -0.5)
        return self


# ------------------------------------------------------ checkpoint reading
def load_fugevik(path: str, device="cpu", dtype=torch.bfloat16,
                 max_position: int | None = None) -> FugevikForCausalLM:
    """config.json + *.safetensors -> model on `device` in `dtype`."""
    from safetensors import safe_open
    root = Path(path)
    c = json.loads((root / "config.json").read_text())
    files = sorted(root.glob("*.safetensors"))
    handles = [safe_open(str(f), framework="pt") for f in files]
    where = {k: h for h in handles for k in h.keys()}

    def get(name):
        return where[name].get_tensor(name)
    cfg = FugevikConfig.from_json(c, name=root.name)
    if max_position is not None:
        cfg.max_position = max_position
    model = FugevikForCausalLM(cfg, device=device, dtype=dtype)
    return model.load_tensors(get).eval()


def save_fugevik(tensors: dict, cfg: FugevikConfig, path: str) -> None:
    """Write checkpoint-named tensors + config.json (tests, tooling)."""
    from safetensors.torch import save_file
    root = Path(path)
    root.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              str(root / "model.safetensors"))
    (root / "config.json").write_text(json.dumps(cfg.to_json(), indent=1))


def _bench_config(name, width, ff, n_layers, heads, kv_heads, dim,
                  vocab=32000, kv_rank=256, rot_dim=64, window=1024,
                  streams=4, taps=4):
    """Blocks of four layers: latent attention, attention with K/V of its
    own, attention sharing them, latent attention."""
    layers = []
    for i in range(n_layers):
        if i % 4 in (0, 3):
            kind, mixer = "latent_attention", LatentAttnSpec(
                heads=heads, dim=dim, rot_dim=rot_dim, vdim=dim,
                kv_rank=kv_rank, scale=(dim + rot_dim) ** -0.5,
                window=window, rot_dims=rot_dim, rot_base=500000.0)
        else:
            kind, mixer = "attention", BiasedAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                scale=dim ** -0.5, window=window, softcap=50.0,
                kv_from=i - 1 if i % 4 == 2 else None)
        layers.append(FLayerSpec(kind=kind, mixer=mixer, ff=ff))
    return FugevikConfig(name=name, vocab_size=vocab, width=width,
                         layers=layers, streams=streams, taps=taps, eps=1e-6)


FUGEVIK_CONFIGS = {
    # a small model with every branch, for smoke runs and CPU tests
    "fugevik-tiny": _bench_config("fugevik-tiny", 128, 320, 4, 4, 2, 32,
                                  vocab=384, kv_rank=48, rot_dim=16,
                                  window=40, streams=3, taps=3),
    # same width / ff / depth / heads as "zudisun-1b", "reperax-1b" and
    # "debug-1b"
    "fugevik-1b": _bench_config("fugevik-1b", 2048, 8192, 16, 16, 8, 128),
    # same width / ff / depth / heads / vocabulary as "llama-3-8b"
    "fugevik-8b": _bench_config("fugevik-8b", 4096, 14336, 32, 32, 8, 128,
                                vocab=128256, kv_rank=512),
}
