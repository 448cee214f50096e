"""Post-norm hybrid decoders: the Zudisun design.

A Zudisun model is a stack of layers `x <- x + norm1(mixer(x))`, `x <- x +
norm2(ff(x))`: the sublayers read the fp32 residual itself and an RMSNorm
sits on each sublayer's *output*.  config.json lists the layers; each names
its mixer and its feed-forward (or none):

  * ``mamba1``    — selective state-space mixer: gated input projection,
    depthwise causal convolution, input-dependent step sizes and B / C, a
    token-serial scan over an fp32 state [inner, state] per sequence
  * ``attention`` — sigmoid attention: per-head unit-RMS q and k, a query
    temperature growing with position, a learned bucketed distance bias, the
    heads' scores mixed by a learned matrix, un-normalised sigmoid weights,
    values optionally blended with the values of the first such layer, a
    per-head sigmoid output gate; no positional rotation
  * feed-forward ``dense`` — ReLU-gated unit with biases; ``moe`` — SiLU-gated
    experts behind a sigmoid router with score correction and group-limited
    top-k, plus an always-on shared expert

Every mechanism is a module parameterised by its spec on the sequence-mixer
op set (ops/seqmix.py): gfx950 kernels on GPU, vendor GEMMs for projections.
K/V pages, scan states and convolution inputs live in `HybridCache`; the
engine's scheduler hands out pages and state slots.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable

import torch
from torch import nn

from ..ops import seqmix as sm
from .hybrid import HybridCache

# a step with at most this many rows runs every expert on every row (static
# shapes, no host round trip); longer steps gather each expert's rows
MOE_STATIC_ROWS = 16


# ------------------------------------------------------------------ specs
@dataclass
class SelectiveSSMSpec:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass
class SigmoidAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_rows: int = 0          # rows of the distance-bias table (0: none)
    bias_max: float = 0.0       # distance at which the last row is reached
    temp_coef: float = 0.0
    temp_every: int = 0         # 0: no query temperature
    v_mix: bool = False


@dataclass
class GluSpec:
    ff: int
    act: str = "relu"
    bias: bool = True


@dataclass
class RoutedSpec:
    experts: int
    top: int
    ff: int
    scale: float = 1.0
    groups: int = 0             # 0: no group limit
    keep: int = 0
    shared_ff: int = 0          # 0: no shared expert
    act: str = "silu"           # "clamped": bounded unit, see ops.glu
    limit: float = 0.0          # bound of the "clamped" unit
    score: str = "sigmoid"      # or "softmax" over all experts
    renorm: bool = True         # weights divided by the chosen scores' sum


@dataclass
class ZLayerSpec:
    kind: str                                   # "mamba1" | "attention"
    mixer: SelectiveSSMSpec | SigmoidAttnSpec
    mlp: GluSpec | RoutedSpec | None = None


@dataclass
class ZudisunConfig:
    name: str = "zudisun"
    vocab_size: int = 512
    width: int = 256
    layers: list = field(default_factory=list)
    eps: float = 1e-6
    max_position: int = 8192    # serving limit (block-table width)

    architecture = "Zudisun"
    # engine-facing traits
    stateful = True
    num_kv_heads = 1
    sliding_window = 0

    @property
    def num_experts(self) -> int:
        return max([ls.mlp.experts for ls in self.layers
                    if isinstance(ls.mlp, RoutedSpec)] or [1])

    def build_model(self, device="cpu", dtype=torch.bfloat16):
        return ZudisunForCausalLM(self, device=device, dtype=dtype)

    def cache_layout(self) -> list:
        """What every layer keeps between steps (HybridCache)."""
        out = []
        for ls in self.layers:
            m = ls.mixer
            if ls.kind == "mamba1":
                out.append({"kv": None, "state": {
                    "ssm": ((m.inner, m.state), "f32"),
                    "conv": ((max(m.conv - 1, 1), m.inner), "model")}})
            else:
                out.append({"kv": (m.kv_heads, m.dim, m.vdim), "state": {}})
        return out

    @staticmethod
    def from_json(c: dict, shape_of: Callable[[str], tuple] | None = None,
                  name: str = "zudisun") -> "ZudisunConfig":
        """Read a checkpoint's config.json.  The number of distance-bias rows
        is a tensor's shape (shape_of(name)); without tensors it is read from
        the mixer's "bias_rows"."""
        layers = []
        for i, lc in enumerate(c["layers"]):
            m = lc["mixer"]
            if lc["type"] == "mamba1":
                mixer = SelectiveSSMSpec(
                    inner=int(m["inner"]), state=int(m["state"]),
                    dt_rank=int(m["dt_rank"]), conv=int(m["conv"]))
            elif lc["type"] == "attention":
                qt = m.get("q_temp") or {}
                rows = (shape_of(f"l{i}.mix.rel")[0] if shape_of is not None
                        else int(m.get("bias_rows", 32)))
                mixer = SigmoidAttnSpec(
                    heads=int(m["heads"]),
                    kv_heads=int(m.get("kv_heads", m["heads"])),
                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                    scale=float(m["scale"]), bias_rows=int(rows),
                    bias_max=float(m["bias_max"]),
                    temp_coef=float(qt.get("coef", 0.0)),
                    temp_every=int(qt.get("every", 0)),
                    v_mix=bool(m.get("v_mix", False)))
            else:
                raise ValueError(f"layer {i}: unknown type {lc['type']}")
            mlp = lc.get("mlp")
            if mlp is None:
                ff = None
            elif mlp.get("kind", "dense") == "dense":
                ff = GluSpec(ff=int(mlp["ff"]), act="relu", bias=True)
            elif mlp["kind"] == "moe":
                r = mlp["router"]
                g = r.get("groups") or {}
                ff = RoutedSpec(
                    experts=int(r["experts"]), top=int(r["top"]),
                    ff=int(mlp["expert"]["ff"]),
                    scale=float(r.get("scale", 1.0)),
                    groups=int(g.get("count", 0)), keep=int(g.get("keep", 0)),
                    shared_ff=int((mlp.get("shared") or {}).get("ff", 0)))
            else:
                raise ValueError(f"layer {i}: unknown mlp kind {mlp['kind']}")
            layers.append(ZLayerSpec(kind=lc["type"], mixer=mixer, mlp=ff))
        return ZudisunConfig(name=name, vocab_size=int(c["vocab"]),
                             width=int(c["width"]), layers=layers,
                             eps=float(c["norm"]["eps"]))

    def to_json(self) -> dict:
        layers = []
        for ls in self.layers:
            m = ls.mixer
            if ls.kind == "mamba1":
                mixer = {"conv": m.conv, "dt_rank": m.dt_rank,
                         "inner": m.inner, "state": m.state}
            else:
                mixer = {"bias_max": m.bias_max, "bias_rows": m.bias_rows,
                         "dim": m.dim, "heads": m.heads,
                         "kv_heads": m.kv_heads, "scale": m.scale,
                         "v_mix": m.v_mix, "vdim": m.vdim}
                if m.temp_every > 0:
                    mixer["q_temp"] = {"coef": m.temp_coef,
                                       "every": m.temp_every}
            f = ls.mlp
            if f is None:
                mlp = None
            elif isinstance(f, GluSpec):
                mlp = {"ff": f.ff, "kind": "dense"}
            else:
                router = {"experts": f.experts, "scale": f.scale, "top": f.top}
                if f.groups > 0:
                    router["groups"] = {"count": f.groups, "keep": f.keep}
                mlp = {"expert": {"ff": f.ff}, "kind": "moe", "router": router}
                if f.shared_ff > 0:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"mixer": mixer, "mlp": mlp, "type": ls.kind})
        return {"architecture": self.architecture, "layers": layers,
                "norm": {"eps": self.eps}, "vocab": self.vocab_size,
                "width": self.width}


def _f32(*shape):
    return torch.zeros(*shape, dtype=torch.float32)


# ----------------------------------------------------------------- mixers
class SelectiveSSM(nn.Module):
    """Mamba-1 mixer.  [x | z] = W_in h; x <- silu(conv(x)); [dt | B | C] =
    W_x x; step = softplus(W_dt dt + b); the scan (ops.selective_scan) with
    A = -exp(A_log) and skip D; times silu(z); W_o."""

    def __init__(self, spec: SelectiveSSMSpec, width: int):
        super().__init__()
        s = self.spec = spec
        self.w_in = nn.Parameter(torch.empty(2 * s.inner, width))
        self.conv = nn.Parameter(torch.empty(s.conv, s.inner))  # tap-major
        self.conv_b = nn.Parameter(torch.empty(s.inner))
        self.w_x = nn.Parameter(torch.empty(s.dt_rank + 2 * s.state, s.inner))
        self.w_dt = nn.Parameter(torch.empty(s.inner, s.dt_rank))
        self.dt_b = nn.Parameter(torch.empty(s.inner))
        self.register_buffer("A", _f32(s.inner, s.state))   # -exp(A_log)
        self.register_buffer("D", _f32(s.inner))
        self.o = nn.Parameter(torch.empty(width, s.inner))

    def forward(self, h, cache: HybridCache, run: int, md, positions, ctx):
        s = self.spec
        xz = sm.matmul(h, self.w_in)
        x = sm.causal_conv(xz[:, :s.inner], self.conv, self.conv_b,
                           cache.state["conv"][run], md, silu=True)
        low = sm.matmul(x, self.w_x)
        dt = sm.matmul(low[:, :s.dt_rank], self.w_dt)
        y = sm.selective_scan(x, dt, self.dt_b, low[:, s.dt_rank:], s.state,
                              xz[:, s.inner:], self.A, self.D,
                              cache.state["ssm"][run], md)
        return sm.matmul(y, self.o)


class SigmoidAttention(nn.Module):
    """Sigmoid attention with grouped K/V heads (ops.qk_unit_cache +
    ops.sigmoid_attention).  q | k | v | gate logits come from one GEMM."""

    def __init__(self, spec: SigmoidAttnSpec, width: int, eps: float):
        super().__init__()
        s = self.spec = spec
        self.eps = eps
        self.nq, self.nk, self.nv = (s.heads * s.dim, s.kv_heads * s.dim,
                                     s.kv_heads * s.vdim)
        rows = self.nq + self.nk + self.nv + s.heads
        self.w_in = nn.Parameter(torch.empty(rows + (-rows) % 8, width))
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))
        self.register_buffer("rel", _f32(max(s.bias_rows, 1), s.heads))
        self.register_buffer("talk", _f32(s.heads, s.heads))
        self.register_buffer("head_bias", _f32(s.heads))
        self.register_buffer(
            "buckets", sm.distance_buckets(s.bias_rows, s.bias_max)
            if s.bias_rows > 0 else torch.zeros(1, dtype=torch.int32))
        self.lam = 0.0          # weight of the first mixing layer's values

    def forward(self, h, cache: HybridCache, run: int, md, positions, ctx):
        s = self.spec
        p = sm.matmul(h, self.w_in)
        a, b, c = self.nq, self.nq + self.nk, self.nq + self.nk + self.nv
        q, k, v, g = p[:, :a], p[:, a:b], p[:, b:c], p[:, c:c + s.heads]
        v_first = ctx.get("v_first") if s.v_mix else None
        qn = sm.qk_unit_cache(q, k, v, s.heads, s.kv_heads, self.eps,
                              cache.k[run], cache.v[run], md.slots, positions,
                              s.temp_coef, s.temp_every, v_first, self.lam)
        if s.v_mix and v_first is None:
            ctx["v_first"] = v
        o = sm.sigmoid_attention(
            qn, cache.k[run], cache.v[run], md, positions, s.scale, s.heads,
            rel=self.rel if s.bias_rows > 0 else None,
            buckets=self.buckets if s.bias_rows > 0 else None,
            talk=self.talk, head_bias=self.head_bias, gate=g)
        return sm.matmul(o, self.o)


# ------------------------------------------------------------ feed-forward
class GluMLP(nn.Module):
    """W_down (act(W_gate h + b) * (W_up h + b)) (+ b): gate and up share one
    GEMM; the down bias is handed to the caller's output norm."""

    def __init__(self, spec: GluSpec, width: int):
        super().__init__()
        self.spec = spec
        self.gate_up = nn.Parameter(torch.empty(2 * spec.ff, width))
        self.down = nn.Parameter(torch.empty(width, spec.ff))
        if spec.bias:
            self.gate_up_b = nn.Parameter(torch.empty(2 * spec.ff))
            self.down_b = nn.Parameter(torch.empty(width))
        else:
            self.gate_up_b = self.down_b = None

    def forward(self, h, md):
        s = self.spec
        a = sm.glu(sm.matmul(h, self.gate_up), s.ff, s.act, self.gate_up_b)
        return sm.matmul(a, self.down), self.down_b


class RoutedExperts(nn.Module):
    """Mixture of gated experts behind a sigmoid or softmax router
    (ops.moe_route) with an optional shared expert.  All gate/up weights sit in one matrix
    [E*2F + 2Fs, W] (expert e: rows e*2F.., gate then up; shared last), all
    down weights in one [W, E*F + Fs].

    Short steps (decode; graph-capturable) run every expert on every row:
    one gate/up GEMM, the gated unit scaled by the router weight (zero for
    experts not chosen), one down GEMM whose K axis sums experts and shared
    expert.  Longer steps sort (row, choice) pairs by expert, run each expert
    on its rows and combine in fp32 in a fixed order."""

    def __init__(self, spec: RoutedSpec, width: int):
        super().__init__()
        s = self.spec = spec
        self.register_buffer("router", _f32(s.experts, width))
        self.register_buffer("correction", _f32(s.experts))
        self.gate_up = nn.Parameter(torch.empty(
            s.experts * 2 * s.ff + 2 * s.shared_ff, width))
        self.down = nn.Parameter(torch.empty(
            width, s.experts * s.ff + s.shared_ff))

    def forward(self, h, md):
        s = self.spec
        E, F, Fs = s.experts, s.ff, s.shared_ff
        T = h.shape[0]
        z = sm.matmul(h.float(), self.router)
        static = (not md.is_prefill) or T <= MOE_STATIC_ROWS
        idx, wts, wd = sm.moe_route(z, self.correction, s.top, s.groups,
                                    s.keep, s.scale, dense=static,
                                    score=s.score, renorm=s.renorm)
        if static:
            gu = sm.matmul(h, self.gate_up)
            act = torch.empty(T, E * F + Fs, dtype=h.dtype, device=h.device)
            sm.glu(gu, F, s.act, units=E, row_weight=wd, out=act,
                   limit=s.limit)
            if Fs > 0:
                sm.glu(gu[:, E * 2 * F:], Fs, s.act, out=act[:, E * F:],
                       limit=s.limit)
            return sm.matmul(act, self.down), None
        # (row, choice) pairs in expert order; one host round trip for sizes
        flat = idx.flatten().long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=E).tolist()
        pos = torch.empty_like(order, dtype=torch.int32)
        pos[order] = torch.arange(order.numel(), dtype=torch.int32,
                                  device=h.device)
        xs = h.index_select(0, torch.div(order, s.top, rounding_mode="floor"))
        ys = torch.empty(T * s.top, h.shape[1], dtype=h.dtype, device=h.device)
        o = 0
        for e, n in enumerate(counts):
            if n == 0:
                continue
            a = sm.glu(sm.matmul(xs[o:o + n],
                                 self.gate_up[e * 2 * F:(e + 1) * 2 * F]),
                       F, s.act, limit=s.limit)
            ys[o:o + n] = sm.matmul(a, self.down[:, e * F:(e + 1) * F])
            o += n
        shared = None
        if Fs > 0:
            a = sm.glu(sm.matmul(h, self.gate_up[E * 2 * F:]), Fs, s.act,
                       limit=s.limit)
            shared = sm.matmul(a, self.down[:, E * F:])
        return sm.moe_combine(ys, pos, wts, shared), None


# ------------------------------------------------------------------- layer
class ZudisunLayer(nn.Module):
    def __init__(self, cfg: ZudisunConfig, spec: ZLayerSpec):
        super().__init__()
        W = cfg.width
        self.spec, self.eps = spec, cfg.eps
        self.norm1 = nn.Parameter(torch.empty(W))
        if spec.kind == "mamba1":
            self.mixer = SelectiveSSM(spec.mixer, W)
        else:
            self.mixer = SigmoidAttention(spec.mixer, W, cfg.eps)
        if spec.mlp is None:
            self.mlp = self.norm2 = None
        else:
            self.norm2 = nn.Parameter(torch.empty(W))
            self.mlp = (GluMLP(spec.mlp, W) if isinstance(spec.mlp, GluSpec)
                        else RoutedExperts(spec.mlp, W))

    def forward(self, x, h, cache, run, md, positions, ctx):
        """x: fp32 residual (updated in place); h: x in the model dtype.
        Returns the new h."""
        dt = self.norm1.dtype
        y = self.mixer(h, cache, run, md, positions, ctx)
        h = sm.norm_residual(x, y, None, self.norm1, self.eps, dt)
        if self.mlp is not None:
            y, bias = self.mlp(h, md)
            h = sm.norm_residual(x, y, bias, self.norm2, self.eps, dt)
        return h


class ZudisunForCausalLM(nn.Module):
    # the engine asks these before wiring a model in
    needs_state_slots = True
    supports_speculation = False    # rejected drafts would need state rollback
    supports_prefix_cache = False   # scan state is not page-addressable

    def __init__(self, cfg: ZudisunConfig, device="cpu",
                 dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        first_mix = None
        for ls in cfg.layers:
            if ls.kind == "attention" and ls.mixer.v_mix:
                m = ls.mixer
                if first_mix is None:
                    first_mix = m
                elif (m.kv_heads, m.vdim) != (first_mix.kv_heads,
                                              first_mix.vdim):
                    raise ValueError("value mixing needs equal kv_heads and "
                                     "vdim in every mixing layer")
        with torch.device(device):
            self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
            self.layers = nn.ModuleList(
                [ZudisunLayer(cfg, ls) for ls in cfg.layers])
            self.final_norm = nn.Parameter(torch.empty(cfg.width))
            self.head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
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
        dt = self.embed.dtype
        x = sm.embed_rows(ids, self.embed)
        h = sm.cast_rows(x, dt)
        ctx: dict = {}
        for run, layer in enumerate(self.layers):
            h = layer(x, h, cache, run, md, positions, ctx)
            if self.record_runs is not None:
                self.record_runs.append(x.clone())
        hn = sm.norm_rows(x, self.final_norm, self.cfg.eps, logit_rows, dt,
                          one_plus=False)
        return sm.matmul(hn, self.head, skinny=False).float()

    # -- weights ------------------------------------------------------------
    @torch.no_grad()
    def load_tensors(self, get: Callable[[str], torch.Tensor]):
        """Fill parameters from checkpoint tensors by name: 'embed', 'head',
        'final.norm', and per layer i 'l<i>.norm1|norm2', 'l<i>.mix.<...>',
        'l<i>.mlp.<...>' (experts 'e<k>.', shared expert 'shared.')."""
        def put(dst, src):
            dst.copy_(src.to(dst.device, dst.dtype))

        def rows(dst, parts):
            t = torch.cat(parts, 0)
            if t.shape[0] < dst.shape[0]:
                t = torch.cat([t, t.new_zeros(dst.shape[0] - t.shape[0],
                                              t.shape[1])], 0)
            put(dst, t)
        put(self.embed, get("embed"))
        put(self.head, get("head"))
        put(self.final_norm, get("final.norm"))
        for i, L in enumerate(self.layers):
            pre, mp = f"l{i}.", f"l{i}.mix."
            put(L.norm1, get(pre + "norm1"))
            m = L.mixer
            if isinstance(m, SelectiveSSM):
                put(m.w_in, get(mp + "in"))
                put(m.conv, get(mp + "conv").t().contiguous())
                put(m.conv_b, get(mp + "conv.b"))
                put(m.w_x, get(mp + "x"))
                put(m.w_dt, get(mp + "dt"))
                put(m.dt_b, get(mp + "dt.b"))
                put(m.A, -torch.exp(get(mp + "A_log").float()))
                put(m.D, get(mp + "D"))
                put(m.o, get(mp + "o"))
            else:
                rows(m.w_in, [get(mp + "q"), get(mp + "k"), get(mp + "v"),
                              get(mp + "g")])
                put(m.o, get(mp + "o"))
                if m.spec.bias_rows > 0:
                    put(m.rel, get(mp + "rel"))
                put(m.talk, get(mp + "talk"))
                put(m.head_bias, get(mp + "pb"))
                if m.spec.v_mix:
                    m.lam = float(get(mp + "vmix").float())
            f = L.mlp
            if f is None:
                continue
            fp = pre + "mlp."
            put(L.norm2, get(pre + "norm2"))
            if isinstance(f, GluMLP):
                rows(f.gate_up, [get(fp + "gate"), get(fp + "up")])
                put(f.down, get(fp + "down"))
                if f.spec.bias:
                    put(f.gate_up_b, torch.cat([get(fp + "gate.b"),
                                                get(fp + "up.b")]))
                    put(f.down_b, get(fp + "down.b"))
            else:
                s = f.spec
                units = [f"e{e}." for e in range(s.experts)] + \
                    (["shared."] if s.shared_ff > 0 else [])
                rows(f.gate_up, [get(fp + u + n) for u in units
                                 for n in ("gate", "up")])
                put(f.down, torch.cat([get(fp + u + "down") for u in units],
                                      1))
                put(f.router, get(fp + "router"))
                put(f.correction, get(fp + "correction"))
        return self

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        """Random weights at scales that keep activations O(1) through depth
        (benchmarks and smoke runs; not a trained model)."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(t, std):
            t.copy_((torch.randn(t.shape, generator=g) * std).to(t.dtype))
        for name, p in list(self.named_parameters()) + \
                list(self.named_buffers()):
            leaf = name.rsplit(".", 1)[-1]
            if leaf == "buckets":
                continue
            if leaf == "A":
                n = p.shape[1]
                p.copy_(-torch.arange(1, n + 1, dtype=torch.float32)
                        .expand(p.shape[0], n))
            elif leaf == "D":
                p.fill_(1.0)
            elif leaf == "dt_b":
                # softplus^-1 of step sizes spread over [1e-3, 1e-1]
                d = torch.exp(torch.rand(p.shape, generator=g)
                              * (math.log(0.1) - math.log(1e-3))
                              + math.log(1e-3))
                p.copy_((d + torch.log(-torch.expm1(-d))).to(p.dtype))
            elif leaf == "talk":
                p.copy_(torch.eye(p.shape[0]) +
                        0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "head_bias":
                p.fill_(-3.0)
            elif leaf in ("rel", "correction"):
                rnd(p, 0.1)
            elif "norm" in leaf:
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g))
                        .to(p.dtype))
            elif p.dim() == 1:
                rnd(p, 0.1)
            elif leaf == "embed":
                rnd(p, 1.0)
            elif leaf == "conv":
                rnd(p, p.shape[0] ** -0.5)
            else:
                rnd(p, p.shape[1] ** -0.5)
        for L in self.layers:
            if isinstance(L.mixer, SigmoidAttention) and L.mixer.spec.v_mix:
                L.mixer.lam = 0.3
        return self


# ------------------------------------------------------ checkpoint reading
def load_zudisun(path: str, device="cpu", dtype=torch.bfloat16,
                 max_position: int | None = None) -> ZudisunForCausalLM:
    """config.json + *.safetensors -> model on `device` in `dtype`."""
    from safetensors import safe_open
    root = Path(path)
    c = json.loads((root / "config.json").read_text())
    files = sorted(root.glob("*.safetensors"))
    handles = [safe_open(str(f), framework="pt") for f in files]
    where = {k: h for h in handles for k in h.keys()}

    def shape_of(name):
        return tuple(where[name].get_slice(name).get_shape())

    def get(name):
        return where[name].get_tensor(name)
    cfg = ZudisunConfig.from_json(c, shape_of, name=root.name)
    if max_position is not None:
        cfg.max_position = max_position
    model = ZudisunForCausalLM(cfg, device=device, dtype=dtype)
    return model.load_tensors(get).eval()


def save_zudisun(tensors: dict, cfg: ZudisunConfig, path: str) -> None:
    """Write checkpoint-named tensors + config.json (tests, tooling)."""
    from safetensors.torch import save_file
    root = Path(path)
    root.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              str(root / "model.safetensors"))
    (root / "config.json").write_text(json.dumps(cfg.to_json(), indent=1))


def _bench_config(name, width, ff, n_layers, heads, kv_heads, dim,
                  vocab=32000, experts=0, top=2, expert_ff=0, shared_ff=0,
                  state=16, moe_every=0):
    """Alternating mamba1 / attention layers; dense feed-forward everywhere,
    or a mixture in every `moe_every`-th layer."""
    layers = []
    for i in range(n_layers):
        if i % 2 == 0:
            kind, mixer = "mamba1", SelectiveSSMSpec(
                inner=2 * width, state=state,
                dt_rank=max(1, width // 16), conv=4)
        else:
            kind, mixer = "attention", SigmoidAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                scale=dim ** -0.5, bias_rows=32, bias_max=128.0,
                temp_coef=0.1, temp_every=256, v_mix=True)
        if experts > 0 and moe_every > 0 and i % moe_every == moe_every - 1:
            mlp = RoutedSpec(experts=experts, top=top, ff=expert_ff,
                             scale=1.0, groups=4, keep=2, shared_ff=shared_ff)
        else:
            mlp = GluSpec(ff=ff)
        layers.append(ZLayerSpec(kind=kind, mixer=mixer, mlp=mlp))
    return ZudisunConfig(name=name, vocab_size=vocab, width=width,
                         layers=layers, eps=1e-6)


ZUDISUN_CONFIGS = {
    # a small model with every branch, for smoke runs and CPU tests
    "zudisun-tiny": _bench_config("zudisun-tiny", 128, 320, 4, 4, 2, 32,
                                  vocab=384, experts=8, top=2, expert_ff=64,
                                  shared_ff=96, state=8, moe_every=2),
    # same width / ff / depth / heads as "reperax-1b" and "debug-1b"
    "zudisun-1b": _bench_config("zudisun-1b", 2048, 8192, 16, 16, 8, 128),
    # same, with a mixture (16 experts of ff 2048, top 4 ~ the dense ff's
    # FLOPs with the shared expert) in every second layer
    "zudisun-1b-moe": _bench_config("zudisun-1b-moe", 2048, 8192, 16, 16, 8,
                                    128, experts=16, top=3, expert_ff=2048,
                                    shared_ff=2048, moe_every=2),
    # same width / ff / depth / heads / vocabulary as "llama-3-8b"
    "zudisun-8b": _bench_config("zudisun-8b", 4096, 14336, 32, 32, 8, 128,
                                vocab=128256),
}
