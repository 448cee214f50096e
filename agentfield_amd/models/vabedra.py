"""Delta-rule decoders with the norm after the residual sum: the Vabedra design.

A Vabedra model is a stack of layers `x <- norm1(alpha x + mixer(x))`, `x <-
norm2(alpha x + ff(x))`: the sublayers read the fp32 residual itself and a
plain-weight RMSNorm sits after each sum.  After the feed-forward every
layer adds a per-token side input: a slice of a second embedding table,
gated by gelu(W x), projected to the model width and RMS-normed.  config.json
lists the layers; each names its mixer:

  * ``delta``    — gated delta rule: q / k / v through short causal
    convolutions and SiLU, unit-length q and k, one decay per head, a sigmoid
    write strength, an fp32 state [dim, vdim] per head and sequence, per-head
    RMSNorm and a SiLU output gate
  * ``parallel`` — two mixers on the same input, each RMS-normed over the
    model width, averaged: sliding-window softmax attention that keeps the
    first tokens visible (projection biases, per-head q/k norm, partial
    rotate-half rotary positions with wavelength-scaled frequencies, soft-
    capped scores, a unit sink in the softmax denominator) beside a delta
    rule whose decay is per key channel (low-rank projection) and whose
    output gate is a low-rank sigmoid

The feed-forward is a mixture of bounded gated units behind a softmax router
with score correction (models/zudisun.py: RoutedExperts).

Every mechanism is a module parameterised by its spec on the sequence-mixer
op set (ops/seqmix.py): gfx950 kernels on GPU, vendor GEMMs for projections.
K/V pages, delta-rule states and convolution inputs live in `HybridCache`;
the engine's scheduler hands out pages and state slots.
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
from .zudisun import RoutedExperts, RoutedSpec


# ------------------------------------------------------------------ specs
@dataclass
class DeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    rank: int = 0           # 0: one decay per head and a full-rank SiLU gate;
                            # > 0: per-key-channel decay and sigmoid gate,
                            # both through projections of this rank
    gate_rank: int = 0


@dataclass
class SinkAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    window: int = 0         # 0: every earlier key
    keep_first: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: dict | None = None


@dataclass
class VLayerSpec:
    kind: str                               # "delta" | "parallel"
    delta: DeltaSpec                        # the mixer, or the right branch
    attn: SinkAttnSpec | None = None        # parallel: the left branch
    mlp: RoutedSpec | None = None


@dataclass
class VabedraConfig:
    name: str = "vabedra"
    vocab_size: int = 512
    width: int = 256
    layers: list = field(default_factory=list)
    eps: float = 1e-6
    alpha: float = 1.0          # residual scale inside the post-sum norm
    embed_scale: float = 1.0
    side_dim: int = 0           # 0: no per-token side input
    max_position: int = 8192    # serving limit (block-table width)

    architecture = "Vabedra"
    # engine-facing traits
    stateful = True
    num_kv_heads = 1
    sliding_window = 0          # the kept first tokens rule out page rolling

    @property
    def num_experts(self) -> int:
        return max([ls.mlp.experts for ls in self.layers
                    if ls.mlp is not None] or [1])

    def build_model(self, device="cpu", dtype=torch.bfloat16):
        return VabedraForCausalLM(self, device=device, dtype=dtype)

    def cache_layout(self) -> list:
        """What every layer keeps between steps (HybridCache)."""
        out = []
        for ls in self.layers:
            d = ls.delta
            need = {"kv": None, "state": {
                "rec": ((d.heads, d.dim, d.vdim), "f32"),
                "conv": ((max(d.conv - 1, 1),
                          2 * d.kv_heads * d.dim + d.heads * d.vdim),
                         "model")}}
            if ls.kind == "parallel":
                a = ls.attn
                need["kv"] = (a.kv_heads, a.dim, a.vdim)
            out.append(need)
        return out

    @staticmethod
    def from_json(c: dict, shape_of: Callable[[str], tuple] | None = None,
                  name: str = "vabedra") -> "VabedraConfig":
        """Read a checkpoint's config.json.  The ranks of the low-rank decay
        and gate projections are tensor shapes (shape_of(name)); without
        tensors they are read from the mixer's "rank" / "gate_rank"."""
        def delta(m, pre, low_rank):
            rank = gate_rank = 0
            if low_rank:
                rank = (shape_of(pre + "a1")[0] if shape_of is not None
                        else int(m.get("rank", 16)))
                gate_rank = (shape_of(pre + "g1")[0] if shape_of is not None
                             else int(m.get("gate_rank", rank)))
            return DeltaSpec(heads=int(m["heads"]),
                             kv_heads=int(m.get("kv_heads", m["heads"])),
                             dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                             conv=int(m["conv"]), rank=rank,
                             gate_rank=gate_rank)
        layers = []
        for i, lc in enumerate(c["layers"]):
            m = lc["mixer"]
            attn = None
            if lc["type"] == "delta":
                d = delta(m, f"l{i}.mix.", False)
            elif lc["type"] == "parallel":
                le = m["left"]
                mask = le.get("mask") or {}
                rot = le.get("rot") or {}
                attn = SinkAttnSpec(
                    heads=int(le["heads"]),
                    kv_heads=int(le.get("kv_heads", le["heads"])),
                    dim=int(le["dim"]), vdim=int(le.get("vdim", le["dim"])),
                    scale=float(le["scale"]),
                    softcap=float(le.get("softcap") or 0.0),
                    window=int(mask.get("size", 0)),
                    keep_first=int(mask.get("keep_first", 0)),
                    rot_dims=int(rot.get("dims", 0)),
                    rot_base=float(rot.get("base", 10000.0)),
                    rot_scaling=dict(rot["scaling"])
                    if rot.get("scaling") else None)
                d = delta(m["right"], f"l{i}.mix.right.", True)
            else:
                raise ValueError(f"layer {i}: unknown type {lc['type']}")
            mlp = lc.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(
                        f"layer {i}: unknown mlp kind {mlp['kind']}")
                ff = RoutedSpec(
                    experts=int(mlp["router"]["experts"]),
                    top=int(mlp["router"]["top"]),
                    ff=int(mlp["expert"]["ff"]), act="clamped",
                    limit=float(mlp["expert"]["limit"]), score="softmax",
                    renorm=False)
            layers.append(VLayerSpec(kind=lc["type"], delta=d, attn=attn,
                                     mlp=ff))
        return VabedraConfig(
            name=name, vocab_size=int(c["vocab"]), width=int(c["width"]),
            layers=layers, eps=float(c["norm"]["eps"]),
            alpha=float(c.get("postln_alpha", 1.0)),
            embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
            side_dim=int((c.get("token_side") or {}).get("dim", 0)))

    def to_json(self) -> dict:
        def delta(d, low_rank):
            m = {"conv": d.conv, "dim": d.dim, "heads": d.heads,
                 "kv_heads": d.kv_heads, "vdim": d.vdim}
            if low_rank:
                m["rank"], m["gate_rank"] = d.rank, d.gate_rank
            return m
        layers = []
        for ls in self.layers:
            if ls.kind == "delta":
                mixer = delta(ls.delta, False)
            else:
                a = ls.attn
                left = {"dim": a.dim, "heads": a.heads,
                        "kv_heads": a.kv_heads, "scale": a.scale,
                        "vdim": a.vdim}
                if a.window > 0 or a.keep_first > 0:
                    left["mask"] = {"keep_first": a.keep_first,
                                    "size": a.window}
                if a.softcap > 0:
                    left["softcap"] = a.softcap
                if a.rot_dims > 0:
                    left["rot"] = {"base": a.rot_base, "dims": a.rot_dims}
                    if a.rot_scaling:
                        left["rot"]["scaling"] = dict(a.rot_scaling)
                mixer = {"left": left, "right": delta(ls.delta, True)}
            f = ls.mlp
            mlp = None if f is None else {
                "expert": {"ff": f.ff, "limit": f.limit}, "kind": "moe",
                "router": {"experts": f.experts, "top": f.top}}
            layers.append({"mixer": mixer, "mlp": mlp, "type": ls.kind})
        out = {"architecture": self.architecture,
               "embedding": {"scale": self.embed_scale}, "layers": layers,
               "norm": {"eps": self.eps}, "postln_alpha": self.alpha,
               "vocab": self.vocab_size, "width": self.width}
        if self.side_dim > 0:
            out["token_side"] = {"dim": self.side_dim}
        return out


def _f32(*shape):
    return torch.zeros(*shape, dtype=torch.float32)


def _pad8(n):
    return n + (-n) % 8


# ----------------------------------------------------------------- mixers
class GatedDeltaRule(nn.Module):
    """q | k | v (then convolution + SiLU), the write-strength logits, the
    decay logits (or their low-rank input) and the gate logits (or their
    low-rank input) come from one GEMM over the mixer's input; the caller
    may put that GEMM's rows into a larger fused one (in_rows / forward's
    `p`).  ops.delta_scan evaluates unit norms, decays and the recurrence."""

    def __init__(self, spec: DeltaSpec, width: int, eps: float):
        super().__init__()
        s = self.spec = spec
        self.eps = eps
        self.nqk, self.nv = s.kv_heads * s.dim, s.heads * s.vdim
        self.nconv = 2 * self.nqk + self.nv
        self.conv = nn.Parameter(torch.empty(s.conv, self.nconv))  # tap-major
        self.register_buffer("rate", _f32(s.heads))     # exp(A_log)
        self.norm = nn.Parameter(torch.empty(s.vdim))
        if s.rank > 0:
            self.a2 = nn.Parameter(torch.empty(s.heads * s.dim, s.rank))
            self.g2 = nn.Parameter(torch.empty(self.nv, s.gate_rank))
            self.register_buffer("dt_bias", _f32(s.heads * s.dim))
        else:
            self.register_buffer("dt_bias", _f32(s.heads))
        self.o = nn.Parameter(torch.empty(width, self.nv))

    def in_blocks(self):
        """(checkpoint tensor, rows) of this mixer's input projection, in
        the order forward() slices them."""
        s = self.spec
        out = [("q", self.nqk), ("k", self.nqk), ("v", self.nv),
               ("b", s.heads)]
        if s.rank > 0:
            return out + [("a1", s.rank), ("g1", s.gate_rank)]
        return out + [("a", s.heads), ("g", self.nv)]

    def in_rows(self) -> int:
        return sum(r for _n, r in self.in_blocks())

    def forward(self, p, cache: HybridCache, run: int, md):
        s = self.spec
        c0 = self.nconv
        qkv = sm.causal_conv(p[:, :c0], self.conv, None,
                             cache.state["conv"][run], md, silu=True)
        beta = p[:, c0:c0 + s.heads]
        c1 = c0 + s.heads
        if s.rank > 0:
            decay = sm.matmul(p[:, c1:c1 + s.rank], self.a2)
            gate = sm.matmul(p[:, c1 + s.rank:c1 + s.rank + s.gate_rank],
                             self.g2)
        else:
            decay = p[:, c1:c1 + s.heads]
            gate = p[:, c1 + s.heads:c1 + s.heads + self.nv]
        o = sm.delta_scan(qkv[:, :self.nqk], qkv[:, self.nqk:2 * self.nqk],
                          qkv[:, 2 * self.nqk:], beta, decay, self.dt_bias,
                          self.rate, cache.rec[run], md, s.heads, s.kv_heads,
                          q_scale=s.dim ** -0.5)
        y = sm.headnorm_gate(o, gate, self.norm, self.eps, s.heads,
                             self.o.dtype,
                             gate_act="sigmoid" if s.rank > 0 else "silu")
        return sm.matmul(y, self.o)


class SinkWindowAttention(nn.Module):
    """Grouped-query softmax attention over a sliding window that keeps the
    first tokens: biases, per-head q/k RMSNorm and rotary positions in
    ops.qk_rope_cache, then ops.masked_attention with soft cap, window,
    kept first keys and a sink of score 0."""

    def __init__(self, spec: SinkAttnSpec, width: int, eps: float):
        super().__init__()
        s = self.spec = spec
        self.eps = eps
        self.nq, self.nk, self.nv = (s.heads * s.dim, s.kv_heads * s.dim,
                                     s.kv_heads * s.vdim)
        self.bias = nn.Parameter(torch.empty(self.nq + self.nk + self.nv))
        self.q_norm = nn.Parameter(torch.empty(s.dim))
        self.k_norm = nn.Parameter(torch.empty(s.dim))
        self.register_buffer("sink", _f32(s.heads))     # score 0: adds 1
        self.register_buffer(
            "inv_freq", sm.scaled_inv_freq(s.rot_dims, s.rot_base,
                                           s.rot_scaling)
            if s.rot_dims > 0 else None)
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))

    def in_blocks(self):
        return [("q", self.nq), ("k", self.nk), ("v", self.nv)]

    def in_rows(self) -> int:
        return self.nq + self.nk + self.nv

    def forward(self, p, cache: HybridCache, run: int, md, positions, ctx):
        s = self.spec
        a, b, c = self.nq, self.nq + self.nk, self.nq + self.nk + self.nv
        tab = None
        if self.inv_freq is not None:
            # layers that rotate alike share the step's cos / sin table
            key = (s.rot_dims, s.rot_base,
                   tuple(sorted((s.rot_scaling or {}).items())))
            tab = ctx.get(key)
            if tab is None:
                tab = ctx[key] = sm.rotary_table(positions, self.inv_freq)
        q = sm.qk_rope_cache(
            p[:, :a], p[:, a:b], p[:, b:c], s.heads, s.kv_heads, self.eps,
            cache.k[run], cache.v[run], md.slots, positions,
            q_bias=self.bias[:a], k_bias=self.bias[a:b],
            v_bias=self.bias[b:c], q_norm=self.q_norm, k_norm=self.k_norm,
            rot_tab=tab)
        o = sm.masked_attention(q, cache.k[run], cache.v[run], md, positions,
                                s.scale, s.heads, window=s.window,
                                sink=self.sink, softcap=s.softcap,
                                keep_first=s.keep_first)
        return sm.matmul(o, self.o)


# ------------------------------------------------------------------- layer
class VabedraLayer(nn.Module):
    def __init__(self, cfg: VabedraConfig, spec: VLayerSpec, index: int):
        super().__init__()
        W = cfg.width
        self.spec, self.eps, self.alpha = spec, cfg.eps, cfg.alpha
        self.index, self.side_dim = index, cfg.side_dim
        self.norm1 = nn.Parameter(torch.empty(W))
        self.delta = GatedDeltaRule(spec.delta, W, cfg.eps)
        rows = self.delta.in_rows()
        if spec.kind == "parallel":
            self.attn = SinkWindowAttention(spec.attn, W, cfg.eps)
            rows += self.attn.in_rows()
            self.left_out = nn.Parameter(torch.empty(W))
            self.right_out = nn.Parameter(torch.empty(W))
        else:
            self.attn = None
        # one GEMM feeds every projection that reads the mixer's input:
        # [attention q | k | v] [delta q | k | v | b | decay | gate]
        self.mix_in = nn.Parameter(torch.empty(_pad8(rows), W))
        # a layer without feed-forward still norms alpha x when its
        # checkpoint carries a second norm weight
        self.norm2 = nn.Parameter(torch.ones(W))
        self.use_norm2 = spec.mlp is not None
        self.mlp = RoutedExperts(spec.mlp, W) if spec.mlp is not None else None
        if cfg.side_dim > 0:
            self.side_gate = nn.Parameter(torch.empty(_pad8(cfg.side_dim), W))
            self.side_proj = nn.Parameter(torch.empty(W, cfg.side_dim))
            self.side_norm = nn.Parameter(torch.empty(W))

    def forward(self, x, h, ids, side_table, cache, run, md, positions, ctx):
        """x: fp32 residual (updated in place); h: x in the model dtype.
        Returns the new h."""
        dt = self.norm1.dtype
        p = sm.matmul(h, self.mix_in)
        if self.attn is not None:
            n = self.attn.in_rows()
            left = self.attn(p[:, :n], cache, run, md, positions, ctx)
            right = self.delta(p[:, n:], cache, run, md)
            h = sm.postnorm_sum(x, left, self.alpha, self.norm1, self.eps, dt,
                                y2=right, wy=self.left_out,
                                wy2=self.right_out)
        else:
            y = self.delta(p, cache, run, md)
            h = sm.postnorm_sum(x, y, self.alpha, self.norm1, self.eps, dt)
        if self.mlp is not None:
            y, _bias = self.mlp(h, md)
            h = sm.postnorm_sum(x, y, self.alpha, self.norm2, self.eps, dt)
        elif self.use_norm2:
            h = sm.postnorm_sum(x, torch.zeros_like(h), self.alpha,
                                self.norm2, self.eps, dt)
        if self.side_dim > 0:
            z = sm.matmul(h, self.side_gate)
            g = sm.gate_gather(z[:, :self.side_dim], side_table, ids,
                               self.index * self.side_dim)
            h = sm.norm_residual(x, sm.matmul(g, self.side_proj), None,
                                 self.side_norm, self.eps, dt)
        return h


class VabedraForCausalLM(nn.Module):
    # the engine asks these before wiring a model in
    needs_state_slots = True
    supports_speculation = False    # rejected drafts would need state rollback
    supports_prefix_cache = False   # recurrent state is not page-addressable

    def __init__(self, cfg: VabedraConfig, device="cpu",
                 dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        with torch.device(device):
            self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
            if cfg.side_dim > 0:
                self.side_embed = nn.Parameter(torch.empty(
                    cfg.vocab_size, cfg.side_dim * len(cfg.layers)))
            else:
                self.side_embed = None
            self.layers = nn.ModuleList(
                [VabedraLayer(cfg, ls, i) for i, ls in enumerate(cfg.layers)])
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
        x = sm.embed_rows(ids, self.embed, scale=self.cfg.embed_scale)
        h = sm.cast_rows(x, dt)
        ctx: dict = {}
        for run, layer in enumerate(self.layers):
            h = layer(x, h, ids, self.side_embed, cache, run, md, positions,
                      ctx)
            if self.record_runs is not None:
                self.record_runs.append(x.clone())
        hn = sm.norm_rows(x, self.final_norm, self.cfg.eps, logit_rows, dt,
                          one_plus=False)
        return sm.matmul(hn, self.head, skinny=False).float()

    # -- weights ------------------------------------------------------------
    @torch.no_grad()
    def load_tensors(self, get: Callable[[str], torch.Tensor]):
        """Fill parameters from checkpoint tensors by name: 'embed', 'head',
        'final.norm', 'side.embed', and per layer i 'l<i>.norm1|norm2',
        'l<i>.mix.<...>' (a parallel layer: 'l<i>.mix.left.<...>',
        'l<i>.mix.right.<...>', 'l<i>.mix.left.out|right.out'),
        'l<i>.mlp.e<k>.gate|up|down', 'l<i>.mlp.router|correction',
        'l<i>.side.gate|proj|norm'."""
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
        if self.side_embed is not None:
            put(self.side_embed, get("side.embed"))
        for i, L in enumerate(self.layers):
            pre = f"l{i}."
            put(L.norm1, get(pre + "norm1"))
            d = L.delta
            dp = pre + ("mix.right." if L.attn is not None else "mix.")
            parts = []
            if L.attn is not None:
                a, ap = L.attn, pre + "mix.left."
                parts += [get(ap + n) for n, _r in a.in_blocks()]
                put(a.bias, torch.cat([get(ap + n + ".b")
                                       for n, _r in a.in_blocks()]))
                put(a.q_norm, get(ap + "q.norm"))
                put(a.k_norm, get(ap + "k.norm"))
                put(a.o, get(ap + "o"))
                put(L.left_out, get(pre + "mix.left.out"))
                put(L.right_out, get(pre + "mix.right.out"))
            parts += [get(dp + n) for n, _r in d.in_blocks()]
            rows(L.mix_in, parts)
            put(d.conv, torch.cat([get(dp + n + ".conv")
                                   for n in ("q", "k", "v")], 0)
                .t().contiguous())
            put(d.rate, torch.exp(get(dp + "A_log").float()))
            put(d.norm, get(dp + "norm"))
            put(d.dt_bias, get(dp + "dt_bias"))
            if d.spec.rank > 0:
                put(d.a2, get(dp + "a2"))
                put(d.g2, get(dp + "g2"))
            put(d.o, get(dp + "o"))
            f = L.mlp
            if f is None:
                try:
                    put(L.norm2, get(pre + "norm2"))
                    L.use_norm2 = True
                except KeyError:
                    L.use_norm2 = False
            else:
                fp = pre + "mlp."
                put(L.norm2, get(pre + "norm2"))
                units = [f"e{e}." for e in range(f.spec.experts)]
                rows(f.gate_up, [get(fp + u + n) for u in units
                                 for n in ("gate", "up")])
                put(f.down, torch.cat([get(fp + u + "down") for u in units],
                                      1))
                put(f.router, get(fp + "router"))
                put(f.correction, get(fp + "correction"))
            if L.side_dim > 0:
                rows(L.side_gate, [get(pre + "side.gate")])
                put(L.side_proj, get(pre + "side.proj"))
                put(L.side_norm, get(pre + "side.norm"))
        return self

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        """Random weights at scales that keep activations O(1) through depth
        (benchmarks and smoke runs; not a trained model)."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(t, std, mean=0.0):
            t.copy_((torch.randn(t.shape, generator=g) * std + mean)
                    .to(t.dtype))
        for name, p in list(self.named_parameters()) + \
                list(self.named_buffers()):
            leaf = name.rsplit(".", 1)[-1]
            if p is None or leaf in ("inv_freq", "sink"):
                continue
            if leaf == "rate":
                p.copy_(torch.exp(torch.randn(p.shape, generator=g) * 0.5
                                  - 1.0))
            elif leaf == "dt_bias":
                rnd(p, 1.0)
            elif leaf == "correction":
                rnd(p, 0.02)
            elif "norm" in leaf or leaf in ("left_out", "right_out"):
                rnd(p, 0.1, 1.0)
            elif p.dim() == 1:
                rnd(p, 0.1)
            elif leaf in ("embed", "side_embed"):
                rnd(p, 1.0)
            elif leaf == "conv":
                rnd(p, p.shape[0] ** -0.5)
            else:
                rnd(p, p.shape[1] ** -0.5)
        return self


# ------------------------------------------------------ checkpoint reading
def load_vabedra(path: str, device="cpu", dtype=torch.bfloat16,
                 max_position: int | None = None) -> VabedraForCausalLM:
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
    cfg = VabedraConfig.from_json(c, shape_of, name=root.name)
    if max_position is not None:
        cfg.max_position = max_position
    model = VabedraForCausalLM(cfg, device=device, dtype=dtype)
    return model.load_tensors(get).eval()


def save_vabedra(tensors: dict, cfg: VabedraConfig, path: str) -> None:
    """Write checkpoint-named tensors + config.json (tests, tooling)."""
    from safetensors.torch import save_file
    root = Path(path)
    root.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              str(root / "model.safetensors"))
    (root / "config.json").write_text(json.dumps(cfg.to_json(), indent=1))


def _bench_config(name, width, n_layers, heads, kv_heads, dim, experts, top,
                  expert_ff, vocab=32000, window=1024, keep_first=64,
                  side_dim=256):
    """Alternating parallel / delta layers with a mixture in every layer."""
    layers = []
    for i in range(n_layers):
        mlp = RoutedSpec(experts=experts, top=top, ff=expert_ff,
                         act="clamped", limit=7.0, score="softmax",
                         renorm=False)
        if i % 2 == 0:
            layers.append(VLayerSpec(
                kind="parallel",
                delta=DeltaSpec(heads=heads // 2, kv_heads=heads // 2,
                                dim=dim, vdim=dim, conv=4, rank=16,
                                gate_rank=16),
                attn=SinkAttnSpec(
                    heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                    scale=dim ** -0.5, softcap=50.0, window=window,
                    keep_first=keep_first, rot_dims=dim // 2, rot_base=5e5,
                    rot_scaling={"factor": 8.0, "low": 1.0, "high": 4.0,
                                 "original": 8192}),
                mlp=mlp))
        else:
            layers.append(VLayerSpec(
                kind="delta",
                delta=DeltaSpec(heads=heads, kv_heads=kv_heads, dim=dim,
                                vdim=dim, conv=4),
                mlp=mlp))
    return VabedraConfig(name=name, vocab_size=vocab, width=width,
                         layers=layers, eps=1e-6, alpha=2.0,
                         embed_scale=width ** 0.5, side_dim=side_dim)


VABEDRA_CONFIGS = {
    # a small model with every branch, for smoke runs and CPU tests
    "vabedra-tiny": _bench_config("vabedra-tiny", 128, 4, 4, 2, 32, 8, 2, 64,
                                  vocab=384, window=48, keep_first=5,
                                  side_dim=8),
    # same width / depth / heads as "reperax-1b" and "zudisun-1b-moe"; the
    # mixture (16 experts of ff 2048, top 4) matches a dense ff of 8192
    "vabedra-1b": _bench_config("vabedra-1b", 2048, 16, 16, 8, 128, 16, 4,
                                2048),
    # the same with 4 experts of ff 2048, all of them chosen: the parameter
    # count of "reperax-1b"'s dense ff, no expert left idle
    "vabedra-1b-e4": _bench_config("vabedra-1b-e4", 2048, 16, 16, 8, 128, 4,
                                   4, 2048),
    # same width / depth / heads / vocabulary as "reperax-8b"
    "vabedra-8b": _bench_config("vabedra-8b", 4096, 32, 32, 8, 128, 16, 4,
                                3584, vocab=128256),
}
