"""Hybrid parallel-residual decoders: the Reperax design.

A Reperax model is a stack of layers, each `x <- x + gate1*mixer(shift(n1))
+ gate2*ff(n2)` with n1, n2 two zero-centred RMSNorms of the same fp32
residual row, a token-shift lerp in front of the mixer, and sigmoid output
gates computed from the un-shifted norms.  Mixers:

  * ``parallel``  — chunk-local softmax attention (GQA, whole-row q/k norm,
    no positional rotation) side by side with gated linear attention
    (per-key-channel data-dependent decay), summed with fixed scales
  * ``retention`` — linear attention with one fixed decay per head and
    partial rotate-half rotary positions

A contiguous span of layers may be looped several times with shared weights;
each pass has its own cache/state, re-injects the embedding output and adds a
learned per-pass vector.  The feed-forward is up -> PolyNorm -> down.  Logits
reuse the embedding table and are soft-capped with tanh.

Every mechanism is a small module parameterised by its spec, running on the
sequence-mixer op set (ops/seqmix.py): hand-written gfx950 kernels on GPU,
vendor GEMMs for the projections.  Per-sequence state (recurrent matrices,
token-shift rows) lives in slots of `HybridCache`, attention K/V in its pages;
the engine's scheduler hands out both.
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


# ------------------------------------------------------------------ specs
@dataclass
class ChunkAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0        # keys visible only within the query's chunk
    window: int = 0       # and/or only the last `window` positions


@dataclass
class GatedLinearSpec:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int             # width of the low-rank decay projection


@dataclass
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_dims: int = 0
    rot_base: float = 10000.0


@dataclass
class LayerSpec:
    kind: str                               # "parallel" | "retention"
    ff: int | None                          # None: no feed-forward
    attn: ChunkAttnSpec | None = None       # parallel: left
    gla: GatedLinearSpec | None = None      # parallel: right
    left_scale: float = 1.0
    right_scale: float = 1.0
    ret: RetentionSpec | None = None


@dataclass
class ReperaxConfig:
    name: str = "reperax"
    vocab_size: int = 512
    width: int = 256
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eps: float = 1e-6
    logit_softcap: float = 0.0
    max_position: int = 8192    # serving limit (block-table width), not a
                                # property of the weights

    architecture = "Reperax"
    # engine-facing traits
    stateful = True             # needs per-sequence state slots
    num_kv_heads = 1
    num_experts = 1
    sliding_window = 0

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start and self.loop_times >= 1

    @property
    def runs(self) -> list[tuple[int, int]]:
        """Execution order as (layer index, pass index); a looped layer
        appears once per pass and owns one cache/state per appearance."""
        n = len(self.layers)
        a, b, times = self.loop_start, self.loop_stop, self.loop_times
        if not self.has_loop:
            return [(i, 0) for i in range(n)]
        out = [(i, 0) for i in range(a)]
        for t in range(times):
            out += [(i, t) for i in range(a, b)]
        out += [(i, 0) for i in range(b, n)]
        return out

    def build_model(self, device="cpu", dtype=torch.bfloat16):
        return ReperaxForCausalLM(self, device=device, dtype=dtype)

    def cache_layout(self) -> list:
        """What every layer run keeps between steps (HybridCache)."""
        out = []
        for li, _p in self.runs:
            ls = self.layers[li]
            m = ls.gla if ls.kind == "parallel" else ls.ret
            need = {"kv": None, "state": {
                "shift": ((self.width,), "f32"),
                "rec": ((m.heads, m.dim, m.vdim), "f32")}}
            if ls.kind == "parallel":
                a = ls.attn
                need["kv"] = (a.kv_heads, a.dim, a.vdim)
            out.append(need)
        return out

    @staticmethod
    def from_json(c: dict, shape_of: Callable[[str], tuple] | None = None,
                  name: str = "reperax") -> "ReperaxConfig":
        """Read a checkpoint's config.json.  Sizes that the JSON leaves to
        the tensors (the decay projection's rank) come from shape_of(name)."""
        layers = []
        for i, lc in enumerate(c["layers"]):
            m = lc["mixer"]
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown mlp kind {mlp['kind']}")
            ff = int(mlp["ff"]) if mlp is not None else None
            if lc["type"] == "parallel":
                le, ri = m["left"], m["right"]
                rank = (shape_of(f"l{i}.mix.right.a1")[0]
                        if shape_of is not None else int(ri.get("rank", 16)))
                layers.append(LayerSpec(
                    kind="parallel", ff=ff,
                    attn=ChunkAttnSpec(
                        heads=int(le["heads"]),
                        kv_heads=int(le.get("kv_heads", le["heads"])),
                        dim=int(le["dim"]), vdim=int(le.get("vdim", le["dim"])),
                        scale=float(le["scale"]),
                        chunk=int((le.get("mask") or {}).get("size", 0))),
                    gla=GatedLinearSpec(
                        heads=int(ri["heads"]), dim=int(ri["dim"]),
                        vdim=int(ri.get("vdim", ri["dim"])),
                        tau=float(ri["tau"]), rank=int(rank)),
                    left_scale=float(m.get("left_scale", 1.0)),
                    right_scale=float(m.get("right_scale", 1.0))))
            elif lc["type"] == "retention":
                rot = m.get("rot") or {}
                layers.append(LayerSpec(
                    kind="retention", ff=ff,
                    ret=RetentionSpec(
                        heads=int(m["heads"]), dim=int(m["dim"]),
                        vdim=int(m.get("vdim", m["dim"])),
                        decay=tuple(float(d) for d in m["decay"]),
                        rot_dims=int(rot.get("dims", 0)),
                        rot_base=float(rot.get("base", 10000.0)))))
            else:
                raise ValueError(f"layer {i}: unknown type {lc['type']}")
        lp = c.get("loop") or {}
        return ReperaxConfig(
            name=name, vocab_size=int(c["vocab"]), width=int(c["width"]),
            layers=layers, loop_start=int(lp.get("start", 0)),
            loop_stop=int(lp.get("stop", 0)), loop_times=int(lp.get("times", 1)),
            eps=float(c["norm"]["eps"]),
            logit_softcap=float(c.get("logit_softcap") or 0.0))

    def to_json(self) -> dict:
        layers = []
        for ls in self.layers:
            mlp = {"ff": ls.ff, "kind": "dense"} if ls.ff is not None else None
            if ls.kind == "parallel":
                a, g = ls.attn, ls.gla
                mixer = {
                    "left": {"dim": a.dim, "heads": a.heads,
                             "kv_heads": a.kv_heads, "mask": {"size": a.chunk},
                             "scale": a.scale, "vdim": a.vdim},
                    "left_scale": ls.left_scale,
                    "right": {"dim": g.dim, "heads": g.heads, "tau": g.tau,
                              "vdim": g.vdim},
                    "right_scale": ls.right_scale}
            else:
                r = ls.ret
                mixer = {"decay": list(r.decay), "dim": r.dim,
                         "heads": r.heads, "vdim": r.vdim,
                         "rot": {"base": r.rot_base, "dims": r.rot_dims}}
            layers.append({"mixer": mixer, "mlp": mlp, "type": ls.kind})
        return {"architecture": self.architecture, "layers": layers,
                "logit_softcap": self.logit_softcap,
                "loop": {"start": self.loop_start, "stop": self.loop_stop,
                         "times": self.loop_times},
                "norm": {"eps": self.eps}, "vocab": self.vocab_size,
                "width": self.width}


# ------------------------------------------------------------------ cache
class HybridCache:
    """Per-run storage for one engine, built from a model's cache layout:
    one entry per layer run (a looped layer counts once per pass) with

      "kv":    (kv_heads, dk, dv) or None - K/V pages [P, G, page, dk] /
               [P, G, page, dv] in the model dtype (dv 0: key pages only,
               for layers whose values are part of the key rows)
      "state": {name: (shape, "f32" | "model")} - per-sequence tensors
               [slots, *shape] (recurrent matrices, token-shift rows,
               convolution inputs, ...)

    Pages live in `k[run]` / `v[run]`, state in `state[name][run]` (`rec` and
    `shift` are the names the linear-recurrence layers use).  Page 0 and slot
    0 are the engine's null page / null slot.  Nothing is cleared when a page
    or slot changes hands: a chunk that starts at position 0 ignores the
    slot's content, and attention never reads a position that the current
    owner has not written."""

    def __init__(self, layout: list, num_pages: int, page_size: int,
                 num_slots: int, device, dtype=torch.bfloat16):
        self.page_size, self.num_pages, self.num_slots = \
            page_size, num_pages, num_slots
        self.k, self.v, self.state = {}, {}, {}
        for r, need in enumerate(layout):
            kv = need.get("kv")
            if kv is not None:
                G, dk, dv = kv
                self.k[r] = torch.zeros(num_pages, G, page_size, dk,
                                        dtype=dtype, device=device)
                if dv > 0:
                    self.v[r] = torch.zeros(num_pages, G, page_size, dv,
                                            dtype=dtype, device=device)
            for name, (shape, kind) in (need.get("state") or {}).items():
                self.state.setdefault(name, {})[r] = torch.zeros(
                    num_slots, *shape, device=device,
                    dtype=torch.float32 if kind == "f32" else dtype)
        self.rec = self.state.get("rec", {})
        self.shift = self.state.get("shift", {})

    @staticmethod
    def bytes_per_page(layout: list, page_size: int, itemsize: int = 2) -> int:
        n = 0
        for need in layout:
            if need.get("kv") is not None:
                G, dk, dv = need["kv"]
                n += G * page_size * (dk + dv) * itemsize
        return max(n, 1)

    @staticmethod
    def bytes_per_slot(layout: list, itemsize: int = 2) -> int:
        n = 0
        for need in layout:
            for shape, kind in (need.get("state") or {}).values():
                n += math.prod(shape) * (4 if kind == "f32" else itemsize)
        return n


# ----------------------------------------------------------------- mixers
class ChunkedAttention(nn.Module):
    """Softmax attention with grouped K/V heads, RMSNorm over the whole q and
    k rows, no positional rotation, keys restricted to the query's chunk
    (and/or a trailing window)."""

    def __init__(self, spec: ChunkAttnSpec, width: int, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        self.q_norm = nn.Parameter(torch.empty(s.heads * s.dim))
        self.k_norm = nn.Parameter(torch.empty(s.kv_heads * s.dim))
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))

    def in_blocks(self):
        s = self.spec
        return [("q", s.heads * s.dim), ("k", s.kv_heads * s.dim),
                ("v", s.kv_heads * s.vdim)]

    def forward(self, p: dict, cache: HybridCache, run: int, md, positions):
        s = self.spec
        q = sm.qk_norm_cache(p["q"], p["k"], p["v"], self.q_norm, self.k_norm,
                             self.eps, cache.k[run], cache.v[run], md.slots)
        o = sm.masked_attention(q, cache.k[run], cache.v[run], md, positions,
                                s.scale, s.heads, chunk=s.chunk,
                                window=s.window)
        return sm.matmul(o, self.o)


class GatedLinearAttention(nn.Module):
    """Linear attention whose state decays per key channel by
    sigmoid(z)^(1/tau), z a low-rank projection of the input plus bias;
    per-head RMSNorm (weight shared by heads) and SiLU output gate."""

    def __init__(self, spec: GatedLinearSpec, width: int, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        self.a2 = nn.Parameter(torch.empty(s.heads * s.dim, s.rank))
        self.register_buffer("a2_b", torch.zeros(s.heads * s.dim,
                                                 dtype=torch.float32))
        self.norm = nn.Parameter(torch.empty(s.vdim))
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))

    def in_blocks(self):
        s = self.spec
        return [("q", s.heads * s.dim), ("k", s.heads * s.dim),
                ("v", s.heads * s.vdim), ("g", s.heads * s.vdim),
                ("a1", s.rank)]

    def forward(self, p: dict, cache: HybridCache, run: int, md, positions):
        s = self.spec
        z = sm.matmul(p["a1"], self.a2)
        o = sm.linear_scan(p["q"], p["k"], p["v"], cache.rec[run], md,
                           positions, s.heads, q_scale=s.dim ** -0.5,
                           decay_logits=z, decay_bias=self.a2_b,
                           inv_tau=1.0 / s.tau)
        y = sm.headnorm_gate(o, p["g"], self.norm, self.eps, s.heads,
                             self.o.dtype)
        return sm.matmul(y, self.o)


class Retention(nn.Module):
    """Linear attention with a fixed decay per head, rotate-half rotary
    positions on the leading dims of q and k, k scaled by dim^-1/2 after the
    rotation, weight-free per-head RMSNorm and SiLU output gate."""

    def __init__(self, spec: RetentionSpec, width: int, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        if len(s.decay) != s.heads:
            raise ValueError("retention: one decay per head expected")
        self.register_buffer("decay", torch.tensor(s.decay,
                                                   dtype=torch.float32))
        self.register_buffer(
            "inv_freq", sm.rotary_inv_freq(s.rot_dims, s.rot_base, "cpu")
            if s.rot_dims > 0 else None)
        self.o = nn.Parameter(torch.empty(width, s.heads * s.vdim))

    def in_blocks(self):
        s = self.spec
        return [("q", s.heads * s.dim), ("k", s.heads * s.dim),
                ("v", s.heads * s.vdim), ("g", s.heads * s.vdim)]

    def forward(self, p: dict, cache: HybridCache, run: int, md, positions):
        s = self.spec
        o = sm.linear_scan(p["q"], p["k"], p["v"], cache.rec[run], md,
                           positions, s.heads, k_scale=s.dim ** -0.5,
                           head_decay=self.decay, inv_freq=self.inv_freq)
        y = sm.headnorm_gate(o, p["g"], None, self.eps, s.heads, self.o.dtype)
        return sm.matmul(y, self.o)


class PolyNormMLP(nn.Module):
    """down(PolyNorm(up(h))); the up projection is fused with whatever else
    reads the same input (the layer's output-gate logits)."""

    def __init__(self, ff: int, width: int, eps: float):
        super().__init__()
        self.ff, self.eps = ff, eps
        self.down = nn.Parameter(torch.empty(width, ff))
        self.register_buffer("act", torch.zeros(4, dtype=torch.float32))

    def forward(self, z):
        return sm.matmul(sm.polynorm(z, self.act, self.eps), self.down)


class ReperaxLayer(nn.Module):
    def __init__(self, cfg: ReperaxConfig, spec: LayerSpec):
        super().__init__()
        W, eps = cfg.width, cfg.eps
        self.spec, self.eps = spec, eps
        self.norm1 = nn.Parameter(torch.empty(W))
        self.shift = nn.Parameter(torch.empty(W))
        self.rg1 = nn.Parameter(torch.empty(W, W))
        self.register_buffer("rg1_b", torch.zeros(W, dtype=torch.float32))
        if spec.kind == "parallel":
            self.mixers = nn.ModuleDict({
                "left": ChunkedAttention(spec.attn, W, eps),
                "right": GatedLinearAttention(spec.gla, W, eps)})
            self.scales = (spec.left_scale, spec.right_scale)
        else:
            self.mixers = nn.ModuleDict({"ret": Retention(spec.ret, W, eps)})
            self.scales = (1.0,)
        # one GEMM feeds every projection that reads the shifted input
        self.blocks = [(mn, bn, rows) for mn, m in self.mixers.items()
                       for bn, rows in m.in_blocks()]
        # fused weights are padded to 64 output rows (the skinny decode GEMM's
        # tile); the padding rows produce columns nobody reads
        def pad64(n):
            return n + (-n) % 64
        self.mix_in = nn.Parameter(torch.empty(
            pad64(sum(r for _, _, r in self.blocks)), W))
        if spec.ff is not None:
            self.norm2 = nn.Parameter(torch.empty(W))
            self.mlp = PolyNormMLP(spec.ff, W, eps)
            # [up | output-gate logits]: both read norm2(x)
            self.ff_in = nn.Parameter(torch.empty(pad64(spec.ff + W), W))
            self.register_buffer("rg2_b", torch.zeros(W, dtype=torch.float32))
        else:
            self.norm2 = None
            self.mlp = None

    def forward(self, x, cache: HybridCache, run: int, md, positions):
        dt = self.mix_in.dtype
        a, s, b = sm.dual_norm_shift(x, self.norm1, self.norm2, self.shift,
                                     self.eps, cache.shift[run], md, dt)
        proj = sm.matmul(s, self.mix_in)
        views, c0 = {}, 0
        for mn, bn, rows in self.blocks:
            views.setdefault(mn, {})[bn] = proj[:, c0:c0 + rows]
            c0 += rows
        outs = [m(views[mn], cache, run, md, positions)
                for mn, m in self.mixers.items()]
        g1 = sm.matmul(a, self.rg1)
        m_out = g2 = b2 = None
        if self.mlp is not None:
            u = sm.matmul(b, self.ff_in)
            m_out = self.mlp(u[:, :self.spec.ff])
            g2 = u[:, self.spec.ff:self.spec.ff + x.shape[1]]
            b2 = self.rg2_b
        sm.gated_residual(x, outs[0], self.scales[0],
                          outs[1] if len(outs) > 1 else None,
                          self.scales[1] if len(outs) > 1 else 0.0,
                          g1, self.rg1_b, m_out, g2, b2)
        return x


class ReperaxForCausalLM(nn.Module):
    # the engine asks these before wiring a model in
    needs_state_slots = True
    supports_speculation = False    # rejected drafts would need state rollback
    supports_prefix_cache = False   # recurrent state is not page-addressable

    def __init__(self, cfg: ReperaxConfig, device="cpu",
                 dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        with torch.device(device):
            self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
            self.layers = nn.ModuleList(
                [ReperaxLayer(cfg, ls) for ls in cfg.layers])
            self.final_norm = nn.Parameter(torch.empty(cfg.width))
            self.register_buffer("loop_step", torch.zeros(
                max(cfg.loop_times, 1), cfg.width, dtype=torch.float32))
        for p in self.parameters():
            p.data = p.data.to(dtype)
            p.requires_grad_(False)
        self.to(device)
        self.record_runs: list | None = None  # set to [] to keep x per run

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
        x = sm.embed_rows(ids, self.embed)
        looped = cfg.has_loop
        e0 = x.clone() if looped and cfg.loop_times > 1 else None
        for run, (li, p) in enumerate(cfg.runs):
            if looped and li == cfg.loop_start:
                sm.add_rows(x, e0 if p > 0 else None, self.loop_step[p])
            x = self.layers[li](x, cache, run, md, positions)
            if self.record_runs is not None:
                self.record_runs.append(x.clone())
        h = sm.norm_rows(x, self.final_norm, cfg.eps, logit_rows,
                         self.embed.dtype)
        # vocabulary-sized N: the vendor GEMM wins there at every row count
        return sm.softcap(sm.matmul(h, self.embed, skinny=False),
                          cfg.logit_softcap)

    # -- weights ------------------------------------------------------------
    @torch.no_grad()
    def load_tensors(self, get: Callable[[str], torch.Tensor]):
        """Fill parameters from checkpoint tensors by name: 'embed',
        'final.norm', 'loop.step', and per layer i 'l<i>.norm1|norm2|shift|
        rg1|rg1.b|rg2|rg2.b', 'l<i>.mix.<...>', 'l<i>.mlp.up|down|act'."""
        def put(dst, src):
            dst.copy_(src.to(dst.device, dst.dtype))
        put(self.embed, get("embed"))
        put(self.final_norm, get("final.norm"))
        cfg = self.cfg
        if cfg.has_loop:
            put(self.loop_step, get("loop.step"))
        for i, L in enumerate(self.layers):
            pre = f"l{i}."
            put(L.norm1, get(pre + "norm1"))
            put(L.shift, get(pre + "shift"))
            put(L.rg1, get(pre + "rg1"))
            put(L.rg1_b, get(pre + "rg1.b"))
            sub = {"left": "mix.left.", "right": "mix.right.", "ret": "mix."}
            def padded(parts, total):
                t = torch.cat(parts, 0)
                if t.shape[0] < total:
                    t = torch.cat([t, t.new_zeros(total - t.shape[0],
                                                  t.shape[1])], 0)
                return t
            rows = [get(pre + sub[mn] + bn) for mn, bn, _ in L.blocks]
            put(L.mix_in, padded(rows, L.mix_in.shape[0]))
            for mn, m in L.mixers.items():
                mp = pre + sub[mn]
                put(m.o, get(mp + "o"))
                if isinstance(m, ChunkedAttention):
                    put(m.q_norm, get(mp + "q.norm"))
                    put(m.k_norm, get(mp + "k.norm"))
                elif isinstance(m, GatedLinearAttention):
                    put(m.a2, get(mp + "a2"))
                    put(m.a2_b, get(mp + "a2.b"))
                    put(m.norm, get(mp + "norm"))
            if L.mlp is not None:
                put(L.norm2, get(pre + "norm2"))
                put(L.ff_in, padded([get(pre + "mlp.up"), get(pre + "rg2")],
                                    L.ff_in.shape[0]))
                put(L.rg2_b, get(pre + "rg2.b"))
                put(L.mlp.down, get(pre + "mlp.down"))
                put(L.mlp.act, get(pre + "mlp.act"))
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
            if p is None or name.endswith(("decay", "inv_freq")):
                continue
            if name.endswith("shift"):
                p.copy_(torch.rand(p.shape, generator=g).to(p.dtype))
            elif name.endswith("act"):
                p.copy_(torch.tensor([0.6, 0.3, 0.1, 0.0]))
            elif p.dim() == 1:
                rnd(p, 0.1)
            elif name == "embed":
                rnd(p, 1.0)
            else:
                rnd(p, p.shape[1] ** -0.5)
        return self


# ------------------------------------------------------ checkpoint reading
def load_reperax(path: str, device="cpu", dtype=torch.bfloat16,
                 max_position: int | None = None) -> ReperaxForCausalLM:
    """config.json + model.safetensors -> model on `device` in `dtype`."""
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
    cfg = ReperaxConfig.from_json(c, shape_of, name=root.name)
    if max_position is not None:
        cfg.max_position = max_position
    model = ReperaxForCausalLM(cfg, device=device, dtype=dtype)
    return model.load_tensors(get).eval()


def save_reperax(tensors: dict, cfg: ReperaxConfig, path: str) -> None:
    """Write checkpoint-named tensors + config.json (tests, tooling)."""
    from safetensors.torch import save_file
    root = Path(path)
    root.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              str(root / "model.safetensors"))
    (root / "config.json").write_text(json.dumps(cfg.to_json(), indent=1))


def _bench_config(name, width, ff, n_par, n_ret, heads, kv_heads, dim,
                  vocab=32000, chunk=512, loop=(0, 0, 1)):
    par = LayerSpec(
        kind="parallel", ff=ff,
        attn=ChunkAttnSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                           scale=dim ** -0.5, chunk=chunk),
        gla=GatedLinearSpec(heads=heads // 2, dim=dim, vdim=dim, tau=16.0,
                            rank=16),
        left_scale=1.0, right_scale=1.0)
    ret = LayerSpec(
        kind="retention", ff=ff,
        ret=RetentionSpec(heads=heads, dim=dim, vdim=dim,
                          decay=tuple(1.0 - 2.0 ** (-5 - 5 * i / max(1, heads - 1))
                                      for i in range(heads)),
                          rot_dims=dim // 2, rot_base=1e6))
    return ReperaxConfig(name=name, vocab_size=vocab, width=width,
                         layers=[par] * n_par + [ret] * n_ret,
                         loop_start=loop[0], loop_stop=loop[1],
                         loop_times=loop[2], eps=1e-6, logit_softcap=30.0)


HYBRID_CONFIGS = {
    # a small looped model for smoke runs and CPU tests
    "reperax-tiny": _bench_config("reperax-tiny", 128, 384, 1, 1, 4, 2, 32,
                                  vocab=384, chunk=32, loop=(0, 2, 2)),
    # same width / ff / depth / heads as the Llama "debug-1b" config
    "reperax-1b": _bench_config("reperax-1b", 2048, 8192, 8, 8, 16, 8, 128),
    # same width / ff / depth / heads / vocabulary as "llama-3-8b"
    "reperax-8b": _bench_config("reperax-8b", 4096, 14336, 16, 16, 32, 8, 128,
                                vocab=128256, chunk=1024),
}
