"""Sequence-mixer op set: masked paged attention for arbitrary head sizes,
decayed linear recurrences with per-sequence state slots, and the norm /
gate / activation glue of parallel-residual hybrid decoders.

Conventions shared by every op here:
  * the residual stream, recurrent state, decays, norms statistics and
    attention scores are fp32; projections / activations are in the model's
    storage dtype (bf16 or fp32) — kernels are instantiated for both
  * a batch is a packed list of row chunks, one per sequence:
    cu [B+1] i32 (row offsets), q_start [B] i32 (absolute position of each
    chunk's first row), row_seq [T] i32 (sequence index of every row),
    state_slots [B] i32 (per-sequence state slot), a decode step being the
    special case of one row per sequence
  * CUDA (=HIP) tensors run the gfx950 kernels of the mixer kernel groups, CPU tensors a
    vectorised torch path used by CPU tests

The recurrences are evaluated strictly token by token in fp32, so results
do not depend on where a prompt was cut into chunks.
"""
from __future__ import annotations

import ctypes
import math
import os

import torch

from . import _lib

_DT = {torch.bfloat16: 0, torch.float32: 1}
# a step whose longest row chunk reaches this many rows runs bf16 attention
# through the MFMA tile kernel; shorter steps (decode) use one wave per row
MFMA_MIN_ROWS = 16
# single rows (decode) with at least this many query heads per K/V head run
# bf16 attention with the heads as matrix-core rows
HEADS_MFMA_MIN = 8
_SKINNY = os.environ.get("AF_MIX_SKINNY", "0") == "1"


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def _L():
    return _lib.mixlib()


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"seqmix ops take bf16 or fp32 storage, got {t.dtype}")


def _rowstride(t: torch.Tensor) -> int:
    assert t.dim() == 2 and t.stride(1) == 1, "rows must be unit-stride"
    return t.stride(0)


# ------------------------------------------------------------------ embed
def embed_rows(ids: torch.Tensor, table: torch.Tensor,
               add: torch.Tensor | None = None,
               scale: float = 1.0) -> torch.Tensor:
    """x[t] = table[ids[t]] * scale (+ add) as an fp32 residual stream
    [T, W]."""
    T = ids.numel()
    W = table.shape[1]
    if not _gpu(table):
        x = table[ids.long()].float() * scale
        return x + add.float() if add is not None else x
    out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    rc = _L().afm_embed(_lib.ptr(out), _lib.ptr(table), _lib.ptr(ids),
                        _lib.ptr(add), float(scale), T, W, _code(table),
                        _lib.cur_stream())
    _lib.check(rc, "afm_embed")
    return out


def add_rows(x: torch.Tensor, other: torch.Tensor | None,
             vec: torch.Tensor | None) -> torch.Tensor:
    """In place x += other (same shape, fp32) + vec (one row, fp32)."""
    if not _gpu(x):
        if other is not None:
            x += other
        if vec is not None:
            x += vec.float()
        return x
    T, W = x.shape
    rc = _L().afm_add_rows(_lib.ptr(x), _lib.ptr(other), _lib.ptr(vec), T, W,
                           _lib.cur_stream())
    _lib.check(rc, "afm_add_rows")
    return x


# ------------------------------------------------------- norms + token shift
def dual_norm_shift(x: torch.Tensor, w1: torch.Tensor,
                    w2: torch.Tensor | None, shift: torch.Tensor | None,
                    eps: float, prev: torch.Tensor | None, md,
                    out_dtype: torch.dtype):
    """Two zero-centred RMSNorms of the same fp32 row (weights applied as
    1 + w) plus the token-shift lerp on the first one.

    a = norm(x)*(1+w1); b = norm(x)*(1+w2); s = a + (a_prev - a)*shift where
    a_prev is the previous position's `a` — the row above inside a chunk,
    the sequence's slot of `prev` [slots, W] fp32 at a chunk's first row,
    zeros at position 0.  `prev` is then updated with each chunk's last `a`.
    Returns (a, s, b) in out_dtype (b None without w2; s is a without shift).
    """
    T, W = x.shape
    B = md.q_start.numel()
    if not _gpu(x):
        r = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        a = x * r * (1.0 + w1.float())
        b = x * r * (1.0 + w2.float()) if w2 is not None else None
        s = a
        if shift is not None:
            cu = md.cu_seqlens.tolist()
            qs = md.q_start.tolist()
            sl = md.state_slots.tolist()
            ap = torch.zeros_like(a)
            ap[1:] = a[:-1]
            for i in range(B):
                if cu[i + 1] == cu[i]:
                    continue
                ap[cu[i]] = prev[sl[i]] if qs[i] > 0 else 0.0
            for i in range(B):
                if cu[i + 1] > cu[i]:
                    prev[sl[i]] = a[cu[i + 1] - 1]
            s = a + (ap - a) * shift.float()
        return (a.to(out_dtype), s.to(out_dtype),
                b.to(out_dtype) if b is not None else None)
    a = torch.empty(T, W, dtype=out_dtype, device=x.device)
    s = torch.empty_like(a) if shift is not None else a
    b = torch.empty_like(a) if w2 is not None else None
    # a decode step (one row per sequence) writes the state slot in place;
    # longer chunks stage their last row and scatter it afterwards, because
    # the chunk's first row still reads the old slot content
    single = not getattr(md, "is_prefill", True)
    last = (torch.empty(B, W, dtype=torch.float32, device=x.device)
            if shift is not None and not single else None)
    rc = _L().afm_dual_norm_shift(
        _lib.ptr(a), _lib.ptr(s), _lib.ptr(b), _lib.ptr(last), _lib.ptr(x),
        _lib.ptr(w1), _lib.ptr(w2), _lib.ptr(shift), _lib.ptr(prev),
        _lib.ptr(md.row_seq), _lib.ptr(md.cu_seqlens), _lib.ptr(md.q_start),
        _lib.ptr(md.state_slots), float(eps), T, W, _code(a),
        _lib.cur_stream())
    _lib.check(rc, "afm_dual_norm_shift")
    if last is not None:
        rc = _L().afm_scatter_state(
            _lib.ptr(prev), _lib.ptr(last), _lib.ptr(md.state_slots),
            _lib.ptr(md.cu_seqlens), B, W, _lib.cur_stream())
        _lib.check(rc, "afm_scatter_state")
    return a, s, b


def norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float,
              rows: torch.Tensor | None, out_dtype: torch.dtype,
              one_plus: bool = True) -> torch.Tensor:
    """RMSNorm of selected fp32 rows: x[rows] / rms * (1 + w) (or * w)."""
    if not _gpu(x):
        xs = x[rows.long()] if rows is not None else x
        r = torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float() + 1.0 if one_plus else w.float()
        return (xs * r * wf).to(out_dtype)
    R = rows.numel() if rows is not None else x.shape[0]
    W = x.shape[1]
    out = torch.empty(R, W, dtype=out_dtype, device=x.device)
    rc = _L().afm_norm_rows(_lib.ptr(out), _lib.ptr(x), _lib.ptr(w),
                            _lib.ptr(rows), float(eps), R, W,
                            1 if one_plus else 0, _code(out),
                            _lib.cur_stream())
    _lib.check(rc, "afm_norm_rows")
    return out


# ----------------------------------------------------------- attention side
def qk_norm_cache(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  qw: torch.Tensor | None, kw: torch.Tensor | None,
                  eps: float, kcache: torch.Tensor, vcache: torch.Tensor,
                  slots: torch.Tensor) -> torch.Tensor:
    """RMSNorm over the WHOLE q row and the whole k row (all heads at once,
    plain weights; skipped when the weight is None), then append k / v to the
    paged caches kcache [P, G, page, dk] / vcache [P, G, page, dv] at `slots`
    [T] i64.  Returns the normed q, contiguous [T, H*dk]."""
    T = q.shape[0]
    _, G, page, dk = kcache.shape
    dv = vcache.shape[3]
    if not _gpu(q):
        qf, kf = q.float(), k.float()
        if qw is not None:
            qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) \
                * qw.float()
        if kw is not None:
            kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) \
                * kw.float()
        pg = torch.div(slots, page, rounding_mode="floor")
        off = slots - pg * page
        kcache[pg, :, off] = kf.view(T, G, dk).to(kcache.dtype)
        vcache[pg, :, off] = v.reshape(T, G, dv).to(vcache.dtype)
        return qf.to(q.dtype)
    out = torch.empty(T, q.shape[1], dtype=q.dtype, device=q.device)
    rc = _L().afm_qk_norm_cache(
        _lib.ptr(out), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(qw),
        _lib.ptr(kw), _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(slots),
        float(eps), T, q.shape[1], G * dk, G * dv, G, dk, dv, page,
        _rowstride(q), _rowstride(k), _rowstride(v), _code(q),
        _lib.cur_stream())
    _lib.check(rc, "afm_qk_norm_cache")
    return out


def masked_attention(q: torch.Tensor, kcache: torch.Tensor,
                     vcache: torch.Tensor | None, md, positions: torch.Tensor,
                     scale: float, heads: int, chunk: int = 0,
                     window: int = 0, sink: torch.Tensor | None = None,
                     softcap: float = 0.0,
                     log_bias: tuple | None = None,
                     v_width: int = 0, keep_first: int = 0) -> torch.Tensor:
    """Softmax attention of packed rows over the paged cache.  Row at
    position i sees key j iff j <= i, and (chunk > 0) floor(j/chunk) ==
    floor(i/chunk), and (window > 0) j > i - window; with keep_first > 0 the
    keys j < keep_first stay visible whatever chunk and window say, at their
    true positions.  Positions are absolute in the sequence.  q [T, H*dk] ->
    [T, H*dv]; scores and softmax in fp32.

    Optional terms, per head h: s = q.k * scale; softcap > 0: s <- softcap *
    tanh(s / softcap); log_bias (r1, r2) [H] fp32 each: s <- s - r1[h] *
    ln(1 + r2[h] * (i - j)); sink [H] fp32: exp(sink[h]) joins the softmax
    denominator (a term without key or value, not scaled).  vcache None: the
    values are the first v_width elements of the key rows."""
    T = q.shape[0]
    _, G, page, dk = kcache.shape
    if vcache is None:
        if not 0 < v_width <= dk:
            raise ValueError("values inside the key rows need 0 < v_width <= dk")
        dv, ldv, vsrc = v_width, dk, kcache
    else:
        dv, ldv, vsrc = vcache.shape[3], vcache.shape[3], vcache
    H = heads
    r1, r2 = log_bias if log_bias is not None else (None, None)
    if not _gpu(q):
        out = torch.zeros(T, H, dv, dtype=torch.float32)
        qf = q.float().view(T, H, dk)
        bt = md.block_table.long()
        rs = md.row_seq.tolist()
        pos = positions.tolist()
        for t in range(T):
            i = pos[t]
            lo = 0
            if chunk > 0:
                lo = (i // chunk) * chunk
            if window > 0:
                lo = max(lo, i - window + 1)
            js = torch.arange(lo, i + 1)
            if keep_first > 0 and lo > 0:
                js = torch.cat([torch.arange(min(keep_first, lo)), js])
            pg = bt[rs[t]][js // page]
            kk = kcache[pg, :, js % page].float()      # [n, G, dk]
            vv = vsrc[pg, :, js % page][..., :dv].float()
            kk = kk.repeat_interleave(H // G, dim=1)
            vv = vv.repeat_interleave(H // G, dim=1)
            s = torch.einsum("nhd,hd->hn", kk, qf[t]) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            if r1 is not None:
                s = s - r1.float()[:, None] * torch.log(
                    1.0 + r2.float()[:, None] * (i - js).float()[None])
            if sink is not None:
                s = torch.cat([s, sink.float()[:, None]], 1)
            w = torch.softmax(s, -1)[:, :js.numel()]
            out[t] = torch.einsum("hn,nhd->hd", w, vv)
        return out.view(T, H * dv).to(q.dtype)
    out = torch.empty(T, H * dv, dtype=q.dtype, device=q.device)
    lens = getattr(md, "seq_lens", None)
    extra = (_lib.ptr(sink), float(softcap), _lib.ptr(r1), _lib.ptr(r2),
             int(ldv), int(keep_first))
    if (q.dtype == torch.bfloat16 and lens is not None and dk <= 576
            and dv <= 512 and max(lens) >= MFMA_MIN_ROWS):
        # prompt portions: 64-row tiles on the matrix cores
        ts, tq = [], []
        for b, ln in enumerate(lens):
            for q0 in range(0, ln, 64):
                ts.append(b)
                tq.append(q0)
        tile_seq = torch.tensor(ts, dtype=torch.int32, device=q.device)
        tile_q0 = torch.tensor(tq, dtype=torch.int32, device=q.device)
        rc = _L().afm_attn_prefill_mfma(
            _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vsrc),
            _lib.ptr(md.block_table), _lib.ptr(md.cu_seqlens),
            _lib.ptr(md.q_start), _lib.ptr(tile_seq), _lib.ptr(tile_q0),
            float(scale), len(ts), H, G, dk, dv, page,
            md.block_table.shape[1], int(chunk), int(window), _rowstride(q),
            *extra, _lib.cur_stream())
        if rc != 9004:          # 9004: no tile kernel for this head geometry
            _lib.check(rc, "afm_attn_prefill_mfma")
            return out
    reach = min(x for x in (chunk, window, md.block_table.shape[1] * page)
                if x > 0) + keep_first
    if (q.dtype == torch.bfloat16 and H // G >= HEADS_MFMA_MIN and dk <= 576
            and dv <= 512):
        # single rows whose many heads share a K/V head: the heads are the
        # rows of the matrix-core tiles; key splits of 64-key multiples
        wgs = T * G * -(-(H // G) // 16)
        nsplit = max(1, min(16, 2048 // max(1, wgs), -(-reach // 64)))
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty(T, H, nsplit, dv, dtype=torch.float32,
                                 device=q.device)
            part_ml = torch.empty(T, H, nsplit, 2, dtype=torch.float32,
                                  device=q.device)
        rc = _L().afm_attn_heads_mfma(
            _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vsrc),
            _lib.ptr(md.block_table), _lib.ptr(md.row_seq),
            _lib.ptr(positions), float(scale), T, H, G, dk, dv, page,
            md.block_table.shape[1], int(chunk), int(window), _rowstride(q),
            nsplit, _lib.ptr(part_o), _lib.ptr(part_ml), *extra,
            _lib.cur_stream())
        if rc != 9004:
            _lib.check(rc, "afm_attn_heads_mfma")
            if nsplit > 1:
                rc = _L().afm_attn_split_combine(
                    _lib.ptr(out), _lib.ptr(part_o), _lib.ptr(part_ml), T * H,
                    nsplit, dv, _code(q), _lib.cur_stream())
                _lib.check(rc, "afm_attn_split_combine")
            return out
    # few rows and many visible keys: cut the keys over several workgroups
    # (about 2048 in flight) and merge the partial softmaxes
    per_wg_heads = min(8, max(1, H // G))
    wgs = T * G * -(-(H // G) // per_wg_heads)
    nsplit = max(1, min(8, 2048 // max(1, wgs), reach // 128))
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty(T, H, nsplit, dv, dtype=torch.float32,
                             device=q.device)
        part_ml = torch.empty(T, H, nsplit, 2, dtype=torch.float32,
                              device=q.device)
    rc = _L().afm_masked_attention(
        _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vsrc),
        _lib.ptr(md.block_table), _lib.ptr(md.row_seq), _lib.ptr(positions),
        float(scale), T, H, G, dk, dv, page, md.block_table.shape[1],
        int(chunk), int(window), _rowstride(q), nsplit, _lib.ptr(part_o),
        _lib.ptr(part_ml), *extra, _code(q), _lib.cur_stream())
    _lib.check(rc, "afm_masked_attention")
    return out


# ---------------------------------------------------------- linear recurrence
def rotary_inv_freq(dims: int, base: float, device) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, fp32 (evaluated in fp64)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).float().to(device)


def linear_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                state: torch.Tensor, md, positions: torch.Tensor,
                heads: int, q_scale: float = 1.0, k_scale: float = 1.0,
                head_decay: torch.Tensor | None = None,
                decay_logits: torch.Tensor | None = None,
                decay_bias: torch.Tensor | None = None,
                inv_tau: float = 1.0,
                inv_freq: torch.Tensor | None = None) -> torch.Tensor:
    """Decayed outer-product recurrence, token by token, fp32:

        S_t = diag(a_t) S_{t-1} + k_t v_t^T,   o_t = S_t^T q_t     per head

    with S [dk, dv] living in `state` [slots, H, dk, dv] fp32 (read unless
    the chunk starts at position 0, written back after the chunk's last row).
    Decay a_t is either one constant per head (head_decay [H] fp32) or one
    value per key channel, sigmoid(z_t + bias)^(inv_tau) from decay_logits
    z [T, H*dk].  inv_freq [r/2] switches on rotate-half rotary embedding of
    the first r dims of q and k (angle = position * f_i, fp32); q_scale and
    k_scale multiply q and k afterwards.  Returns o [T, H*dv] fp32."""
    T = q.shape[0]
    H = heads
    dk = q.shape[1] // H
    dv = v.shape[1] // H
    if not _gpu(q):
        qf = q.float().reshape(T, H, dk).clone()
        kf = k.float().reshape(T, H, dk).clone()
        vf = v.float().reshape(T, H, dv)
        if inv_freq is not None:
            r2 = inv_freq.numel()
            ang = positions.float()[:, None] * inv_freq.float()[None]
            c, s = ang.cos()[:, None], ang.sin()[:, None]
            for t_ in (qf, kf):
                u = t_[..., :r2].clone()
                w = t_[..., r2:2 * r2].clone()
                t_[..., :r2] = u * c - w * s
                t_[..., r2:2 * r2] = w * c + u * s
        qf *= q_scale
        kf *= k_scale
        if decay_logits is not None:
            z = decay_logits.float() + decay_bias.float()
            a = torch.exp(torch.nn.functional.logsigmoid(z) * inv_tau)
            a = a.view(T, H, dk, 1)
        else:
            a = head_decay.float().view(1, H, 1, 1).expand(T, H, 1, 1)
        out = torch.empty(T, H, dv, dtype=torch.float32)
        cu, qs, sl = (md.cu_seqlens.tolist(), md.q_start.tolist(),
                      md.state_slots.tolist())
        for b in range(len(qs)):
            if cu[b + 1] == cu[b]:
                continue
            S = state[sl[b]].clone() if qs[b] > 0 else \
                torch.zeros(H, dk, dv)
            for t in range(cu[b], cu[b + 1]):
                S = a[t] * S + kf[t][:, :, None] * vf[t][:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S, qf[t])
            state[sl[b]] = S
        return out.view(T, H * dv)
    out = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
    B = md.q_start.numel()
    rot = 2 * inv_freq.numel() if inv_freq is not None else 0
    rc = _L().afm_linear_scan(
        _lib.ptr(out), _lib.ptr(state), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v),
        _lib.ptr(decay_logits), _lib.ptr(decay_bias), _lib.ptr(head_decay),
        _lib.ptr(inv_freq), _lib.ptr(positions), _lib.ptr(md.cu_seqlens),
        _lib.ptr(md.q_start), _lib.ptr(md.state_slots),
        float(q_scale), float(k_scale), float(inv_tau), B, H, dk, dv, rot,
        _rowstride(q), _rowstride(k), _rowstride(v),
        _rowstride(decay_logits) if decay_logits is not None else 0,
        _code(q), _lib.cur_stream())
    _lib.check(rc, "afm_linear_scan")
    return out


def headnorm_gate(o: torch.Tensor, g: torch.Tensor,
                  weight: torch.Tensor | None, eps: float, heads: int,
                  out_dtype: torch.dtype,
                  gate_act: str = "silu") -> torch.Tensor:
    """Per-head RMSNorm of o [T, H*dv] fp32 (optional plain weight [dv]
    shared by heads) times silu(g) (gate_act "sigmoid": times sigmoid(g));
    g [T, H*dv] may be a strided view."""
    T, HD = o.shape
    dv = HD // heads
    if not _gpu(o):
        of = o.view(T, heads, dv)
        of = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            of = of * weight.float()
        gf = g.float()
        gate = torch.sigmoid(gf) if gate_act == "sigmoid" else \
            gf * torch.sigmoid(gf)
        return (of.reshape(T, HD) * gate).to(out_dtype)
    out = torch.empty(T, HD, dtype=out_dtype, device=o.device)
    rc = _L().afm_headnorm_gate(_lib.ptr(out), _lib.ptr(o), _lib.ptr(g),
                                _lib.ptr(weight), float(eps), T, heads, dv,
                                _rowstride(g),
                                1 if gate_act == "sigmoid" else 0, _code(out),
                                _lib.cur_stream())
    _lib.check(rc, "afm_headnorm_gate")
    return out


# ------------------------------------------------------------ feed-forward
def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """PolyNorm activation per row: c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3,
    N(u) = u / sqrt(mean(u^2) + eps) over the row; coef [4] fp32."""
    T, F = z.shape
    if not _gpu(z):
        zf = z.float()
        c = coef.float()

        def n(u):
            return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
        return (c[0] * n(zf) + c[1] * n(zf * zf) + c[2] * n(zf * zf * zf)
                + c[3]).to(z.dtype)
    out = torch.empty(T, F, dtype=z.dtype, device=z.device)
    rc = _L().afm_polynorm(_lib.ptr(out), _lib.ptr(z), _lib.ptr(coef),
                           float(eps), T, F, _rowstride(z), _code(z),
                           _lib.cur_stream())
    _lib.check(rc, "afm_polynorm")
    return out


def gated_residual(x: torch.Tensor, a: torch.Tensor, a_scale: float,
                   b: torch.Tensor | None, b_scale: float,
                   gate1: torch.Tensor, bias1: torch.Tensor,
                   m: torch.Tensor | None = None,
                   gate2: torch.Tensor | None = None,
                   bias2: torch.Tensor | None = None) -> torch.Tensor:
    """In place on the fp32 residual:
    x += sigmoid(gate1 + bias1) * (a_scale*a + b_scale*b)
       + sigmoid(gate2 + bias2) * m          (b and the m term optional).
    gate1/gate2 may be strided views; biases fp32 [W]."""
    T, W = x.shape
    if not _gpu(x):
        mix = a_scale * a.float()
        if b is not None:
            mix = mix + b_scale * b.float()
        x += torch.sigmoid(gate1.float() + bias1.float()) * mix
        if m is not None:
            x += torch.sigmoid(gate2.float() + bias2.float()) * m.float()
        return x
    rc = _L().afm_gated_residual(
        _lib.ptr(x), _lib.ptr(a), float(a_scale), _lib.ptr(b), float(b_scale),
        _lib.ptr(gate1), _rowstride(gate1), _lib.ptr(bias1), _lib.ptr(m),
        _lib.ptr(gate2), _rowstride(gate2) if gate2 is not None else 0,
        _lib.ptr(bias2), T, W, _code(a), _lib.cur_stream())
    _lib.check(rc, "afm_gated_residual")
    return x


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(logits / cap) as fp32 (cap <= 0: plain fp32 copy)."""
    if not _gpu(logits):
        lf = logits.float()
        return cap * torch.tanh(lf / cap) if cap > 0 else lf
    logits = logits.contiguous()
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    rc = _L().afm_softcap(_lib.ptr(out), _lib.ptr(logits), float(cap),
                          logits.numel(), _code(logits), _lib.cur_stream())
    _lib.check(rc, "afm_softcap")
    return out


def matmul(x: torch.Tensor, w: torch.Tensor,
           skinny: bool = True) -> torch.Tensor:
    """x [M, K] @ w [N, K]^T through the vendor GEMM (hipBLASLt / rocBLAS);
    fp32 operands run in true fp32 (no reduced-precision matrix mode).

    AF_MIX_SKINNY=1 sends decode-sized bf16 products (<= 64 rows, N and K
    multiples of 64) to the framework's MFMA skinny-GEMM kernel instead, with
    the per-shape policy ops.linear uses for the Llama family.  Measured on
    MI355X for this family the two are equal in GEMM time (1.33 vs 1.34 ms
    per 64-row step at width 2048, and the same tokens/s at width 4096) while
    the skinny path adds a combine launch per product, so the vendor GEMM is
    the default."""
    M, K = x.shape
    N = w.shape[0]
    if (skinny and _SKINNY and x.is_cuda and x.dtype == torch.bfloat16
            and N % 64 == 0 and K % 64 == 0
            and ((M <= 64 and K <= 8192)
                 or (32 < M <= 128 and K >= 8192 and N <= 8192))
            and x.is_contiguous() and w.is_contiguous()
            and _lib.main_lib_ready()):
        from . import linear_skinny
        return linear_skinny(x, w)
    return x @ w.t()


# =====================================================================
# Ops of post-norm hybrid decoders: sublayers read the residual itself, a
# norm sits on each sublayer's output; selective state-space mixer, sigmoid
# attention with distance bias and head mixing, gated units, sigmoid router.
# =====================================================================
def cast_rows(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The fp32 residual in the storage dtype (itself when that is fp32)."""
    if x.dtype == dtype:
        return x
    if not _gpu(x):
        return x.to(dtype)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    rc = _L().afm_cast_rows(_lib.ptr(out), _lib.ptr(x), x.numel(), _code(out),
                            _lib.cur_stream())
    _lib.check(rc, "afm_cast_rows")
    return out


def norm_residual(x: torch.Tensor, y: torch.Tensor,
                  bias: torch.Tensor | None, w: torch.Tensor, eps: float,
                  dtype: torch.dtype) -> torch.Tensor:
    """In place on the fp32 residual: u = y (+ bias); x += u / rms(u) * w.
    y [T, W] is in the storage dtype or fp32.  Returns the new residual in
    `dtype` (x itself for fp32), the next sublayer's input."""
    T, W = x.shape
    if not _gpu(x):
        u = y.float()
        if bias is not None:
            u = u + bias.float()
        x += u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        return x.to(dtype) if dtype != torch.float32 else x
    h = None if dtype == torch.float32 else \
        torch.empty(T, W, dtype=dtype, device=x.device)
    rc = _L().afm_norm_residual(
        _lib.ptr(x), _lib.ptr(h), _lib.ptr(y), _rowstride(y),
        1 if y.dtype == torch.float32 else 0, _lib.ptr(bias), _lib.ptr(w),
        float(eps), T, W, _code(w), _lib.cur_stream())
    _lib.check(rc, "afm_norm_residual")
    return x if h is None else h


GLU_ACTS = {"silu": 0, "relu": 1, "gelu_tanh": 2, "clamped": 3}


def _act(name: str, a: torch.Tensor) -> torch.Tensor:
    if name == "silu":
        return a * torch.sigmoid(a)
    if name == "relu":
        return torch.relu(a)
    return 0.5 * a * (1.0 + torch.tanh(
        0.7978845608028654 * (a + 0.044715 * a ** 3)))


def glu(gu: torch.Tensor, F: int, act: str,
        bias: torch.Tensor | None = None, units: int = 1,
        row_weight: torch.Tensor | None = None,
        out: torch.Tensor | None = None, limit: float = 0.0) -> torch.Tensor:
    """act(gate + bg) * (up + bu) (* row_weight) for `units` gated units
    laid side by side in every row of gu [T, >= units*2F], unit e being
    [gate_e (F) | up_e (F)].  bias [2F] = [bg | bu] (units == 1 only);
    row_weight [T, units] fp32.  act "clamped" is the bounded unit g' *
    sigmoid(1.702 g') * (u' + 1) with g' = min(gate, limit), u' = clamp(up,
    -limit, limit).  Writes out [T, >= units*F] (allocated [T, units*F] when
    not given)."""
    T = gu.shape[0]
    if out is None:
        out = torch.empty(T, units * F, dtype=gu.dtype, device=gu.device)
    if not _gpu(gu):
        v = gu[:, :units * 2 * F].float().reshape(T, units, 2 * F)
        g, u = v[..., :F], v[..., F:]
        if bias is not None:
            g, u = g + bias[:F].float(), u + bias[F:].float()
        if act == "clamped":
            g = g.clamp(max=limit)
            o = g * torch.sigmoid(1.702 * g) * (u.clamp(-limit, limit) + 1.0)
        else:
            o = _act(act, g) * u
        if row_weight is not None:
            o = o * row_weight.float().reshape(T, units, 1)
        out[:, :units * F] = o.reshape(T, units * F).to(out.dtype)
        return out
    rc = _L().afm_glu(
        _lib.ptr(out), _rowstride(out), F, _lib.ptr(gu),
        ctypes.c_void_p(gu.data_ptr() + F * gu.element_size()),
        _rowstride(gu), 2 * F, units,
        _lib.ptr(bias[:F]) if bias is not None else None,
        _lib.ptr(bias[F:]) if bias is not None else None,
        _lib.ptr(row_weight), T * units, F, GLU_ACTS[act], float(limit),
        _code(gu), _lib.cur_stream())
    _lib.check(rc, "afm_glu")
    return out


def moe_route(z: torch.Tensor, correction: torch.Tensor | None, top: int,
              n_groups: int = 0, keep: int = 0, scale: float = 1.0,
              dense: bool = False, score: str = "sigmoid",
              renorm: bool = True):
    """Router with score correction and group-limited top-k.

    z [T, E] fp32 logits; s = sigmoid(z) (score "softmax": softmax(z) over
    all experts); choice = s + correction.  With
    n_groups > 0 the experts form equal groups of neighbours, a group scores
    the sum of its two largest choice scores and only experts of the `keep`
    best groups can be chosen.  The `top` largest choice scores win; weights
    = s / (sum of the chosen s + 1e-20) * scale (renorm False: s * scale).
    Returns (idx [T, top] i32,
    weights [T, top] fp32, dense weights [T, E] fp32 or None)."""
    T, E = z.shape
    if not _gpu(z):
        s = torch.softmax(z.float(), -1) if score == "softmax" else \
            torch.sigmoid(z.float())
        choice = s + correction.float() if correction is not None else s.clone()
        if n_groups > 0 and keep < n_groups:
            size = E // n_groups
            gs = choice.view(T, n_groups, size).topk(min(2, size), -1)[0].sum(-1)
            kept = torch.zeros(T, n_groups, dtype=torch.bool)
            kept.scatter_(1, gs.topk(keep, -1)[1], True)
            choice = choice.masked_fill(
                ~kept.repeat_interleave(size, dim=1), -math.inf)
        idx = choice.topk(top, -1)[1]
        w = s.gather(1, idx)
        w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale if renorm \
            else w * scale
        wd = None
        if dense:
            wd = torch.zeros(T, E).scatter_(1, idx, w)
        return idx.to(torch.int32), w, wd
    z = z.contiguous()
    idx = torch.empty(T, top, dtype=torch.int32, device=z.device)
    w = torch.empty(T, top, dtype=torch.float32, device=z.device)
    wd = torch.empty(T, E, dtype=torch.float32, device=z.device) \
        if dense else None
    rc = _L().afm_moe_route(_lib.ptr(idx), _lib.ptr(w), _lib.ptr(wd),
                            _lib.ptr(z), _lib.ptr(correction), T, E, top,
                            int(n_groups), int(keep), float(scale),
                            1 if score == "softmax" else 0,
                            1 if renorm else 0, _lib.cur_stream())
    _lib.check(rc, "afm_moe_route")
    return idx, w, wd


def moe_combine(ys: torch.Tensor, pos: torch.Tensor, weights: torch.Tensor,
                shared: torch.Tensor | None) -> torch.Tensor:
    """y[t] = sum_r weights[t, r] * ys[pos[t*top + r]] (+ shared[t]), fp32,
    summed in the order r = 0..top-1.  ys [T*top, W] holds the experts'
    outputs in expert-sorted order, pos [T*top] i32 the place of every
    (token, choice) in it."""
    T, top = weights.shape
    W = ys.shape[1]
    if not _gpu(ys):
        y = (ys.float()[pos.long()].view(T, top, W)
             * weights.float()[:, :, None])
        out = shared.float().clone() if shared is not None else \
            torch.zeros(T, W)
        for r in range(top):
            out += y[:, r]
        return out
    out = torch.empty(T, W, dtype=torch.float32, device=ys.device)
    rc = _L().afm_moe_combine(_lib.ptr(out), _lib.ptr(ys), _lib.ptr(pos),
                              _lib.ptr(weights), _lib.ptr(shared), T, top, W,
                              _code(ys), _lib.cur_stream())
    _lib.check(rc, "afm_moe_combine")
    return out


# ------------------------------------------------- selective state space
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None,
                state: torch.Tensor, md, silu: bool = True) -> torch.Tensor:
    """Depthwise causal convolution over packed chunks: out[t, c] = act(b[c]
    + sum_j w[j, c] x[t - (taps-1-j), c]); w is tap-major [taps, C], its last
    row weighing the current token.  Inputs from before a chunk come from the sequence's slot
    of `state` [slots, taps-1, C] (storage dtype, oldest first), inputs
    before position 0 are zero; afterwards the slot holds the sequence's last
    taps-1 inputs.  x [T, C] may be a strided view."""
    T, C = x.shape
    taps = w.shape[0]
    B = md.q_start.numel()
    if not _gpu(x):
        out = torch.empty(T, C, dtype=torch.float32)
        cu, qs, sl = (md.cu_seqlens.tolist(), md.q_start.tolist(),
                      md.state_slots.tolist())
        wf = w.float()
        for b in range(B):
            r0, r1 = cu[b], cu[b + 1]
            if r1 == r0:
                continue
            hist = state[sl[b]][:taps - 1].float() if qs[b] > 0 else \
                torch.zeros(taps - 1, C)
            cat = torch.cat([hist, x[r0:r1].float()], 0)
            acc = torch.zeros(r1 - r0, C)
            if bias is not None:
                acc += bias.float()
            for j in range(taps):
                acc += wf[j] * cat[j:j + r1 - r0]
            out[r0:r1] = acc
            if taps > 1:
                state[sl[b]][:taps - 1] = cat[-(taps - 1):].to(state.dtype)
        if silu:
            out = out * torch.sigmoid(out)
        return out.to(x.dtype)
    out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    rc = _L().afm_causal_conv(
        _lib.ptr(out), _lib.ptr(x), _rowstride(x), _lib.ptr(w),
        _lib.ptr(bias), _lib.ptr(state), _lib.ptr(md.row_seq),
        _lib.ptr(md.cu_seqlens), _lib.ptr(md.q_start),
        _lib.ptr(md.state_slots), T, B, C, taps, 1 if silu else 0, _code(x),
        _lib.cur_stream())
    _lib.check(rc, "afm_causal_conv")
    return out


def selective_scan(x: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor,
                   bc: torch.Tensor, N: int, z: torch.Tensor,
                   A: torch.Tensor, D: torch.Tensor, state: torch.Tensor,
                   md) -> torch.Tensor:
    """Selective scan, token by token in fp32, per channel c and state n:

        d = softplus(dt[t, c] + dt_bias[c])
        S[c, n] <- exp(d A[c, n]) S[c, n] + d x[t, c] B[t, n]
        y[t, c] = (sum_n S[c, n] C[t, n] + D[c] x[t, c]) * silu(z[t, c])

    bc [T, >= 2N] holds [B | C] per row (may be a strided view, as may z);
    A [C, N], D [C] fp32; state [slots, C, N] fp32 is read unless the chunk
    starts at position 0 and written after the chunk's last row."""
    T, C = x.shape
    B = md.q_start.numel()
    if not _gpu(x):
        d = torch.nn.functional.softplus(dt.float() + dt_bias.float(),
                                         threshold=20.0)
        xf, zf = x.float(), z.float()
        Bm, Cm = bc[:, :N].float(), bc[:, N:2 * N].float()
        y = torch.empty(T, C, dtype=torch.float32)
        cu, qs, sl = (md.cu_seqlens.tolist(), md.q_start.tolist(),
                      md.state_slots.tolist())
        for b in range(B):
            if cu[b + 1] == cu[b]:
                continue
            S = state[sl[b]].clone() if qs[b] > 0 else torch.zeros(C, N)
            for t in range(cu[b], cu[b + 1]):
                S = torch.exp(d[t][:, None] * A) * S + \
                    (d[t] * xf[t])[:, None] * Bm[t][None]
                y[t] = S @ Cm[t] + D * xf[t]
            state[sl[b]] = S
        return (y * zf * torch.sigmoid(zf)).to(x.dtype)
    out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    rc = _L().afm_selective_scan(
        _lib.ptr(out), _lib.ptr(state), _lib.ptr(x.contiguous()),
        _lib.ptr(dt.contiguous()), _lib.ptr(dt_bias), _lib.ptr(bc),
        _rowstride(bc), _lib.ptr(z), _rowstride(z), _lib.ptr(A), _lib.ptr(D),
        _lib.ptr(md.cu_seqlens), _lib.ptr(md.q_start),
        _lib.ptr(md.state_slots), B, C, N, _code(x), _lib.cur_stream())
    _lib.check(rc, "afm_selective_scan")
    return out


# ------------------------------------------------------ sigmoid attention
def distance_buckets(rows: int, dmax: float) -> torch.Tensor:
    """Bucket of every distance below dmax for a learned distance bias with
    `rows` rows: n itself below rows/2, then logarithmic steps that reach the
    last row at dmax; distances from dmax on all take the last row (callers
    clamp).  i32 [ceil(dmax)], evaluated in double precision on the host."""
    half = rows // 2
    out = []
    for n in range(max(int(math.ceil(dmax)), half)):
        if n < half:
            out.append(n)
            continue
        if dmax <= half or half == 0:      # no logarithmic range at all
            out.append(rows - 1)
            continue
        v = math.log(n / half) / math.log(dmax / half) * (rows - half)
        out.append(min(rows - 1, half + int(math.floor(v + 1e-9))))
    return torch.tensor(out or [rows - 1], dtype=torch.int32)


def qk_unit_cache(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  heads: int, kv_heads: int, eps: float,
                  kcache: torch.Tensor, vcache: torch.Tensor,
                  slots: torch.Tensor, positions: torch.Tensor,
                  temp_coef: float = 0.0, temp_every: int = 0,
                  v_first: torch.Tensor | None = None,
                  lam: float = 0.0) -> torch.Tensor:
    """Per head: q and k divided by their root mean square (no weight); q
    times 1 + temp_coef * ln(floor((p+1)/temp_every) + 1) at position p
    (temp_every 0: no temperature); v <- (1-lam) v + lam v_first when v_first
    is given.  k and v are appended to the paged caches at `slots`.  Inputs
    may be strided views.  Returns q, contiguous [T, H*dk]."""
    T = q.shape[0]
    H, G = heads, kv_heads
    dk = q.shape[1] // H
    dv = v.shape[1] // G
    page = kcache.shape[2]
    if not _gpu(q):
        qf = q.float().reshape(T, H, dk)
        kf = k.float().reshape(T, G, dk)
        qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps)
        kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps)
        if temp_every > 0:
            steps = torch.div(positions + 1, temp_every,
                              rounding_mode="floor").float()
            qf = qf * (1.0 + temp_coef * torch.log(steps + 1.0))[:, None, None]
        vf = v.float()
        if v_first is not None:
            vf = (1.0 - lam) * vf + lam * v_first.float()
        pg = torch.div(slots, page, rounding_mode="floor")
        off = slots - pg * page
        kcache[pg, :, off] = kf.to(kcache.dtype)
        vcache[pg, :, off] = vf.reshape(T, G, dv).to(vcache.dtype)
        return qf.reshape(T, H * dk).to(q.dtype)
    out = torch.empty(T, H * dk, dtype=q.dtype, device=q.device)
    rc = _L().afm_qk_unit_cache(
        _lib.ptr(out), _lib.ptr(q), _rowstride(q), _lib.ptr(k), _rowstride(k),
        _lib.ptr(v), _rowstride(v), _lib.ptr(v_first),
        _rowstride(v_first) if v_first is not None else 0, float(lam),
        _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(slots),
        _lib.ptr(positions), float(eps), float(temp_coef), int(temp_every),
        T, H, G, dk, dv, page, _code(q), _lib.cur_stream())
    _lib.check(rc, "afm_qk_unit_cache")
    return out


def sigmoid_attention(q: torch.Tensor, kcache: torch.Tensor,
                      vcache: torch.Tensor, md, positions: torch.Tensor,
                      scale: float, heads: int,
                      rel: torch.Tensor | None = None,
                      buckets: torch.Tensor | None = None,
                      talk: torch.Tensor | None = None,
                      head_bias: torch.Tensor | None = None,
                      gate: torch.Tensor | None = None,
                      window: int = 0) -> torch.Tensor:
    """Attention with un-normalised sigmoid weights over the paged cache.
    For the row at position i and every key j <= i (and j > i - window when
    window > 0), per head h:

        s_h = q_h . k_g(h) * scale + rel[bucket(i - j), h]
        m_h = sum_g talk[h, g] s_g                 (all heads of the pair)
        o_h = sum_j sigmoid(m_h + head_bias[h]) v_j,   o_h *= sigmoid(gate_h)

    rel [rows, H], talk [H, H], head_bias [H] fp32 (each optional); buckets
    i32 from distance_buckets (distances past its end use the last row);
    gate [T, H] logits in the storage dtype (may be a strided view).
    q [T, H*dk] -> [T, H*dv]."""
    T = q.shape[0]
    _, G, page, dk = kcache.shape
    dv = vcache.shape[3]
    H = heads
    RB = rel.shape[0] if rel is not None else 0
    if not _gpu(q):
        out = torch.zeros(T, H, dv, dtype=torch.float32)
        qf = q.float().view(T, H, dk)
        bt = md.block_table.long()
        rs = md.row_seq.tolist()
        pos = positions.tolist()
        for t in range(T):
            i = pos[t]
            lo = max(0, i - window + 1) if window > 0 else 0
            js = torch.arange(lo, i + 1)
            pg = bt[rs[t]][js // page]
            kk = kcache[pg, :, js % page].float()      # [n, G, dk]
            vv = vcache[pg, :, js % page].float()
            kk = kk.repeat_interleave(H // G, dim=1)
            vv = vv.repeat_interleave(H // G, dim=1)
            s = torch.einsum("nhd,hd->hn", kk, qf[t]) * scale
            if rel is not None:
                dist = (i - js).clamp(max=buckets.numel())
                bk = torch.cat([buckets.long(),
                                torch.tensor([RB - 1])])[dist]
                s = s + rel.float()[bk].t()
            if talk is not None:
                s = talk.float() @ s
            if head_bias is not None:
                s = s + head_bias.float()[:, None]
            out[t] = torch.einsum("hn,nhd->hd", torch.sigmoid(s), vv)
        if gate is not None:
            out = out * torch.sigmoid(gate.float())[:, :, None]
        return out.view(T, H * dv).to(q.dtype)
    out = torch.empty(T, H * dv, dtype=q.dtype, device=q.device)
    lens = getattr(md, "seq_lens", None)
    if (q.dtype == torch.bfloat16 and lens is not None and window == 0
            and dk <= 128 and dv <= 128 and H <= 32
            and max(lens) >= MFMA_MIN_ROWS):
        # prompt portions: 16-row tiles x all heads on the matrix cores
        # (falls back to the row kernel when LDS cannot hold a tile)
        ts, tq = [], []
        for b, ln in enumerate(lens):
            for q0 in range(0, ln, 16):
                ts.append(b)
                tq.append(q0)
        tile_seq = torch.tensor(ts, dtype=torch.int32, device=q.device)
        tile_q0 = torch.tensor(tq, dtype=torch.int32, device=q.device)
        rc = _L().afm_sigattn_prefill_mfma(
            _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache),
            _lib.ptr(md.block_table), _lib.ptr(md.cu_seqlens),
            _lib.ptr(md.q_start), _lib.ptr(tile_seq), _lib.ptr(tile_q0),
            _lib.ptr(rel), _lib.ptr(buckets),
            buckets.numel() if buckets is not None else 0, RB,
            _lib.ptr(talk), _lib.ptr(head_bias), _lib.ptr(gate),
            _rowstride(gate) if gate is not None else 0, float(scale),
            len(ts), H, G, dk, dv, page, md.block_table.shape[1],
            _lib.cur_stream())
        if rc != 9004:          # 9004: a tile does not fit in LDS
            _lib.check(rc, "afm_sigattn_prefill_mfma")
            return out
    # few rows and a long reach: cut each row's keys over several workgroups
    reach = md.block_table.shape[1] * page
    if window > 0:
        reach = min(reach, window)
    nsplit = max(1, min(32, 2048 // max(1, T), reach // 64))
    part = torch.empty(T, nsplit, H * dv, dtype=torch.float32,
                       device=q.device)
    rc = _L().afm_sigmoid_attention(
        _lib.ptr(out), _lib.ptr(part), _lib.ptr(q), _lib.ptr(kcache),
        _lib.ptr(vcache), _lib.ptr(md.block_table), _lib.ptr(md.row_seq),
        _lib.ptr(positions), _lib.ptr(rel), _lib.ptr(buckets),
        buckets.numel() if buckets is not None else 0, RB, _lib.ptr(talk),
        _lib.ptr(head_bias), _lib.ptr(gate),
        _rowstride(gate) if gate is not None else 0, float(scale), T, H, G,
        dk, dv, page, md.block_table.shape[1], nsplit, int(window), _code(q),
        _lib.cur_stream())
    _lib.check(rc, "afm_sigmoid_attention")
    return out


# =====================================================================
# Ops of hyper-connected decoders: several fp32 residual streams per token
# mixed by learned matrices, a norm and a short causal convolution in front
# of every sublayer, latent attention (one normed latent + one rotary key
# part per token in the pages), squared-ReLU feed-forward.
# =====================================================================
def embed_streams(ids: torch.Tensor, table: torch.Tensor,
                  streams: int) -> torch.Tensor:
    """x[t, s] = table[ids[t]] for every stream s: fp32 [T, streams, W]."""
    T, W = ids.numel(), table.shape[1]
    if not _gpu(table):
        return table[ids.long()].float()[:, None, :].repeat(1, streams, 1)
    x = torch.empty(T, streams, W, dtype=torch.float32, device=table.device)
    rc = _L().afm_embed_streams(_lib.ptr(x), _lib.ptr(table), _lib.ptr(ids), T,
                                streams, W, _code(table), _lib.cur_stream())
    _lib.check(rc, "afm_embed_streams")
    return x


def hyper_step(x: torch.Tensor, y: torch.Tensor | None,
               mix: torch.Tensor | None, out_w: torch.Tensor | None,
               in_w: torch.Tensor | None, norm_w: torch.Tensor | None,
               eps: float, _tail: tuple | None = None) -> torch.Tensor | None:
    """One step of the stream mixer, in place on x [T, S, W] fp32.

    With y [T, W] (a sublayer's output): every stream at once from the old
    ones, x_r <- sum_s mix[s, r] x_s + out_w[r] y.  With in_w [S]: returns
    u = sum_r in_w[r] x_r of the (updated) streams as fp32 [T, W], RMS-normed
    as u / rms(u) * (1 + norm_w) when norm_w is given.  mix [S, S], out_w and
    in_w are fp32."""
    T, S, W = x.shape
    if not _gpu(x):
        if y is not None:
            x.copy_(torch.einsum("sr,tsw->trw", mix.float(), x)
                    + out_w.float()[None, :, None] * y.float()[:, None, :])
        if in_w is None:
            return None
        u = torch.einsum("s,tsw->tw", in_w.float(), x)
        if norm_w is not None:
            u = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) \
                * (1.0 + norm_w.float())
        return u
    n = torch.empty(T, W, dtype=torch.float32, device=x.device) \
        if in_w is not None else None
    ref = y if y is not None else norm_w
    h = None
    tail = (None, None, None, None, 0, None)
    if _tail is not None:
        conv_w, state, md, positions = _tail
        h = torch.empty(T, W, dtype=conv_w.dtype, device=x.device)
        tail = (_lib.ptr(conv_w), _lib.ptr(state), _lib.ptr(md.state_slots),
                _lib.ptr(positions), conv_w.shape[1], _lib.ptr(h))
    rc = _L().afm_hyper_step(
        _lib.ptr(x), _lib.ptr(y), _rowstride(y) if y is not None else 0,
        _lib.ptr(mix), _lib.ptr(out_w), _lib.ptr(in_w), _lib.ptr(norm_w),
        float(eps), _lib.ptr(n), T, S, W, 1 if norm_w is not None else 0,
        *tail, _code(ref) if ref is not None else 1, _lib.cur_stream())
    _lib.check(rc, "afm_hyper_step")
    return n if h is None else h


def hyper_conv_step(x: torch.Tensor, y: torch.Tensor | None,
                    mix: torch.Tensor | None, out_w: torch.Tensor | None,
                    in_w: torch.Tensor, norm_w: torch.Tensor, eps: float,
                    conv_w: torch.Tensor, state: torch.Tensor, md,
                    positions: torch.Tensor,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """hyper_step (write y in, read the next input out, norm) followed by
    canon_conv: a sublayer's input in out_dtype.  Steps of one row per
    sequence (decode) run as a single kernel on GPU."""
    if _gpu(x) and not getattr(md, "is_prefill", True) \
            and conv_w.dtype == out_dtype and norm_w.dtype == out_dtype:
        return hyper_step(x, y, mix, out_w, in_w, norm_w, eps,
                          _tail=(conv_w, state, md, positions))
    n = hyper_step(x, y, mix, out_w, in_w, norm_w, eps)
    return canon_conv(n, conv_w, state, md, out_dtype)


def canon_conv(n: torch.Tensor, w: torch.Tensor, state: torch.Tensor, md,
               out_dtype: torch.dtype) -> torch.Tensor:
    """h[t] = n[t] + sum_j w[:, j] n[t - (taps-1-j)]: a depthwise causal
    convolution over time added to its own input.  n [T, W] fp32 packed
    chunks, w [W, taps].  Inputs from before a chunk come from the sequence's
    slot of `state` [slots, max(taps-1, 1), W] fp32 (oldest first), inputs
    before position 0 are zero; afterwards the slot holds the sequence's last
    taps-1 inputs.  Returns h in out_dtype."""
    T, W = n.shape
    taps = w.shape[1]
    B = md.q_start.numel()
    if not _gpu(n):
        out = torch.empty(T, W, dtype=torch.float32)
        cu, qs, sl = (md.cu_seqlens.tolist(), md.q_start.tolist(),
                      md.state_slots.tolist())
        wf = w.float()
        for b in range(B):
            r0, r1 = cu[b], cu[b + 1]
            if r1 == r0:
                continue
            hist = state[sl[b]][:taps - 1].clone()
            if qs[b] < taps - 1:      # places before position 0
                hist[:taps - 1 - qs[b]] = 0.0
            cat = torch.cat([hist, n[r0:r1]], 0)
            acc = n[r0:r1].clone()
            for j in range(taps):
                acc += wf[:, j] * cat[j:j + r1 - r0]
            out[r0:r1] = acc
            if taps > 1:
                state[sl[b]][:taps - 1] = cat[-(taps - 1):]
        return out.to(out_dtype)
    h = torch.empty(T, W, dtype=out_dtype, device=n.device)
    if w.dtype != out_dtype:
        raise TypeError("canon_conv: weights must be in the output dtype")
    rc = _L().afm_canon_conv(
        _lib.ptr(h), _lib.ptr(n), _lib.ptr(w), _lib.ptr(state),
        _lib.ptr(md.row_seq), _lib.ptr(md.cu_seqlens), _lib.ptr(md.q_start),
        _lib.ptr(md.state_slots), T, B, W, taps, _code(h), _lib.cur_stream())
    _lib.check(rc, "afm_canon_conv")
    return h


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor,
                 inv_freq: torch.Tensor) -> torch.Tensor:
    """Interleaved rotary embedding of the leading 2*len(inv_freq) elements
    of the last axis (element 2i pairs with 2i+1; angle = position * f_i);
    x [T, ..., d] fp32, CPU helper of latent_prep."""
    r = 2 * inv_freq.numel()
    ang = positions.float()[:, None] * inv_freq.float()[None]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [r // 2]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    u, v = x[..., 0:r:2], x[..., 1:r:2]
    out = x.clone()
    out[..., 0:r:2] = u * c - v * s
    out[..., 1:r:2] = v * c + u * s
    return out


def latent_prep(q: torch.Tensor, dkv: torch.Tensor, qf: torch.Tensor,
                norm_w: torch.Tensor, eps: float,
                inv_freq: torch.Tensor | None, positions: torch.Tensor,
                kcache: torch.Tensor, slots: torch.Tensor, heads: int,
                dim: int) -> torch.Tensor:
    """Row steps of latent attention.  dkv [T, R + rd] (may be a strided
    view) holds the latent and one rotary key part: the latent is RMS-normed
    with a plain weight, the key part rotated (interleaved pairs on its first
    2*len(inv_freq) elements), and [latent | key part] is appended to the key
    pages kcache [P, 1, page, R + rd] at `slots`.  q [T, H*(dim + rd)] holds
    per head [unrotated | rotary part].  qf [T, H*(R + rd)] are the attention
    queries, per head [unrotated part carried into latent space | rotated
    rotary part]: the caller has filled the first R elements of every head,
    the rotary slices are written here.  Returns qf."""
    T = q.shape[0]
    H = heads
    R = norm_w.numel()
    rd = dkv.shape[1] - R
    dkc = R + rd
    page = kcache.shape[2]
    rot = 2 * inv_freq.numel() if inv_freq is not None else 0
    if not _gpu(q):
        d = dkv.float()
        c = d[:, :R] * torch.rsqrt(d[:, :R].pow(2).mean(-1, keepdim=True)
                                   + eps) * norm_w.float()
        kr = d[:, R:]
        qr = q.float().view(T, H, dim + rd)[..., dim:]
        if rot:
            kr = rotate_pairs(kr, positions, inv_freq)
            qr = rotate_pairs(qr, positions, inv_freq)
        pg = torch.div(slots, page, rounding_mode="floor")
        off = slots - pg * page
        kcache[pg, 0, off] = torch.cat([c, kr], 1).to(kcache.dtype)
        qf.view(T, H, dkc)[..., R:] = qr.to(qf.dtype)
        return qf
    assert qf.is_contiguous() and qf.shape == (T, H * dkc)
    rc = _L().afm_latent_prep(
        _lib.ptr(qf), _lib.ptr(kcache), _lib.ptr(q), _rowstride(q),
        _lib.ptr(dkv), _rowstride(dkv), _lib.ptr(norm_w),
        _lib.ptr(inv_freq), _lib.ptr(positions), _lib.ptr(slots), float(eps),
        T, H, dim, rd, R, rot, _code(q), _lib.cur_stream())
    _lib.check(rc, "afm_latent_prep")
    return qf


def gate_heads(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """out[t, h*dv + d] = o[h, t, d] * sigmoid(gate[t, h*dv + d]): per-head
    results [H, T, dv] back to token rows, times an element-wise output gate
    (logits [T, H*dv], may be a strided view)."""
    H, T, dv = o.shape
    if not _gpu(o):
        return (o.float().transpose(0, 1).reshape(T, H * dv)
                * torch.sigmoid(gate.float())).to(o.dtype)
    o = o.contiguous()
    out = torch.empty(T, H * dv, dtype=o.dtype, device=o.device)
    rc = _L().afm_gate_heads(_lib.ptr(out), _lib.ptr(o), _lib.ptr(gate),
                             _rowstride(gate), T, H, dv, _code(o),
                             _lib.cur_stream())
    _lib.check(rc, "afm_gate_heads")
    return out


def relu2(z: torch.Tensor) -> torch.Tensor:
    """max(z, 0)^2, element-wise; z [T, F] may be a strided view."""
    T, F = z.shape
    if not _gpu(z):
        return torch.relu(z.float()).pow(2).to(z.dtype)
    out = torch.empty(T, F, dtype=z.dtype, device=z.device)
    rc = _L().afm_relu2(_lib.ptr(out), _lib.ptr(z), _rowstride(z), T, F,
                        _code(z), _lib.cur_stream())
    _lib.check(rc, "afm_relu2")
    return out


# =====================================================================
# Ops of delta-rule decoders with the norm after the residual sum: gated
# delta rule over per-sequence fp32 state, per-head q/k norm with partial
# rotary positions (optionally wavelength-scaled frequencies), sublayer
# outputs summed into a scaled residual and normed, per-token side tables.
# =====================================================================
def scaled_inv_freq(dims: int, base: float,
                    scaling: dict | None = None) -> torch.Tensor:
    """Rotary frequencies f_i = base^(-2i/dims), i < dims/2, as float64.

    scaling {factor, low, high, original} rescales by wavelength l = 2 pi /
    f: l < original/high keeps f; l > original/low gives f / factor; in
    between, with s = (original/l - low) / (high - low), the blend (1 - s) *
    f / factor + s * f."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            orig, fac = float(scaling["original"]), float(scaling["factor"])
            lo, hi = float(scaling["low"]), float(scaling["high"])
            wl = 2.0 * math.pi / f
            if wl > orig / lo:
                f = f / fac
            elif wl >= orig / hi:
                s = (orig / wl - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rotary_table(positions: torch.Tensor,
                 inv_freq: torch.Tensor) -> torch.Tensor:
    """[cos | sin] of position * f_i per row as fp32 [T, 2*len(inv_freq)];
    inv_freq float64, the product and the functions in double precision.
    One table serves every layer of a step that rotates alike."""
    T, half = positions.numel(), inv_freq.numel()
    if not _gpu(positions):
        ang = positions.double()[:, None] * inv_freq.double()[None]
        return torch.cat([ang.cos(), ang.sin()], 1).float()
    tab = torch.empty(T, 2 * half, dtype=torch.float32,
                      device=positions.device)
    rc = _L().afm_rotary_table(_lib.ptr(tab), _lib.ptr(positions),
                               _lib.ptr(inv_freq), T, half,
                               _lib.cur_stream())
    _lib.check(rc, "afm_rotary_table")
    return tab


def qk_rope_cache(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  heads: int, kv_heads: int, eps: float,
                  kcache: torch.Tensor, vcache: torch.Tensor,
                  slots: torch.Tensor, positions: torch.Tensor,
                  q_bias: torch.Tensor | None = None,
                  k_bias: torch.Tensor | None = None,
                  v_bias: torch.Tensor | None = None,
                  q_norm: torch.Tensor | None = None,
                  k_norm: torch.Tensor | None = None,
                  inv_freq: torch.Tensor | None = None,
                  rot_tab: torch.Tensor | None = None) -> torch.Tensor:
    """Row steps in front of rotary attention.  q [T, H*dk], k [T, G*dk], v
    [T, G*dv] (strided views allowed) get their biases; every q and k head
    is RMS-normed over dk with a plain weight [dk] shared by heads (skipped
    without one); the first 2*len(inv_freq) dims of each head are rotated,
    dim i paired with i + len(inv_freq), by the angle position * f_i
    (inv_freq float64; product, sine and cosine in double precision; or the
    rows' ready rotary_table as rot_tab); k and v are appended to the paged
    caches at `slots`.  Returns q, contiguous [T, H*dk]."""
    T = q.shape[0]
    H, G = heads, kv_heads
    dk = q.shape[1] // H
    dv = v.shape[1] // G
    page = kcache.shape[2]
    if rot_tab is None and inv_freq is not None and inv_freq.numel() > 0:
        rot_tab = rotary_table(positions, inv_freq)
    half = rot_tab.shape[1] // 2 if rot_tab is not None else 0
    if not _gpu(q):
        qf = q.float()
        kf = k.float()
        vf = v.float()
        if q_bias is not None:
            qf = qf + q_bias.float()
        if k_bias is not None:
            kf = kf + k_bias.float()
        if v_bias is not None:
            vf = vf + v_bias.float()
        qf, kf = qf.reshape(T, H, dk), kf.reshape(T, G, dk)
        if q_norm is not None:
            qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) \
                * q_norm.float()
        if k_norm is not None:
            kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) \
                * k_norm.float()
        if half:
            c, s = rot_tab[:, None, :half], rot_tab[:, None, half:]

            def rot(x):
                u, w = x[..., :half], x[..., half:2 * half]
                return torch.cat([u * c - w * s, w * c + u * s,
                                  x[..., 2 * half:]], -1)
            qf, kf = rot(qf), rot(kf)
        pg = torch.div(slots, page, rounding_mode="floor")
        off = slots - pg * page
        kcache[pg, :, off] = kf.to(kcache.dtype)
        vcache[pg, :, off] = vf.reshape(T, G, dv).to(vcache.dtype)
        return qf.reshape(T, H * dk).to(q.dtype)
    out = torch.empty(T, H * dk, dtype=q.dtype, device=q.device)
    rc = _L().afm_qk_rope_cache(
        _lib.ptr(out), _lib.ptr(q), _rowstride(q), _lib.ptr(k), _rowstride(k),
        _lib.ptr(v), _rowstride(v), _lib.ptr(q_bias), _lib.ptr(k_bias),
        _lib.ptr(v_bias), _lib.ptr(q_norm), _lib.ptr(k_norm),
        _lib.ptr(rot_tab), 2 * half, _lib.ptr(kcache), _lib.ptr(vcache),
        _lib.ptr(slots), float(eps), T, H, G, dk, dv, page, _code(q),
        _lib.cur_stream())
    _lib.check(rc, "afm_qk_rope_cache")
    return out


# a step whose longest row chunk reaches this many rows runs the delta rule
# in its prompt layout (rows of the state over the lanes of a DPP row)
DELTA_LONG_ROWS = 32


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
               beta: torch.Tensor, decay: torch.Tensor,
               decay_bias: torch.Tensor, rate: torch.Tensor,
               state: torch.Tensor, md, heads: int, kv_heads: int,
               q_scale: float = 1.0) -> torch.Tensor:
    """Gated delta rule, token by token in fp32, per head h with its q/k
    head g = h // (heads / kv_heads) and state S [dk, dv]:

        q' = q_g / sqrt(|q_g|^2 + 1e-6) * q_scale,  k' = k_g / sqrt(|k_g|^2 + 1e-6)
        a  = exp(-rate[h] * softplus(decay + decay_bias))
        S <- a * S;  u = sigmoid(beta[h]) * (v_h - S^T k');  S <- S + k' u^T
        o_h = S^T q'                       (the read-out sees the write)

    q, k [T, G*dk], v [T, H*dv], beta [T, H] logits (strided views allowed).
    decay [T, H] gives one decay per head (decay_bias [H]); decay [T, H*dk]
    one per head and key channel, scaling the rows of S (decay_bias [H*dk]).
    rate, decay_bias fp32.  S lives in `state` [slots, H, dk, dv] fp32: read
    unless the chunk starts at position 0, written after the chunk's last
    row.  Returns o [T, H*dv] fp32."""
    T = q.shape[0]
    H, G = heads, kv_heads
    dk = q.shape[1] // G
    dv = v.shape[1] // H
    per_channel = dk > 1 and decay.shape[1] == H * dk
    if decay.shape[1] not in (H, H * dk):
        raise ValueError("delta_scan: decay must be [T, H] or [T, H*dk]")
    if not _gpu(q):
        qf = q.float().reshape(T, G, dk)
        kf = k.float().reshape(T, G, dk)
        qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + 1e-6) * q_scale
        kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + 1e-6)
        qf = qf.repeat_interleave(H // G, dim=1)
        kf = kf.repeat_interleave(H // G, dim=1)
        vf = v.float().reshape(T, H, dv)
        bt = torch.sigmoid(beta.float())
        z = torch.nn.functional.softplus(decay.float() + decay_bias.float(),
                                         threshold=20.0)
        if per_channel:
            a = torch.exp(-rate.float()[None, :, None] * z.view(T, H, dk))
            a = a[..., None]
        else:
            a = torch.exp(-rate.float()[None] * z)[..., None, None]
        out = torch.empty(T, H, dv, dtype=torch.float32)
        cu, qs, sl = (md.cu_seqlens.tolist(), md.q_start.tolist(),
                      md.state_slots.tolist())
        for b in range(len(qs)):
            if cu[b + 1] == cu[b]:
                continue
            S = state[sl[b]].clone() if qs[b] > 0 else torch.zeros(H, dk, dv)
            for t in range(cu[b], cu[b + 1]):
                S = a[t] * S
                u = bt[t][:, None] * (vf[t] - torch.einsum("hkv,hk->hv", S,
                                                           kf[t]))
                S = S + kf[t][:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S, qf[t])
            state[sl[b]] = S
        return out.view(T, H * dv)
    out = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
    B = md.q_start.numel()
    # prompt portions amortise the state's load and store over many tokens
    # and take the layout with the shortest per-token chain; short chunks and
    # decode steps take the one whose state accesses coalesce
    lens = getattr(md, "seq_lens", None)
    long_chunks = lens is not None and max(lens) >= DELTA_LONG_ROWS
    rc = _L().afm_delta_scan(
        _lib.ptr(out), _lib.ptr(state), _lib.ptr(q), _rowstride(q),
        _lib.ptr(k), _rowstride(k), _lib.ptr(v), _rowstride(v),
        _lib.ptr(beta), _rowstride(beta), _lib.ptr(decay), _rowstride(decay),
        _lib.ptr(decay_bias), _lib.ptr(rate), _lib.ptr(md.cu_seqlens),
        _lib.ptr(md.q_start), _lib.ptr(md.state_slots), B, H, G, dk, dv,
        1 if per_channel else 0, float(q_scale), 1 if long_chunks else 0,
        _code(q), _lib.cur_stream())
    _lib.check(rc, "afm_delta_scan")
    return out


def postnorm_sum(x: torch.Tensor, y: torch.Tensor, alpha: float,
                 w: torch.Tensor, eps: float, dtype: torch.dtype,
                 y2: torch.Tensor | None = None,
                 wy: torch.Tensor | None = None,
                 wy2: torch.Tensor | None = None) -> torch.Tensor:
    """In place on the fp32 residual: x <- (alpha x + u) / rms(alpha x + u)
    * w, the norm sitting after the sum.  u = y, or with a second branch u =
    (y / rms(y) * wy + y2 / rms(y2) * wy2) / 2.  y (and y2) [T, W] in the
    storage dtype or fp32.  Returns the new residual in `dtype` (x itself for
    fp32), the next sublayer's input."""
    T, W = x.shape
    if not _gpu(x):
        def n(u, wt):
            return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) \
                * wt.float()
        u = y.float()
        if y2 is not None:
            u = 0.5 * (n(u, wy) + n(y2.float(), wy2))
        x.copy_(n(alpha * x + u, w))
        return x.to(dtype) if dtype != torch.float32 else x
    h = None if dtype == torch.float32 else \
        torch.empty(T, W, dtype=dtype, device=x.device)
    if y2 is not None and y2.dtype != y.dtype:
        raise TypeError("postnorm_sum: both branches in one dtype")
    rc = _L().afm_postnorm_sum(
        _lib.ptr(x), _lib.ptr(h), _lib.ptr(y), _rowstride(y),
        1 if y.dtype == torch.float32 else 0, _lib.ptr(y2),
        _rowstride(y2) if y2 is not None else 0, _lib.ptr(wy), _lib.ptr(wy2),
        _lib.ptr(w), float(alpha), float(eps), T, W, _code(w),
        _lib.cur_stream())
    _lib.check(rc, "afm_postnorm_sum")
    return x if h is None else h


def gate_gather(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor,
                offset: int) -> torch.Tensor:
    """out[t, c] = gelu_tanh(z[t, c]) * table[ids[t], offset + c]: a gate
    on a slice of a per-token table row.  z [T, C] may be a strided view."""
    T, C = z.shape
    if not _gpu(z):
        e = table[ids.long()][:, offset:offset + C].float()
        return (_act("gelu_tanh", z.float()) * e).to(z.dtype)
    out = torch.empty(T, C, dtype=z.dtype, device=z.device)
    rc = _L().afm_gate_gather(_lib.ptr(out), _lib.ptr(z), _rowstride(z),
                              _lib.ptr(table), table.stride(0), int(offset),
                              _lib.ptr(ids), T, C, _code(z),
                              _lib.cur_stream())
    _lib.check(rc, "afm_gate_gather")
    return out
