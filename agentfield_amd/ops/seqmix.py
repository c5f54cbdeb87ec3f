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
  * CUDA (=HIP) tensors run the gfx950 kernels in libafmix.so, CPU tensors a
    vectorised torch path used by CPU tests

The recurrences are evaluated strictly token by token in fp32, so results
do not depend on where a prompt was cut into chunks.
"""
from __future__ import annotations

import math
import os

import torch

from . import _lib

_DT = {torch.bfloat16: 0, torch.float32: 1}
# a step whose longest row chunk reaches this many rows runs bf16 attention
# through the MFMA tile kernel; shorter steps (decode) use one wave per row
MFMA_MIN_ROWS = 16
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
               add: torch.Tensor | None = None) -> torch.Tensor:
    """x[t] = table[ids[t]] (+ add) as an fp32 residual stream [T, W]."""
    T = ids.numel()
    W = table.shape[1]
    if not _gpu(table):
        x = table[ids.long()].float()
        return x + add.float() if add is not None else x
    out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    rc = _L().afm_embed(_lib.ptr(out), _lib.ptr(table), _lib.ptr(ids),
                        _lib.ptr(add), T, W, _code(table), _lib.cur_stream())
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
                     vcache: torch.Tensor, md, positions: torch.Tensor,
                     scale: float, heads: int, chunk: int = 0,
                     window: int = 0) -> torch.Tensor:
    """Softmax attention of packed rows over the paged cache.  Row at
    position i sees key j iff j <= i, and (chunk > 0) floor(j/chunk) ==
    floor(i/chunk), and (window > 0) j > i - window.  Positions are absolute
    in the sequence.  q [T, H*dk] -> [T, H*dv]; scores and softmax in fp32."""
    T = q.shape[0]
    _, G, page, dk = kcache.shape
    dv = vcache.shape[3]
    H = heads
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
            pg = bt[rs[t]][js // page]
            kk = kcache[pg, :, js % page].float()      # [n, G, dk]
            vv = vcache[pg, :, js % page].float()
            kk = kk.repeat_interleave(H // G, dim=1)
            vv = vv.repeat_interleave(H // G, dim=1)
            s = torch.einsum("nhd,hd->hn", kk, qf[t]) * scale
            out[t] = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), vv)
        return out.view(T, H * dv).to(q.dtype)
    out = torch.empty(T, H * dv, dtype=q.dtype, device=q.device)
    lens = getattr(md, "seq_lens", None)
    if (q.dtype == torch.bfloat16 and lens is not None and dk <= 128
            and dv <= 128 and max(lens) >= MFMA_MIN_ROWS):
        # prompt portions: 64-row tiles on the matrix cores
        ts, tq = [], []
        for b, ln in enumerate(lens):
            for q0 in range(0, ln, 64):
                ts.append(b)
                tq.append(q0)
        tile_seq = torch.tensor(ts, dtype=torch.int32, device=q.device)
        tile_q0 = torch.tensor(tq, dtype=torch.int32, device=q.device)
        rc = _L().afm_attn_prefill_mfma(
            _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache),
            _lib.ptr(md.block_table), _lib.ptr(md.cu_seqlens),
            _lib.ptr(md.q_start), _lib.ptr(tile_seq), _lib.ptr(tile_q0),
            float(scale), len(ts), H, G, dk, dv, page,
            md.block_table.shape[1], int(chunk), int(window), _rowstride(q),
            _lib.cur_stream())
        _lib.check(rc, "afm_attn_prefill_mfma")
        return out
    # few rows and many visible keys: cut the keys over several workgroups
    # (about 2048 in flight) and merge the partial softmaxes
    reach = min(x for x in (chunk, window, md.block_table.shape[1] * page)
                if x > 0)
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
        _lib.ptr(out), _lib.ptr(q), _lib.ptr(kcache), _lib.ptr(vcache),
        _lib.ptr(md.block_table), _lib.ptr(md.row_seq), _lib.ptr(positions),
        float(scale), T, H, G, dk, dv, page, md.block_table.shape[1],
        int(chunk), int(window), _rowstride(q), nsplit, _lib.ptr(part_o),
        _lib.ptr(part_ml), _code(q), _lib.cur_stream())
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
                  out_dtype: torch.dtype) -> torch.Tensor:
    """Per-head RMSNorm of o [T, H*dv] fp32 (optional plain weight [dv]
    shared by heads) times silu(g); g [T, H*dv] may be a strided view."""
    T, HD = o.shape
    dv = HD // heads
    if not _gpu(o):
        of = o.view(T, heads, dv)
        of = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            of = of * weight.float()
        gf = g.float()
        return (of.reshape(T, HD) * gf * torch.sigmoid(gf)).to(out_dtype)
    out = torch.empty(T, HD, dtype=out_dtype, device=o.device)
    rc = _L().afm_headnorm_gate(_lib.ptr(out), _lib.ptr(o), _lib.ptr(g),
                                _lib.ptr(weight), float(eps), T, heads, dv,
                                _rowstride(g), _code(out), _lib.cur_stream())
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
