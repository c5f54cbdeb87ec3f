"""Slow, plain float64 statement of the Reperax equations — the oracle the
framework's kernels, cache and scheduler are tested against.  One function
per mechanism, whole sequences only (no cache, no batching, no chunking),
written token by token from the definitions.  Shares no code with
agentfield_amd.

Weights come as a dict of checkpoint-named tensors, the model description as
the config.json dict.
"""
import math

import torch

F64 = torch.float64


def unit_rms(u, eps):
    """u / sqrt(mean(u^2) + eps) along the last axis."""
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu with h_{-1} = 0."""
    out = torch.empty_like(h)
    for t in range(h.shape[0]):
        before = h[t - 1] if t > 0 else torch.zeros_like(h[0])
        out[t] = h[t] + (before - h[t]) * mu
    return out


def chunk_attention(h, Wq, Wk, Wv, Wo, gq, gk, heads, kv_heads, dim, vdim,
                    scale, chunk, eps):
    """Softmax attention; whole-row q/k norm; key j visible from i iff
    j <= i and both lie in the same chunk (chunk 0: plain causal)."""
    T = h.shape[0]
    q = unit_rms(h @ Wq.T, eps) * gq
    k = unit_rms(h @ Wk.T, eps) * gk
    v = h @ Wv.T
    per = heads // kv_heads
    cat = torch.zeros(T, heads * vdim, dtype=F64)
    for i in range(T):
        first = (i // chunk) * chunk if chunk > 0 else 0
        for a in range(heads):
            b = a // per
            qi = q[i, a * dim:(a + 1) * dim]
            scores = torch.stack([
                (qi * k[j, b * dim:(b + 1) * dim]).sum() * scale
                for j in range(first, i + 1)])
            wts = torch.exp(scores - scores.max())
            wts = wts / wts.sum()
            acc = torch.zeros(vdim, dtype=F64)
            for n, j in enumerate(range(first, i + 1)):
                acc += wts[n] * v[j, b * vdim:(b + 1) * vdim]
            cat[i, a * vdim:(a + 1) * vdim] = acc
    return cat @ Wo.T


def decayed_recurrence(q, k, v, decay):
    """S_t = diag(decay_t) S_{t-1} + k_t v_t^T ; o_t = S_t^T q_t for one
    head.  q, k [T, dk]; v [T, dv]; decay [T, dk]."""
    T, dk = k.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=F64)
    out = torch.zeros(T, dv, dtype=F64)
    for t in range(T):
        S = decay[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def gated_linear_attention(h, Wq, Wk, Wv, Wg, Wo, Wa1, Wa2, ba, gn, heads,
                           dim, vdim, tau, eps):
    T = h.shape[0]
    q = (h @ Wq.T) / math.sqrt(dim)
    k = h @ Wk.T
    v = h @ Wv.T
    z = (h @ Wa1.T) @ Wa2.T + ba
    alpha = torch.sigmoid(z) ** (1.0 / tau)
    cat = torch.zeros(T, heads * vdim, dtype=F64)
    for a in range(heads):
        ks, vs = slice(a * dim, (a + 1) * dim), slice(a * vdim, (a + 1) * vdim)
        o = decayed_recurrence(q[:, ks], k[:, ks], v[:, vs], alpha[:, ks])
        cat[:, vs] = unit_rms(o, eps) * gn
    gate = h @ Wg.T
    return (cat * gate * torch.sigmoid(gate)) @ Wo.T


def rotate_half(x, pos, dims, base):
    """Rotate the first `dims` entries of x; entry i pairs with i + dims/2."""
    y = x.clone()
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        y[i] = x[i] * c - x[i + half] * s
        y[i + half] = x[i + half] * c + x[i] * s
    return y


def retention(h, Wq, Wk, Wv, Wg, Wo, heads, dim, vdim, decay, rot_dims,
              rot_base, eps):
    T = h.shape[0]
    q, k, v = h @ Wq.T, h @ Wk.T, h @ Wv.T
    cat = torch.zeros(T, heads * vdim, dtype=F64)
    for a in range(heads):
        ks, vs = slice(a * dim, (a + 1) * dim), slice(a * vdim, (a + 1) * vdim)
        qa = torch.stack([rotate_half(q[t, ks], t, rot_dims, rot_base)
                          for t in range(T)])
        ka = torch.stack([rotate_half(k[t, ks], t, rot_dims, rot_base)
                          for t in range(T)]) / math.sqrt(dim)
        d = torch.full((T, dim), float(decay[a]), dtype=F64)
        cat[:, vs] = unit_rms(decayed_recurrence(qa, ka, v[:, vs], d), eps)
    gate = h @ Wg.T
    return (cat * gate * torch.sigmoid(gate)) @ Wo.T


def polynorm_ff(h, Wup, Wdown, coef, eps):
    z = h @ Wup.T
    act = (coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z ** 2, eps)
           + coef[2] * unit_rms(z ** 3, eps) + coef[3])
    return act @ Wdown.T


def layer(x, i, lc, w, eps):
    p = f"l{i}."
    g = lambda n: w[p + n].to(F64)  # noqa: E731
    n1 = zero_centred_norm(x, g("norm1"), eps)
    hs = token_shift(n1, g("shift"))
    m = lc["mixer"]
    if lc["type"] == "parallel":
        le, ri = m["left"], m["right"]
        left = chunk_attention(
            hs, g("mix.left.q"), g("mix.left.k"), g("mix.left.v"),
            g("mix.left.o"), g("mix.left.q.norm"), g("mix.left.k.norm"),
            le["heads"], le["kv_heads"], le["dim"], le["vdim"], le["scale"],
            le["mask"]["size"], eps)
        right = gated_linear_attention(
            hs, g("mix.right.q"), g("mix.right.k"), g("mix.right.v"),
            g("mix.right.g"), g("mix.right.o"), g("mix.right.a1"),
            g("mix.right.a2"), g("mix.right.a2.b"), g("mix.right.norm"),
            ri["heads"], ri["dim"], ri["vdim"], ri["tau"], eps)
        mixed = m["left_scale"] * left + m["right_scale"] * right
    else:
        mixed = retention(
            hs, g("mix.q"), g("mix.k"), g("mix.v"), g("mix.g"), g("mix.o"),
            m["heads"], m["dim"], m["vdim"], m["decay"], m["rot"]["dims"],
            m["rot"]["base"], eps)
    y = mixed * torch.sigmoid(n1 @ g("rg1").T + g("rg1.b"))
    if lc["mlp"] is not None:
        n2 = zero_centred_norm(x, g("norm2"), eps)
        ff = polynorm_ff(n2, g("mlp.up"), g("mlp.down"), g("mlp.act"), eps)
        y = y + ff * torch.sigmoid(n2 @ g("rg2").T + g("rg2.b"))
    return x + y


def forward(tokens, cfg, w, keep_runs=False):
    """Logits [T, vocab] (float64) for one whole sequence from position 0."""
    eps = cfg["norm"]["eps"]
    emb = w["embed"].to(F64)
    x = emb[torch.tensor(tokens)]
    x0 = x.clone()
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    n = len(cfg["layers"])
    runs = []

    def go(i, x):
        x = layer(x, i, cfg["layers"][i], w, eps)
        runs.append(x.clone())
        return x
    i = 0
    while i < n:
        if lp["stop"] > lp["start"] and i == lp["start"]:
            for t in range(lp["times"]):
                if t > 0:
                    x = x + x0
                x = x + w["loop.step"].to(F64)[t]
                for j in range(lp["start"], lp["stop"]):
                    x = go(j, x)
            i = lp["stop"]
        else:
            x = go(i, x)
            i += 1
    h = zero_centred_norm(x, w["final.norm"].to(F64), eps)
    logits = h @ emb.T
    cap = cfg.get("logit_softcap") or 0.0
    if cap > 0:
        logits = cap * torch.tanh(logits / cap)
    return (logits, runs) if keep_runs else logits


# ------------------------------------------------ random models for tests
def random_weights(cfg, seed=0, dtype=torch.float32):
    """Checkpoint-named random tensors for a config dict.  Values are
    rounded to `dtype` (so bf16 runs see exactly these numbers) and scaled to
    keep activations O(1)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def mat(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(n, s=0.2):
        return torch.randn(n, generator=g) * s
    w["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    w["final.norm"] = vec(W)
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        w["loop.step"] = torch.randn(lp["times"], W, generator=g) * 0.5
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        w[p + "norm1"] = vec(W)
        w[p + "shift"] = torch.rand(W, generator=g)
        w[p + "rg1"] = mat(W, W)
        w[p + "rg1.b"] = vec(W, 0.5)
        m = lc["mixer"]
        if lc["type"] == "parallel":
            le, ri = m["left"], m["right"]
            q = p + "mix.left."
            w[q + "q"] = mat(le["heads"] * le["dim"], W)
            w[q + "k"] = mat(le["kv_heads"] * le["dim"], W)
            w[q + "v"] = mat(le["kv_heads"] * le["vdim"], W)
            w[q + "q.norm"] = 1.0 + vec(le["heads"] * le["dim"])
            w[q + "k.norm"] = 1.0 + vec(le["kv_heads"] * le["dim"])
            w[q + "o"] = mat(W, le["heads"] * le["vdim"])
            r = p + "mix.right."
            rank = ri.get("rank", 4)
            w[r + "q"] = mat(ri["heads"] * ri["dim"], W)
            w[r + "k"] = mat(ri["heads"] * ri["dim"], W)
            w[r + "v"] = mat(ri["heads"] * ri["vdim"], W)
            w[r + "g"] = mat(ri["heads"] * ri["vdim"], W)
            w[r + "o"] = mat(W, ri["heads"] * ri["vdim"])
            w[r + "norm"] = 1.0 + vec(ri["vdim"])
            w[r + "a1"] = mat(rank, W)
            w[r + "a2"] = mat(ri["heads"] * ri["dim"], rank, 2.0)
            w[r + "a2.b"] = vec(ri["heads"] * ri["dim"], 1.0) + 2.0
        else:
            q = p + "mix."
            w[q + "q"] = mat(m["heads"] * m["dim"], W)
            w[q + "k"] = mat(m["heads"] * m["dim"], W)
            w[q + "v"] = mat(m["heads"] * m["vdim"], W)
            w[q + "g"] = mat(m["heads"] * m["vdim"], W)
            w[q + "o"] = mat(W, m["heads"] * m["vdim"])
        if lc["mlp"] is not None:
            w[p + "norm2"] = vec(W)
            w[p + "mlp.up"] = mat(lc["mlp"]["ff"], W)
            w[p + "mlp.down"] = mat(W, lc["mlp"]["ff"])
            w[p + "mlp.act"] = torch.tensor([0.7, 0.25, 0.1, 0.05])
            w[p + "rg2"] = mat(W, W)
            w[p + "rg2.b"] = vec(W, 0.5)
    return {k: v.to(dtype).contiguous() for k, v in w.items()}
