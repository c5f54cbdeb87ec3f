"""Plain float64 statement of the Zudisun decoder, one function per mechanism.

Whole sequences only, no cache, no batching, no kernels: every function takes
the full [T, ...] input of one sequence and loops where the definition loops.
It shares no code with the package and is the yardstick of test_zudisun.py.

Tensors are looked up by checkpoint name in a dict `P` (values are cast to
float64 on use); `cfg` is the parsed config.json.
"""
import math

import torch

F64 = torch.float64


def _f(t):
    return t.to(F64)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * _f(w)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ mamba1
def causal_conv(x, w, b):
    """Depthwise causal convolution: out[t, c] = b[c] + sum_j w[c, j] *
    x[t - (taps - 1 - j), c]; the last column weighs the current token and
    inputs before the start are zero."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = _f(b).clone()
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                acc = acc + _f(w)[:, j] * x[s]
        out[t] = acc
    return out


def selective_scan(x, dt, A, Bm, Cm, D):
    """S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;
    y_c = sum_n S[c, n] C_n + D_c x_c, state zero at the start."""
    T, C = x.shape
    N = A.shape[1]
    S = torch.zeros(C, N, dtype=F64)
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + \
            (dt[t] * x[t])[:, None] * Bm[t][None, :]
        y[t] = S @ Cm[t] + D * x[t]
    return y


def mamba1(h, P, pre, m):
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ _f(P[pre + "in"]).t()
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, P[pre + "conv"], P[pre + "conv.b"]))
    low = x @ _f(P[pre + "x"]).t()
    dt, Bm, Cm = low[:, :R], low[:, R:R + N], low[:, R + N:R + 2 * N]
    dt = softplus(dt @ _f(P[pre + "dt"]).t() + _f(P[pre + "dt.b"]))
    A = -torch.exp(_f(P[pre + "A_log"]))
    y = selective_scan(x, dt, A, Bm, Cm, _f(P[pre + "D"]))
    return (y * silu(z)) @ _f(P[pre + "o"]).t()


# --------------------------------------------------------------- attention
def distance_bucket(n, rows, dmax):
    """Exact for small distances, logarithmic up to dmax, then the last."""
    half = rows // 2
    if n < half:
        return n
    v = math.log(n / half) / math.log(dmax / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(v + 1e-9)))


def query_temperature(p, coef, every):
    return 1.0 + coef * math.log((p + 1) // every + 1)


def sigmoid_attention(h, P, pre, m, eps, v_first=None):
    """Returns (mixer output, the values this layer used)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ _f(P[pre + "q"]).t()).view(T, H, dk)
    k = (h @ _f(P[pre + "k"]).t()).view(T, G, dk)
    v = (h @ _f(P[pre + "v"]).t()).view(T, G, dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    qt = m.get("q_temp")
    if qt:
        for p in range(T):
            q[p] = q[p] * query_temperature(p, qt["coef"], qt["every"])
    if v_first is not None:
        lam = float(P[pre + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    rel = _f(P[pre + "rel"])
    talk, pb = _f(P[pre + "talk"]), _f(P[pre + "pb"])
    gate = torch.sigmoid(h @ _f(P[pre + "g"]).t())           # [T, H]
    out = torch.zeros(T, H, dv, dtype=F64)
    rep = H // G
    bucket = torch.tensor([distance_bucket(n, rel.shape[0], m["bias_max"])
                           for n in range(T)])
    for i in range(T):
        s = torch.zeros(H, i + 1, dtype=F64)
        bias = rel[bucket[:i + 1].flip(0)]                   # [i+1, H], by j
        for hh in range(H):
            s[hh] = (k[:i + 1, hh // rep] @ q[i, hh]) * m["scale"] \
                + bias[:, hh]
        w = torch.sigmoid(talk @ s + pb[:, None])            # [H, i+1]
        for hh in range(H):
            out[i, hh] = w[hh] @ v[:i + 1, hh // rep]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ _f(P[pre + "o"]).t(), v


# ------------------------------------------------------------ feed-forward
def glu(h, P, pre, act, bias):
    g = h @ _f(P[pre + "gate"]).t()
    u = h @ _f(P[pre + "up"]).t()
    if bias:
        g, u = g + _f(P[pre + "gate.b"]), u + _f(P[pre + "up.b"])
    y = (act(g) * u) @ _f(P[pre + "down"]).t()
    return y + _f(P[pre + "down.b"]) if bias else y


def route(z, corr, r):
    """Router of one token.  z: logits [E].  Returns (experts, weights)."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    choice = s + corr
    groups = r.get("groups")
    if groups:
        size = E // groups["count"]
        gs = []
        for g in range(groups["count"]):
            part = sorted(choice[g * size:(g + 1) * size].tolist(),
                          reverse=True)
            gs.append(sum(part[:2]))
        keep = sorted(range(len(gs)), key=lambda g: (-gs[g], g))
        keep = set(keep[:groups["keep"]])
        choice = choice.clone()
        for e in range(E):
            if e // size not in keep:
                choice[e] = -math.inf
    order = sorted(range(E), key=lambda e: (-float(choice[e]), e))[:top]
    w = torch.stack([s[e] for e in order])
    return order, w / (w.sum() + 1e-20) * r["scale"]


def moe_ff(h, P, pre, mlp):
    r = mlp["router"]
    T, W = h.shape
    z = h @ _f(P[pre + "router"]).t()
    corr = _f(P[pre + "correction"])
    out = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        experts, w = route(z[t], corr, r)
        for e, we in zip(experts, w):
            out[t] += we * glu(h[t:t + 1], P, f"{pre}e{e}.", silu, False)[0]
    if mlp.get("shared"):
        out = out + glu(h, P, pre + "shared.", silu, False)
    return out


# ------------------------------------------------------------------- model
def forward(tokens, cfg, P, keep_layers=False):
    """tokens: list[int] of one sequence -> logits [T, vocab] (and, on
    request, the residual stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = _f(P["embed"])[torch.tensor(tokens)]
    v_first, layers = None, []
    for i, lc in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", lc["mixer"]
        if lc["type"] == "mamba1":
            y = mamba1(x, P, pre, m)
        elif lc["type"] == "attention":
            mixing = bool(m.get("v_mix"))
            y, v = sigmoid_attention(x, P, pre, m, eps,
                                     v_first if mixing else None)
            if mixing and v_first is None:
                v_first = v
        else:
            raise ValueError(lc["type"])
        x = x + rms_norm(y, P[f"l{i}.norm1"], eps)
        mlp = lc.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = glu(x, P, f"l{i}.mlp.", torch.relu, True)
            else:
                y = moe_ff(x, P, f"l{i}.mlp.", mlp)
            x = x + rms_norm(y, P[f"l{i}.norm2"], eps)
        if keep_layers:
            layers.append(x.clone())
    logits = rms_norm(x, P["final.norm"], eps) @ _f(P["head"]).t()
    return (logits, layers) if keep_layers else logits


# ------------------------------------------------------------ test weights
def random_weights(cfg, seed, dtype=torch.float32):
    """Checkpoint-named random tensors for a config (values rounded to
    `dtype`), at scales that keep every branch alive: step sizes spread over
    two decades, distinct distance-bias rows, a head-mixing matrix away from
    the identity, corrections that change which experts win."""
    g = torch.Generator().manual_seed(seed)

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(dtype)
    W, V = cfg["width"], cfg["vocab"]
    P = {"embed": r(V, W), "head": r(V, W, std=W ** -0.5),
         "final.norm": r(W, std=0.2, mean=1.0)}
    for i, lc in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", lc["mixer"]
        P[f"l{i}.norm1"] = r(W, std=0.2, mean=1.0)
        if lc["type"] == "mamba1":
            C, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            P[pre + "in"] = r(2 * C, W, std=W ** -0.5)
            P[pre + "conv"] = r(C, K, std=K ** -0.5)
            P[pre + "conv.b"] = r(C, std=0.2)
            P[pre + "x"] = r(R + 2 * N, C, std=C ** -0.5)
            P[pre + "dt"] = r(C, R, std=R ** -0.5)
            P[pre + "dt.b"] = r(C, std=1.5, mean=-2.0)
            P[pre + "A_log"] = torch.log(
                torch.rand(C, N, generator=g) * 4 + 0.05).to(dtype)
            P[pre + "D"] = r(C, std=0.5, mean=1.0)
            P[pre + "o"] = r(W, C, std=C ** -0.5)
        else:
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            P[pre + "q"] = r(H * dk, W, std=W ** -0.5)
            P[pre + "k"] = r(G * dk, W, std=W ** -0.5)
            P[pre + "v"] = r(G * dv, W, std=W ** -0.5)
            P[pre + "g"] = r(H, W, std=W ** -0.5)
            P[pre + "o"] = r(W, H * dv, std=(H * dv) ** -0.5)
            P[pre + "rel"] = r(m.get("bias_rows", 32), H, std=0.7)
            P[pre + "talk"] = (torch.eye(H) + torch.randn(H, H, generator=g)
                               * 0.4).to(dtype)
            P[pre + "pb"] = r(H, std=0.5, mean=-2.0)
            P[pre + "vmix"] = torch.tensor(0.35).to(dtype)
        mlp = lc.get("mlp")
        if mlp is None:
            continue
        fp = f"l{i}.mlp."
        P[f"l{i}.norm2"] = r(W, std=0.2, mean=1.0)

        def unit(p, F, bias):
            P[p + "gate"] = r(F, W, std=W ** -0.5)
            P[p + "up"] = r(F, W, std=W ** -0.5)
            P[p + "down"] = r(W, F, std=F ** -0.5)
            if bias:
                P[p + "gate.b"], P[p + "up.b"] = r(F, std=0.3), r(F, std=0.3)
                P[p + "down.b"] = r(W, std=0.3)
        if mlp["kind"] == "dense":
            unit(fp, mlp["ff"], True)
        else:
            E = mlp["router"]["experts"]
            for e in range(E):
                unit(f"{fp}e{e}.", mlp["expert"]["ff"], False)
            if mlp.get("shared"):
                unit(fp + "shared.", mlp["shared"]["ff"], False)
            P[fp + "router"] = r(E, W, std=0.5 * W ** -0.5)
            P[fp + "correction"] = r(E, std=0.6, mean=-0.4)
    return P


def greedy(tokens, n, cfg, P):
    """n greedy continuation tokens of a prompt."""
    toks, out = list(tokens), []
    for _ in range(n):
        nxt = int(forward(toks, cfg, P)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
