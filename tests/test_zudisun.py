"""Zudisun (post-norm hybrid decoder: selective state-space mixer, sigmoid
attention, routed experts) against the plain float64 oracle in
zudisun_oracle.py: every mechanism alone, then whole models through the
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

import zudisun_oracle as orc  # noqa: E402
from agentfield_amd.engine import LLMEngine, SamplingParams  # noqa: E402
from agentfield_amd.models import load_model  # noqa: E402
from agentfield_amd.models.zudisun import (RoutedExperts,  # noqa: E402
                                           RoutedSpec, SelectiveSSM,
                                           SelectiveSSMSpec, ZudisunConfig,
                                           ZudisunForCausalLM, save_zudisun)
from agentfield_amd.ops import seqmix as sm  # noqa: E402

REPO = Path(__file__).resolve().parent.parent
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


# ------------------------------------------------------------ model zoo
def _moe(experts, top, ff, groups=None, shared=None, scale=1.0):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def cfg_mixed():
    """Unequal sizes everywhere; attention first; a layer without
    feed-forward; a non-mixing attention layer between mixing ones; state
    size past one 16-lane group."""
    att = lambda **kw: {"type": "attention", "mixer": dict(  # noqa: E731
        {"heads": 6, "kv_heads": 3, "dim": 12, "vdim": 20, "scale": 0.3,
         "bias_rows": 10, "bias_max": 23, "v_mix": True,
         "q_temp": {"coef": 0.7, "every": 5}}, **kw)}
    a0 = att(); a0["mlp"] = {"kind": "dense", "ff": 40}
    a1 = att(v_mix=False, heads=3, kv_heads=3, vdim=8, bias_rows=7,
             bias_max=9.5)
    a1["mlp"] = None
    a2 = att(heads=3, q_temp={"coef": 0.2, "every": 1})
    a2["mlp"] = _moe(6, 2, 24, groups=(3, 2), shared=16, scale=1.7)
    m0 = {"type": "mamba1", "mlp": _moe(10, 3, 12, groups=(5, 2), shared=8),
          "mixer": {"inner": 40, "state": 20, "dt_rank": 3, "conv": 4}}
    m1 = {"type": "mamba1", "mlp": {"kind": "dense", "ff": 56},
          "mixer": {"inner": 72, "state": 5, "dt_rank": 2, "conv": 3}}
    return {"architecture": "Zudisun", "vocab": 96, "width": 48,
            "layers": [a0, m0, a1, m1, a2], "norm": {"eps": 1e-5}}


def cfg_degenerate():
    """Values a model may happen to make equal or 1: one head, kv_heads ==
    heads, dim == vdim, dt_rank 1, state 1, two taps, top 1, one group, keep
    == count, no shared expert, a single mixing layer."""
    att = {"type": "attention", "mlp": _moe(4, 1, 16, groups=(1, 1)),
           "mixer": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8,
                     "scale": 1.0, "bias_rows": 2, "bias_max": 4,
                     "v_mix": True, "q_temp": {"coef": 1.0, "every": 3}}}
    att2 = {"type": "attention", "mlp": _moe(4, 4, 8, groups=(2, 2)),
            "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8,
                      "scale": 0.5, "bias_rows": 4, "bias_max": 64,
                      "v_mix": False}}
    mam = {"type": "mamba1", "mlp": {"kind": "dense", "ff": 32},
           "mixer": {"inner": 32, "state": 1, "dt_rank": 1, "conv": 2}}
    return {"architecture": "Zudisun", "vocab": 40, "width": 32,
            "layers": [mam, att, att2], "norm": {"eps": 1e-6}}


def cfg_odd():
    """Nothing divisible by 4 or 8 (scalar kernel paths), nine query heads on
    three K/V heads, more experts than a wavefront has lanes, a one-tap
    convolution."""
    att = {"type": "attention", "mlp": _moe(70, 5, 6, groups=(7, 3),
                                            shared=5, scale=2.5),
           "mixer": {"heads": 9, "kv_heads": 3, "dim": 6, "vdim": 10,
                     "scale": 0.41, "bias_rows": 9, "bias_max": 31.5,
                     "v_mix": True, "q_temp": {"coef": 0.3, "every": 7}}}
    mam = {"type": "mamba1", "mlp": {"kind": "dense", "ff": 25},
           "mixer": {"inner": 22, "state": 33, "dt_rank": 5, "conv": 1}}
    mam2 = {"type": "mamba1", "mlp": None,
            "mixer": {"inner": 18, "state": 7, "dt_rank": 2, "conv": 5}}
    return {"architecture": "Zudisun", "vocab": 33, "width": 30,
            "layers": [mam, att, mam2, att], "norm": {"eps": 1e-4}}


ZOO = {"mixed": cfg_mixed, "degenerate": cfg_degenerate, "odd": cfg_odd}


def build(cfg_json, device, dtype, seed=0, page=8, pages=64, live=4,
          paced=True, graphs=False):
    w = orc.random_weights(cfg_json, seed, dtype)
    cfg = ZudisunConfig.from_json(cfg_json, lambda n: tuple(w[n].shape))
    cfg.max_position = 512
    model = ZudisunForCausalLM(cfg, device=device, dtype=dtype)
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


def model_close(got, want, dtype):
    """Whole-model comparison.  fp32: every row at rounding level.  bf16: a
    router fed bf16-rounded activations now and then prefers another expert
    than the float64 oracle does where two scores nearly tie, which moves
    that row by more than rounding (with one expert per token, by as much
    as the logits themselves); so nine rows in ten are held to bf16 rounding,
    the median row to half of it, and every row to the scale of the logits."""
    d = got.to(F64).cpu() - want
    d = d - d.mean(-1, keepdim=True)
    rows = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    if dtype == torch.float32:
        return float(rows.max()) < tol(dtype)
    return (float(rows.quantile(0.9)) < tol(dtype)
            and float(rows.median()) < tol(dtype) / 2
            and float(rows.max()) < 2.0)


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


def md_for(chunks, starts, slots, device, page=8, pages_per_seq=16):
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
                         seq_lens=list(chunks), is_prefill=True)
    return md, t(pos, torch.int32)


PORTIONS = ((0, 11), (11, 13), (13, 14), (14, 31), (31, 33), (33, 90))


# ====================================================== mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
def test_kernel_groups_present(device):
    if device == "cuda":
        from agentfield_amd.ops import _lib
        assert _lib.mixgroup("glue") is not None
        assert _lib.mixgroup("ssm") is not None  # no eager fallback on GPU


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(40, 20, 3, 4), (32, 1, 1, 2),
                                   (22, 33, 5, 1), (16, 130, 2, 6)])
def test_selective_ssm_alone(device, dtype, shape):
    """The mixer in portions (state and convolution inputs carried in a slot
    that held something else before) against the whole-sequence oracle."""
    C, N, R, K = shape
    torch.manual_seed(11)
    W, T = 24, 90
    mspec = {"inner": C, "state": N, "dt_rank": R, "conv": K}
    cfg = {"width": W, "vocab": 4, "norm": {"eps": 1e-5},
           "layers": [{"type": "mamba1", "mixer": mspec, "mlp": None}]}
    P = orc.random_weights(cfg, 5, dtype)
    h = torch.randn(T, W).to(dtype)
    want = orc.mamba1(h.to(F64), P, "l0.mix.", mspec)
    mod = SelectiveSSM(SelectiveSSMSpec(C, N, R, K), W)
    for name, src in (("w_in", "in"), ("conv", "conv"), ("conv_b", "conv.b"),
                      ("w_x", "x"), ("w_dt", "dt"), ("dt_b", "dt.b"),
                      ("o", "o")):
        w = P["l0.mix." + src]
        getattr(mod, name).data = (w.t().contiguous() if name == "conv"
                                   else w.clone())
    mod.A.copy_(-torch.exp(P["l0.mix.A_log"].float()))
    mod.D.copy_(P["l0.mix.D"].float())
    mod = mod.to(device)
    cache = SimpleNamespace(state={
        "ssm": {0: torch.full((3, C, N), 9.0, device=device)},
        "conv": {0: torch.full((3, max(K - 1, 1), C), 9.0, device=device,
                               dtype=dtype)}})
    got = []
    with torch.no_grad():
        for lo, hi in PORTIONS:
            md, pos = md_for([hi - lo], [lo], [2], device)
            got.append(mod(h[lo:hi].to(device), cache, 0, md, pos, {}).cpu())
    assert rel_err(torch.cat(got), want) < tol(dtype)
    assert float(cache.state["ssm"][0][1].min()) == 9.0  # other slots intact


@pytest.mark.parametrize("device", DEVICES)
def test_conv_history_shorter_than_taps(device):
    """One- and two-token portions with six taps: the carried inputs are a
    mix of old history and new rows."""
    torch.manual_seed(12)
    C, K, T = 10, 6, 17
    x = torch.randn(T, C)
    w, b = torch.randn(C, K), torch.randn(C)
    want = orc.silu(orc.causal_conv(x.to(F64), w, b))
    state = torch.full((2, K - 1, C), 5.0, device=device)
    got, lo = [], 0
    for n in (1, 2, 1, 1, 3, 2, 7):
        md, _ = md_for([n], [lo], [1], device)
        got.append(sm.causal_conv(x[lo:lo + n].to(device),
                                  w.t().contiguous().to(device),
                                  b.to(device), state, md).cpu())
        lo += n
    assert torch.allclose(torch.cat(got).to(F64), want, atol=1e-5)
    assert torch.allclose(state[1].cpu(), x[-(K - 1):], atol=1e-6)


def _attn_case(H, G, dk, dv, rows, dmax, every, dtype, seed=0, T=90, W=24):
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.45,
         "bias_rows": rows, "bias_max": dmax, "v_mix": True,
         "q_temp": {"coef": 0.6, "every": every}}
    cfg = {"width": W, "vocab": 4, "norm": {"eps": 1e-5},
           "layers": [{"type": "attention", "mixer": m, "mlp": None}]}
    P = orc.random_weights(cfg, seed, dtype)
    torch.manual_seed(seed)
    h = torch.randn(T, W).to(dtype)
    v_first = torch.randn(T, G, dv).to(dtype)
    return m, P, h, v_first


def _attn_run(m, P, h, v_first, device, dtype, portions, page=8):
    """q/k/v/gate projections with torch, then the two attention ops."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pre = "l0.mix."
    kc = torch.zeros(20, G, page, dk, dtype=dtype, device=device)
    vc = torch.zeros(20, G, page, dv, dtype=dtype, device=device)
    dev = lambda n: P[pre + n].to(device)  # noqa: E731
    f32 = lambda n: P[pre + n].float().to(device)  # noqa: E731
    buckets = sm.distance_buckets(m["bias_rows"], m["bias_max"]).to(device)
    got = []
    for lo, hi in portions:
        md, pos = md_for([hi - lo], [lo], [1], device, page, 18)
        x = h[lo:hi].to(device)
        vf = v_first[lo:hi].reshape(hi - lo, G * dv).to(device)
        q = sm.qk_unit_cache(x @ dev("q").T, x @ dev("k").T, x @ dev("v").T,
                             H, G, 1e-5, kc, vc, md.slots, pos,
                             m["q_temp"]["coef"], m["q_temp"]["every"], vf,
                             float(P[pre + "vmix"]))
        got.append(sm.sigmoid_attention(
            q, kc, vc, md, pos, m["scale"], H, rel=f32("rel"),
            buckets=buckets, talk=f32("talk"), head_bias=f32("pb"),
            gate=(x @ dev("g").T).contiguous()).cpu())
    return torch.cat(got)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 16, 8, 32, 120, 16),
                                   (1, 1, 8, 8, 2, 4, 3),
                                   (9, 3, 6, 10, 9, 31.5, 7),
                                   (6, 6, 24, 40, 12, 50, 1),
                                   (20, 2, 8, 8, 16, 64, 1000),
                                   (32, 8, 16, 24, 6, 33, 5),
                                   (12, 4, 8, 8, 4, 9, 2)])
def test_sigmoid_attention_alone(device, dtype, shape):
    H, G, dk, dv, rows, dmax, every = shape
    m, P, h, v_first = _attn_case(H, G, dk, dv, rows, dmax, every, dtype)
    eye = torch.eye(H * dv, dtype=F64)
    want, _ = orc.sigmoid_attention(h.to(F64), dict(P, **{"l0.mix.o": eye}),
                                    "l0.mix.", m, 1e-5, v_first.to(F64))
    got = _attn_run(m, P, h, v_first, device, dtype, PORTIONS)
    assert rel_err(got, want) < tol(dtype)


@pytest.mark.parametrize("rows,dmax", [(32, 120), (32, 128), (32, 256),
                                       (2, 4), (9, 31.5), (10, 23), (16, 8.5)])
def test_distance_buckets_match_definition(rows, dmax):
    tab = sm.distance_buckets(rows, dmax).tolist()
    for n in range(int(dmax) + 40):
        got = tab[n] if n < len(tab) else rows - 1
        assert got == orc.distance_bucket(n, rows, dmax), n


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_distance_bias_selects_rows(device, dtype):
    """With zero queries the weight of key j is sigmoid(rel[bucket(i-j)]):
    one open row of the table at a time shows exactly the keys of that
    bucket, in prompts and when the position is decoded alone, across page
    borders and past the last bucket."""
    rows, dmax, T, page, dv = 8, 37, 120, 8, 4
    for row in range(rows):
        rel = torch.full((rows, 1), -30.0)
        rel[row] = 30.0
        v = torch.arange(T, dtype=torch.float32)[:, None].expand(T, dv) / 8
        kc = torch.zeros(20, 1, page, 8, dtype=dtype, device=device)
        vc = torch.zeros(20, 1, page, dv, dtype=dtype, device=device)
        md, pos = md_for([T], [0], [1], device, page, 18)
        z = torch.zeros(T, 8, dtype=dtype, device=device)
        q = sm.qk_unit_cache(z, z, v.to(device, dtype), 1, 1, 1e-5, kc, vc,
                             md.slots, pos)
        tab = sm.distance_buckets(rows, dmax).to(device)
        o = sm.sigmoid_attention(q, kc, vc, md, pos, 1.0, 1,
                                 rel=rel.to(device), buckets=tab).cpu()
        for i in (0, 3, 7, 8, 36, 37, 38, 63, 64, 119):
            want = sum(j / 8 for j in range(i + 1)
                       if orc.distance_bucket(i - j, rows, dmax) == row)
            assert abs(float(o[i, 0]) - want) < 2e-2 * max(1.0, want), (row, i)
            md1, pos1 = md_for([1], [i], [1], device, page, 18)
            o1 = sm.sigmoid_attention(q[i:i + 1], kc, vc, md1, pos1, 1.0, 1,
                                      rel=rel.to(device), buckets=tab).cpu()
            assert abs(float(o1[0, 0]) - want) < 2e-2 * max(1.0, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_stands_out(device, dtype):
    """Among hundreds of keys whose weights are closed by a negative head
    bias, one far key matching the query returns its value: position 0, keys
    at a page's last and first place, the query's own position."""
    page, dk, dv, T = 8, 8, 8, 700
    torch.manual_seed(13)
    u = torch.zeros(dk)
    u[2] = 1.0
    for key_pos, query_pos in ((0, 699), (7, 650), (8, 650), (255, 256),
                               (256, 699), (699, 699), (1, 2)):
        k = torch.randn(T, dk)
        k[:, :4] = 0.0              # queries and keys live on disjoint
        q = torch.randn(T, dk)      # channels: only the marked pair matches
        q[:, 2:] = 0.0
        k[key_pos], q[query_pos] = u, u
        v = torch.randn(T, dv) * 0.1
        v[key_pos] = 3.0
        kc = torch.zeros(100, 1, page, dk, dtype=dtype, device=device)
        vc = torch.zeros(100, 1, page, dv, dtype=dtype, device=device)
        md, pos = md_for([T], [0], [1], device, page, 90)
        qn = sm.qk_unit_cache(q.to(device, dtype), k.to(device, dtype),
                              v.to(device, dtype), 1, 1, 1e-6, kc, vc,
                              md.slots, pos)
        # unit-RMS rows have q.k = dk for the matching pair, ~0 otherwise
        pb = torch.tensor([-60.0], device=device)
        o = sm.sigmoid_attention(qn, kc, vc, md, pos, 15.0, 1, head_bias=pb)
        assert torch.allclose(o[query_pos].float().cpu(),
                              torch.full((dv,), 3.0), atol=5e-2)
        other = (query_pos + 1) % T if query_pos + 1 < T else query_pos - 1
        assert float(o[other].float().abs().max()) < 1e-2
        md1, pos1 = md_for([1], [query_pos], [1], device, page, 90)
        o1 = sm.sigmoid_attention(qn[query_pos:query_pos + 1], kc, vc, md1,
                                  pos1, 15.0, 1, head_bias=pb)
        assert torch.allclose(o1[0].float().cpu(), torch.full((dv,), 3.0),
                              atol=5e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_query_temperature_steps(device):
    """q grows exactly at positions p with (p + 1) a multiple of `every`."""
    T, dk, every, coef = 20, 8, 4, 0.5
    q = torch.ones(T, dk)
    kc = torch.zeros(8, 1, 8, dk, device=device)
    vc = torch.zeros(8, 1, 8, dk, device=device)
    md, pos = md_for([T], [0], [1], device)
    qn = sm.qk_unit_cache(q.to(device), q.to(device), q.to(device), 1, 1, 0.0,
                          kc, vc, md.slots, pos, coef, every).cpu()
    for p in range(T):
        want = orc.query_temperature(p, coef, every)
        assert abs(float(qn[p, 0]) - want) < 1e-5, p
    assert float(qn[2, 0]) == 1.0 and float(qn[3, 0]) > 1.3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("case", [(12, 3, (4, 3), 2.0), (10, 3, (5, 2), 1.0),
                                  (4, 1, (1, 1), 1.0), (4, 4, (2, 2), 0.5),
                                  (70, 5, (7, 3), 2.5), (6, 2, None, 1.0),
                                  (8, 2, (8, 3), 1.0), (130, 6, (2, 1), 1.0)])
def test_router_alone(device, case):
    """Choice by corrected score inside the kept groups, weights from the
    uncorrected score.  Corrections are negative enough that a masked expert
    counted as 0 instead of minus infinity would win."""
    E, top, groups, scale = case
    torch.manual_seed(14)
    T = 64
    z = torch.randn(T, E) * 2
    corr = torch.randn(E) * 0.6 - 0.9
    r = {"experts": E, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    idx, w, wd = sm.moe_route(z.to(device), corr.to(device), top,
                              groups[0] if groups else 0,
                              groups[1] if groups else 0, scale, dense=True)
    idx, w, wd = idx.cpu(), w.cpu(), wd.cpu()
    for t in range(T):
        want_e, want_w = orc.route(z[t].to(F64), corr.to(F64), r)
        got = dict(zip(idx[t].tolist(), w[t].tolist()))
        assert sorted(got) == sorted(want_e), t
        for e, we in zip(want_e, want_w):
            assert abs(got[e] - float(we)) < 1e-5
            assert abs(float(wd[t, e]) - float(we)) < 1e-5
        assert int((wd[t] != 0).sum()) == top


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [5, 40])
def test_routed_experts_both_dispatches(device, dtype, rows):
    """Few rows take the every-expert path, many the gathered path; both
    agree with the oracle, also with an expert nobody chose."""
    torch.manual_seed(15)
    W = 24
    mlp = _moe(10, 3, 12, groups=(5, 2), shared=8, scale=1.3)
    cfg = {"width": W, "vocab": 4, "norm": {"eps": 1e-5}, "layers": [
        {"type": "mamba1", "mlp": mlp,
         "mixer": {"inner": 8, "state": 2, "dt_rank": 1, "conv": 2}}]}
    P = orc.random_weights(cfg, 3, dtype)
    h = torch.randn(rows, W).to(dtype)
    want = orc.moe_ff(h.to(F64), P, "l0.mlp.", mlp)
    mod = RoutedExperts(RoutedSpec(10, 3, 12, 1.3, 5, 2, 8), W)
    units = [f"e{e}." for e in range(10)] + ["shared."]
    mod.gate_up.data = torch.cat([P[f"l0.mlp.{u}{n}"] for u in units
                                  for n in ("gate", "up")])
    mod.down.data = torch.cat([P[f"l0.mlp.{u}down"] for u in units], 1)
    mod.router.copy_(P["l0.mlp.router"].float())
    mod.correction.copy_(P["l0.mlp.correction"].float())
    mod = mod.to(device)
    with torch.no_grad():
        y, _ = mod(h.to(device), SimpleNamespace(is_prefill=True))
    assert rel_err(y.float(), want) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_residual_and_glu(device, dtype):
    torch.manual_seed(16)
    T, W, F = 7, 30, 22
    x = torch.randn(T, W)
    y, b, w = (torch.randn(*s).to(dtype) for s in ((T, W), (W,), (W,)))
    want = x.to(F64) + orc.rms_norm(y.to(F64) + b.to(F64), w, 1e-5)
    xd = x.clone().to(device)
    h = sm.norm_residual(xd, y.to(device), b.to(device), w.to(device), 1e-5,
                         dtype)
    assert torch.allclose(xd.cpu().to(F64), want, atol=1e-5)
    assert torch.allclose(h.cpu().to(F64), want,
                          atol=1e-5 if dtype == torch.float32 else 5e-2)
    yf = torch.randn(T, W)                      # fp32 sublayer output
    xd2 = x.clone().to(device)
    sm.norm_residual(xd2, yf.to(device), None, w.to(device), 1e-5, dtype)
    assert torch.allclose(xd2.cpu().to(F64),
                          x.to(F64) + orc.rms_norm(yf.to(F64), w, 1e-5),
                          atol=1e-5)
    gu, bias = torch.randn(T, 2 * F).to(dtype), torch.randn(2 * F).to(dtype)
    for act, fn in (("relu", torch.relu), ("silu", orc.silu),
                    ("gelu_tanh", lambda a: 0.5 * a * (1 + torch.tanh(
                        math.sqrt(2 / math.pi) * (a + 0.044715 * a ** 3))))):
        g = gu[:, :F].to(F64) + bias[:F].to(F64)
        u = gu[:, F:].to(F64) + bias[F:].to(F64)
        got = sm.glu(gu.to(device), F, act, bias.to(device)).cpu()
        assert torch.allclose(got.to(F64), fn(g) * u,
                              atol=1e-5 if dtype == torch.float32 else 8e-2)


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
    assert model_close(got, want, dtype)
    assert len(eng.model.record_runs) == len(layers)
    for g, r in zip(eng.model.record_runs, layers):
        assert model_close(g, r, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(ZOO))
def test_prefill_then_token_by_token(device, dtype, name):
    """The first tokens of a sequence one by one, a prompt portion, then long
    decoding: past every temperature step, bucket edge and page border."""
    cj = ZOO[name]()
    eng, w = build(cj, device, dtype, pages=40)
    toks = tokens_for(cj, 200, 2)
    want = orc.forward(toks, cj, w)
    sched = [[("a", 1)]] * 6 + [[("a", 44)]] + [[("a", 1)]] * 150
    got = run_schedule(eng, {"a": toks}, sched)["a"]
    assert model_close(got, want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_down_to_two_tokens(device, dtype):
    cj = cfg_mixed()
    eng, w = build(cj, device, dtype)
    toks = tokens_for(cj, 120, 3)
    want = orc.forward(toks, cj, w)
    cuts = [2, 2, 3, 2, 17, 2, 40, 5, 2, 16, 1, 2, 26]
    assert sum(cuts) == len(toks)
    got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert model_close(got, want, dtype)
    whole = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    # how a prompt is cut changes nothing beyond rounding
    assert model_close(got, whole.to(F64), dtype)
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
    assert model_close(torch.cat([got[n] for n in reqs]),
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
    slack = 0.35 if dtype == torch.bfloat16 else \
        (0.03 if device == "cuda" else 1e-3)
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
    cj = cfg_degenerate()
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
    cfg = ZudisunConfig.from_json(cj, lambda n: tuple(w[n].shape))
    again = ZudisunConfig.from_json(cfg.to_json())
    assert again.layers == cfg.layers and again.eps == cfg.eps
    save_zudisun(w, cfg, str(tmp_path / "ckpt"))
    model = load_model(str(tmp_path / "ckpt"), device="cpu",
                       dtype=torch.float32)
    assert isinstance(model, ZudisunForCausalLM)
    assert model.cfg.layers == cfg.layers


def test_trace_runner_subprocess(tmp_path):
    """bin/trace_run on a checkpoint directory: a mixed schedule with reuse,
    logits compared with the oracle."""
    cj = cfg_degenerate()
    w = orc.random_weights(cj, 6, torch.bfloat16)
    cfg = ZudisunConfig.from_json(cj, lambda n: tuple(w[n].shape))
    save_zudisun(w, cfg, str(tmp_path / "m"))
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
