"""Nolavik on the GPU against the plain implementation (tests/plain_nolavik.py, float64 on the CPU): each mechanism
alone, then whole models of small made-up sizes in every way of cutting a request into steps, with pages and state
slots that are freed and used again, and greedy generation through the entry point.

Which experts a token uses is a discrete choice: the 32-bit engine makes the plain implementation's choices, so every
position is compared there.  Whole models in bfloat16 are held to three times what rounding operands of
matrix products to bfloat16 alone does to the plain logits (norms on both sides of every sublayer carry a sublayer's relative error into
the stream at full size, so a fixed bound says little)."""

import math
import random
from types import SimpleNamespace

import pytest
import torch

import plain_nolavik as pn
import traces
from nolavik_configs import SMALL, SMALL_B, SMALL_C, SMALL_D, config_of, delta, latent, moe, parallel

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def close(got, ref, dtype, what="", loose=1.0):
    got, ref = got.double().cpu(), ref.double()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    scale = max(1e-6, float(ref.abs().max()))
    worst = float((got - ref).abs().max()) / scale
    assert worst <= loose * (2.0 ** -6 if dtype == torch.bfloat16 else 2e-5), f"{what}: off by {worst:.2e} of the largest value"


def dev(x, dtype=torch.float32):
    return x.to(dtype).to(DEV).contiguous()


def ints(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def step_of(counts, lengths, slots):
    """What the recurrent kernels read of a step: request b brings counts[b] tokens and is lengths[b] long afterwards."""
    positions = [length - c + i for c, length in zip(counts, lengths) for i in range(c)]
    token_seq = [b for b, c in enumerate(counts) for _ in range(c)]
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    return SimpleNamespace(token_seq=ints(token_seq), positions=ints(positions), cu_seqlens=ints(cu), context_lens=ints(lengths),
                           state_slots=ints(slots), num_seqs=len(counts), max_count=max(counts))


def in_portions(total, portions):
    a, i = 0, 0
    while a < total:
        n = min(portions[i % len(portions)], total - a)
        i += 1
        yield a, n
        a += n


# ------------------------------------------------------------------------------ the stream's kernels
@pytest.mark.parametrize("hidden", [40, 72, 256, 1100])
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sum_through_a_norm_and_the_next_norm_in_one_kernel(hidden, dtype):
    from llmserve.ops import library as ops

    n = 9
    x, y = rnd(n, hidden, seed=1, scale=3.0), rnd(n, hidden, seed=2, scale=40.0)
    wb, w = rnd(hidden, seed=3) + 1, rnd(hidden, seed=4) + 1
    stream = dev(x)
    out = torch.full((n, hidden), float("nan"), dtype=dtype, device=DEV)
    ops.normed_add_norm(out, stream, dev(w), 1e-5, y=dev(y), y_weight=dev(wb), y_eps=1e-3)
    summed = x + pn.rms(y, 1e-3, wb)
    close(stream, summed, torch.float32, "the stream")
    close(out, pn.rms(summed, 1e-5, w), dtype, "the normed row")
    # picked rows: nothing is stored
    before = stream.clone()
    picked = torch.full((3, hidden), float("nan"), dtype=dtype, device=DEV)
    ops.normed_add_norm(picked, stream, dev(w), 1e-5, y=dev(y), y_weight=dev(wb), y_eps=1e-3, rows=ints([6, 0, 3]))
    close(picked, pn.rms(summed + pn.rms(y, 1e-3, wb), 1e-5, w)[[6, 0, 3]], dtype, "picked rows")
    assert torch.equal(stream, before)
    # nothing joins: the norm alone; and a vector added to every row
    ops.normed_add_norm(out, stream, dev(w), 1e-5)
    close(out, pn.rms(summed, 1e-5, w), dtype, "the norm alone")
    v = rnd(hidden, seed=5)
    ops.add_vector(stream, dev(v))
    close(stream, summed + v, torch.float32, "a vector on every row")


# ------------------------------------------------------------------------------ convolution and its ring
@pytest.mark.parametrize("taps,channels", [(3, 20), (4, 300), (2, 7), (1, 33)])
def test_the_convolution_in_portions_down_to_one_token(taps, channels):
    """Two requests in alternating portions on slots 2 and 0 of four; the other slots hold NaN, and so does each ring
    before its request starts (a token before position 0 counts as zero, whatever the ring holds)."""
    from llmserve.ops import library as ops

    lengths, pad, off = [37, 22], 3, 11
    u = [rnd(n, pad + channels + 2, seed=10 + i) for i, n in enumerate(lengths)]
    w, bias = rnd(channels, taps, seed=20), rnd(channels, seed=21)
    want = [pn.silu(pn.causal_conv(x[:, pad: pad + channels], w, bias)) for x in u]
    state = torch.full((4, off + max(taps - 1, 1) * channels + 5), float("nan"), dtype=torch.float32, device=DEV)
    state[:, :off] = 7.0
    state[:, off + (taps - 1) * channels:] = 7.0
    got = [torch.zeros(n, channels, dtype=F64) for n in lengths]
    cuts = [list(in_portions(lengths[0], (5, 1, 1, 2, 9))), list(in_portions(lengths[1], (1, 3, 1, 1, 8, 2)))]
    for step in range(max(len(c) for c in cuts)):
        who = [b for b in (0, 1) if step < len(cuts[b])]
        counts = [cuts[b][step][1] for b in who]
        ends = [cuts[b][step][0] + cuts[b][step][1] for b in who]
        rows = dev(torch.cat([u[b][cuts[b][step][0]: ends[i]] for i, b in enumerate(who)]))
        batch = step_of(counts, ends, [[2, 0][b] for b in who])
        out32 = torch.full((rows.shape[0], channels), float("nan"), dtype=torch.float32, device=DEV)
        out16 = torch.full((rows.shape[0], channels), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.conv_act(rows, pad, channels, dev(w), bias=dev(bias), state=state, ring_offset=off, batch=batch, out32=out32, out16=out16)
        assert torch.equal(out16, out32.to(torch.bfloat16))
        a = 0
        for i, b in enumerate(who):
            got[b][cuts[b][step][0]: ends[i]] = out32[a: a + counts[i]].double().cpu()
            a += counts[i]
    for b in (0, 1):
        close(got[b], want[b], torch.float32, f"request {b}")
    assert bool((state[:, :off] == 7.0).all()) and bool((state[:, off + (taps - 1) * channels:] == 7.0).all())
    assert bool(torch.isnan(state[1]).sum() == (taps - 1) * channels) and bool(torch.isnan(state[3]).sum() == (taps - 1) * channels)


# ------------------------------------------------------------------------------ the selective scan
def scan_weights(width, inner, states, rank, taps, seed):
    return {"in": rnd(2 * inner, width, seed=seed, scale=0.3), "conv": rnd(inner, taps, seed=seed + 1, scale=0.5),
            "conv.b": rnd(inner, seed=seed + 2, scale=0.2), "x": rnd(rank + 2 * states, inner, seed=seed + 3, scale=0.4),
            "dt": rnd(inner, rank, seed=seed + 4, scale=0.5), "dt.b": rnd(inner, seed=seed + 5) - 1.0,
            "A_log": rnd(inner, states, seed=seed + 6, scale=0.7), "D": rnd(inner, seed=seed + 7) + 1.0,
            "o": torch.eye(inner, dtype=F64)}


@pytest.mark.parametrize("inner,states,rank,taps", [(56, 5, 6, 4), (9, 24, 1, 1), (40, 37, 3, 2), (64, 16, 8, 4), (33, 100, 4, 3)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_selective_scan_whole_and_in_portions(inner, states, rank, taps, dtype):
    """The kernels behind the projections against the plain recurrence, in one portion and in many; the state of the
    request lies in slot 1 of three behind an offset, the others hold NaN."""
    from llmserve.ops import library as ops

    t, width = 75, 24
    h, w = rnd(t, width, seed=30), scan_weights(width, inner, states, rank, taps, seed=31)
    want = pn.selective_scan(h, w, "", {"inner": inner, "state": states, "dt_rank": rank, "conv": taps})
    xz = h @ w["in"].T
    for portions in ((1000,), (7, 2, 1, 19, 1, 1)):
        numbers = inner * states + (taps - 1) * inner
        state = torch.full((3, numbers), float("nan"), dtype=torch.float32, device=DEV)
        state[1] = 0.0
        outs = []
        for a, n in in_portions(t, portions):
            batch = step_of([n], [a + n], [1])
            proj = dev(xz[a: a + n])
            x32 = torch.empty((n, inner), dtype=torch.float32, device=DEV)
            ops.conv_act(proj, 0, inner, dev(w["conv"]), bias=dev(w["conv.b"]), state=state, ring_offset=inner * states, batch=batch,
                         out32=x32)
            low = dev(x32.double().cpu() @ w["x"].T)
            many = n > 2  # (portions of several tokens: silu(z) formed beside the recurrence, as the part does)
            dt = ops.step_sizes(torch.empty((n, inner), dtype=torch.float32, device=DEV), low, 0, dev(w["dt"].T), dev(w["dt.b"]),
                                z=proj if many else None, z_col=inner)
            close(dt, pn.softplus(low.double().cpu()[:, :rank] @ w["dt"].T + w["dt.b"]), torch.float32, "step sizes", loose=3)
            out = torch.full((n, inner), float("nan"), dtype=dtype, device=DEV)
            ops.selective_scan(out, x32, proj, inner, low, rank, rank + states, dt, dev(-torch.exp(w["A_log"])), dev(w["D"]), state, 0,
                               batch, z_prepared=many)
            outs.append(out.cpu())
        close(torch.cat(outs), want, dtype, f"portions {portions}", loose=3)
        assert bool(torch.isnan(state[0]).all()) and bool(torch.isnan(state[2]).all())


def test_a_scan_whose_state_must_last():
    """A channel that decays by next to nothing and reads its state back far later: what the first token wrote is the
    whole result at the last, so a state that is lost or cleared between portions shows."""
    from llmserve.ops import library as ops

    inner, states, t = 4, 3, 400
    x = torch.zeros(t, inner, dtype=F64)
    x[0] = 5.0
    low = torch.zeros(t, 2 * states, dtype=F64)
    low[0, :states] = 1.0          # B of the first token
    low[t - 1, states:] = 1.0      # C of the last
    dt = 1.25
    steps = torch.full((t, inner), dt, dtype=F64)
    a_neg = torch.full((inner, states), -1e-4, dtype=F64)
    want_last = states * dt * 5.0 * math.exp(-1e-4 * dt * (t - 1))
    state = torch.zeros((1, inner * states), dtype=torch.float32, device=DEV)
    z = torch.full((t, inner), 30.0, dtype=F64)  # silu(30) = 30
    last = None
    for a, n in in_portions(t, (64, 1, 1, 130, 2)):
        out = torch.empty((n, inner), dtype=torch.float32, device=DEV)
        ops.selective_scan(out, dev(x[a: a + n]), dev(z[a: a + n]), 0, dev(low[a: a + n]), 0, states, dev(steps[a: a + n]),
                           dev(a_neg), dev(torch.zeros(inner, dtype=F64)), state, 0, step_of([n], [a + n], [0]))
        last = out[-1].cpu()
    assert float(last[0]) == pytest.approx(30.0 * want_last, rel=1e-4)


# ------------------------------------------------------------------------------ the gated delta rule
def delta_weights(width, heads, kv, dk, dv, taps, seed):
    return {"q": rnd(kv * dk, width, seed=seed, scale=0.4), "k": rnd(kv * dk, width, seed=seed + 1, scale=0.4),
            "v": rnd(heads * dv, width, seed=seed + 2, scale=0.4), "q.conv": rnd(kv * dk, taps, seed=seed + 3, scale=0.6),
            "k.conv": rnd(kv * dk, taps, seed=seed + 4, scale=0.6), "v.conv": rnd(heads * dv, taps, seed=seed + 5, scale=0.6),
            "b": rnd(heads, width, seed=seed + 6, scale=0.3), "a": rnd(heads, width, seed=seed + 7, scale=0.3),
            "A_log": rnd(heads, seed=seed + 8) - 1.0, "dt_bias": rnd(heads, seed=seed + 9), "g": rnd(heads * dv, width, seed=seed + 10, scale=0.3),
            "norm": rnd(dv, seed=seed + 11) + 1.0, "o": torch.eye(heads * dv, dtype=F64)}


def run_delta(h, w, heads, kv, dk, dv, taps, eps, dtype, portions, fused=True):
    from llmserve.ops import library as ops

    t = h.shape[0]
    cq, cv = kv * dk, heads * dv
    channels = 2 * cq + cv
    proj_all = torch.cat([h @ w[x].T for x in ("q", "k", "v", "g", "a", "b")], dim=1)
    taps_w = dev(torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]]))
    scan = heads * dk * dv
    state = torch.full((3, scan + (taps - 1) * channels), float("nan"), dtype=torch.float32, device=DEV)
    state[2] = 0.0
    outs = []
    for a, n in in_portions(t, portions):
        batch = step_of([n], [a + n], [2])
        proj = dev(proj_all[a: a + n])
        qkv = torch.empty((n, channels), dtype=torch.float32, device=DEV)
        gates = dict(gates=proj, a_col=channels + cv, b_col=channels + cv + heads, a_log=dev(w["A_log"]), dt_bias=dev(w["dt_bias"]),
                     heads=heads)
        many = n > 2  # (decay and beta formed beside the recurrence, as the part does for portions of several tokens)
        if fused:  # the convolution, the unit vectors and the gates in one launch, as the part does
            ops.conv_heads(proj, 0, channels, taps_w, qkv, q_heads=kv, k_heads=kv, dk=dk, eps=1e-6, q_factor=dk ** -0.5, state=state,
                           ring_offset=scan, batch=batch, gates=gates if many else None)
        else:
            ops.conv_act(proj, 0, channels, taps_w, state=state, ring_offset=scan, batch=batch, out32=qkv)
            ops.unit_heads(qkv, q_col=0, k_col=cq, q_heads=kv, k_heads=kv, dk=dk, eps=1e-6, q_factor=dk ** -0.5,
                           gates=gates if many else None)
        o = torch.full((n, cv), float("nan"), dtype=torch.float32, device=DEV)
        ops.delta_scan(o, qkv, q_col=0, k_col=cq, v_col=2 * cq, kv_heads=kv, dk=dk, dv=dv, state=state, scan_offset=0, batch=batch,
                       prepared=many, **gates)
        out = torch.full((n, cv), float("nan"), dtype=dtype, device=DEV)
        ops.delta_finish(out, o, proj, channels, dev(w["norm"]), heads=heads, dv=dv, eps=eps)
        outs.append(out.cpu())
    assert bool(torch.isnan(state[0]).all()) and bool(torch.isnan(state[1]).all())
    return torch.cat(outs)


@pytest.mark.parametrize("heads,kv,dk,dv,taps", [(4, 2, 12, 20, 3), (1, 1, 72, 8, 1), (2, 2, 40, 8, 2), (6, 3, 16, 64, 4), (2, 1, 130, 17, 3)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_delta_rule_whole_and_in_portions(heads, kv, dk, dv, taps, dtype):
    t, width, eps = 70, 24, 1e-5
    h, w = rnd(t, width, seed=40), delta_weights(width, heads, kv, dk, dv, taps, seed=41)
    want = pn.gated_delta(h, w, "", {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "conv": taps}, eps)
    close(run_delta(h, w, heads, kv, dk, dv, taps, eps, dtype, (1000,)), want, dtype, "whole", loose=3)
    in_portions_fused = run_delta(h, w, heads, kv, dk, dv, taps, eps, dtype, (7, 2, 1, 19, 1, 1))
    close(in_portions_fused, want, dtype, "in portions", loose=3)
    # the kernels the fused launch stands for give the same numbers
    in_portions_apart = run_delta(h, w, heads, kv, dk, dv, taps, eps, dtype, (7, 2, 1, 19, 1, 1), fused=False)
    close(in_portions_apart, want, dtype, "in portions, convolution and unit vectors apart", loose=3)
    assert (in_portions_apart.double() - in_portions_fused.double()).abs().max() <= 1e-5 * float(want.abs().max())


def test_the_read_out_sees_the_tokens_own_write():
    """One token, a state of zero: o = (k . q) beta v, which is nothing if the read-out came before the write."""
    from llmserve.ops import library as ops

    dk, dv = 16, 8
    qkv = torch.zeros(1, 2 * dk + dv, dtype=F64)
    qkv[0, :dk] = 0.25
    qkv[0, dk: 2 * dk] = 0.25   # k . q = 1
    qkv[0, 2 * dk:] = torch.arange(1, dv + 1, dtype=F64)
    gates = torch.tensor([[0.0, 0.0]], dtype=F64)  # decay from a = 0, beta = 1/2
    state = torch.zeros((1, dk * dv), dtype=torch.float32, device=DEV)
    o = torch.empty((1, dv), dtype=torch.float32, device=DEV)
    ops.delta_scan(o, dev(qkv), q_col=0, k_col=dk, v_col=2 * dk, gates=dev(gates), a_col=0, b_col=1, a_log=dev(torch.zeros(1, dtype=F64)),
                   dt_bias=dev(torch.zeros(1, dtype=F64)), heads=1, kv_heads=1, dk=dk, dv=dv, state=state, scan_offset=0,
                   batch=step_of([1], [1], [0]))
    close(o[0], 0.5 * torch.arange(1, dv + 1, dtype=F64), torch.float32, "the first token's result")
    # and the state holds k u^T (kept column by column)
    close(state.view(dv, dk).t(), torch.outer(qkv[0, dk: 2 * dk], 0.5 * qkv[0, 2 * dk:]), torch.float32, "the state")


# ------------------------------------------------------------------------------ attention with a sink
def paged(t, k_heads, dk, v_heads, dv, bs, dtype, seed=0, spare=3):
    need = -(-t // bs)
    order = torch.randperm(need + spare, generator=torch.Generator().manual_seed(seed)).tolist()[:need]
    k_pool = torch.full((need + spare, k_heads, bs, dk), float("nan"), dtype=dtype, device=DEV)
    v_pool = torch.full((need + spare, v_heads, dv, bs), float("nan"), dtype=dtype, device=DEV)
    slots = [order[p // bs] * bs + p % bs for p in range(t)]
    return k_pool, v_pool, ints(order).reshape(1, need), slots


def sink_attention(proj, m, eps, dtype, bs, portions=(1000,), matrix_cores=False):
    """The engine's kernels on one request that comes in portions, from the projected q, k, v [t, ...] (float64): the
    rotation, the norm and the store, then the attention per portion over shuffled pages."""
    from llmserve.ops import library as ops
    from llmserve.parts.attention_composed import scaled_frequencies

    t = proj.shape[0]
    heads, kv, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    freq = scaled_frequencies(rot.get("base", 1e4), int(rot.get("dims", 0)), rot.get("scaling"))
    freq = dev(torch.tensor(freq, dtype=F64)) if freq else None
    k_pool, v_pool, table, slots = paged(t, kv, dk, kv, dv, bs, dtype)
    outs = []
    for a, n in in_portions(t, portions):
        p = dev(proj[a: a + n])
        q = torch.empty((n, heads * dk), dtype=dtype, device=DEV)
        ops.norm_store(q, p, q_heads=heads, k_heads=kv, dk=dk, v_heads=kv, dv=dv, eps=eps, positions=ints(range(a, a + n)),
                       slots=ints(slots[a: a + n]), k_pool=k_pool, v_pool=v_pool, block_size=bs, freq=freq, unit_norm=True)
        out = torch.full((n, heads * dv), float("nan"), dtype=dtype, device=DEV)
        common = dict(heads=heads, kv_heads=kv, dk=dk, dv=dv, block_size=bs, scale=float(m["scale"]), sink=True)
        if matrix_cores:
            ops.attend_composed_mfma(out, q, k_pool, v_pool, table, ints([0, n]), ints([a + n]), 0, 1, n, **common)
        else:
            ops.attend_composed(out, q, k_pool, v_pool, table, ints([0] * n), ints(range(a, a + n)), **common)
        outs.append(out.cpu())
    return torch.cat(outs)


def attention_case(heads, kv, dk, dv, dims, scaling, t, seed, dtype):
    width = 32
    m = {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "scale": 6.0 / math.sqrt(dk),
         "rot": {"base": 200.0, "dims": dims, "scaling": scaling}}
    h = rnd(t, width, seed=seed)
    w = {"q": rnd(heads * dk, width, seed=seed + 1), "k": rnd(kv * dk, width, seed=seed + 2), "v": rnd(kv * dv, width, seed=seed + 3),
         "o": torch.eye(heads * dv, dtype=F64)}
    if dtype == torch.bfloat16:
        h, w = h.to(dtype).double(), {k: v.to(dtype).double() for k, v in w.items()}
    proj = torch.cat([h @ w["q"].T, h @ w["k"].T, h @ w["v"].T], dim=1)
    return m, h, w, proj


SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48}
SINK_CASES = [  # heads, kv_heads, dk, dv, turned dimensions, stretched, block size, tokens
    (4, 2, 24, 12, 16, SCALING, 8, 90),
    (3, 3, 8, 8, 8, None, 4, 50),
    (5, 1, 24, 12, 0, None, 16, 260),
    (6, 3, 80, 48, 2, SCALING, 16, 70),
    (1, 1, 10, 6, 10, None, 8, 20),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,dims,scaling,bs,t", SINK_CASES)
def test_turned_and_normed_queries_and_keys_and_the_sink(dtype, heads, kv, dk, dv, dims, scaling, bs, t):
    eps = 1e-5
    m, h, w, proj = attention_case(heads, kv, dk, dv, dims, scaling, t, 60, dtype)
    want = pn.sink_attention(h, w, "", m, eps)
    close(sink_attention(proj, m, eps, dtype, bs), want, dtype, "whole", loose=3)
    close(sink_attention(proj, m, eps, dtype, bs, portions=(7, 2, 1, 19, 1, 1)), want, dtype, "in portions", loose=3)


MATRIX_CORE_CASES = [  # heads, kv_heads, dk, dv, turned dimensions, stretched, block size, tokens
    (6, 2, 128, 96, 32, SCALING, 16, 300),
    (8, 1, 64, 64, 32, None, 16, 420),
    (6, 3, 80, 48, 16, SCALING, 8, 150),
    (3, 3, 32, 16, 32, None, 4, 70),
]


@pytest.mark.parametrize("heads,kv,dk,dv,dims,scaling,bs,t", MATRIX_CORE_CASES)
def test_the_sink_on_the_matrix_cores(heads, kv, dk, dv, dims, scaling, bs, t):
    """The same through the bfloat16 kernel on the matrix cores: whole, in portions, and token by token."""
    eps, dtype = 1e-5, torch.bfloat16
    m, h, w, proj = attention_case(heads, kv, dk, dv, dims, scaling, t, 61, dtype)
    want = pn.sink_attention(h, w, "", m, eps)
    close(sink_attention(proj, m, eps, dtype, bs, matrix_cores=True), want, dtype, "whole", loose=3)
    close(sink_attention(proj, m, eps, dtype, bs, portions=(7, 2, 1, 19, 1, 1, 64), matrix_cores=True), want, dtype, "in portions", loose=3)
    close(sink_attention(proj, m, eps, dtype, bs, portions=(t - 40,) + (1,) * 40, matrix_cores=True), want, dtype, "token by token",
          loose=3)


@pytest.mark.parametrize("matrix_cores", [False, True])
def test_the_sink_takes_its_share_and_a_far_key_is_found(matrix_cores):
    """Queries and keys are unit-RMS vectors, so a score is at most dk * scale.  (1) Every key at right angles to the
    query: all scores are 0, the sink holds one part in t + 1 and the result is the mean of the values times t / (t + 1):
    without the sink it would be the mean itself.  (2) One key far back equal to the query, with a large scale: it takes
    all the weight, at a page's border and in the first page alike."""
    dk, dv, bs = 16, 16, 16
    dtype = torch.bfloat16 if matrix_cores else torch.float32
    m = {"heads": 1, "kv_heads": 1, "dim": dk, "vdim": dv, "scale": 1.0, "rot": {"dims": 0}}
    for t in (1, 2, 17, 100):
        q = torch.zeros(t, dk, dtype=F64)
        q[:, 0] = 1.0
        k = torch.zeros(t, dk, dtype=F64)
        k[:, 1] = 1.0
        v = torch.arange(t, dtype=F64)[:, None].expand(t, dv) * 0.125 + 1.0
        got = sink_attention(torch.cat([q, k, v], dim=1), m, 1e-6, dtype, bs, portions=(t - 1, 1) if t > 1 else (1,),
                             matrix_cores=matrix_cores)
        want = v[:, 0].cumsum(0) / (torch.arange(t, dtype=F64) + 2.0)
        close(got[:, 0], want, dtype, f"{t} keys at right angles", loose=2)
    t, m["scale"] = 700, 4.0  # a match scores dk * 4 = 64, everything else 0
    for far in (0, 15, 16, 31, 32, 333, 698):
        q = torch.zeros(t, dk, dtype=F64)
        q[:, 0] = 1.0
        k = torch.zeros(t, dk, dtype=F64)
        k[:, 1] = 1.0
        k[far] = 0.0
        k[far, 0] = 1.0
        v = torch.arange(t, dtype=F64)[:, None].expand(t, dv).clone()
        got = sink_attention(torch.cat([q, k, v], dim=1), m, 1e-6, dtype, bs, portions=(t - 1, 1), matrix_cores=matrix_cores)
        assert float(got[t - 1, 0]) == pytest.approx(float(far), abs=0.02 * far + 1e-3), f"the key at {far}"


# ------------------------------------------------------------------------------ latent attention, pairs a half apart
@pytest.mark.parametrize("dr,dims", [(8, 8), (12, 4), (16, 16), (6, 0)])
def test_the_rotated_parts_turn_in_pairs_a_half_apart(dr, dims):
    from llmserve.ops import library as ops

    n, heads, dn, r, q_rank = 7, 3, 10, 20, 12
    positions = [0, 1, 2, 700, 5, 31, 1500]
    freq64 = pn.frequencies(50.0, dims)
    freq = dev(freq64) if dims else None
    q = rnd(n, heads, dn + dr, seed=70)
    plain = torch.empty((n, heads * dn), dtype=torch.float32, device=DEV)
    folded = torch.zeros((n, heads * (r + dr)), dtype=torch.float32, device=DEV)
    ops.latent_query(plain, folded, dev(q.reshape(n, -1)), heads=heads, dn=dn, dr=dr, r=r, freq=freq, positions=ints(positions),
                     pairing="half")
    want = torch.stack([pn.rotate_half(q[i: i + 1, :, dn:].expand(p + 1, heads, dr), freq64, torch.arange(p + 1))[p]
                        for i, p in enumerate(positions)])
    close(folded.view(n, heads, r + dr)[:, :, r:], want, torch.float32, "queries", loose=20)
    close(plain.view(n, heads, dn), q[..., :dn], torch.float32, "unrotated parts")
    z = rnd(n, q_rank + r + dr, seed=71)
    wq, wc = rnd(q_rank, seed=72) + 1, rnd(r, seed=73) + 1
    pool = torch.full((2, 1, 8, r + dr), float("nan"), dtype=torch.float32, device=DEV)
    cq = torch.empty((n, q_rank), dtype=torch.float32, device=DEV)
    ops.latent_prepare(dev(z), col_q=0, q_rank=q_rank, col_c=q_rank, r=r, dr=dr, wq=dev(wq), wc=dev(wc), freq=freq,
                       positions=ints(positions), eps=1e-5, cq=cq, pool=pool, slots=ints([8, 9, 10, 3, 4, 5, 15]), pairing="half")
    rows = pool.view(16, r + dr)[[8, 9, 10, 3, 4, 5, 15]]
    close(cq, pn.rms(z[:, :q_rank], 1e-5, wq), torch.float32, "the query latent")
    close(rows[:, :r], pn.rms(z[:, q_rank: q_rank + r], 1e-5, wc), torch.float32, "the latent")
    want_k = torch.stack([pn.rotate_half(z[i: i + 1, None, q_rank + r:].expand(p + 1, 1, dr), freq64, torch.arange(p + 1))[p, 0]
                          for i, p in enumerate(positions)])
    close(rows[:, r:], want_k, torch.float32, "the shared key part", loose=20)


# ------------------------------------------------------------------------------ routing and experts
def expert_weights(width, experts, ff, shared, seed):
    t = {"router": rnd(experts, width, seed=seed), "router.b": rnd(experts, seed=seed + 1, scale=2.0)}
    for e in range(experts):
        t[f"e{e}.gate"], t[f"e{e}.up"] = rnd(ff, width, seed=seed + 10 + 3 * e, scale=0.3), rnd(ff, width, seed=seed + 11 + 3 * e, scale=0.3)
        t[f"e{e}.down"] = rnd(width, ff, seed=seed + 12 + 3 * e, scale=0.3)
    if shared:
        t["shared.gate"], t["shared.up"] = rnd(shared, width, seed=seed + 2, scale=0.3), rnd(shared, width, seed=seed + 3, scale=0.3)
        t["shared.down"], t["shared.sg"] = rnd(width, shared, seed=seed + 4, scale=0.3), rnd(1, width, seed=seed + 5, scale=0.5)
    return t


@pytest.mark.parametrize("experts,top", [(6, 2), (16, 4), (5, 1), (4, 4), (9, 3)])
def test_the_router_adds_its_bias_and_weighs_the_chosen_alone(experts, top):
    from llmserve.ops import library as ops

    n, width = 40, 24
    h = rnd(n, width, seed=80)
    t = expert_weights(width, experts, 4, 0, seed=81)
    extra = rnd(2, width, seed=82)
    chosen = torch.empty((n, top), dtype=torch.int32, device=DEV)
    weight = torch.empty((n, top), dtype=torch.float32, device=DEV)
    extra_out = torch.full((n, 2), float("nan"), dtype=torch.float32, device=DEV)
    ops.moe_router(chosen, weight, dev(h), dev(torch.cat([t["router"], extra])), renormalize=True, scores="softmax",
                   bias=dev(t["router.b"]), extra_out=extra_out)
    idx, w = pn.route(h, t, "", top)
    assert torch.equal(chosen.cpu().long(), idx)
    close(weight, w, torch.float32, "weights", loose=3)
    close(extra_out, h @ extra.T, torch.float32, "the rows behind the experts'", loose=3)
    # the bias decides: without it other experts are chosen somewhere
    ops.moe_router(chosen, weight, dev(h), dev(t["router"]), renormalize=True, scores="softmax")
    assert not torch.equal(chosen.cpu().long(), idx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,ff,shared,rows", [(6, 2, 24, 40, 150), (3, 1, 40, 0, 1), (8, 8, 4, 12, 37), (16, 4, 16, 16, 600)])
def test_experts_and_the_shared_expert_against_the_plain_sum(dtype, experts, top, ff, shared, rows):
    from llmserve.parts import model  # noqa: F401  (registers the built-in parts)
    from llmserve.parts.registry import FEED_FORWARDS, BuildContext
    from llmserve.parts.spec import PartSpec

    width = 32
    t = expert_weights(width, experts, ff, shared, seed=90)
    h = rnd(rows, width, seed=91)
    if dtype == torch.bfloat16:
        h, t = h.to(dtype).double(), {k: v.to(dtype).double() for k, v in t.items()}
    part = FEED_FORWARDS.build(PartSpec("experts", {
        "hidden": width, "intermediate": ff, "experts": experts, "top": top, "unit": "silu", "scores": "softmax", "renormalize": True,
        "weight_on": "output", "router_bias": True, "shared": {"intermediate": shared, "gate": True} if shared else None}),
        BuildContext(dtype, DEV))
    assert set(part.param_infos()) == set(t)
    part.load({k: dev(v, dtype) for k, v in t.items()})
    mlp = {"router": {"experts": experts, "top": top}, "shared": {"ff": shared} if shared else None}
    close(part.forward(dev(h, dtype)), pn.mixture(h, t, "", mlp), dtype, "experts", loose=4)


# ------------------------------------------------------------------------------ whole models
def write_model(folder, config, seed):
    from safetensors.torch import load_file, save_file

    from llmserve.weights import write_random_model

    # stored in bfloat16, so that both engines and the plain implementation hold the same numbers
    write_random_model(folder, config, seed=seed, dtype=torch.bfloat16, std=0.08, norm_std=0.05)
    tensors = load_file(str(folder / "model.safetensors"))
    for name in tensors:  # routers that decide: with logits this close together, most choices would be a coin's toss in bfloat16
        if name.endswith(".mlp.router"):
            tensors[name] = (tensors[name].float() * 8.0).to(torch.bfloat16)
    save_file(tensors, str(folder / "model.safetensors"))
    return {k: v.double() for k, v in tensors.items()}


def position_errors(got, ref, scale):
    d = got.double() - ref.double()
    d = d - d.mean(dim=-1, keepdim=True)
    return d.pow(2).mean(dim=-1).sqrt() / scale


def bf16(h):
    return h.to(torch.bfloat16).double()


def logits_close(got, ref, dtype, what, noise=None):
    """Per position: the difference of the logits (mean taken off, root mean square over the vocabulary) against the
    root mean square of the logits themselves.  32-bit: every position.  bfloat16: against `noise`, the plain logits
    with nothing but operands of matrix products rounded to bfloat16 (sublayer inputs, what the last projections read,
    queries, keys, values and latents), which no bfloat16 engine avoids: the median and the upper quartile of the
    engine's differences stay within three times those of that rounding alone."""
    got, ref = (torch.cat(list(x)) if isinstance(x, (list, tuple)) else x for x in (got, ref))
    scale = ref.double().pow(2).mean().sqrt()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    err = position_errors(got, ref, scale)
    worst = int(err.argmax())
    if dtype == torch.float32:
        assert float(err.max()) <= 1e-4, f"{what}: position {worst} is off by {float(err.max()):.2e}"
        return
    floor = position_errors(torch.cat(list(noise)) if isinstance(noise, (list, tuple)) else noise, ref, scale)
    for q in (0.5, 0.75):
        a, b = float(err.quantile(q)), float(floor.quantile(q))
        assert a <= 3.0 * b + 2e-3, f"{what}: quantile {q} of the positions is off by {a:.2e}, rounding alone by {b:.2e}"


MODELS = {"small": (SMALL, 8), "small_b": (SMALL_B, 16), "small_c": (SMALL_C, 4), "small_d": (SMALL_D, 16)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, (config, bs)) in enumerate(MODELS.items()):
        folder = tmp_path_factory.mktemp(f"nolavik_{name}")
        out[name] = (folder, config, write_model(folder, config, seed=270 + i), bs)
    return out


def poison(runner):
    """Pages and state slots hold NaN until the engine writes them."""
    runner.storage.poison()
    for t in runner.storage.state.values():
        t.fill_(float("nan"))


def run_trace(runner, steps):
    from llmserve.engine.replay import Replayer

    rep, outputs = Replayer(runner), {}
    for rec in steps:
        out = rep.run(rec)
        runner.manager.check_invariants()
        if out.shape[0]:
            outputs[rec["step"]] = out.float().cpu()
    return traces.collect(steps, outputs)


@pytest.mark.parametrize("name", list(MODELS))
def test_the_stream_after_every_layer_run(models, name):
    """Layer run by layer run against the plain implementation, in 32-bit, the shifts of the loop included."""
    from llmserve.config import EngineConfig
    from llmserve.engine.batch import build_batch
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    ids = traces.random_ids(config["vocab"], 45, 5)
    want = []
    pn.forward(config, w, ids, collect=want)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=16, max_num_seqs=2,
                                                          use_graphs=False))
    runner.add_sequence("a")
    layout = runner.manager.append(["a"], [len(ids)])
    batch = build_batch(layout, [ids], [0], runner._uploader, runner.storage)
    model = runner.model
    x, delta = model.embedding.forward(batch.token_ids), None
    sources = model.cache_sources()
    assert len(want) == len(model.spec.schedule)
    for pos, index in enumerate(model.spec.schedule):
        if pos in model._shift_rows:
            model._shift(x, delta, model._shift_rows[pos])
        x, delta = model.blocks[index].forward(x, delta, batch, runner.storage.layer_cache(pos, sources[pos]))
        joined = pn.rms(delta.y.double().cpu(), delta.eps, delta.weight.double().cpu())
        # per token, against the root mean square of the stream: the median token within rounding, and no token far off (a
        # norm behind every sublayer carries the rounding of a small result into the stream at full size)
        got = x[:, 0].double().cpu() + joined
        err = (got - want[pos]).pow(2).mean(-1).sqrt() / want[pos].pow(2).mean().sqrt()
        assert torch.isfinite(got).all() and float(err.median()) <= 5e-5 and float(err.max()) <= 5e-4, \
            f"after layer run {pos}: median {float(err.median()):.2e}, worst {float(err.max()):.2e}"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("graphs", [True, False])
def test_every_way_of_cutting_gives_the_plain_logits(models, name, dtype_name, graphs):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    dtype = getattr(torch, dtype_name)
    seqs = {f"r{i}": traces.random_ids(config["vocab"], n, 300 + i) for i, n in enumerate([67, 1, 30, 41, 2, 75])}
    ref = {rid: pn.forward(config, w, ids) for rid, ids in seqs.items()}
    noise = [pn.forward(config, w, ids, rounded=bf16) for ids in seqs.values()] if dtype == torch.bfloat16 else None
    modes = {"whole": traces.whole(seqs), "decode": traces.prefill_then_decode(seqs, tail=40),
             "portions": traces.portions(seqs), "mixed": traces.mixed(seqs, seed=3, live_max=3)}
    for mode, steps in modes.items():
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                              max_num_seqs=3, use_graphs=graphs))
        assert runner._use_graphs == graphs  # every part of the model can be captured
        poison(runner)
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], dtype, f"{name} {mode} {dtype_name}", noise)
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
        if graphs and mode == "decode":
            assert runner._graphs, "steps of single tokens were not replayed from a graph"


def test_a_batch_gives_each_request_what_it_gets_alone(models):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, _w, bs = models["small"]
    seqs = {f"b{i}": traces.random_ids(config["vocab"], n, 500 + i) for i, n in enumerate([50, 13, 29])}
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=64, max_num_seqs=3))
    alone = run_trace(runner, traces.portions(seqs))
    together = run_trace(runner, traces.mixed(seqs, seed=9, live_max=3))
    for rid in seqs:
        assert (alone[rid] - together[rid]).abs().max() <= 2e-5 * float(alone[rid].abs().max())


def test_long_decoding_and_the_prompt_of_the_same_tokens_agree(models):
    """280 tokens: whole in one step, and most of them one by one through the states and the pages; then again on the
    slot and the pages that came back."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small_c"]
    ids = traces.random_ids(config["vocab"], 280, 77)
    ref = pn.forward(config, w, ids)
    for graphs in (True, False):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=-(-280 // bs) + 1,
                                                              max_num_seqs=2, use_graphs=graphs))
        poison(runner)
        got = run_trace(runner, traces.prefill_then_decode({"long": ids}, tail=250))
        logits_close(got["long"], ref, torch.float32, "long decoding")
        whole = run_trace(runner, traces.whole({"again": ids}))
        logits_close(whole["again"], ref, torch.float32, "the whole prompt on the slot and pages that came back")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_long_request_at_matrix_core_sizes(models, dtype_name):
    """650 tokens through every kind of layer at sizes the matrix-core kernels take: the prompt in one step and its last
    tokens one by one (keys shared out to several workgroups, several tiles a wave), then in portions on the pages
    and the slot that came back."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small_d"]
    dtype = getattr(torch, dtype_name)
    ids = traces.random_ids(config["vocab"], 650, 78)
    ref = pn.forward(config, w, ids)
    noise = pn.forward(config, w, ids, rounded=bf16) if dtype == torch.bfloat16 else None
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=-(-650 // bs) + 1,
                                                          max_num_seqs=2))
    poison(runner)
    got = run_trace(runner, traces.prefill_then_decode({"long": ids}, tail=48))
    logits_close(got["long"], ref, dtype, f"a long prompt, then token by token, {dtype_name}", noise)
    again = run_trace(runner, traces.portions({"again": ids}, sizes=[200, 7, 2, 130, 64, 1, 33]))
    logits_close(again["again"], ref, dtype, f"the same in portions, {dtype_name}", noise)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(models, dtype_name):
    from llmserve import LLM, EngineConfig, SamplingParams

    folder, config, w, bs = models["small"]
    prompts = [traces.random_ids(config["vocab"], n, 600 + i) for i, n in enumerate([19, 3, 33, 8, 1])]
    llm = LLM(folder, dtype=dtype_name, engine=EngineConfig(block_size=bs, num_blocks=40, max_num_seqs=3,
                                                            max_num_batched_tokens=16))
    assert llm.runner.takes_device_tokens  # decode steps are replayed graphs, fed from the sampler's ids
    results = llm.generate(prompts, SamplingParams(max_new_tokens=24))
    for prompt, result in zip(prompts, results):
        assert len(result.tokens) == 24
        ref = pn.forward(config, w, prompt + result.tokens)
        far = 0
        for i, tok in enumerate(result.tokens):
            row = ref[len(prompt) - 1 + i]
            if dtype_name == "float32":  # the plain implementation's own choice, but for a tie within rounding
                far += float(row.max() - row[tok]) > 1e-4 * float(ref.pow(2).mean().sqrt())
            else:
                far += float(row.max() - row[tok]) > 0.25 * float(ref.pow(2).mean().sqrt()) + 1e-3
        assert far <= (0 if dtype_name == "float32" else 2)
    assert llm.runner.manager.num_free_slots == 3


def test_named_sizes_run_from_the_command_line_entry(capsys):
    from llmserve.cli import main

    assert main(["--model", "nolavik-tiny", "--random-weights", "--max-new-tokens", "5", "--dtype", "float32"]) == 0
    assert "decode=" in capsys.readouterr().out


def drawn_config(seed: int) -> tuple[dict, int]:
    """A configuration drawn at random from what config.json allows: the three kinds of layer in any order, layers
    without feed-forward, with and without a shared expert, a loop anywhere (or none) of 1 to 3 passes, 1 to 6 heads, 1
    to all of them key/value heads, sizes from 2 up and beyond 64, rotations over all, a part or nothing of a head with
    plain or stretched frequencies, 1 to 40 states a channel, 1 to 5 taps; and a page size."""
    rng = random.Random(seed)

    def rot(within, may_be_none=True):
        dims = rng.choice([within, within // 2 // 2 * 2, 2] + ([0] if may_be_none else []))
        r = {"base": rng.choice([10.0, 10000.0, 1e6]), "dims": min(dims, within // 2 * 2)}
        if rng.random() < 0.5 and r["dims"]:
            r["scaling"] = {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]),
                            "original": rng.choice([16, 64, 512])}
        return r

    def mlp():
        if rng.random() < 0.2:
            return None
        experts = rng.randint(1, 9)
        return moe(experts, rng.randint(1, min(4, experts)), rng.choice([8, 24, 40]), rng.choice([0, 8, 40]))

    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(["latent", "delta", "parallel"])
        if kind == "latent":
            dr = rng.choice([2, 4, 8, 16])
            layers.append(latent(heads=rng.randint(1, 5), dim=rng.choice([4, 8, 16, 20, 32]), rot_dim=dr, vdim=rng.choice([4, 8, 16, 40]),
                                 q_rank=rng.choice([8, 16, 24]), kv_rank=rng.choice([8, 16, 32, 48]), scale=rng.choice([0.1, 0.2, 0.35]),
                                 rot=rot(dr, False), mlp=mlp()))
        elif kind == "delta":
            kv = rng.choice([1, 2, 3])
            layers.append(delta(heads=kv * rng.choice([1, 2]), kv_heads=kv, dim=rng.choice([4, 8, 20, 32, 72]),
                                vdim=rng.choice([4, 8, 24, 64]), conv=rng.randint(1, 5), mlp=mlp()))
        else:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([4, 8, 16, 32, 48, 64, 96])
            layers.append(parallel(
                left={"heads": kv * rng.choice([1, 2, 3]), "kv_heads": kv, "dim": dim, "vdim": rng.choice([4, 8, 16, 64, dim, dim]),
                      "scale": rng.choice([0.2, 1.0, 8.0]) / math.sqrt(dim), "rot": rot(dim)},
                right={"inner": rng.choice([8, 24, 40, 100]), "state": rng.choice([1, 4, 16, 17, 40]), "dt_rank": rng.choice([1, 4, 8]),
                       "conv": rng.randint(1, 5)},
                left_scale=rng.choice([0.5, 1.0]), right_scale=rng.choice([0.3, 1.1]), mlp=mlp()))
    loop = None
    if rng.random() < 0.8:
        start = rng.randrange(len(layers))
        loop = (start, rng.randint(start + 1, len(layers)), rng.randint(1, 3))
    return config_of(layers, width=rng.choice([40, 64, 72, 100]), vocab=rng.choice([61, 128, 257]),
                     eps=rng.choice([1e-6, 1e-5]), loop=loop), rng.choice([4, 8, 16])


@pytest.mark.parametrize("seed", list(range(10)))
def test_configurations_drawn_at_random(tmp_path, seed):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    config, bs = drawn_config(seed)
    w = write_model(tmp_path, config, seed=900 + seed)
    seqs = {f"q{i}": traces.random_ids(config["vocab"], n, 40 * seed + i) for i, n in enumerate([90, 3, 47, 160, 18])}
    ref = {rid: pn.forward(config, w, ids) for rid, ids in seqs.items()}
    noise = [pn.forward(config, w, ids, rounded=bf16) for ids in seqs.values()]
    for dtype_name in ("float32", "bfloat16"):
        steps = traces.mixed(seqs, seed=seed, live_max=3, tail=30)
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(tmp_path, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                                max_num_seqs=3))
        poison(runner)
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], getattr(torch, dtype_name),
                     f"seed {seed} {dtype_name}: {config['layers']} {config.get('loop')}", noise)
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
