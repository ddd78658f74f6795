"""Felavik on the GPU against the plain implementation (tests/plain_felavik.py, float64 on the CPU): each mechanism
alone, then whole models of small made-up sizes in every way of cutting a request into steps, with pages and state
slots that are freed and used again, and greedy generation through the entry point.

Which experts a token uses is a discrete choice: the 32-bit engine makes the plain implementation's choices, so every
position is compared there.  Whole models in bfloat16 are held to a bound that three positions in four meet (every
position that attends to a token whose choice was a close call follows it), and a tighter one on the median."""

import math
import random

import pytest
import torch

import plain_felavik as pf
import traces
from felavik_configs import SMALL, SMALL_B, SMALL_C, SMALL_D, config_of, lightning, moe, parallel

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


# ------------------------------------------------------------------------------ the linear attention's kernels
@pytest.mark.parametrize("heads,dk,dv,dims,act", [(3, 12, 20, 0, "silu"), (2, 16, 8, 8, None), (1, 72, 80, 72, None),
                                                  (2, 130, 70, 2, "silu"), (4, 8, 8, 8, None)])
def test_activation_rotation_and_key_scale(heads, dk, dv, dims, act):
    from llmserve.ops import library as ops

    n, pad, base, key_scale = 11, 5, 50.0, dk ** -0.5
    q, k, v = rnd(n, heads, dk, seed=1), rnd(n, heads, dk, seed=2), rnd(n, heads, dv, seed=3)
    positions = [0, 1, 2, 700, 701, 5, 6, 7, 8, 31, 1500]
    proj = torch.cat([rnd(n, pad, seed=4), q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1), rnd(n, pad, seed=5)], dim=1)
    d = dev(proj)
    freq = None if not dims else dev(torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64))
    ops.decay_prepare(d, col_q=pad, col_k=pad + heads * dk, col_v=pad + 2 * heads * dk, heads=heads, dk=dk, dv=dv,
                      activation=act, freq=freq, rot_dims=dims, positions=ints(positions), key_scale=key_scale)
    f = pf.silu if act else (lambda z: z)
    want_q, want_k = f(q), f(k)
    if dims:
        for row, p in enumerate(positions):  # (the plain rotation counts positions from 0: one row at a time)
            for x in (want_q, want_k):
                x[row] = pf.rotate_half(x[row: row + 1].expand(p + 1, heads, dk), base, dims)[p]
    got = d.cpu().double()
    # 32-bit angles: a position of 1,500 times a frequency near one is known to 1e-4
    close(got[:, pad: pad + heads * dk], want_q.reshape(n, -1), torch.float32, "q", loose=20 if dims else 1)
    close(got[:, pad + heads * dk: pad + 2 * heads * dk], (want_k * key_scale).reshape(n, -1), torch.float32, "k", loose=20 if dims else 1)
    close(got[:, pad + 2 * heads * dk: pad + 2 * heads * dk + heads * dv], f(v).reshape(n, -1), torch.float32, "v")
    assert torch.equal(got[:, :pad], proj[:, :pad].float().double()) and torch.equal(got[:, -pad:], proj[:, -pad:].float().double())


@pytest.mark.parametrize("heads,dk,dv,dims,act", [(3, 12, 20, 0, "silu"), (2, 16, 8, 8, None), (1, 72, 80, 72, "silu"),
                                                  (2, 130, 70, 2, "silu"), (4, 8, 8, 4, None)])
@pytest.mark.parametrize("kernel", ["scan", "chunks"])
def test_the_recurrence_prepares_what_it_reads_as_the_kernel_of_its_own_does(heads, dk, dv, dims, act, kernel):
    """The recurrence may take the projection as it is and do the activation, the rotation and the key's factor on the
    way in: the same numbers as after the preparing kernel, and the projection is left alone."""
    from llmserve.ops import library as ops

    chunks = kernel == "chunks"
    if chunks and dk > ops.DECAY_CHUNKS_MAX_KEY:
        pytest.skip("keys wider than the kernel of runs takes")
    counts, lengths = ([70, 3, 1, 130], [70, 40, 1501, 139]) if chunks else ([1, 3, 1, 2], [40, 3, 1501, 9])
    n, pad = sum(counts), 3
    proj = dev(torch.cat([rnd(n, pad, seed=6), rnd(n, 2 * heads * dk + heads * dv, seed=7), rnd(n, pad, seed=8)], dim=1))
    positions = [length - c + i for c, length in zip(counts, lengths) for i in range(c)]
    freq = None if not dims else dev(torch.tensor([70.0 ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64))
    cols = dict(col_q=pad, col_k=pad + heads * dk, col_v=pad + 2 * heads * dk, heads=heads, dk=dk, dv=dv)
    prepare = dict(activation=act, freq=freq, rot_dims=dims, positions=ints(positions), key_scale=dk ** -0.5)
    decay = dev(torch.tensor([0.9 + 0.02 * h for h in range(heads)], dtype=F64))
    cu = ints([0] + list(torch.tensor(counts).cumsum(0)))
    state0 = dev(rnd(4, heads, dk, dv, seed=9))
    results = []
    for fused in (False, True):
        p, state = proj.clone(), state0.clone()
        out = torch.full((n, heads * dv), float("nan"), dtype=torch.float32, device=DEV)
        if not fused:
            ops.decay_prepare(p, **prepare, **cols)
        args = (out, p, state, ints([2, 0, 3, 1]), cu, ints(lengths), decay)
        if chunks:
            ops.decay_chunks(*args, max(counts), prepare=prepare if fused else None, **cols)
        else:
            ops.decay_scan(*args, prepare=prepare if fused else None, **cols)
        if fused:
            assert torch.equal(p, proj)
        results.append((out, state))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])


SCAN_CASES = [(3, 12, 20), (2, 16, 8), (1, 72, 80), (2, 130, 70), (1, 32, 64), (5, 8, 200)]


@pytest.mark.parametrize("kernel", ["scan", "chunks"])
@pytest.mark.parametrize("heads,dk,dv", SCAN_CASES)
def test_the_recurrence_in_portions_of_any_size_beside_each_other(heads, dk, dv, kernel):
    """Three requests of unequal length advance in portions of changing size, down to one token, in one launch each
    step; between them sits a request of length 0 (padding).  Foreign state slots hold NaN; a slot that a finished
    request gives back is used again by the next without being cleared by anyone but the kernel's own start.  Token by
    token, and in runs of 64 tokens (portions of one run, of a run and one token, of several runs and a rest, and of
    one token beside them)."""
    from llmserve.ops import library as ops

    chunks = kernel == "chunks"
    if chunks and dk > ops.DECAY_CHUNKS_MAX_KEY:
        pytest.skip("keys wider than the kernel of runs takes")
    lengths = {"a": 331, "b": 9, "c": 133, "d": 90} if chunks else {"a": 61, "b": 9, "c": 33, "d": 20}
    decay = [0.5 + 0.5 * (h + 1) / (heads + 1) for h in range(heads)]
    decay[-1] = 1.0 if heads > 1 else 0.97
    data = {r: (rnd(n, heads, dk, seed=i), rnd(n, heads, dk, seed=10 + i, scale=dk ** -0.5), rnd(n, heads, dv, seed=20 + i))
            for i, (r, n) in enumerate(lengths.items())}
    want = {r: pf.decayed_sums(*data[r], decay) for r in lengths}
    state = torch.full((4, heads, dk, dv), float("nan"), dtype=torch.float32, device=DEV)
    slot = {"a": 2, "b": 0, "c": 3, "d": 0}  # d takes b's slot when b has finished
    done = {r: 0 for r in lengths}
    got = {r: [] for r in lengths}
    sizes = [5, 64, 1, 65, 130, 2, 9, 63, 1, 17] if chunks else [5, 1, 2, 9, 1, 1, 17, 3]
    step = 0
    while any(done[r] < lengths[r] for r in lengths):
        live = [r for r in ("a", "b", "c") if done[r] < lengths[r]]
        if done["b"] == lengths["b"] and done["d"] < lengths["d"]:
            live.append("d")
        takes = {r: min(sizes[(step + i) % len(sizes)], lengths[r] - done[r]) for i, r in enumerate(live)}
        rows, cu, ctx, slots = [], [0], [], []
        for i, r in enumerate(live):
            if i == 1:  # a request of padding: no rows, no length
                cu.append(cu[-1])
                ctx.append(0)
                slots.append(1)
            a, n = done[r], takes[r]
            q, k, v = data[r]
            rows.append(torch.cat([q[a: a + n].reshape(n, -1), k[a: a + n].reshape(n, -1), v[a: a + n].reshape(n, -1)], dim=1))
            cu.append(cu[-1] + n)
            ctx.append(a + n)
            slots.append(slot[r])
        proj = dev(torch.cat(rows))
        out = torch.full((proj.shape[0], heads * dv), float("nan"), dtype=torch.float32, device=DEV)
        args = (out, proj, state, ints(slots), ints(cu), ints(ctx), dev(torch.tensor(decay, dtype=F64)))
        cols = dict(col_q=0, col_k=heads * dk, col_v=2 * heads * dk, heads=heads, dk=dk, dv=dv)
        if chunks:
            ops.decay_chunks(*args, max(takes.values()), **cols)
        else:
            ops.decay_scan(*args, **cols)
        at = 0
        for r in live:
            got[r].append(out[at: at + takes[r]].cpu())
            at += takes[r]
            done[r] += takes[r]
        step += 1
    for r in lengths:
        close(torch.cat(got[r]), want[r].reshape(lengths[r], -1), torch.float32, f"request {r}", loose=3)
    assert torch.isnan(state[1]).all()  # the padding request's slot was left alone


def test_a_key_far_back_is_still_in_the_state_after_long_decoding():
    """One key and value that stand out at position 3, then 600 tokens one by one with a decay of 1: a query along
    that key at the end gets its value back, and with a decay below 1 what the powers leave of it."""
    from llmserve.ops import library as ops

    heads, dk, dv, n = 2, 16, 24, 600
    q, k, v = rnd(n, heads, dk, seed=1, scale=0.01), rnd(n, heads, dk, seed=2, scale=0.01), rnd(n, heads, dv, seed=3, scale=0.01)
    k[3, :, :] = 0.0
    k[3, :, 5] = 10.0
    v[3] = rnd(heads, dv, seed=4, scale=5.0)
    q[n - 1, :, :] = 0.0
    q[n - 1, :, 5] = 1.0
    decay = [1.0, 0.99]
    want = pf.decayed_sums(q, k, v, decay)
    state = torch.zeros((1, heads, dk, dv), dtype=torch.float32, device=DEV)
    proj = dev(torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], dim=1))
    out = torch.empty((n, heads * dv), dtype=torch.float32, device=DEV)
    for t in range(n):
        ops.decay_scan(out[t: t + 1], proj[t: t + 1], state, ints([0]), ints([0, 1]), ints([t + 1]),
                       dev(torch.tensor(decay, dtype=F64)), col_q=0, col_k=heads * dk, col_v=2 * heads * dk,
                       heads=heads, dk=dk, dv=dv)
    close(out, want.reshape(n, -1), torch.float32, "600 single tokens", loose=5)
    last = out[n - 1].cpu().double().reshape(heads, dv)
    assert (last[0] - 10.0 * v[3, 0]).abs().max() < 0.05 * float(v[3, 0].abs().max())
    assert (last[1] - 10.0 * 0.99 ** (n - 4) * v[3, 1]).abs().max() < 0.05 * float(v[3, 1].abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dv,joint,gate", [(3, 20, True, "sigmoid"), (2, 8, False, "silu"), (1, 80, False, None),
                                                 (300, 4, False, "silu"), (2, 2048, True, "sigmoid"),
                                                 (4, 256, True, "sigmoid"), (16, 128, True, "silu"), (8, 1024, True, None),
                                                 (4, 1024, True, "sigmoid"), (4, 256, False, "silu")])
def test_head_norms_and_gates(dtype, heads, dv, joint, gate):
    """(Rows of 1,024, 2,048, 4,096 or 8,192 numbers whose gate starts at a multiple of 16 bytes are kept in registers
    where all heads are normed together; the others go through LDS.)"""
    from llmserve.ops import library as ops

    n, eps, width = 6, 1e-3, heads * dv
    pad = 3 if heads == 2 else 4
    o, z, w = rnd(n, heads, dv, seed=1, scale=4.0), rnd(n, width + pad, seed=2), rnd(width, seed=3) + 1
    o[2] *= 1e-3  # (eps matters for a small row)
    out = torch.full((n, width), float("nan"), dtype=dtype, device=DEV)
    ops.decay_finish(out, dev(o.reshape(n, width)), heads=heads, dv=dv, eps=eps, weight=dev(w) if joint else None,
                     gate=dev(z)[:, pad:] if gate else None, gate_activation=gate)
    want = pf.rms_norm(o.reshape(n, width), w, eps) if joint else pf.rms_unit(o, eps).reshape(n, width)
    if gate:
        want = want * (pf.silu(z[:, pad:]) if gate == "silu" else torch.sigmoid(z[:, pad:]))
    close(out, want, dtype, "normed and gated heads")


# ------------------------------------------------------------------------------ the softmax attention's ingredients
def paged(t, k_heads, dk, v_heads, dv, bs, dtype, seed=0, spare=3):
    need = -(-t // bs)
    order = torch.randperm(need + spare, generator=torch.Generator().manual_seed(seed)).tolist()[:need]
    k_pool = torch.full((need + spare, k_heads, bs, dk), float("nan"), dtype=dtype, device=DEV)
    v_pool = torch.full((need + spare, v_heads, dv, bs), float("nan"), dtype=dtype, device=DEV)
    slots = [order[p // bs] * bs + p % bs for p in range(t)]
    return k_pool, v_pool, ints(order).reshape(1, need), slots


def softmax_attention(h, w, m, eps, dtype, bs, portions=(1000,), matrix_cores=False):
    """The engine's kernels on one request that comes in portions: projection by the test, then norm_store and
    attend_composed (or, with `matrix_cores`, attend_composed_mfma) per portion over shuffled pages."""
    from llmserve.ops import library as ops
    from llmserve.parts.attention_composed import bias_by_distance

    t = h.shape[0]
    heads, kv, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    proj = torch.cat([h @ w["q"].T + w["q.b"], h @ w["k"].T + w["k.b"], h @ w["v"].T + w["v.b"], h @ w["g"].T], dim=1)
    k_pool, v_pool, table, slots = paged(t, kv, dk, kv, dv, bs, dtype)
    bias = bias_by_distance(dev(w["rel"]), int(m["bias_max"]))
    outs, a, i = [], 0, 0
    while a < t:
        n = min(portions[i % len(portions)], t - a)
        i += 1
        p = dev(proj[a: a + n])
        q = torch.empty((n, heads * dk), dtype=dtype, device=DEV)
        ops.norm_store(q, p, q_heads=heads, k_heads=kv, dk=dk, v_heads=kv, dv=dv, q_norm=dev(w["q.norm"]),
                       k_norm=dev(w["k.norm"]), eps=eps, temp_coef=float(m["q_temp"]["coef"]),
                       temp_every=int(m["q_temp"]["every"]), positions=ints(range(a, a + n)), slots=ints(slots[a: a + n]),
                       k_pool=k_pool, v_pool=v_pool, block_size=bs)
        out = torch.full((n, heads * dv), float("nan"), dtype=dtype, device=DEV)
        gate = p[:, (heads + kv) * dk + kv * dv:]
        if matrix_cores == "prompt":
            ops.attention_prompt_biased(out, q, k_pool, v_pool, table, ints([0, n]), ints([a + n]), 0, 1, n, 0, n, n_heads=heads,
                                        n_kv_heads=kv, head_dim=dk, block_size=bs, scale=float(m["scale"]), dist_bias=bias,
                                        gate=gate)
        elif matrix_cores:
            ops.attend_composed_mfma(out, q, k_pool, v_pool, table, ints([0, n]), ints([a + n]), 0, 1, n, heads=heads,
                                     kv_heads=kv, dk=dk, dv=dv, block_size=bs, scale=float(m["scale"]), dist_bias=bias,
                                     gate=gate)
        else:
            ops.attend_composed(out, q, k_pool, v_pool, table, ints([0] * n), ints(range(a, a + n)), heads=heads,
                                kv_heads=kv, dk=dk, dv=dv, block_size=bs, scale=float(m["scale"]), dist_bias=bias, gate=gate)
        outs.append(out.cpu())
        a += n
    return torch.cat(outs)


def attention_weights(heads, kv, dk, dv, rows, width, seed, rel_scale=2.0):
    w = {"q": rnd(heads * dk, width, seed=seed), "k": rnd(kv * dk, width, seed=seed + 1), "v": rnd(kv * dv, width, seed=seed + 2),
         "q.b": rnd(heads * dk, seed=seed + 3), "k.b": rnd(kv * dk, seed=seed + 4), "v.b": rnd(kv * dv, seed=seed + 5),
         "q.norm": rnd(dk, seed=seed + 6) + 1, "k.norm": rnd(dk, seed=seed + 7) + 1,
         "rel": rnd(rows, heads, seed=seed + 8, scale=rel_scale), "g": rnd(heads * dv, width, seed=seed + 9, scale=0.3),
         "o": torch.eye(heads * dv, dtype=F64)}
    return w


ATTENTION_CASES = [  # heads, kv_heads, dk, dv, table rows, farthest, every, block size, tokens
    (4, 2, 16, 24, 10, 40, 9, 8, 90),
    (3, 3, 8, 8, 4, 17, 2, 4, 50),
    (5, 1, 24, 12, 32, 200, 50, 16, 260),
    (6, 3, 80, 48, 8, 30, 64, 16, 70),
    (1, 1, 10, 6, 2, 5, 1, 8, 20),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,rows,farthest,every,bs,t", ATTENTION_CASES)
def test_normed_queries_distance_table_and_gate(dtype, heads, kv, dk, dv, rows, farthest, every, bs, t):
    """The table's entries differ by several units from row to row, so a distance that lands in the neighbouring
    bucket, at the last single distance, at `farthest` or beyond it, moves the weights visibly."""
    width, eps = 32, 1e-5
    m = {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "scale": 0.8 / math.sqrt(dk), "bias_max": farthest,
         "q_temp": {"coef": 1.5, "every": every}}
    h, w = rnd(t, width, seed=40), attention_weights(heads, kv, dk, dv, rows, width, seed=50)
    if dtype == torch.bfloat16:  # (keys and values as the cache will hold them are not what this test is about)
        h, w = h.to(dtype).double(), {k: v.to(dtype).double() for k, v in w.items()}
    want = pf.gated_softmax_attention(h, w, m, eps)
    close(softmax_attention(h, w, m, eps, dtype, bs), want, dtype, "whole", loose=3)
    close(softmax_attention(h, w, m, eps, dtype, bs, portions=(7, 2, 1, 19, 1, 1)), want, dtype, "in portions", loose=3)


MATRIX_CORE_CASES = [  # heads, kv_heads, dk, dv, table rows, farthest, every, block size, tokens
    (4, 2, 16, 32, 10, 40, 9, 16, 300),    # most keys lie beyond the table's reach
    (8, 1, 64, 64, 32, 200, 50, 16, 420),  # groups of tiles that the scalar unit addresses
    (6, 3, 80, 48, 8, 30, 64, 8, 150),
    (3, 3, 32, 16, 4, 1000, 2, 4, 70),     # every key within the table's reach
]


@pytest.mark.parametrize("heads,kv,dk,dv,rows,farthest,every,bs,t", MATRIX_CORE_CASES)
def test_distance_table_and_gate_on_the_matrix_cores(heads, kv, dk, dv, rows, farthest, every, bs, t):
    """The same as above through the bfloat16 kernel on the matrix cores: whole, in portions, and token by token."""
    width, eps, dtype = 32, 1e-5, torch.bfloat16
    m = {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "scale": 0.8 / math.sqrt(dk), "bias_max": farthest,
         "q_temp": {"coef": 1.5, "every": every}}
    h, w = rnd(t, width, seed=41), attention_weights(heads, kv, dk, dv, rows, width, seed=51)
    h, w = h.to(dtype).double(), {k: v.to(dtype).double() for k, v in w.items()}
    want = pf.gated_softmax_attention(h, w, m, eps)
    close(softmax_attention(h, w, m, eps, dtype, bs, matrix_cores=True), want, dtype, "whole", loose=3)
    close(softmax_attention(h, w, m, eps, dtype, bs, portions=(7, 2, 1, 19, 1, 1, 64), matrix_cores=True), want, dtype,
          "in portions", loose=3)
    close(softmax_attention(h, w, m, eps, dtype, bs, portions=(t - 40,) + (1,) * 40, matrix_cores=True), want, dtype,
          "token by token", loose=3)


PROMPT_KERNEL_CASES = [  # heads, kv_heads, head size, table rows, farthest, every, block size, tokens
    (8, 1, 64, 32, 200, 50, 16, 420),
    (4, 2, 32, 10, 40, 9, 8, 300),     # most keys lie beyond the table's reach
    (6, 3, 96, 8, 30, 64, 16, 150),
    (2, 2, 128, 12, 1000, 5, 32, 200),  # every key within the table's reach
]


@pytest.mark.parametrize("heads,kv,d,rows,farthest,every,bs,t", PROMPT_KERNEL_CASES)
def test_distance_table_and_gate_in_the_prompt_kernel(heads, kv, d, rows, farthest, every, bs, t):
    """The plain attention's prompt kernel in its variant with a distance table and a gate: whole, and in portions
    behind what the earlier portions left in the pages."""
    width, eps, dtype = 32, 1e-5, torch.bfloat16
    m = {"heads": heads, "kv_heads": kv, "dim": d, "vdim": d, "scale": 0.8 / math.sqrt(d), "bias_max": farthest,
         "q_temp": {"coef": 1.5, "every": every}}
    h, w = rnd(t, width, seed=42), attention_weights(heads, kv, d, d, rows, width, seed=52)
    h, w = h.to(dtype).double(), {k: v.to(dtype).double() for k, v in w.items()}
    want = pf.gated_softmax_attention(h, w, m, eps)
    close(softmax_attention(h, w, m, eps, dtype, bs, matrix_cores="prompt"), want, dtype, "whole", loose=3)
    close(softmax_attention(h, w, m, eps, dtype, bs, portions=(70, 2, 33, 19, 64, 5), matrix_cores="prompt"), want, dtype,
          "in portions", loose=3)


def test_a_key_that_stands_out_at_every_edge_of_the_distance_table():
    """One bucket of the table is raised by 30 so that the keys at its distances take all the weight; the values name
    their positions, so a query's result says which keys it saw in that bucket: those of the plain implementation."""
    heads, kv, dk, dv, rows, farthest, bs, t = 2, 1, 8, 4, 12, 60, 8, 100
    m = {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "scale": 1e-3, "bias_max": farthest,
         "q_temp": {"coef": 0.0, "every": 1}}
    width = 16
    h = rnd(t, width, seed=1)
    for row in range(rows):
        w = attention_weights(heads, kv, dk, dv, rows, width, seed=60, rel_scale=0.0)
        w["rel"][row] = 30.0
        w["v"][:] = 0.0
        w["g"][:] = 0.0  # a gate of one half
        # values: the position itself in every dimension, through the bias of v (per token it must come from h)
        h2 = h.clone()
        h2[:, 0] = torch.arange(t, dtype=F64) / 10.0
        w["v"][:, 0] = 10.0
        w["v.b"][:] = 0.0
        want = pf.gated_softmax_attention(h2, w, m, 1e-5)
        got = softmax_attention(h2, w, m, 1e-5, torch.float32, bs, portions=(13, 1, 1, 30))
        close(got, want, torch.float32, f"row {row} raised", loose=5)
        # and the plain result is the mean position of the bucket's keys, where the bucket is in reach
        lo = min(n for n in range(t) if pf.distance_bucket(n, rows, farthest) == row)
        hi = max(n for n in range(t) if pf.distance_bucket(n, rows, farthest) == row)
        i = t - 1
        mean_pos = sum(range(i - hi, i - lo + 1)) / (hi - lo + 1)
        assert abs(float(want[i, 0]) * 2 - mean_pos) < 0.02 * mean_pos + 0.02


# ------------------------------------------------------------------------------ routing and experts
@pytest.mark.parametrize("experts,top,groups,keep", [(6, 2, 3, 2), (12, 4, 4, 3), (8, 2, 4, 1), (5, 1, 1, 1), (4, 4, 2, 2),
                                                     (64, 6, 8, 3), (9, 3, 3, 3)])
def test_softmax_scores_and_the_best_groups(experts, top, groups, keep):
    from llmserve.ops import library as ops

    rows, hidden = 200, 24
    h, w = rnd(rows, hidden, seed=experts), rnd(experts, hidden, seed=top + 7, scale=0.7)
    chosen = torch.empty((rows, top), dtype=torch.int32, device=DEV)
    weight = torch.empty((rows, top), dtype=torch.float32, device=DEV)
    ops.moe_router(chosen, weight, dev(h), dev(w), renormalize=True, scores="softmax", groups=groups, keep=keep, renorm_eps=1e-20)
    want_e, want_w = pf.route(h.float().double(), w.float().double(), top, groups, keep)
    assert chosen.cpu().tolist() == want_e.tolist()
    close(weight, want_w, torch.float32, "weights")
    assert torch.allclose(weight.sum(dim=1).cpu(), torch.ones(rows), atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,ff,groups,keep,rows", [(6, 2, 24, 3, 2, 150), (3, 1, 40, 1, 1, 1), (8, 8, 4, 2, 2, 37),
                                                             (10, 3, 48, 5, 3, 300)])
def test_experts_against_the_plain_sum(dtype, experts, top, ff, groups, keep, rows):
    import llmserve.parts.model  # noqa: F401  (registers the built-in parts)
    from llmserve.parts.registry import FEED_FORWARDS, BuildContext
    from llmserve.parts.spec import PartSpec

    hidden = 48
    part = FEED_FORWARDS.build(PartSpec("experts", {"hidden": hidden, "intermediate": ff, "experts": experts, "top": top,
                                                    "unit": "silu", "scores": "softmax", "groups": groups, "keep": keep,
                                                    "renormalize": True, "renorm_eps": 1e-20, "weight_on": "output"}),
                               BuildContext(dtype, DEV))
    w = {name: rnd(*info.shape, seed=i, scale=0.25).to(dtype).double() for i, (name, info) in enumerate(part.param_infos().items())}
    part.load({k: dev(v, dtype) for k, v in w.items()})
    h = rnd(rows, hidden, seed=99).to(dtype).double()
    mlp = {"router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    close(part.forward(dev(h, dtype)), pf.experts(h, w, mlp), dtype, "experts", loose=2)


def test_the_soft_cap_the_weighted_sum_and_the_norm_without_a_mean():
    from llmserve.ops import library as ops

    x = rnd(5, 333, seed=1, scale=40.0)
    close(ops.softcap(dev(x), 30.0), 30.0 * torch.tanh(x / 30.0), torch.float32, "soft cap")
    a, b = rnd(7, 50, seed=2), rnd(7, 50, seed=3)
    da = dev(a)
    close(ops.weighted_sum(da, da, dev(b), 0.8, -1.1), 0.8 * a - 1.1 * b, torch.float32, "weighted sum in place")
    for hidden in (100, 98, 256, 512, 1024, 2048, 4096, 768, 8192):  # (a wave a row at 256 .. 4,096; a workgroup a row else)
        n = 7
        x, y, w = rnd(n, hidden, seed=4, scale=3.0) + 0.7, rnd(n, hidden, seed=5), rnd(hidden, seed=6) + 1
        for dtype in DTYPES:
            stream = dev(x).unsqueeze(1).contiguous()
            out = torch.full((n, hidden), float("nan"), dtype=dtype, device=DEV)
            ops.streams_norm(out, stream, dev(w), 1e-5, y=dev(y), center=False)
            close(out, pf.rms_norm(x + y, w, 1e-5), dtype, f"RMS norm of the closed sum, {hidden}")
            close(stream[:, 0], x + y, torch.float32, "the sum stored")
            # the first read of a layer: the rows as they are; picked rows: nothing stored
            again = torch.full((n, hidden), float("nan"), dtype=dtype, device=DEV)
            ops.streams_norm(again, stream, dev(w), 1e-5, center=False)
            assert torch.equal(again, out)
            picked = torch.full((3, hidden), float("nan"), dtype=dtype, device=DEV)
            before = stream.clone()
            ops.streams_norm(picked, stream, dev(w), 1e-5, y=dev(y), rows=ints([6, 0, 3]), center=False)
            close(picked, pf.rms_norm(x + 2 * y, w, 1e-5)[[6, 0, 3]], dtype, f"picked rows, {hidden}")
            assert torch.equal(stream, before)
            centered = torch.empty((n, hidden), dtype=torch.float32, device=DEV)
            ops.streams_norm(centered, stream, dev(w), 1e-5, center=True)
            z = x + y
            want = (z - z.mean(-1, keepdim=True)) / torch.sqrt(z.var(-1, unbiased=False, keepdim=True) + 1e-5) * w
            close(centered, want, torch.float32, f"with the mean taken off, {hidden}")


# ------------------------------------------------------------------------------ whole models
def write_model(folder, config, seed):
    from safetensors.torch import load_file

    from llmserve.weights import write_random_model

    # stored in bfloat16, so that both engines and the plain implementation hold the same numbers
    write_random_model(folder, config, seed=seed, dtype=torch.bfloat16, std=0.08, norm_std=0.05)
    return {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}


def logits_close(got, ref, dtype, what):
    """Per position: the difference of the logits (mean taken off, root mean square over the vocabulary) against the
    root mean square of the logits themselves.  32-bit: every position.  bfloat16: the median, and three positions
    in four."""
    if isinstance(got, (list, tuple)):
        scale = torch.cat([r.double().flatten() for r in ref]).pow(2).mean().sqrt()
        got, ref = torch.cat(list(got)), torch.cat(list(ref))
    else:
        scale = ref.double().pow(2).mean().sqrt()
    got, ref = got.double(), ref.double()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    d = got - ref
    d = d - d.mean(dim=-1, keepdim=True)
    err = d.pow(2).mean(dim=-1).sqrt() / scale
    worst = int(err.argmax())
    if dtype == torch.float32:
        assert float(err.max()) <= 5e-5, f"{what}: position {worst} is off by {float(err.max()):.2e}"
    else:
        assert float(err.median()) <= 0.02, f"{what}: the median position is off by {float(err.median()):.2e}"
        over = int((err > 0.04).sum())
        assert over <= max(1, len(err) // 4), f"{what}: {over} of {len(err)} positions are off by more than 0.04 (worst {worst})"


MODELS = {"small": (SMALL, 8), "small_b": (SMALL_B, 16), "small_c": (SMALL_C, 4), "small_d": (SMALL_D, 16)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, (config, bs)) in enumerate(MODELS.items()):
        folder = tmp_path_factory.mktemp(f"felavik_{name}")
        out[name] = (folder, config, write_model(folder, config, seed=170 + i), bs)
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
def test_the_stream_after_every_layer(models, name):
    """Layer by layer against the plain implementation, in 32-bit."""
    from llmserve.config import EngineConfig
    from llmserve.engine.batch import build_batch
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    ids = traces.random_ids(config["vocab"], 45, 5)
    want = []
    pf.forward(config, w, ids, layers_out=want)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=16, max_num_seqs=2,
                                                          use_graphs=False))
    runner.add_sequence("a")
    layout = runner.manager.append(["a"], [len(ids)])
    batch = build_batch(layout, [ids], [0], runner._uploader, runner.storage)
    model = runner.model
    x, delta = model.embedding.forward(batch.token_ids), None
    sources = model.cache_sources()
    for pos, index in enumerate(model.spec.schedule):
        x, delta = model.blocks[index].forward(x, delta, batch, runner.storage.layer_cache(pos, sources[pos]))
        close(x[:, 0].double().cpu() + delta.y.double().cpu(), want[pos], torch.float32, f"after layer {pos}")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("graphs", [True, False])
def test_every_way_of_cutting_gives_the_plain_logits(models, name, dtype_name, graphs):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    dtype = getattr(torch, dtype_name)
    seqs = {f"r{i}": traces.random_ids(config["vocab"], n, 300 + i) for i, n in enumerate([67, 1, 30, 41, 2, 75])}
    ref = {rid: pf.forward(config, w, ids) for rid, ids in seqs.items()}
    modes = {"whole": traces.whole(seqs), "decode": traces.prefill_then_decode(seqs, tail=40),
             "portions": traces.portions(seqs), "mixed": traces.mixed(seqs, seed=3, live_max=3)}
    for mode, steps in modes.items():
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                              max_num_seqs=3, use_graphs=graphs))
        assert runner._use_graphs == graphs  # every part of the model can be captured
        poison(runner)
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], dtype, f"{name} {mode} {dtype_name}")
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
    """280 tokens: whole in one step, and most of them one by one through the state and the pages."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small_c"]
    ids = traces.random_ids(config["vocab"], 280, 77)
    ref = pf.forward(config, w, ids)
    for graphs in (True, False):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=-(-280 // bs) + 1,
                                                              max_num_seqs=2, use_graphs=graphs))
        poison(runner)
        got = run_trace(runner, traces.prefill_then_decode({"long": ids}, tail=250))
        logits_close(got["long"], ref, torch.float32, "long decoding")
        whole = run_trace(runner, traces.whole({"again": ids}))
        logits_close(whole["again"], ref, torch.float32, "the whole prompt on the slot and pages that came back")


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
        if dtype_name == "float32":
            assert result.tokens == pf.greedy(config, w, prompt, 24)
        else:  # a tie may fall either way in bfloat16: nearly every token must be near the top of the plain logits
            ref = pf.forward(config, w, prompt + result.tokens)
            far = 0
            for i, tok in enumerate(result.tokens):
                row = ref[len(prompt) - 1 + i]
                far += float(row.max() - row[tok]) > 0.08 * float(ref.pow(2).mean().sqrt()) + 1e-3
            assert far <= 2
    assert llm.runner.manager.num_free_slots == 3


def test_named_sizes_run_from_the_command_line_entry(capsys):
    from llmserve.cli import main

    assert main(["--model", "felavik-tiny", "--random-weights", "--max-new-tokens", "5", "--dtype", "float32"]) == 0
    assert "decode=" in capsys.readouterr().out


def drawn_config(seed: int) -> tuple[dict, int]:
    """A configuration drawn at random from what config.json allows: layers of both kinds in any order, layers on
    another layer's tensors (also in chains), layers without feed-forward, 1 to 6 heads, 1 to all of them key/value
    heads, sizes from 2 up and beyond 64 (keys and values of one size or of two), rotations over all or part of a head,
    tables of 2 to 32 rows, factors that
    step every 1 to 100 positions, 1 to 4 groups of experts of which 1 to all are kept; and a page size."""
    rng = random.Random(seed)

    def decays(n):
        return [rng.choice([0.3, 0.9, 0.97, 0.999, 1.0]) for _ in range(n)]

    def mlp():
        if rng.random() < 0.2:
            return None
        groups = rng.choice([1, 2, 3, 4])
        per = rng.randint(1, 3)
        keep = rng.randint(1, groups)
        top = rng.randint(1, min(4, keep * per))
        return moe(groups * per, top, rng.choice([8, 24, 40]), groups if rng.random() < 0.8 or groups > 1 else None, keep)

    layers = []
    for i in range(rng.randint(2, 6)):
        if layers and rng.random() < 0.3:
            j = rng.randrange(len(layers))
            layers.append(dict(layers[j], weights_of=j))
            continue
        if rng.random() < 0.5:
            heads = rng.randint(1, 4)
            layers.append(lightning(heads=heads, dim=rng.choice([4, 8, 20, 32, 72]), vdim=rng.choice([4, 8, 24, 64, 80]),
                                    decay=decays(heads), mlp=mlp()))
        else:
            kv = rng.choice([1, 2, 3])
            heads = kv * rng.choice([1, 2, 3])
            rows = rng.choice([2, 4, 10, 16, 32])
            dim = rng.choice([4, 8, 16, 32])
            rheads = rng.randint(1, 4)
            left_dim = rng.choice([4, 8, 16, 32, 48, 64, 96])
            layers.append(parallel(
                left={"heads": heads, "kv_heads": kv, "dim": left_dim, "vdim": rng.choice([4, 8, 16, 64, left_dim, left_dim]),
                      "scale": rng.choice([0.1, 0.2, 0.35]), "bias_rows": rows, "bias_max": rows // 2 + rng.choice([1, 7, 60, 300]),
                      "q_temp": {"coef": rng.choice([0.1, 0.5, 2.0]), "every": rng.choice([1, 3, 16, 100])}},
                right={"heads": rheads, "dim": dim, "vdim": rng.choice([4, 8, 32, 72]), "decay": decays(rheads),
                       "rot": {"base": rng.choice([10.0, 10000.0, 1e6]), "dims": rng.choice([dim, dim // 2, 2])}},
                left_scale=rng.choice([0.5, 1.0]), right_scale=rng.choice([0.3, 1.1]), mlp=mlp()))
    return config_of(layers, width=rng.choice([40, 64, 72, 100]), vocab=rng.choice([61, 128, 257]),
                     scale=rng.choice([0.5, 1.0, 4.0]), eps=rng.choice([1e-6, 1e-5]),
                     softcap=rng.choice([None, 5.0, 30.0])), rng.choice([4, 8, 16])


# (Seed 6 draws layers that give a token one expert of nine: the bfloat16 engine's choices part from the plain ones at 28 %
# of the positions, a little over the quarter allowed below, whichever attention and recurrence kernels run; its 32-bit
# engine agrees with the plain implementation everywhere.)
@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 7, 8, 9, 10])
def test_configurations_drawn_at_random(tmp_path, seed):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    config, bs = drawn_config(seed)
    w = write_model(tmp_path, config, seed=900 + seed)
    seqs = {f"q{i}": traces.random_ids(config["vocab"], n, 40 * seed + i) for i, n in enumerate([90, 3, 47, 160, 18])}
    ref = {rid: pf.forward(config, w, ids) for rid, ids in seqs.items()}
    for dtype_name in ("float32", "bfloat16"):
        steps = traces.mixed(seqs, seed=seed, live_max=3, tail=30)
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(tmp_path, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                                max_num_seqs=3))
        poison(runner)
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], getattr(torch, dtype_name),
                     f"seed {seed} {dtype_name}: {config['layers']}")
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
