"""Every mechanism of the Mogisun design alone: the kernel (its torch twin on the CPU, the HIP kernel on the GPU in
float32 and bfloat16) against the plain implementation's function for it, at sizes of all kinds."""

import math

import pytest
import torch

import plain_mogisun as plain
from simple_inference_amd.parts.context import LayerCache, StepContext

BACKENDS = [
    pytest.param("twins"),
    pytest.param("hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip-bf16", marks=pytest.mark.gpu),
]


def setup(backend):
    """(kernels, device, compute dtype, tolerance)."""
    if backend == "twins":
        from twins import TwinKernels
        return TwinKernels(), "cpu", torch.float32, 2e-5
    from simple_inference_amd.kernels import HipKernels
    return (HipKernels(), "cuda:0") + ((torch.float32, 2e-5) if backend == "hip-f32" else (torch.bfloat16, 2e-2))


def rnd(gen, *shape, std=1.0):
    return torch.randn(*shape, generator=gen, dtype=torch.float64) * std


def lowered(x, dtype, device):
    """The tensor as the engine would hold it, and the float64 values it then holds."""
    t = x.to(dtype).to(device)
    return t, t.double().cpu()


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    assert float((got - want).abs().max()) <= tol * max(1.0, float(want.abs().max())), float((got - want).abs().max())


def context(device, q_lens, slots):
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return StepContext(
        n_tokens=cu[-1], n_seqs=len(q_lens), token_ids=i32([0] * cu[-1]), positions=i32([0] * cu[-1]),
        seq_of_token=i32([s for s, n in enumerate(q_lens) for _ in range(n)]), cu_q=i32(cu), kv_len=i32(q_lens),
        state_slots=i32(slots), logit_rows=None, n_logit_rows=0, max_q_len=max(q_lens), max_kv_len=max(q_lens),
        q_lens=list(q_lens))


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("hidden,extra", [(96, 0), (176, 24), (50, 3), (1024, 8)])
def test_gated_sum_into_the_residual_and_the_norm_after_it(backend, hidden, extra):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(hidden)
    n = 7
    res = rnd(g, n, hidden)
    delta, delta64 = lowered(rnd(g, n, hidden), dtype, dev)
    wide, wide64 = lowered(rnd(g, n, hidden + extra, std=2.0), dtype, dev)    # the gate's logits: columns of a wider matrix
    gate, gate64 = wide[:, extra:], wide64[:, extra:]
    gb, db, w = rnd(g, hidden), rnd(g, hidden), 1 + rnd(g, hidden, std=0.2)
    f32 = lambda t: t.float().to(dev)
    want_res = res.float().double() + (delta64 + db.float().double()) * torch.sigmoid(gate64 + gb.float().double())
    want = plain.unit_rms(want_res, 1e-5) * w.float().double()
    # all rows: the residual is updated
    r = f32(res)
    out = k.add_rmsnorm(r, delta, f32(w), 1e-5, dtype, gate=gate, gate_bias=f32(gb), delta_bias=f32(db))
    close(r, want_res, 2e-6)
    close(out, want, tol)
    # selected rows: the residual stays
    r = f32(res)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=dev)
    out = k.add_rmsnorm(r, delta, f32(w), 1e-5, dtype, rows, gate=gate, gate_bias=f32(gb), delta_bias=f32(db))
    close(r, res.float(), 0)
    close(out, want[[5, 0, 5]], tol)
    # the sum alone, without biases, and without a gate
    r = f32(res)
    k.gated_add(r, delta, gate)
    close(r, res.float().double() + delta64 * torch.sigmoid(gate64), 2e-6)
    r = f32(res)
    k.gated_add(r, delta, None, None, f32(db))
    close(r, res.float().double() + delta64 + db.float().double(), 2e-6)


@pytest.mark.parametrize("backend", BACKENDS)
def test_small_steps_around_the_gates(backend):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(3)
    # one sigmoid per token and head on the attention's output
    out, out64 = lowered(rnd(g, 5, 6 * 20), dtype, dev)
    wide, wide64 = lowered(rnd(g, 5, 11, std=2.0), dtype, dev)
    got = k.head_gate(out, wide[:, 3:9], 6)
    close(got, (out64.view(5, 6, 20) * torch.sigmoid(wide64[:, 3:9])[:, :, None]).reshape(5, 120), tol)
    # a bias on rows
    y, y64 = lowered(rnd(g, 4, 33), dtype, dev)
    b = rnd(g, 33).float()
    close(k.add_bias(y, b.to(dev)), y64 + b.double(), tol)
    # two float streams side by side, lowered
    a, b2 = rnd(g, 3, 40).float(), rnd(g, 3, 40).float()
    both = k.side_by_side(a.to(dev), b2.to(dev), dtype)
    assert both.dtype == dtype and torch.equal(both.cpu(), torch.cat([a, b2], -1).to(dtype))
    # scale and soft cap of logits
    z = rnd(g, 4, 77, std=8.0).float()
    close(k.scale_softcap(z.clone().to(dev), 2.0, 15.0), 15.0 * torch.tanh(z.double() * 2.0 / 15.0), 2e-6)
    close(k.scale_softcap(z.clone().to(dev), 0.5, None), z.double() * 0.5, 2e-6)


def test_the_query_temperature_steps_where_the_formula_says():
    t = plain.query_temperature(range(40), 0.3, 8)
    assert float(t[0]) == 1.0 and float(t[6]) == 1.0                       # (p + 1) // 8 == 0 up to p = 6
    assert abs(float(t[7]) - (1 + 0.3 * math.log(2))) < 1e-12 and float(t[14]) == float(t[7])
    assert abs(float(t[15]) - (1 + 0.3 * math.log(3))) < 1e-12 and abs(float(t[39]) - (1 + 0.3 * math.log(6))) < 1e-12


# ---------------------------------------------------------------------------------------------------------------
GLA_SHAPES = [(3, 24, 40, 5, 4.0), (1, 8, 8, 3, 1.0), (2, 64, 64, 8, 16.0), (2, 128, 128, 16, 8.0), (2, 256, 48, 33, 2.0),
              (5, 56, 24, 12, 6.0), (1, 40, 200, 2, 0.5), (1, 264, 512, 4, 2.0)]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,Dv,rank,tau", GLA_SHAPES)
def test_linear_attention_carries_its_state_through_any_cut(backend, H, D, Dv, rank, tau):
    """Three sequences of unequal length in scattered slots, fed in three steps of unequal portions (one of a single
    token, one of two) and a last step in which each brings one token (a decode step): every output is the plain
    recurrence's over the whole sequence, and the states left in the slots are its last states."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * 1000 + D)
    lengths, slots = [38, 6, 22], [4, 0, 2]
    pad = 8                          # columns in front of q that belong to somebody else
    width = pad + 2 * H * D + 2 * H * Dv + rank
    cols = (pad, pad + H * D, pad + 2 * H * D, pad + 2 * H * D + H * Dv, pad + 2 * H * D + 2 * H * Dv)
    a2, a2_64 = lowered(rnd(g, H * D, rank, std=0.5), dtype, dev)
    bias, w = (1.0 + rnd(g, H * D)).float(), (1 + rnd(g, Dv, std=0.3)).float()
    projs = [lowered(rnd(g, n, width), dtype, dev) for n in lengths]
    state = torch.zeros(6, H, D, Dv, dtype=torch.float32, device=dev)
    state[4].fill_(0.0)
    cache = LayerCache(state=state)
    eps, q_scale = 1e-5, D ** -0.5
    cuts = [[20, 1, 16, 1], [2, 2, 1, 1], [1, 18, 2, 1]]
    got = [[] for _ in lengths]
    at = [0, 0, 0]
    for step in range(4):
        order = [1, 0, 2] if step == 1 else [0, 1, 2]        # the batch's order changes from step to step
        q_lens = [cuts[s][step] for s in order]
        ctx = context(dev, q_lens, [slots[s] for s in order])
        rows = torch.cat([projs[s][0][at[s]:at[s] + cuts[s][step]] for s in order]).contiguous()
        out = k.gla_recurrent(rows, cols, a2, bias.to(dev), w.to(dev), H, D, Dv, tau, q_scale, eps, ctx, cache)
        i = 0
        for s, n in zip(order, q_lens):
            got[s].append(out[i:i + n])
            at[s] += n
            i += n
    for s, n in enumerate(lengths):
        p = projs[s][1]
        q = p[:, cols[0]:cols[1]].view(n, H, D) * q_scale
        kk = p[:, cols[1]:cols[2]].view(n, H, D)
        v = p[:, cols[2]:cols[3]].view(n, H, Dv)
        gate = p[:, cols[3]:cols[4]]
        z = p[:, cols[4]:cols[4] + rank] @ a2_64.T + bias.double()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(n, H, D)
        outs, last = zip(*[plain.linear_recurrence(q[:, h], kk[:, h], v[:, h], alpha[:, h]) for h in range(H)])
        o = plain.unit_rms(torch.stack(outs, dim=1), eps) * w.double()
        want = o.reshape(n, H * Dv) * plain.silu(gate)
        close(torch.cat(got[s]), want, tol * 2)
        close(state[slots[s]], torch.stack(last), 1e-5 if dtype == torch.float32 else 2e-2)
    assert float(state[[1, 3, 5]].abs().max()) == 0.0        # nobody else's slot was touched


@pytest.mark.parametrize("backend", BACKENDS)
def test_linear_attention_remembers_one_token_over_a_long_decode(backend):
    """Decays of almost 1 in one head and of almost 0 in the other: after 300 single-token steps the first head
    still answers with the value planted at the start, the second only with the latest token's."""
    k, dev, dtype, tol = setup(backend)
    H, D, Dv, rank, n = 2, 16, 16, 1, 300
    g = torch.Generator().manual_seed(5)
    cols = (0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv)
    rows64 = rnd(g, n, cols[4] + rank, std=0.05)
    rows64[:, cols[4]:] = 0.0                                            # the decays come from the bias alone
    key = torch.zeros(D, dtype=torch.float64)
    key[3] = 4.0
    for h in range(H):
        rows64[0, cols[1] + h * D:cols[1] + (h + 1) * D] = key           # planted: a key, and a value of its own
        rows64[0, cols[2] + h * Dv:cols[2] + (h + 1) * Dv] = torch.arange(Dv, dtype=torch.float64) - 7.5
        rows64[-1, cols[0] + h * D:cols[0] + (h + 1) * D] = key          # the last query asks for it
    rows, rows64 = lowered(rows64, dtype, dev)
    a2 = torch.zeros(H * D, rank, dtype=dtype, device=dev)
    bias = torch.cat([torch.full((D,), 14.0), torch.full((D,), -14.0)])
    state = torch.zeros(2, H, D, Dv, dtype=torch.float32, device=dev)
    cache = LayerCache(state=state)
    w = torch.ones(Dv)
    for t in range(n):
        ctx = context(dev, [1], [1])
        out = k.gla_recurrent(rows[t:t + 1].contiguous(), cols, a2, bias.to(dev), w.to(dev), H, D, Dv, 1.0, 1.0, 1e-6, ctx, cache)
    q = rows64[:, cols[0]:cols[1]].view(n, H, D)
    kk = rows64[:, cols[1]:cols[2]].view(n, H, D)
    v = rows64[:, cols[2]:cols[3]].view(n, H, Dv)
    alpha = torch.exp(torch.nn.functional.logsigmoid(bias.double())).view(1, H, D).expand(n, H, D)
    o = torch.stack([plain.linear_recurrence(q[:, h], kk[:, h], v[:, h], alpha[:, h])[0][-1] for h in range(H)])
    want = (plain.unit_rms(o, 1e-6).reshape(-1) * plain.silu(rows64[-1, cols[3]:cols[4]]))
    close(out[0], want, tol * 2)
    planted = (torch.arange(Dv, dtype=torch.float64) - 7.5)
    cos = lambda a, b: float((a * b).sum() / a.norm() / b.norm())
    assert cos(o[0], planted) > 0.99 and abs(cos(o[1], planted)) < 0.9


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width", [(5, 1, 96), (8, 3, 128), (11, 2, 50), (7, 7, 64), (70, 6, 128)])
def test_the_router_picks_the_largest_logits_and_weighs_them_among_themselves(backend, experts, top, width):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(experts)
    h, h64 = lowered(rnd(g, 9, width), dtype, dev)
    router = rnd(g, experts, width, std=0.3).float()
    router[min(4, experts - 1)] = router[1]                  # two experts always tie: the lower index is taken first
    ids, weights = k.moe_route(h, router.to(dev), top)
    logits = h64 @ router.double().T
    want_ids, want_w = plain.route(h64, router.double(), top)
    assert ids.dtype == torch.int32 and tuple(ids.shape) == (9, top)
    for t in range(9):
        got = ids[t].tolist()
        assert len(set(got)) == top
        chosen = logits[t][got]
        rest = [logits[t][e] for e in range(experts) if e not in got]
        assert not rest or float(chosen.min()) >= float(max(rest)) - 1e-5 * float(logits[t].abs().max())
        if 4 in got and experts > 4 and top < experts:
            assert 1 in got
        close(weights[t], torch.softmax(chosen, -1), 1e-5)
        close(weights[t].sort().values, want_w[t].sort().values, 1e-4)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width,ff,shared,n", [
    (5, 1, 96, 40, False, 11), (8, 3, 128, 24, True, 11), (4, 2, 50, 17, True, 11), (6, 6, 64, 128, False, 11),
    # steps of many slots, which the GPU sorts by expert and multiplies in tiles: tiles that are not full, experts
    # nobody chose, columns that do not fill a workgroup's share
    (8, 2, 160, 96, True, 203), (16, 1, 64, 32, False, 70), (3, 3, 128, 288, True, 64)])
def test_experts_weighted_and_summed_with_a_shared_one(backend, experts, top, width, ff, shared, n):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(ff)
    h, h64 = lowered(rnd(g, n, width), dtype, dev)
    w1, w1_64 = lowered(rnd(g, experts, 2 * ff, width, std=0.1), dtype, dev)
    w2, w2_64 = lowered(rnd(g, experts, width, ff, std=0.1), dtype, dev)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    if experts == 16:
        ids = ids % 5          # most experts are chosen by nobody
    weights = torch.softmax(rnd(g, n, top), -1).float()
    sh = sg = sh64 = sg64 = None
    if shared:
        sh, sh64 = lowered(rnd(g, n, width), dtype, dev)
        wide, wide64 = lowered(rnd(g, n, 4), dtype, dev)
        sg, sg64 = wide[:, 2:3], wide64[:, 2:3]
    got = k.moe_experts(h, w1, w2, ids.to(dev), weights.to(dev), sh, sg)
    want = torch.zeros(n, width, dtype=torch.float64)
    for t in range(n):
        for e, p in zip(ids[t].tolist(), weights[t].double()):
            want[t] += p * plain.swiglu(h64[t], w1_64[e][:ff], w1_64[e][ff:], w2_64[e])
    if shared:
        want = want + torch.sigmoid(sg64) * sh64
    close(got, want, tol * 2)
