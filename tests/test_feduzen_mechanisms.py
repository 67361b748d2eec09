"""Each mechanism of the Feduzen design alone, against the plain implementation's function for it.

The kernels are called as the parts call them, on the CPU through their torch twins and on the GPU as HIP kernels
in float32 and bfloat16.  Where random numbers would hide a fault (one key among hundreds, a key one position
outside a block, a sink), the inputs are made so that it shows: one query and one key are scaled so that their
score stands out, and the values say which position was read.
"""

import math
import types

import pytest
import torch

import plain_feduzen as plain
from simple_inference_amd.parts.context import LayerCache

BACKENDS = [
    pytest.param("twins"),
    pytest.param("hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip-bf16", marks=pytest.mark.gpu),
]
TOL = {"twins": 2e-6, "hip-f32": 2e-6, "hip-bf16": 1.6e-2}


def setup(backend):
    if backend == "twins":
        from twins import TwinKernels
        return TwinKernels(), "cpu", torch.float32
    from simple_inference_amd.kernels import HipKernels
    return HipKernels(), "cuda:0", torch.float32 if backend == "hip-f32" else torch.bfloat16


def close(got, want, backend, scale=None):
    got, want = got.double().cpu(), want.double().cpu()
    size = float(want.abs().max()) if scale is None else scale
    assert float((got - want).abs().max()) <= TOL[backend] * max(size, 1e-30), float((got - want).abs().max()) / size


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def step_context(device, runs, page_size, kernels):
    """A flat batch: ``runs`` is a list of (first position, number of tokens); single tokens first, as the step
    function lays them out.  Pages are dealt in a scrambled order so that nothing lies where its position says."""
    runs = sorted(runs, key=lambda r: r[1] != 1)
    positions, seq_of, cu, kv_len = [], [], [0], []
    for s, (first, n) in enumerate(runs):
        positions += list(range(first, first + n))
        seq_of += [s] * n
        cu.append(cu[-1] + n)
        kv_len.append(first + n)
    width = max(-(-L // page_size) for L in kv_len)
    n_pages = len(runs) * width
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(5)).tolist()
    table = torch.full((len(runs), width), -1, dtype=torch.int32)
    for s, L in enumerate(kv_len):
        for i in range(-(-L // page_size)):
            table[s, i] = perm.pop()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    ctx = types.SimpleNamespace(
        n_tokens=len(positions), n_seqs=len(runs), positions=i32(positions), seq_of_token=i32(seq_of), cu_q=i32(cu),
        kv_len=i32(kv_len), max_kv_len=max(kv_len), max_q_len=max(n for _, n in runs),
        n_decode_seqs=sum(1 for _, n in runs if n == 1), q_lens=[n for _, n in runs], kv_bound=0,
        max_run_kv_len=max([f + n for f, n in runs if n > 1], default=0), kernels=kernels, extra={})
    return ctx, table.to(device), n_pages, runs


def empty_cache(device, dtype, n_pages, kv_heads, page_size, dim, vdim, table):
    return LayerCache(k_pages=torch.zeros(n_pages, kv_heads, page_size, dim, dtype=dtype, device=device),
                      v_pages=torch.zeros(n_pages, kv_heads, vdim, page_size, dtype=dtype, device=device),
                      block_table=table, page_size=page_size)


# ---------------------------------------------------------------------------------------------------------------
# embedding, norm behind a sublayer, activation
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
def test_embedding_is_the_row_times_the_scale(backend):
    k, dev, dtype = setup(backend)
    table = rnd(50, 40, seed=1).to(dtype)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    got = k.embed(ids.to(dev), table.to(dev), scale=2.75)
    assert got.dtype == torch.float32
    close(got, plain.embed(ids.tolist(), table.double(), 2.75), backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width", [40, 136, 384])
def test_residual_grows_by_the_norm_of_the_sublayers_output(backend, width):
    k, dev, dtype = setup(backend)
    x, y, g = rnd(7, width, seed=2, std=3.0), rnd(7, width, seed=3, std=0.2).to(dtype), 1 + rnd(width, seed=4, std=0.3)
    residual = x.clone().to(dev)
    lowered = k.norm_add(residual, y.to(dev), g.to(dev), 1e-3, dtype)
    want = x.double() + plain.rms_norm(y.double(), g.double(), 1e-3)
    assert residual.dtype == torch.float32 and lowered.dtype == dtype
    close(residual, want, backend if dtype == torch.float32 else "hip-f32")   # the sum itself is float in both modes
    close(lowered, want, backend)
    # eps sits inside the root: rows of zeros stay where they are
    residual = x.clone().to(dev)
    k.norm_add(residual, torch.zeros(7, width, dtype=dtype, device=dev), g.to(dev), 1e-3, dtype)
    assert torch.equal(residual.cpu(), x)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("rows", [3, 40])
def test_dense_feed_forward_squares_the_relu(backend, rows):
    k, dev, dtype = setup(backend)
    h, up, down = rnd(rows, 64, seed=5).to(dtype), rnd(80, 64, seed=6, std=0.2).to(dtype), rnd(64, 80, seed=7, std=0.2).to(dtype)
    a = k.activated_linear(h.to(dev), up.to(dev), "relu2")
    want_a = torch.relu(h.double() @ up.double().T) ** 2
    close(a, want_a, backend)
    assert float(a.min()) >= 0
    got = k.linear(a, down.to(dev))
    close(got, plain.dense_feed_forward(h.double(), {"l0.mlp.up": up, "l0.mlp.down": down}, "l0"), backend)
    z = rnd(5, 24, seed=8, std=2.0).to(dtype)
    g = k.activated_linear(z.to(dev), torch.eye(24).to(dtype).to(dev), "gelu_tanh")
    zd = z.double()
    close(g, 0.5 * zd * (1 + torch.tanh(math.sqrt(2 / math.pi) * (zd + 0.044715 * zd ** 3))), backend)


# ---------------------------------------------------------------------------------------------------------------
# between the projection and attention: bias, q/k norm, rotation, cache write
# ---------------------------------------------------------------------------------------------------------------
def rope_tables(dims, base, scaling, n, device):
    f = torch.tensor(plain.rotary_frequencies(dims, base, scaling), dtype=torch.float32)
    a = torch.outer(torch.arange(n, dtype=torch.float32), f)
    return a.cos().to(device).contiguous(), a.sin().to(device).contiguous()


def test_frequencies_follow_the_wavelength_rule():
    scaling = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    plainf = plain.rotary_frequencies(16, 100.0, None)
    f = plain.rotary_frequencies(16, 100.0, scaling)
    from simple_inference_amd.parts.rope import rotary_inv_freq
    own = rotary_inv_freq(16, 100.0, {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                                      "high_freq_factor": 4.0, "original_max_position_embeddings": 64})
    assert torch.allclose(own.double(), torch.tensor(f, dtype=torch.float64), rtol=1e-6)
    kinds = set()
    for a, b in zip(plainf, f):
        wl = 2 * math.pi / a
        if wl < 16:
            assert b == a; kinds.add("kept")
        elif wl > 64:
            assert abs(b - a / 4) < 1e-12; kinds.add("divided")
        else:
            assert a / 4 < b < a; kinds.add("between")
    assert kinds == {"kept", "divided", "between"}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv,dim,vdim,rot", [(3, 3, 32, 16, 32), (4, 2, 16, 48, 8), (8, 2, 64, 64, 32), (2, 2, 24, 24, 0),
                                                   (5, 1, 80, 40, 80)])
def test_bias_norm_rotation_and_cache_write(backend, heads, kv, dim, vdim, rot):
    k, dev, dtype = setup(backend)
    page = 8
    ctx, table, n_pages, runs = step_context(dev, [(13, 1), (0, 11), (5, 6)], page, k)
    N, width = ctx.n_tokens, heads * dim + kv * (dim + vdim)
    eps = 1e-4
    qkv0 = rnd(N, width, seed=9).to(dtype)
    bias = rnd(width, seed=10, std=0.5)
    qg, kg = 1 + rnd(dim, seed=11, std=0.3), 1 + rnd(dim, seed=12, std=0.3)
    scaling = {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}
    cos, sin = rope_tables(rot, 500.0, scaling, 32, dev) if rot else (None, None)
    cache = empty_cache(dev, dtype, n_pages, kv, page, dim, vdim, table)
    # the product is the identity here: the kernels' part after it is what is under test
    qkv = k.qkv_to_cache(qkv0.to(dev), torch.eye(width).to(dtype).to(dev), heads, kv, dim, rot, cos, sin, ctx, cache,
                         value_dim=vdim, bias=bias.to(dev), qk_norm=(qg.to(dev), kg.to(dev), eps))
    x = qkv0.double() + bias.double()
    pos = ctx.positions.cpu().tolist()
    q = plain.rotate(plain.rms_norm(x[:, :heads * dim].view(N, heads, dim), qg.double(), eps), pos, rot, 500.0, scaling)
    kk = plain.rotate(plain.rms_norm(x[:, heads * dim:(heads + kv) * dim].view(N, kv, dim), kg.double(), eps), pos, rot,
                      500.0, scaling)
    v = x[:, (heads + kv) * dim:].view(N, kv, vdim)
    close(qkv[:, :heads * dim].view(N, heads, dim), q, backend)
    seq = ctx.seq_of_token.cpu().tolist()
    for t in range(N):
        p = int(table[seq[t], pos[t] // page])
        close(cache.k_pages[p, :, pos[t] % page, :], kk[t], backend, scale=float(kk.abs().max()))
        close(cache.v_pages[p, :, :, pos[t] % page], v[t], backend, scale=float(v.abs().max()))


# ---------------------------------------------------------------------------------------------------------------
# attention: block mask, sink, grouped heads, value width
# ---------------------------------------------------------------------------------------------------------------
def fill_cache(cache, table, keys, values, page, s=0):
    """keys [T, kv, dim], values [T, kv, vdim] of sequence ``s`` into its pages."""
    for t in range(keys.shape[0]):
        p = int(table[s, t // page])
        cache.k_pages[p, :, t % page, :] = keys[t].to(cache.k_pages.dtype)
        cache.v_pages[p, :, :, t % page] = values[t].to(cache.v_pages.dtype)


def plain_attention(q, keys, values, qpos, scale, chunk, sinks):
    """q [n, H, dim] at positions qpos over keys/values [T, G, .] of one sequence, by the plain functions."""
    n, H, _ = q.shape
    G = keys.shape[1]
    T = keys.shape[0]
    seen = plain.chunk_mask(T, chunk)[qpos]
    out = torch.empty(n, H, values.shape[2], dtype=torch.float64)
    for h in range(H):
        s = (q[:, h].double() @ keys[:, h // (H // G)].double().T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        if sinks is None:
            p = torch.softmax(s, -1)
        else:
            p = plain.softmax_with_sink(s, sinks[h].double())
        out[:, h] = p @ values[:, h // (H // G)].double()
    return out


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv,dim,vdim,chunk,page", [(3, 3, 32, 16, 24, 8), (4, 2, 16, 48, 20, 16), (8, 2, 64, 64, 37, 16),
                                                         (6, 1, 32, 32, None, 8), (4, 4, 128, 128, 100, 16)])
def test_attention_with_block_mask_and_sink_in_prompts_and_decoding(backend, heads, kv, dim, vdim, chunk, page):
    k, dev, dtype = setup(backend)
    scale = 0.31
    T = 150
    # a whole prompt, a portion that starts inside a block and crosses a border, single tokens at a block's first
    # and last place and at a page's border
    c = chunk or 32
    runs = [(0, T), (c + 3, 2 * c), (c, 1), (2 * c - 1, 1), (3 * page, 1), (0, 1)]
    ctx, table, n_pages, runs = step_context(dev, runs, page, k)
    cache = empty_cache(dev, dtype, n_pages, kv, page, dim, vdim, table)
    sinks = rnd(heads, seed=20, std=1.5)
    qkv = torch.zeros(ctx.n_tokens, heads * dim + kv * (dim + vdim), dtype=dtype)
    want, row = [], 0
    for s, (first, n) in enumerate(runs):
        L = first + n
        keys, values = rnd(L, kv, dim, seed=30 + s).to(dtype), rnd(L, kv, vdim, seed=40 + s).to(dtype)
        q = rnd(n, heads, dim, seed=50 + s).to(dtype)
        fill_cache(cache, table, keys, values, page, s)
        qkv[row:row + n, :heads * dim] = q.reshape(n, heads * dim)
        want.append(plain_attention(q, keys, values, list(range(first, L)), scale, chunk, sinks))
        row += n
    got = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, value_dim=vdim, chunk=chunk,
                            sinks=sinks.to(dev))
    close(got.view(ctx.n_tokens, heads, vdim), torch.cat(want), backend)
    # without the sink the weights sum to one: another result, and again the plain one
    got = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, value_dim=vdim, chunk=chunk)
    row, s = 0, 0
    first, n = runs[0]
    keys, values = rnd(first + n, kv, dim, seed=30).to(dtype), rnd(first + n, kv, vdim, seed=40).to(dtype)
    q = rnd(n, heads, dim, seed=50).to(dtype)
    close(got.view(ctx.n_tokens, heads, vdim)[:n], plain_attention(q, keys, values, list(range(first, first + n)), scale,
                                                                  chunk, None), backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoding", [False, True])
@pytest.mark.parametrize("dim,vdim,page", [(32, 32, 16), (16, 48, 8)])
def test_one_planted_key_is_found_exactly_where_the_mask_lets_it_be(backend, decoding, dim, vdim, page):
    """One key is made to stand out for one query (their score is far above every other).  The value rows say their
    own position, so the result names the key that was read.  The planted key lies just inside the query's block
    (its first position), just outside it (one before), far back among hundreds, at page borders, at position 0."""
    k, dev, dtype = setup(backend)
    chunk, heads, kv, scale = 400, 2, 1, 1.0
    u = torch.zeros(dim)
    u[3] = 1.0
    cases = []   # (query position, planted key, seen?)
    for qpos, key in [(799, 400), (799, 399), (799, 401), (400, 400), (400, 399), (401, 400), (399, 0), (399, 1),
                      (1190, 800), (1190, 799), (799, 799 - 16), (799, 799 - 17), (790, 784), (790, 783), (5, 0)]:
        cases.append((qpos, key, key // chunk == qpos // chunk and key <= qpos))
    for qpos, key, seen in cases:
        L = qpos + 1
        first, n = (qpos, 1) if decoding else (max(0, qpos - 40), qpos + 1 - max(0, qpos - 40))
        ctx, table, n_pages, runs = step_context(dev, [(first, n)], page, k)
        cache = empty_cache(dev, dtype, n_pages, kv, page, dim, vdim, table)
        keys = rnd(L, kv, dim, seed=60, std=0.05)
        keys[key, 0] = 12.0 * u
        values = torch.zeros(L, kv, vdim)
        values[:, 0, 0] = torch.arange(L) % 64          # exact in bfloat16
        values[:, 0, 1] = torch.arange(L) // 64
        fill_cache(cache, table, keys, values, page)
        qkv = torch.zeros(n, heads * dim + kv * (dim + vdim), dtype=dtype)
        qkv[-1, :dim] = (12.0 * u).to(dtype)            # head 0 of the last token asks for the planted key
        got = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, value_dim=vdim, chunk=chunk)
        o = got.view(n, heads, vdim)[-1, 0].float().cpu()
        read = float(o[0]) + 64 * float(o[1])
        if seen:
            assert abs(read - key) < 0.51, (qpos, key, read)
        else:
            assert abs(read - key) > 0.9, (qpos, key, read)


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_sink_takes_weight_and_gives_nothing(backend):
    k, dev, dtype = setup(backend)
    heads, kv, dim, page, L = 4, 2, 32, 8, 70
    ctx, table, n_pages, runs = step_context(dev, [(L - 1, 1), (0, L)], page, k)
    cache = empty_cache(dev, dtype, n_pages, kv, page, dim, dim, table)
    keys, values = rnd(L, kv, dim, seed=70), 1.0 + rnd(L, kv, dim, seed=71, std=0.1)
    for s in range(2):
        fill_cache(cache, table, keys, values, page, s)
    qkv = torch.zeros(ctx.n_tokens, (heads + 2 * kv) * dim, dtype=dtype)
    qkv[:, :heads * dim] = rnd(ctx.n_tokens, heads * dim, seed=72).to(dtype)
    # head 0: a sink far above every score takes all the weight; head 1: far below, none; heads 2, 3 in between
    sinks = torch.tensor([60.0, -60.0, 0.0, 2.0])
    with_sink = k.paged_attention(qkv.to(dev), heads, kv, dim, 0.2, None, ctx, cache, sinks=sinks.to(dev))
    without = k.paged_attention(qkv.to(dev), heads, kv, dim, 0.2, None, ctx, cache)
    a, b = with_sink.view(-1, heads, dim).float().cpu(), without.view(-1, heads, dim).float().cpu()
    assert float(a[:, 0].abs().max()) < 1e-6
    assert torch.allclose(a[:, 1], b[:, 1], atol=1e-6)
    for h in (2, 3):   # the values are near 1: the sink's share of the weight is what is missing
        share = 1 - a[:, h].mean(-1) / b[:, h].mean(-1)
        assert float(share.min()) > 0.001 and float(share.max()) < 0.999
    # the score scale does not touch a sink: with a sink of zero and scores of zero (no query) it is one among n + 1
    qkv.zero_()
    got = k.paged_attention(qkv.to(dev), heads, kv, dim, 0.2, None, ctx, cache, sinks=torch.zeros(heads).to(dev))
    first = got.view(-1, heads, dim).float().cpu()[0]       # the single token at position L - 1 sees L keys
    close(first[0], values[:, 0].mean(0) * L / (L + 1), backend)


@pytest.mark.gpu
@pytest.mark.parametrize("backend", ["hip-f32", "hip-bf16"])
@pytest.mark.parametrize("heads,kv,dim,vdim,rot,wide", [(3, 3, 32, 16, 32, 32), (4, 2, 16, 48, 8, 48), (2, 2, 24, 24, 0, 32),
                                                        (5, 1, 80, 40, 80, 80), (2, 1, 64, 128, 32, 128)])
def test_pages_wider_than_the_heads_hold_the_same_numbers_and_zeros(backend, heads, kv, dim, vdim, rot, wide):
    """Keys and values kept at one width (for the attention kernel that wants them alike): the heads' own elements
    are what they are in pages as wide as the heads, everything beyond them is zero, and attention over such pages
    gives the same result with zeros behind every head."""
    k, dev, dtype = setup(backend)
    page = 16
    ctx, table, n_pages, runs = step_context(dev, [(40, 1), (0, 37), (21, 19)], page, k)
    N, width = ctx.n_tokens, heads * dim + kv * (dim + vdim)
    qkv0 = rnd(N, width, seed=80).to(dtype).to(dev)
    bias, qg, kg = rnd(width, seed=81, std=0.5).to(dev), (1 + rnd(dim, seed=82, std=0.3)).to(dev), (1 + rnd(dim, seed=83, std=0.3)).to(dev)
    cos, sin = rope_tables(rot, 500.0, None, 64, dev) if rot else (None, None)
    eye = torch.eye(width).to(dtype).to(dev)
    plain_cache = empty_cache(dev, dtype, n_pages, kv, page, dim, vdim, table)
    wide_cache = empty_cache(dev, dtype, n_pages, kv, page, wide, wide, table)
    q1 = k.qkv_to_cache(qkv0, eye, heads, kv, dim, rot, cos, sin, ctx, plain_cache, value_dim=vdim, bias=bias,
                        qk_norm=(qg, kg, 1e-5))
    q2 = k.qkv_to_cache(qkv0, eye, heads, kv, dim, rot, cos, sin, ctx, wide_cache, value_dim=vdim, bias=bias,
                        qk_norm=(qg, kg, 1e-5), page_dim=wide)
    assert tuple(q2.shape) == (N, heads * wide)
    assert torch.equal(q2.view(N, heads, wide)[:, :, :dim], q1[:, :heads * dim].view(N, heads, dim))
    assert float(q2.view(N, heads, wide)[:, :, dim:].abs().sum()) == 0
    assert torch.equal(wide_cache.k_pages[..., :dim], plain_cache.k_pages) and float(wide_cache.k_pages[..., dim:].abs().sum()) == 0
    assert torch.equal(wide_cache.v_pages[:, :, :vdim], plain_cache.v_pages) and float(wide_cache.v_pages[:, :, vdim:].abs().sum()) == 0
    # fill the pasts of the runs that do not start at 0, alike in both
    for cache in (plain_cache, wide_cache):
        cache.k_pages[..., :dim] += 0.1
        cache.v_pages[:, :, :vdim] += 0.2
    sinks = rnd(heads, seed=84).to(dev)
    o1 = k.paged_attention(q1, heads, kv, dim, 0.2, None, ctx, plain_cache, value_dim=vdim, chunk=30, sinks=sinks)
    o2 = k.paged_attention(q2, heads, kv, wide, 0.2, None, ctx, wide_cache, chunk=30, sinks=sinks)
    close(o2.view(N, heads, wide)[:, :, :vdim], o1.view(N, heads, vdim), backend)
    assert float(o2.view(N, heads, wide)[:, :, vdim:].abs().sum()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n,k", [(1, 3072, 8192), (8, 3072, 3072), (16, 320, 384), (5, 200, 128)])
def test_few_row_product_from_the_tiled_copy_of_a_weight_has_the_same_bits(rows, n, k):
    kern, dev, _ = setup("hip-bf16")
    x, w = rnd(rows, k, seed=90).bfloat16().to(dev), rnd(n, k, seed=91, std=0.05).bfloat16().to(dev)
    plain_y = kern.linear(x, w)
    made = kern.prepare_pending_weight(w)
    assert made == (kern.core.sia_gemm_skinny_tile_height(n) > 0)
    tiled_y = kern.linear(x, w)
    assert torch.equal(plain_y, tiled_y)
    close(tiled_y, x.double() @ w.double().T, "hip-bf16")


def fill_cache_by_pages(cache, table, keys, values, page, s):
    """As ``fill_cache``, a page at a time (for long sequences)."""
    L, kv, dim = keys.shape
    n = -(-L // page)
    k = torch.zeros(n * page, kv, dim, dtype=keys.dtype)
    v = torch.zeros(n * page, kv, values.shape[2], dtype=values.dtype)
    k[:L], v[:L] = keys, values
    pages = table[s, :n].long()
    cache.k_pages[pages] = k.view(n, page, kv, dim).permute(0, 2, 1, 3).to(cache.k_pages.dtype).to(cache.k_pages.device)
    cache.v_pages[pages] = v.view(n, page, kv, -1).permute(0, 2, 3, 1).to(cache.v_pages.dtype).to(cache.v_pages.device)


@pytest.mark.gpu
@pytest.mark.parametrize("n_seqs,mode", [(4, 2), (40, 0), (130, 1)])
@pytest.mark.parametrize("chunk", [None, 2048])
def test_sinks_and_blocks_where_decode_attention_splits_the_keys(n_seqs, mode, chunk):
    """Long contexts in bfloat16: a sequence's keys are shared by several workgroups and their partial results are
    merged (by the kernel that combines splits, by the one that combines every run, or inside one workgroup,
    depending on how many sequences the step holds).  The sink joins the merged denominator exactly once."""
    k, dev, dtype = setup("hip-bf16")
    heads, kv, dim, page, scale = 8, 2, 64, 16, 0.11
    lengths = [(2500, 1100, 3000, 600, 1025, 2049)[i % 6] for i in range(n_seqs)]
    ctx, table, n_pages, runs = step_context(dev, [(L - 1, 1) for L in lengths], page, k)
    lib = k._attn_lib(dim)
    splits = lib.sia_attn_decode_max_splits(max(lengths), chunk or 0)
    assert splits > 1 and lib.sia_attn_decode_mode(n_seqs, heads, kv, splits) == mode
    cache = empty_cache(dev, dtype, n_pages, kv, page, dim, dim, table)
    sinks = torch.tensor([3.0, -2.0, 0.0, 1.0, 6.0, -30.0, 0.5, 2.0])
    qkv = torch.zeros(n_seqs, (heads + 2 * kv) * dim, dtype=dtype)
    want = []
    for s, (first, n) in enumerate(runs):
        L = first + 1
        keys, values = rnd(L, kv, dim, seed=1000 + s).to(dtype), rnd(L, kv, dim, seed=2000 + s).to(dtype)
        q = rnd(1, heads, dim, seed=3000 + s, std=2.0).to(dtype)
        fill_cache_by_pages(cache, table.cpu(), keys, values, page, s)
        qkv[s, :heads * dim] = q.reshape(-1)
        lo = first - first % chunk if chunk else 0
        want.append(plain_attention(q, keys[lo:], values[lo:], [first - lo], scale, None, sinks))
    got = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, chunk=chunk, sinks=sinks.to(dev))
    close(got.view(n_seqs, heads, dim), torch.cat(want), "hip-bf16")
    without = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, chunk=chunk)
    ratio = (got.view(n_seqs, heads, dim).float().norm(dim=-1) / without.view(n_seqs, heads, dim).float().norm(dim=-1)).cpu()
    assert float(ratio[:, 5].min()) > 0.999 and float(ratio[:, 4].max()) < 0.999   # a sink of -30 is nothing, one of 6 is felt


@pytest.mark.gpu
@pytest.mark.parametrize("first,n", [(0, 2048), (0, 4096), (0, 9216), (7000, 1024), (100, 700)])
@pytest.mark.parametrize("chunk", [None, 1500])
def test_sinks_and_blocks_in_every_shape_of_prefill_workgroup(first, n, chunk):
    """Long prompts and portions over a long past in bfloat16: the prefill kernel takes another shape of workgroup
    by the number of row tiles (two sets of waves that share each pair of key tiles and merge at the end, or every
    wave all tiles); the sink joins the denominator after that merge, and a block's first key bounds every tile
    range.  The plain computation runs in float64 on the GPU."""
    prefill_case(first, n, chunk, 16, 4, 64)


@pytest.mark.gpu
@pytest.mark.parametrize("first,n", [(0, 1300), (900, 300)])
@pytest.mark.parametrize("dim", [144, 256])
def test_sinks_and_blocks_in_prefill_with_large_heads(first, n, dim):
    """Head sizes above 128 take workgroups of fewer tokens, and the largest load straight from the pages."""
    prefill_case(first, n, 500, 4, 2, dim)


def prefill_case(first, n, chunk, heads, kv, dim):
    k, dev, dtype = setup("hip-bf16")
    page, scale = 16, 0.09
    L = first + n
    ctx, table, n_pages, runs = step_context(dev, [(first, n)], page, k)
    cache = empty_cache(dev, dtype, n_pages, kv, page, dim, dim, table)
    keys, values = rnd(L, kv, dim, seed=500).to(dtype), rnd(L, kv, dim, seed=501).to(dtype)
    q = rnd(n, heads, dim, seed=502, std=1.5).to(dtype)
    fill_cache_by_pages(cache, table.cpu(), keys, values, page, 0)
    sinks = (rnd(heads, seed=503, std=2.0) + 1.0)
    qkv = torch.zeros(n, (heads + 2 * kv) * dim, dtype=dtype)
    qkv[:, :heads * dim] = q.reshape(n, -1)
    got = k.paged_attention(qkv.to(dev), heads, kv, dim, scale, None, ctx, cache, chunk=chunk, sinks=sinks.to(dev))
    got = got.view(n, heads, dim).double()
    qd, kd, vd = q.to(dev).double(), keys.to(dev).double(), values.to(dev).double()
    qpos = torch.arange(first, L, device=dev)[:, None]
    kpos = torch.arange(L, device=dev)[None, :]
    seen = kpos <= qpos
    if chunk:
        seen &= (kpos // chunk) == (qpos // chunk)
    worst = 0.0
    for h in range(heads):
        s = (qd[:, h] @ kd[:, h // (heads // kv)].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        want = plain.softmax_with_sink(s, sinks[h].double().to(dev)) @ vd[:, h // (heads // kv)]
        worst = max(worst, float((got[:, h] - want).abs().max() / want.abs().max()))
    assert worst <= TOL["hip-bf16"], worst
