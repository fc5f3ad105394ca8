"""Every mechanism of the Vovalix decoder alone: the kernel against the plain function of
``tests/plain/vovalix.py``, at sizes of the tests' own, whole and in steps, beside other
requests and padding, from slots that hold another request's leftovers, with inputs made so
that a far token, a chunk's edge or a lost state shows."""

from __future__ import annotations

import math

import pytest
import torch

from tests.plain import vovalix as plain
from tests.vovalix_helpers import batch_tensors

pytestmark = pytest.mark.gpu

DEV = "cuda"


def gpu(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def rel(got, want):
    return float((got.double().cpu() - want).pow(2).mean().sqrt() / (want.pow(2).mean().sqrt() + 1e-30))


# ------------------------------------------------------------------ the matrix state
def new_state(slots, heads, dim, vdim, fill=float("nan")):
    """Slots as the engine keeps them (NaN where a request must not read: another's leftovers)."""
    from kvcore_amd.ops import library as ops

    return torch.full((slots, heads, ops.linear_state_rows(dim), vdim), fill, device=DEV)


def run_scan(q, k, v, decay, beta, state, reqs, *, heads, qk_heads, dim, vdim, delta, q_scale=1.0):
    from kvcore_amd.ops import library as ops

    batch, T = batch_tensors(reqs)
    out = torch.full((T, heads * vdim), float("nan"), device=DEV)
    ops.linear_state_scan(out, q, k, v, decay, beta, state, heads=heads, qk_heads=qk_heads, dim=dim, vdim=vdim,
                          delta_rule=delta, q_scale=q_scale, **batch)
    return out


@pytest.mark.parametrize("heads,qk_heads,dim,vdim", [(3, 3, 24, 40), (1, 1, 8, 5), (2, 2, 200, 80), (4, 4, 64, 64),
                                                       (2, 2, 32, 130)])
def test_key_decay_recurrence_whole_in_steps_and_beside_others(heads, qk_heads, dim, vdim):
    gen = torch.Generator().manual_seed(dim + vdim)
    T = 83
    q = torch.randn(T, heads, dim, generator=gen, dtype=torch.float64)
    k = torch.randn(T, heads, dim, generator=gen, dtype=torch.float64) * 0.5
    v = torch.randn(T, heads, vdim, generator=gen, dtype=torch.float64)
    a = torch.rand(T, heads, dim, generator=gen, dtype=torch.float64) * 0.5 + 0.5
    want = torch.stack([plain.gated_linear_recurrence(q[:, h] * 0.3, k[:, h], v[:, h], a[:, h]) for h in range(heads)], 1)
    want = want.reshape(T, -1)
    qg, kg, vg, ag = (gpu(t.reshape(T, -1)) for t in (q, k, v, a))
    kw = dict(heads=heads, qk_heads=qk_heads, dim=dim, vdim=vdim, delta=False, q_scale=0.3)
    # the slots hold another request's leftovers (NaN where nothing may be read)
    state = new_state(3, heads, dim, vdim)
    out = run_scan(qg, kg, vg, ag, None, state, [(1, 0, T)], **kw)
    assert rel(out, want) < 2e-6
    # in steps of every size down to one token, cut inside the stages of 16
    state = new_state(3, heads, dim, vdim)
    at, got = 0, []
    for n in (2, 1, 17, 3, 1, 16, 31, 2, 10):
        got.append(run_scan(qg[at:at + n], kg[at:at + n], vg[at:at + n], ag[at:at + n], None, state, [(2, at, n)], **kw))
        at += n
    assert at == T
    assert rel(torch.cat(got), want) < 2e-6
    # beside a padded row and another request that is further on: rows [other | pad | this]
    other = new_state(3, heads, dim, vdim, 0.0)
    mixed_q = torch.cat([qg[40:41], qg[:1], qg[:20]])
    mixed_k = torch.cat([kg[40:41], kg[:1], kg[:20]])
    mixed_v = torch.cat([vg[40:41], vg[:1], vg[:20]])
    mixed_a = torch.cat([ag[40:41], ag[:1], ag[:20]])
    run_scan(qg[:40], kg[:40], vg[:40], ag[:40], None, other, [(0, 0, 40)], **kw)
    out = run_scan(mixed_q, mixed_k, mixed_v, mixed_a, None, other, [(0, 40, 1), None, (1, 0, 20)], **kw)
    assert rel(out[0:1], want[40:41]) < 2e-6 and rel(out[2:], want[:20]) < 2e-6
    assert float(out[1].abs().max()) == 0.0


@pytest.mark.parametrize("heads,qk_heads,dim,vdim", [(4, 2, 24, 20), (1, 1, 8, 1), (3, 1, 8, 1), (2, 1, 130, 72),
                                                       (2, 2, 64, 64)])
def test_delta_rule_whole_in_steps_and_beside_others(heads, qk_heads, dim, vdim):
    gen = torch.Generator().manual_seed(dim * 3 + vdim)
    T = 70
    q = plain.unit_vector(torch.randn(T, qk_heads, dim, generator=gen, dtype=torch.float64))
    k = plain.unit_vector(torch.randn(T, qk_heads, dim, generator=gen, dtype=torch.float64))
    v = torch.randn(T, heads, vdim, generator=gen, dtype=torch.float64)
    beta = torch.rand(T, heads, generator=gen, dtype=torch.float64)
    g = torch.rand(T, heads, generator=gen, dtype=torch.float64) * 0.3 + 0.7
    rep = heads // qk_heads
    want = torch.stack([plain.delta_recurrence(q[:, h // rep], k[:, h // rep], v[:, h], beta[:, h], g[:, h])
                        for h in range(heads)], 1).reshape(T, -1)
    qg, kg, vg = (gpu(t.reshape(T, -1)) for t in (q, k, v))
    bg, gg = gpu(beta), gpu(g)
    kw = dict(heads=heads, qk_heads=qk_heads, dim=dim, vdim=vdim, delta=True)
    state = new_state(2, heads, dim, vdim)
    out = run_scan(qg, kg, vg, gg, bg, state, [(1, 0, T)], **kw)
    assert rel(out, want) < 5e-6
    state = new_state(2, heads, dim, vdim)
    at, got = 0, []
    for n in (1, 2, 16, 1, 19, 2, 29):
        got.append(run_scan(qg[at:at + n], kg[at:at + n], vg[at:at + n], gg[at:at + n], bg[at:at + n], state,
                            [(0, at, n)], **kw))
        at += n
    assert at == T
    assert rel(torch.cat(got), want) < 5e-6
    # a column view of a wider row, as the mixers hand their projections over
    wide = torch.cat([qg, kg, vg], dim=1).contiguous()
    nq = qk_heads * dim
    state = new_state(2, heads, dim, vdim, 0.0)
    out = run_scan(wide[:, :nq], wide[:, nq:2 * nq], wide[:, 2 * nq:], gg, bg, state, [(0, 0, T)], **kw)
    assert rel(out, want) < 5e-6


def test_a_token_written_six_hundred_tokens_ago_is_still_read():
    """A decay of almost one: the first token's value, written at a key of its own, comes back
    for a query of that key 600 tokens later (in one step, and token by token), scaled by the
    decay's 600th power; with the state lost on the way it would be zero."""
    T, d, dv = 601, 16, 8
    gen = torch.Generator().manual_seed(4)
    k = torch.randn(T, 1, d, generator=gen, dtype=torch.float64) * 0.05
    k[:, 0, 0] = 0.0
    k[0, 0] = 0.0
    k[0, 0, 0] = 1.0  # channel 0 is the first token's alone
    v = torch.randn(T, 1, dv, generator=gen, dtype=torch.float64)
    q = torch.zeros(T, 1, d, dtype=torch.float64)
    q[:, 0, 0] = 1.0
    a = torch.full((T, 1, d), 0.999, dtype=torch.float64)
    want = plain.gated_linear_recurrence(q[:, 0], k[:, 0], v[:, 0], a[:, 0])
    assert torch.allclose(want[600], v[0, 0] * 0.999 ** 600, atol=1e-9)
    qg, kg, vg, ag = (gpu(t.reshape(T, -1)) for t in (q, k, v, a))
    kw = dict(heads=1, qk_heads=1, dim=d, vdim=dv, delta=False)
    state = new_state(1, 1, d, dv)
    out = run_scan(qg, kg, vg, ag, None, state, [(0, 0, T)], **kw)
    assert rel(out[600], want[600]) < 1e-4
    state = new_state(1, 1, d, dv)
    run_scan(qg[:300], kg[:300], vg[:300], ag[:300], None, state, [(0, 0, 300)], **kw)
    for t in range(300, T):
        out = run_scan(qg[t:t + 1], kg[t:t + 1], vg[t:t + 1], ag[t:t + 1], None, state, [(0, t, 1)], **kw)
    assert rel(out[0], want[600]) < 1e-4


def test_small_kernels_around_the_recurrences():
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(8)
    T = 37
    # sigmoid(z + b) ^ (1 / tau), through the logarithm, also far out in the tails
    z = torch.randn(T, 48, generator=gen, dtype=torch.float64) * 6
    b = torch.randn(48, generator=gen, dtype=torch.float64)
    out = torch.empty(T, 48, device=DEV)
    ops.sigmoid_power(out, gpu(z), gpu(b), 1 / 12.0)
    assert rel(out, torch.sigmoid(z + b).pow(1 / 12.0)) < 1e-6
    # decay and write strength of the delta rule
    a_raw, b_raw = (torch.randn(T, 5, generator=gen, dtype=torch.float64) * 3 for _ in range(2))
    a_log, dt_bias = (torch.randn(5, generator=gen, dtype=torch.float64) for _ in range(2))
    g, beta = torch.empty(T, 5, device=DEV), torch.empty(T, 5, device=DEV)
    wide = gpu(torch.cat([a_raw, b_raw], 1))
    ops.decay_and_write_gates(g, beta, wide[:, :5], wide[:, 5:], gpu(a_log), gpu(dt_bias))
    assert rel(g, torch.exp(-torch.exp(a_log) * plain.softplus(a_raw + dt_bias))) < 1e-6
    assert rel(beta, torch.sigmoid(b_raw)) < 1e-6
    # unit vectors per head, in place, in a column view
    x = torch.randn(T, 3 * 24 + 7, generator=gen, dtype=torch.float64)
    xg = gpu(x)
    ops.unit_heads(xg[:, :72], 3, 24, 1e-6, 24 ** -0.5)
    want = plain.unit_vector(x[:, :72].reshape(T, 3, 24)).reshape(T, 72) * 24 ** -0.5
    assert rel(xg[:, :72], want) < 1e-6 and torch.equal(xg[:, 72:].cpu().double(), x[:, 72:].float().double())
    # the first heads with a scale of their own (q before k in one launch)
    xg = gpu(x)
    ops.unit_heads(xg[:, :72], 3, 24, 1e-6, 1.0, first_heads=1, first_scale=0.25)
    want = plain.unit_vector(x[:, :72].reshape(T, 3, 24))
    want[:, 0] *= 0.25
    assert rel(xg[:, :72], want.reshape(T, 72)) < 1e-6
    # the head norm with its gate, heads of 40 and of 1 and of 130 values
    for heads, dv in ((3, 40), (4, 1), (2, 130)):
        o = torch.randn(T, heads, dv, generator=gen, dtype=torch.float64)
        gate = torch.randn(T, heads * dv, generator=gen, dtype=torch.float64)
        gain = torch.randn(dv, generator=gen, dtype=torch.float64)
        want = (plain.rms_unit(o, 1e-5) * gain).reshape(T, -1) * plain.silu(gate)
        for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 6e-3)):
            out = torch.empty(T, heads * dv, device=DEV, dtype=dtype)
            gate_rows = gpu(gate) if dtype == torch.float32 else gpu(gate, torch.bfloat16)
            ref = want if dtype == torch.float32 else (plain.rms_unit(o, 1e-5) * gain).reshape(T, -1) * plain.silu(
                gate.to(torch.bfloat16).double())
            ops.head_rmsnorm_gate(out, gpu(o.reshape(T, -1)), gate_rows, gpu(gain), 1e-5, heads, dv)
            assert rel(out, ref) < tol
    # the experts' activation
    gu = torch.randn(T, 2 * 24, generator=gen, dtype=torch.float64) * 3
    out = torch.empty(T, 24, device=DEV)
    ops.clamped_glu(out, gpu(gu), 1.3, 1.702)
    gg, uu = torch.clamp(gu[:, :24], max=1.3), torch.clamp(gu[:, 24:], -1.3, 1.3)
    assert rel(out, gg * torch.sigmoid(1.702 * gg) * (uu + 1)) < 1e-6


# ------------------------------------------------------------------------- attention
def paged(q, k, v, page, *, scale, slopes, chunk, dtype, positions=None, shuffle=True, kernel="general"):
    """Attention of ``q [T, H, d]`` (tokens at ``positions``, default 0..T-1) over keys and values
    ``k, v [S, G, d / dv]`` laid into pages in a shuffled order, through the general kernel, or
    (bfloat16) the matrix-core kernel for portions (``"portion"``) or for single tokens
    (``"single"``, one launch a token)."""
    from kvcore_amd.ops import library as ops

    S, G, d = k.shape
    dv = v.shape[2]
    T, H, _ = q.shape
    n_pages = -(-S // page)
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1)) if shuffle else torch.arange(n_pages)
    k_cache = torch.full((n_pages + 1, G, page, d), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((n_pages + 1, G, dv, page), float("nan"), dtype=dtype, device=DEV)
    table = torch.zeros((2, n_pages), dtype=torch.int32, device=DEV)
    for p in range(n_pages):
        pid = int(order[p]) + 1
        table[1, p] = pid
        n = min(page, S - p * page)
        k_cache[pid, :, :n] = gpu(k[p * page:p * page + n].transpose(0, 1), dtype)
        v_cache[pid, :, :, :n] = gpu(v[p * page:p * page + n].permute(1, 2, 0), dtype)
    pos = list(range(T)) if positions is None else positions
    out = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    slope_t = None if slopes is None else gpu(torch.tensor(slopes))
    if kernel == "portion":
        assert ops.prefill_attention_supported(H, G, d, page, dtype) and dv == d
        ops.prefill_attention(out, gpu(q.reshape(T, -1), dtype), k_cache, v_cache, table=table,
                              positions=torch.tensor(pos, dtype=torch.int32, device=DEV),
                              q_start=torch.tensor([0, T], dtype=torch.int32, device=DEV),
                              slots=torch.tensor([1], dtype=torch.int32, device=DEV), num_reqs=1, nh=H, nkv=G, d=d,
                              scale=scale, slopes=slope_t, chunk=chunk)
        assert ops.last_variant("prefill_attention").startswith("prefill_attention_kernel")
        return out.double().cpu().view(T, H, dv)
    if kernel == "single":
        assert ops.decode_attention_supported(H, G, d, page, dtype) and dv == d
        for i in range(T):
            ops.decode_attention(out[i:i + 1], gpu(q[i:i + 1].reshape(1, -1), dtype), k_cache, v_cache, table=table,
                                 positions=torch.tensor(pos[i:i + 1], dtype=torch.int32, device=DEV),
                                 token_req=torch.zeros(1, dtype=torch.int32, device=DEV),
                                 slots=torch.tensor([1], dtype=torch.int32, device=DEV), nh=H, nkv=G, d=d,
                                 scale=scale, slopes=slope_t, chunk=chunk)
        return out.double().cpu().view(T, H, dv)
    ops.paged_attention(out, gpu(q.reshape(T, -1), dtype), k_cache, v_cache, table=table,
                        positions=torch.tensor(pos, dtype=torch.int32, device=DEV),
                        token_req=torch.zeros(T, dtype=torch.int32, device=DEV),
                        slots=torch.tensor([1], dtype=torch.int32, device=DEV), nh=H, nkv=G, d=d, dv=dv,
                        scale=scale, slopes=None if slopes is None else gpu(torch.tensor(slopes)), chunk=chunk)
    return out.double().cpu().view(T, H, dv)


def normalised(x):
    """Heads with a mean square of exactly one, which the plain function's own norm leaves alone."""
    return x / x.pow(2).mean(dim=-1, keepdim=True).sqrt()


@pytest.mark.parametrize("H,G,d,dv,chunk,page", [(4, 2, 32, 16, 24, 8), (6, 6, 16, 16, 10, 16), (1, 1, 16, 32, 1, 4),
                                                  (2, 1, 16, 16, 0, 4), (3, 1, 48, 72, 100, 16)])
def test_chunked_attention_with_a_distance_bias(H, G, d, dv, chunk, page):
    gen = torch.Generator().manual_seed(H * 100 + chunk)
    T = 131
    q = normalised(torch.randn(T, H, d, generator=gen, dtype=torch.float64))
    k = normalised(torch.randn(T, G, d, generator=gen, dtype=torch.float64))
    v = torch.randn(T, G, dv, generator=gen, dtype=torch.float64)
    want = plain.chunked_distance_attention(q, k, v, 0.3, chunk or None, 0.0)
    got = paged(q, k, v, page, scale=0.3, slopes=plain.distance_slopes(H), chunk=chunk, dtype=torch.float32)
    assert rel(got, want) < 2e-6
    # the bias matters: without it the result differs
    flat = paged(q, k, v, page, scale=0.3, slopes=None, chunk=chunk, dtype=torch.float32)
    if chunk != 1:
        assert rel(flat, want) > 1e-3
    got = paged(q, k, v, page, scale=0.3, slopes=plain.distance_slopes(H), chunk=chunk, dtype=torch.bfloat16)
    qb, kb, vb = (t.to(torch.bfloat16).double() for t in (q, k, v))
    want_b = plain.chunked_distance_attention(qb, kb, vb, 0.3, chunk or None, 0.0)
    # q and k are rounded after their norm here, which moves their mean squares by 1e-3
    assert rel(got, want_b) < 2e-2


@pytest.mark.parametrize("single", [False, True], ids=["portion", "single"])
def test_a_key_that_stands_out_at_a_chunk_s_edges_and_far_back(single):
    """One key is made to outscore all others for every query.  A query sees it iff it lies in
    the query's chunk and not after it: the first position of the chunk (just inside), the last
    of the chunk before (just outside), a page's first and last slot, a key hundreds of tokens
    back in a long chunk.  The queries come as a portion of a prompt or as single tokens."""
    H, G, d, dv, page = 2, 1, 16, 8, 16
    for chunk, T, marked, query in ((64, 200, 64, 127), (64, 200, 63, 64), (64, 200, 128, 128), (64, 200, 127, 191),
                                    (400, 420, 0, 399), (400, 420, 15, 399), (400, 420, 16, 399), (400, 420, 399, 400),
                                    (0, 420, 3, 419), (48, 200, 95, 96), (48, 200, 96, 143), (48, 200, 96, 144)):
        gen = torch.Generator().manual_seed(marked + query)
        k = torch.randn(T, G, d, generator=gen, dtype=torch.float64) * 0.3
        k[:, 0, 0] = 0.0
        k[marked, 0] = 0.0
        k[marked, 0, 0] = 1.0
        v = torch.randn(T, G, dv, generator=gen, dtype=torch.float64)
        q = torch.randn(T, H, d, generator=gen, dtype=torch.float64) * 0.3
        q[:, :, 0] = 60.0
        visible = marked <= query and (chunk == 0 or marked // chunk == query // chunk)
        want = plain.chunked_distance_attention(normalised(q), normalised(k), v, 1.0, chunk or None, 0.0)
        # head 1's slope is 2^-8: the marked key wins even from 400 tokens away
        assert torch.allclose(want[query, 1], v[marked, 0], atol=1e-3) == visible
        qs = normalised(q)[query:query + 1] if single else normalised(q)[query - 2:query + 1]
        pos = [query] if single else [query - 2, query - 1, query]
        got = paged(qs, normalised(k), v, page, scale=1.0, slopes=plain.distance_slopes(H), chunk=chunk,
                    dtype=torch.float32, positions=pos)
        assert rel(got[-1], want[query]) < 1e-5, (chunk, marked, query)
        assert torch.allclose(got[-1, 1], v[marked, 0], atol=1e-3) == visible, (chunk, marked, query)


@pytest.mark.parametrize("kernel", ["portion", "single"])
@pytest.mark.parametrize("H,G,d,chunk", [(8, 2, 64, 48), (4, 4, 128, 0), (8, 1, 64, 200), (16, 2, 64, 1)])
def test_matrix_core_kernels_with_bias_and_chunks(kernel, H, G, d, chunk):
    """The bfloat16 kernels for portions and for single tokens against the plain function on the
    same rounded values: every position of a prompt of 300 tokens (chunks that are no multiple of
    the kernels' tiles of 16 and 64 keys, a chunk of one position, no chunk), then the key that
    stands out at a chunk's edges."""
    gen = torch.Generator().manual_seed(H + d + chunk)
    T, page = 300, 16
    q = normalised(torch.randn(T, H, d, generator=gen, dtype=torch.float64)).to(torch.bfloat16).double()
    k = normalised(torch.randn(T, G, d, generator=gen, dtype=torch.float64)).to(torch.bfloat16).double()
    v = torch.randn(T, G, d, generator=gen, dtype=torch.float64).to(torch.bfloat16).double()
    # the plain function norms again: take that out by its own factor (the rounded rows' mean squares are not 1)
    want = plain.chunked_distance_attention(q * q.pow(2).mean(-1, keepdim=True).sqrt(),
                                            k * k.pow(2).mean(-1, keepdim=True).sqrt(), v, 0.3, chunk or None, 0.0)
    rows = list(range(T)) if kernel == "portion" else [0, 1, 15, 16, 47, 48, 95, 96, 143, 144, 199, 200, 255, 256, 299]
    got = paged(q[rows] if kernel == "single" else q, k, v, page, scale=0.3, slopes=plain.distance_slopes(H),
                chunk=chunk, dtype=torch.bfloat16, positions=rows, kernel=kernel)
    assert rel(got, want[rows]) < 1e-2
    for size, marked, query in ((48, 95, 96), (48, 96, 143), (48, 96, 144), (48, 48, 95), (200, 0, 199), (200, 15, 199),
                                (200, 199, 200), (0, 3, 299)):
        k2 = (torch.randn(T, G, d, generator=gen, dtype=torch.float64) * 0.3)
        k2[:, :, 0] = 0.0
        k2[marked] = 0.0
        k2[marked, :, 0] = 1.0
        q2 = torch.randn(T, H, d, generator=gen, dtype=torch.float64) * 0.3
        q2[:, :, 0] = 60.0
        q2, k2 = normalised(q2).to(torch.bfloat16).double(), normalised(k2).to(torch.bfloat16).double()
        visible = marked <= query and (size == 0 or marked // size == query // size)
        rows = [query - 2, query - 1, query] if kernel == "portion" else [query]
        got = paged(q2[rows], k2, v, page, scale=1.0, slopes=plain.distance_slopes(H), chunk=size,
                    dtype=torch.bfloat16, positions=rows, kernel=kernel)
        # the last head's slope is 2^-8: the marked key wins even from 300 tokens away
        assert torch.allclose(got[-1, H - 1], v[marked, G - 1], atol=2e-2) == visible, (size, marked, query)


# --------------------------------------------------------------------- routed experts
@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (8, 3, 1, 1), (2, 2, 2, 2), (3, 1, 3, 1), (16, 4, 4, 1),
                                               (16, 4, 4, 2), (12, 3, 4, 3), (5, 5, 1, 1), (70, 6, 10, 3)])
def test_routing_against_the_plain_rule(E, top, groups, keep):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(E * 7 + top)
    T = 57
    logits = torch.randn(T, E, generator=gen, dtype=torch.float64) * 2
    logits[3] = 0.0  # all equal: the lowest indices of the first groups
    logits = logits.float().double()
    choice = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_route(choice, weight, gpu(logits), top=top, groups=groups, keep=keep)
    scores = torch.softmax(logits, dim=-1)
    for t in range(T):
        want_e, want_w = plain.route(scores[t], top, groups, keep)
        got_e = choice[t].tolist()
        live = min(top, keep * (E // groups))  # fewer allowed experts than choices: the rest weigh nothing
        assert got_e[:live] == want_e[:live], t
        assert torch.allclose(weight[t, :live].double().cpu(), want_w[:live], atol=1e-6), t
        assert float(weight[t, live:].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("E,top,groups,keep,H,T", [(6, 2, 3, 2, 96, 75), (32, 4, 8, 4, 256, 1100), (2, 2, 2, 2, 40, 1),
                                                   (70, 6, 10, 3, 130, 9), (130, 3, 1, 1, 64, 20)])
def test_router_product_and_choice_in_one_kernel(dtype, E, top, groups, keep, H, T):
    """The fused router against the plain rule on the same rows; the logits are float32 sums of the
    rows as they are, the same for a token alone and among a thousand (blocks of 4 and of 16 tokens)."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(E + T)
    x = torch.randn(T, H, generator=gen, dtype=torch.float64)
    x = x.to(dtype).double()
    w = (torch.randn(E, H, generator=gen, dtype=torch.float64) * 0.5).float().double()
    choice = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_router(choice, weight, gpu(x, dtype), gpu(w), top=top, groups=groups, keep=keep)
    logits = x @ w.T
    scores = torch.softmax(logits, dim=-1)
    checked = 0
    for t in range(T):
        if plain.route_margin(logits[t], top, groups, keep) < 1e-4:
            continue  # a tie within float32's reach
        want_e, want_w = plain.route(scores[t], top, groups, keep)
        assert choice[t].tolist() == want_e, t
        assert torch.allclose(weight[t].double().cpu(), want_w, atol=1e-5), t
        checked += 1
    assert checked >= T * 0.9
    # a token's result does not depend on the batch: the first rows alone give the same bits
    n = min(T, 3)
    c2 = torch.empty(n, top, dtype=torch.int32, device=DEV)
    w2 = torch.empty(n, top, dtype=torch.float32, device=DEV)
    ops.moe_router(c2, w2, gpu(x[:n], dtype), gpu(w), top=top, groups=groups, keep=keep)
    assert torch.equal(c2, choice[:n]) and torch.equal(w2, weight[:n])


def expert_weights(E, H, I, gen, shared=0):
    w = {"router": torch.randn(E, H, generator=gen, dtype=torch.float64) * 0.5}
    for e in range(E):
        w[f"e{e}.gate"] = torch.randn(I, H, generator=gen, dtype=torch.float64) * 0.3
        w[f"e{e}.up"] = torch.randn(I, H, generator=gen, dtype=torch.float64) * 0.3
        w[f"e{e}.down"] = torch.randn(H, I, generator=gen, dtype=torch.float64) * 0.3
    if shared:
        w["shared.gate"] = torch.randn(shared, H, generator=gen, dtype=torch.float64) * 0.3
        w["shared.up"] = torch.randn(shared, H, generator=gen, dtype=torch.float64) * 0.3
        w["shared.down"] = torch.randn(H, shared, generator=gen, dtype=torch.float64) * 0.3
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("E,top,groups,keep,H,I,shared,T", [(6, 2, 3, 2, 96, 40, 56, 75), (8, 3, 1, 1, 128, 64, 0, 300),
                                                            (2, 2, 2, 2, 40, 8, 0, 1), (3, 1, 3, 1, 40, 16, 8, 2),
                                                            (16, 4, 4, 1, 64, 32, 32, 33), (5, 2, 1, 1, 36, 20, 12, 19),
                                                            (4, 2, 1, 1, 96, 32, 0, 200), (2, 1, 1, 1, 160, 96, 16, 150),
                                                            (2, 2, 2, 2, 64, 32, 0, 300), (3, 1, 1, 1, 96, 64, 24, 800)])
def test_the_feed_forward_of_routed_experts(dtype, E, top, groups, keep, H, I, shared, T):
    """The part itself on rows of its own: routing, the arrangement by expert, both products,
    the weighted sum and the shared expert, against the plain function token by token.  Sizes
    that 16-byte loads do not divide (36, 20, 12) take the kernel without them; many rows an expert
    take tiles of 64 rows (also with sums of 96, 160 and 32 terms, which end inside a pass of 64)."""
    from kvcore_amd.engine.context import StepBuffers, StepContext
    from kvcore_amd.parts.base import Runtime
    from kvcore_amd.parts.moe import RoutedExperts

    gen = torch.Generator().manual_seed(E + T)
    w = expert_weights(E, H, I, gen, shared)
    if dtype == torch.bfloat16:
        w = {k: (v if k == "router" else v.to(torch.bfloat16).double()) for k, v in w.items()}
    part = RoutedExperts(hidden_size=H, experts=E, top=top, expert_size=I, limit=1.2, groups=groups, keep=keep,
                         shared_size=shared, shared_limit=0.8,
                         tensor_names={"router": "router", "expert": "e{e}", "shared": "shared", "gate": "gate",
                                       "up": "up", "down": "down"})
    part.setup(Runtime(dtype=dtype, device=torch.device(DEV)))
    params = {}
    for ps in part.param_specs():
        t = torch.empty(ps.shape, dtype=torch.float32 if ps.kind == "vector" else dtype, device=DEV)
        for src in ps.resolved_sources():
            t[src.row:src.row + src.rows] = gpu(w[src.name], t.dtype)
        params[ps.name] = t
    part.bind(params)
    x = torch.randn(T, H, generator=gen, dtype=torch.float64)
    if dtype == torch.bfloat16:
        x = x.to(torch.bfloat16).double()
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}},
           "expert": {"ff": I, "limit": 1.2}, "shared": {"ff": shared, "limit": 0.8} if shared else None}
    want = plain.moe_feed_forward(x, {f"p.{k}": v for k, v in w.items()}, "p", mlp)
    buffers = StepBuffers(torch.device(DEV), token_capacity=T)
    none = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = StepContext(num_tokens=T, num_reqs=1, token_ids=none, positions=none, token_req=none, q_start=none,
                      seq_lens=none, slots=none, groups=[], states=[], buffers=buffers, dtype=dtype,
                      device=torch.device(DEV))
    out = part.forward(gpu(x, dtype), ctx, None)
    assert out.dtype == torch.float32 and out.shape == (T, H)
    assert rel(out, want) < (3e-6 if dtype == torch.float32 else 8e-3)
    # the form that adds into a stream, with another branch's rows taken along
    stream = torch.randn(T, H, generator=gen, dtype=torch.float64)
    other = torch.randn(T, H, generator=gen, dtype=torch.float64)
    first = out.double().cpu().clone()
    stream_gpu = gpu(stream)
    part.forward_into(stream_gpu, gpu(x, dtype), ctx, None, add=gpu(other))
    assert rel(stream_gpu, stream.float().double() + (other.float().double() + first)) < 1e-6
    # the same rows again among others, in another order: a row's result does not depend on its place
    out = part.forward(gpu(x, dtype), ctx, None)
    if T > 2:
        first = out.cpu().clone()  # the result lives in a step buffer that the next call rewrites
        perm = torch.randperm(T, generator=gen)
        again = part.forward(gpu(x[perm], dtype), ctx, None)
        assert rel(again, first[perm].double()) < 1e-6


def test_offset_norm_keeps_a_gain_of_one_plus_the_stored_weight():
    from kvcore_amd.parts.base import Runtime
    from kvcore_amd.parts.rmsnorm import RMSNorm

    gen = torch.Generator().manual_seed(2)
    H, T = 96, 9
    w = torch.randn(H, generator=gen, dtype=torch.float64) * 0.2
    r = torch.randn(T, H, generator=gen, dtype=torch.float64) * 3
    norm = RMSNorm(hidden_size=H, eps=1e-5, weight_offset=1.0, weight_name="")
    assert [s.name for s in norm.param_specs()[0].resolved_sources()] == [""]
    norm.setup(Runtime(dtype=torch.float32, device=torch.device(DEV)))
    norm.bind({"weight": gpu(w)})
    norm.weights_loaded()
    out = torch.empty(T, H, device=DEV)
    norm.forward_fused(out, gpu(r), None)
    assert rel(out, plain.offset_rms_norm(r, w, 1e-5)) < 1e-6
    assert math.isclose(float(norm.as_gain()[0][0]), 1.0 + float(w[0].float()), rel_tol=1e-6)
