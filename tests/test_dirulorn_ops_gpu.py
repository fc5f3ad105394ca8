"""Each mechanism of the Dirulorn decoder alone: the kernel against the plain implementation
of ``tests/plain/dirulorn.py`` (float64 on the CPU), whole and cut into steps, with state slots
used again, and with inputs made so that a fault would show."""

from __future__ import annotations

import math

import pytest
import torch

from tests.dirulorn_helpers import batch_tensors
from tests.plain import dirulorn as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from kvcore_amd.ops import library

    library.load()
    return library


def rnd(*shape, seed=0, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def close(got, want, atol, rtol=1e-5):
    got, want = got.detach().cpu().double(), want.double()
    assert torch.isfinite(got).all()
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert (err <= bound).all(), f"worst error {float(err.max()):.3e} at {int(torch.argmax(err - bound))}"


# ------------------------------------------------------------------------------ norms
@pytest.mark.parametrize("H", [40, 96, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_norm_with_the_residual_sum(ops, H, dtype):
    T = 7
    res = rnd(T, H, seed=1) * 3 + 5.0  # a mean far from zero: the variance is of the deviations
    delta = rnd(T, H, seed=2).to(dtype)
    w, b = rnd(H, seed=3) + 1, rnd(H, seed=4)
    r = res.clone().to(DEV)
    out = torch.empty(T, H, dtype=dtype, device=DEV)
    ops.add_layernorm(out, r, delta.to(DEV), w.to(DEV), b.to(DEV), 1e-5)
    total = res.double() + delta.double()
    close(r, total, 1e-6)
    want = plain.layer_norm(total, w.double(), b.double(), 1e-5)
    tol = dict(atol=2e-5) if dtype == torch.float32 else dict(atol=1e-2, rtol=8e-3)  # one rounding to 8 bits
    close(out, want, **tol)
    ops.add_layernorm(out, r, None, w.to(DEV), None, 1e-5)  # no pending sum, no shift
    close(out, plain.layer_norm(total, w.double(), torch.zeros(H, dtype=torch.float64), 1e-5), **tol)


@pytest.mark.parametrize("n", [1, 2, 3])
def test_mean_of_branches_each_over_its_root_mean_square(ops, n):
    T, H = 5, 72
    xs = [rnd(T, H, seed=10 + b) * (10.0 ** b) for b in range(n)]  # branches of very different size
    gs = [rnd(H, seed=20 + b) + 1 for b in range(n)]
    out = torch.empty(T, H, device=DEV)
    ops.rms_branches_mean(out, [(x.to(DEV), g.to(DEV)) for x, g in zip(xs, gs)], 1e-6)
    want = sum(plain.rms_unit(x.double(), 1e-6) * g.double() for x, g in zip(xs, gs)) / n
    close(out, want, 1e-5)


def test_gate_then_norm_in_equal_parts(ops):
    T, width, parts = 6, 60, 3
    y, z, g = rnd(T, width, seed=1), rnd(T, width + 9, seed=2), rnd(width, seed=3) + 1
    y[:, :20] *= 50.0  # one part far larger than the others: each part has its own root mean square
    out = torch.empty(T, width, device=DEV)
    zd = z.to(DEV)
    ops.gated_group_rmsnorm(out, y.to(DEV), zd[:, 4: 4 + width], g.to(DEV), 1e-6, parts)
    v = y.double() * plain.silu(z[:, 4: 4 + width].double())
    want = plain.rms_unit(v.view(T, parts, width // parts), 1e-6).reshape(T, width) * g.double()
    close(out, want, 1e-5)


def test_loop_entry_pieces(ops):
    T, H = 4, 24
    a, b, v = rnd(T, H, seed=1), rnd(T, H, seed=2), rnd(H, seed=3)
    both = torch.empty(T, 2 * H, device=DEV)
    ops.concat2(both, a.to(DEV), b.to(DEV))
    assert torch.equal(both.cpu(), torch.cat([a, b], dim=1))
    x = a.clone().to(DEV)
    ops.add_row(x, v.to(DEV))
    assert torch.equal(x.cpu(), a + v)


# ------------------------------------------------------------------------ convolution
def run_conv_in_steps(ops, x, w, b, cuts, act, slot, state, junk_rows=3):
    """One request's tokens cut at ``cuts``; other requests ride along in the batch."""
    T, C = x.shape
    K = w.shape[1]
    outs = []
    start = 0
    other = rnd(64, C + 5, seed=99)
    for n in cuts:
        # the request sits between two others, its channels inside wider rows
        reqs = [((slot + 1) % state.shape[0], 7, junk_rows), (slot, start, n), None]
        batch, total = batch_tensors(reqs)
        rows = torch.zeros(total, C + 5)
        rows[:junk_rows] = other[:junk_rows]
        rows[junk_rows: junk_rows + n, 2: 2 + C] = x[start: start + n]
        rows_d = rows.to(DEV)
        out = torch.full((total, C), float("nan"), device=DEV)
        ops.causal_conv(out, rows_d[:, 2: 2 + C], w.to(DEV), None if b is None else b.to(DEV), state,
                        act=act, **batch)
        outs.append(out[junk_rows: junk_rows + n].cpu())
        assert torch.equal(out[-1].cpu(), torch.zeros(C))  # the padding token's row
        start += n
    return torch.cat(outs)


@pytest.mark.parametrize("K", [1, 2, 4, 5])
@pytest.mark.parametrize("act", ["none", "silu"])
def test_causal_convolution_whole_and_in_steps(ops, K, act):
    T, C = 53, 70  # steps of 32 tokens and more run the kernel that slides a window along
    x, w, b = rnd(T, C, seed=K), rnd(C, K, seed=K + 10), rnd(C, seed=K + 20)
    want = plain.causal_conv(x.double(), w.double(), b.double())
    if act == "silu":
        want = plain.silu(want)
    for cuts in ([T], [1] * T, [2, 2, 1, 3, 1, 1, 2, 11, 30], [5, 1, 1, 1, 15, 30], [52, 1], [1, 52]):
        # a slot that another request has left full of its inputs: the first tokens see zeros
        state = torch.full((3, max(K - 1, 1), C), 7.0, device=DEV)[:, : K - 1]
        got = run_conv_in_steps(ops, x, w, b, cuts, act, slot=1, state=state)
        close(got, want, 1e-5)


@pytest.mark.parametrize("K", [1, 2, 4])
def test_convolution_of_single_tokens_moves_its_state_on_in_the_same_kernel(ops, K):
    """A step in which every request brings one token (as the caller vouches): two requests at
    different positions and a padded row between them, token after token."""
    T, C = 19, 40
    xa, xb = rnd(T, C, seed=1), rnd(T, C, seed=2)
    w, b = rnd(C, K, seed=3), rnd(C, seed=4)
    want_a = plain.causal_conv(xa.double(), w.double(), b.double())
    want_b = plain.causal_conv(xb.double(), w.double(), b.double())
    state = torch.full((3, max(K - 1, 1), C), 5.0, device=DEV)[:, : K - 1]
    got_a, got_b = [], []
    for t in range(T):
        reqs = [(2, t, 1), None] + ([(0, t - 4, 1)] if t >= 4 else [])  # the second starts four steps later
        batch, total = batch_tensors(reqs)
        rows = torch.zeros(total, C)
        rows[0] = xa[t]
        if t >= 4:
            rows[2] = xb[t - 4]
        out = torch.full((total, C), float("nan"), device=DEV)
        ops.causal_conv(out, rows.to(DEV), w.to(DEV), b.to(DEV), state, single_tokens=True, **batch)
        got_a.append(out[0].cpu())
        if t >= 4:
            got_b.append(out[2].cpu())
    close(torch.stack(got_a), want_a, 1e-5)
    close(torch.stack(got_b), want_b[: T - 4], 1e-5)


def test_convolution_reads_bfloat16_rows_and_writes_them(ops):
    T, C, K = 9, 32, 4
    x, w = rnd(T, C, seed=1, dtype=torch.bfloat16), rnd(C, K, seed=2)
    state = torch.zeros(1, K - 1, C, device=DEV)
    batch, _ = batch_tensors([(0, 0, T)])
    out = torch.empty(T, C, dtype=torch.bfloat16, device=DEV)
    ops.causal_conv(out, x.to(DEV), w.to(DEV), None, state, **batch)
    close(out, plain.causal_conv(x.double(), w.double(), torch.zeros(C, dtype=torch.float64)), 2e-2, 1e-2)
    # the state afterwards: the last K-1 inputs, oldest first
    assert torch.equal(state[0].cpu(), x[T - (K - 1):].float())


# ------------------------------------------------------------ gated linear recurrence
def plain_recurrence(u, y, wa, wi, ba, bi, lam, c):
    T, W = u.shape
    nb = wa.shape[0]
    ub = u.view(T, nb, W // nb)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", wa, ub) + ba).reshape(T, W)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", wi, ub) + bi).reshape(T, W)
    a = torch.exp(-c * r * plain.softplus(lam))
    drive = torch.sqrt(1 - a * a) * i * u
    S = torch.zeros(W, dtype=u.dtype)
    out = torch.empty_like(u)
    for t in range(T):
        S = a[t] * S + drive[t]
        out[t] = S * plain.gelu_tanh(y[t])
    return out, S


@pytest.mark.parametrize("W,nb", [(40, 1), (72, 3), (160, 2), (130, 130)])
def test_gated_linear_recurrence_whole_and_in_steps(ops, W, nb):
    T = 41
    bw = W // nb
    u, y = rnd(T, W, seed=1), rnd(T, W, seed=2)
    wa, wi = rnd(nb, bw, bw, seed=3, std=0.5), rnd(nb, bw, bw, seed=4, std=0.5)
    ba, bi = rnd(nb, bw, seed=5), rnd(nb, bw, seed=6)
    lam = rnd(W, seed=7) * 2 - 3  # decays from almost 1 to almost 0
    want, last = plain_recurrence(*(t.double() for t in (u, y, wa, wi, ba, bi, lam)), 8.0)
    d = [t.to(DEV) for t in (wa, wi, ba, bi, lam)]
    for cuts in ([T], [1] * T, [2, 3, 17, 1, 1, 2, 15], [40, 1]):
        state = torch.full((4, W), float("nan"), device=DEV)  # nobody reads a slot before writing it
        outs, start = [], 0
        for n in cuts:
            batch, total = batch_tensors([None, (2, start, n), (3, 5, 2)])
            uu = torch.zeros(total, W)
            yy = torch.zeros(total, W + 3)
            uu[1: 1 + n], yy[1: 1 + n, 3:] = u[start: start + n], y[start: start + n]
            state[3] = 0.5
            a = torch.empty(total, W, device=DEV)
            drive = torch.empty(total, W, device=DEV)
            ops.rglru_gates(a, drive, uu.to(DEV), *d, 8.0)
            out = torch.empty(total, W, device=DEV)
            ops.rglru_scan(out, a, drive, yy.to(DEV)[:, 3:], state, **batch)
            outs.append(out[1: 1 + n].cpu())
            start += n
        close(torch.cat(outs), want, 2e-5, 2e-5)
        close(state[2], last, 2e-5, 2e-5)


def test_long_portions_are_scanned_in_segments_side_by_side(ops):
    """With a workspace, requests longer than a segment are cut into segments that are scanned
    side by side and joined in order: the same results, whatever the portions, beside short
    requests and a padded one, from a state that an earlier step left."""
    T, W, nb = 333, 96, 2
    bw = W // nb
    u, y = rnd(T, W, seed=1), rnd(T, W, seed=2)
    wa, wi = rnd(nb, bw, bw, seed=3, std=0.5), rnd(nb, bw, bw, seed=4, std=0.5)
    ba, bi = rnd(nb, bw, seed=5), rnd(nb, bw, seed=6)
    lam = rnd(W, seed=7) * 2 - 3
    want, last = plain_recurrence(*(t.double() for t in (u, y, wa, wi, ba, bi, lam)), 8.0)
    d = [t.to(DEV) for t in (wa, wi, ba, bi, lam)]
    for cuts in ([T], [64, 65, 1, 129, 74], [200, 133], [3, 330]):
        state = torch.full((4, W), float("nan"), device=DEV)
        outs, start = [], 0
        for n in cuts:
            batch, total = batch_tensors([(3, 5, 2), (2, start, n), None, (0, 0, 70)])
            uu = torch.zeros(total, W)
            yy = torch.zeros(total, W)
            uu[2: 2 + n], yy[2: 2 + n] = u[start: start + n], y[start: start + n]
            uu[3 + n:], yy[3 + n:] = u[:70], y[:70]  # a second request: the first 70 tokens again
            state[3] = 0.5
            a = torch.empty(total, W, device=DEV)
            drive = torch.empty(total, W, device=DEV)
            ops.rglru_gates(a, drive, uu.to(DEV), *d, 8.0)
            out = torch.empty(total, W, device=DEV)
            longest = max(n, 70)
            ws = torch.full((ops.rglru_scan_workspace_floats(4, W, longest),), float("nan"), device=DEV)
            ops.rglru_scan(out, a, drive, yy.to(DEV), state, max_query_len=longest, workspace=ws, **batch)
            outs.append(out[2: 2 + n].cpu())
            close(out[3 + n:], want[:70], 2e-5, 2e-5)
            assert torch.equal(out[2 + n].cpu(), torch.zeros(W))
            start += n
        close(torch.cat(outs), want, 2e-5, 2e-5)
        close(state[2], last, 2e-5, 2e-5)


def test_recurrence_keeps_a_far_token(ops):
    """A channel whose decay is almost 1 still carries its first input after 600 tokens, through
    steps of every size; a channel whose decay is almost 0 carries nothing."""
    T, W = 600, 64
    u = torch.zeros(T, W)
    u[0] = 1.0
    lam = torch.full((W,), -12.0)
    lam[W // 2:] = 3.0
    wa = wi = torch.zeros(1, W, W)
    ba = bi = torch.zeros(1, W)
    y = torch.ones(T, W)
    want, _ = plain_recurrence(*(t.double() for t in (u, y, wa, wi, ba, bi, lam)), 8.0)
    assert want[-1, 0] > 0.5 * want[0, 0] and want[-1, -1] == 0
    state = torch.zeros(1, W, device=DEV)
    outs, start = [], 0
    for n in [100, 1, 1, 254, 2, 200, 41, 1]:
        batch, total = batch_tensors([(0, start, n)])
        a = torch.empty(total, W, device=DEV)
        drive = torch.empty(total, W, device=DEV)
        ops.rglru_gates(a, drive, u[start: start + n].to(DEV), wa.to(DEV), wi.to(DEV), ba.to(DEV), bi.to(DEV),
                        lam.to(DEV), 8.0)
        out = torch.empty(total, W, device=DEV)
        ops.rglru_scan(out, a, drive, y[start: start + n].to(DEV), state, **batch)
        outs.append(out.cpu())
        start += n
    close(torch.cat(outs), want, 1e-5, 1e-4)


# ------------------------------------------------------------------------ state space
def plain_state_space(x, B, C, dt_raw, dt_bias, a_log, d_skip, G):
    T, nh, P = x.shape
    N = B.shape[2]
    dt = plain.softplus(dt_raw + dt_bias)
    dec = torch.exp(-torch.exp(a_log) * dt)
    y = torch.empty(T, nh, P, dtype=x.dtype)
    S = torch.zeros(nh, N, P, dtype=x.dtype)
    for t in range(T):
        for h in range(nh):
            g = h // (nh // G)
            S[h] = dec[t, h] * S[h] + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S[h].T @ C[t, g] + d_skip[h] * x[t, h]
    return y.reshape(T, nh * P), S


@pytest.mark.parametrize("nh,P,N,G", [(1, 5, 3, 1), (6, 20, 24, 3), (7, 1, 9, 7), (2, 80, 200, 1), (4, 64, 128, 2)])
def test_state_space_recurrence_whole_and_in_steps(ops, nh, P, N, G):
    T = 37
    x, B, C = rnd(T, nh, P, seed=1), rnd(T, G, N, seed=2), rnd(T, G, N, seed=3)
    dt_raw, dt_bias = rnd(T, nh, seed=4), rnd(nh, seed=5)
    a_log, d_skip = rnd(nh, seed=6) - 0.5, rnd(nh, seed=7) + 1
    want, last = plain_state_space(*(t.double() for t in (x, B, C, dt_raw, dt_bias, a_log, d_skip)), G)
    xbc = torch.cat([x.reshape(T, -1), B.reshape(T, -1), C.reshape(T, -1)], dim=1)
    width = xbc.shape[1]
    for cuts in ([T], [1] * T, [2, 3, 16, 1, 15], [17, 20]):
        state = torch.full((3, nh, N, P), float("nan"), device=DEV)
        outs, start = [], 0
        for n in cuts:
            batch, total = batch_tensors([(0, 3, 1), (1, start, n), None])
            state[0] = 0.25
            rows = torch.zeros(total, width + 4)
            rows[1: 1 + n, :width] = xbc[start: start + n]
            dts = torch.zeros(total, nh + 2)
            dts[1: 1 + n, 2:] = dt_raw[start: start + n]
            y = torch.full((total, nh * P), float("nan"), device=DEV)
            ops.ssm_scan(y, rows.to(DEV)[:, :width], dts.to(DEV)[:, 2:], dt_bias.to(DEV), a_log.to(DEV),
                         d_skip.to(DEV), state, heads=nh, head_dim=P, state_size=N, groups=G, **batch)
            assert torch.isfinite(y).all()
            outs.append(y[1: 1 + n].cpu())
            start += n
        close(torch.cat(outs), want, 3e-5, 3e-5)
        close(state[1], last, 3e-5, 3e-5)


# -------------------------------------------------------------------------- attention
def attention_setup(ops, T_cap, nkv, d, dv, page, dtype, planes=1):
    pages = -(-T_cap // page) + 3
    kc = torch.full((pages, nkv, page, d), float("nan"), dtype=dtype, device=DEV)
    vc = [torch.full((pages, nkv, dv // planes, page), float("nan"), dtype=dtype, device=DEV)
          for _ in range(planes)]
    return kc, vc[0] if planes == 1 else vc


def run_attention_in_steps(ops, qkv, cuts, nh, nkv, d, dv, scale, freqs, interleaved, gains, eps, page, dtype,
                           table_pages, planes=1):
    """Norm, rotation, cache write and attention of one request cut at ``cuts``; pages in the
    order ``table_pages``; the values in ``planes`` planes, each attended to by itself."""
    T = qkv.shape[0]
    kc, vc = attention_setup(ops, T + 64, nkv, d, dv, page, dtype, planes)
    table = torch.zeros(2, len(table_pages), dtype=torch.int32, device=DEV)
    table[1] = torch.tensor(table_pages, dtype=torch.int32)
    inv_freq = torch.tensor(freqs, dtype=torch.float32, device=DEV)
    outs, start = [], 0
    for n in cuts:
        batch, total = batch_tensors([(1, start, n)])
        rows = qkv[start: start + n].to(dtype).to(DEV).contiguous()
        cos = torch.empty(total, len(freqs), device=DEV)
        sin = torch.empty(total, len(freqs), device=DEV)
        if freqs:
            ops.rope_table(cos, sin, batch["positions"], inv_freq)
        kv_slot = torch.empty(total, dtype=torch.int32, device=DEV)
        ops.kv_slots(kv_slot, positions=batch["positions"], token_req=batch["token_req"], slots=batch["slots"],
                     table=table, page_size=page, num_pages=kc.shape[0])
        ops.qk_norm_rope_kv_write(rows, kc, vc, cos, sin, rot_dim=2 * len(freqs), interleaved=interleaved,
                                  kv_slot=kv_slot, nh=nh, nkv=nkv, d=d, dv=dv,
                                  q_gain=None if gains is None else gains[0].to(DEV),
                                  k_gain=None if gains is None else gains[1].to(DEV), eps=eps)
        if planes == 1:
            out = torch.empty(total, nh * dv, dtype=dtype, device=DEV)
            ops.paged_attention(out, rows, kc, vc, table=table, positions=batch["positions"],
                                token_req=batch["token_req"], slots=batch["slots"], nh=nh, nkv=nkv, d=d, dv=dv,
                                scale=scale)
        else:
            per = []
            for plane in vc:
                o = torch.empty(total, nh * dv // planes, dtype=dtype, device=DEV)
                ops.paged_attention(o, rows, kc, plane, table=table, positions=batch["positions"],
                                    token_req=batch["token_req"], slots=batch["slots"], nh=nh, nkv=nkv, d=d,
                                    dv=dv // planes, scale=scale)
                per.append(o.view(total, nh, 1, dv // planes))
            out = torch.cat(per, dim=2).reshape(total, nh * dv)
        outs.append(out.float().cpu())
        start += n
    return torch.cat(outs)


def plain_attention(qkv, nh, nkv, d, dv, scale, freqs, gains, eps):
    T = qkv.shape[0]
    q = qkv[:, : nh * d].view(T, nh, d)
    k = qkv[:, nh * d: (nh + nkv) * d].view(T, nkv, d)
    v = qkv[:, (nh + nkv) * d:].view(T, nkv, dv)
    if gains is not None:
        q = plain.rms_unit(q, eps) * gains[0].double()
        k = plain.rms_unit(k, eps) * gains[1].double()
    if freqs:
        q, k = plain.rotate_interleaved(q, freqs), plain.rotate_interleaved(k, freqs)
    return plain.softmax_attention(q, k, v, scale).reshape(T, nh * dv)


@pytest.mark.parametrize("nh,nkv,d,dv,rot", [(4, 2, 32, 16, 8), (6, 3, 24, 40, 24), (1, 1, 16, 16, 2),
                                             (3, 1, 48, 72, 0), (2, 2, 20, 12, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_head_norm_rotation_and_value_size(ops, nh, nkv, d, dv, rot, dtype):
    T, page = 45, 8
    qkv = rnd(T, (nh + nkv) * d + nkv * dv, seed=d)
    if dtype == torch.bfloat16:
        qkv = qkv.to(torch.bfloat16).float()
    gains = (rnd(d, seed=1) * 0.2 + 1, rnd(d, seed=2) * 0.2 + 1)
    freqs = plain.rotary_frequencies(rot, 50.0, {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}) if rot else []
    want = plain_attention(qkv.double(), nh, nkv, d, dv, 0.3, freqs, gains, 1e-5)
    pages = [5, 2, 7, 1, 4, 3, 6, 8]  # not in order
    for cuts in ([T], [20] + [1] * 25, [3, 5, 8, 2, 2, 9, 16]):
        got = run_attention_in_steps(ops, qkv, cuts, nh, nkv, d, dv, 0.3, freqs, True, gains, 1e-5, page, dtype, pages)
        close(got, want, 2e-5 if dtype == torch.float32 else 3e-2, 1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("planes", [2, 3])
def test_values_kept_in_several_planes(ops, planes):
    """Element i of a value head lies in plane i / (dv / planes): attending to each plane by
    itself and laying the results side by side within every head gives the whole."""
    T, nh, nkv, d, page = 37, 4, 2, 16, 8
    dv = planes * d
    qkv = rnd(T, (nh + nkv) * d + nkv * dv, seed=planes)
    want = plain_attention(qkv.double(), nh, nkv, d, dv, 0.25, [], None, 0.0)
    for cuts in ([T], [9, 1, 1, 2, 24]):
        got = run_attention_in_steps(ops, qkv, cuts, nh, nkv, d, dv, 0.25, [], True, None, 0.0, page, torch.float32,
                                     [3, 1, 4, 2, 6, 5], planes=planes)
        close(got, want, 2e-5, 1e-4)


@pytest.mark.parametrize("far", [0, 1, 7, 8, 15, 16, 17, 250])
def test_a_far_key_that_stands_out_is_found(ops, far):
    """One key among 300 has a score far above the rest: the output at the last positions is
    that key's value, whether it lies at a page's edge or far back, in a prompt's portion or for
    a single token."""
    T, nh, nkv, d, dv, page = 300, 2, 1, 16, 24, 16
    qkv = rnd(T, (nh + nkv) * d + nkv * dv, seed=3) * 0.1
    qkv[far, nh * d: (nh + nkv) * d] = 0.0
    qkv[far, nh * d] = 30.0          # the key at `far` points along the first axis
    qkv[T - 3:, 0] = 30.0            # and so do the last queries of head 0
    want = plain_attention(qkv.double(), nh, nkv, d, dv, 1.0, [], None, 0.0)
    v_far = qkv[far, (nh + nkv) * d:].double()
    assert (want[T - 1, :dv] - v_far).abs().max() < 1e-6  # the plain result is that value
    pages = list(range(1, 20))
    for cuts in ([T], [T - 3, 1, 1, 1], [far + 1, T - far - 3, 2] if far + 3 < T else [T]):
        got = run_attention_in_steps(ops, qkv, cuts, nh, nkv, d, dv, 1.0, [], True, None, 0.0, page,
                                     torch.float32, pages)
        close(got, want, 2e-5, 1e-4)


def test_rotation_pairs_neighbours_and_leaves_the_rest(ops):
    """Interleaved pairs (2i, 2i+1) of the first ``dims`` elements turn by position * f_i; the
    elements behind them pass; values are not rotated."""
    nh = nkv = 1
    d, dv, page = 16, 16, 4
    T = 6
    qkv = torch.zeros(T, 3 * d)
    qkv[:, 0] = 1.0       # q: first of the first pair
    qkv[:, d + 0] = 1.0   # k likewise
    qkv[:, 2 * d:] = rnd(T, dv, seed=1)
    freqs = [0.5, 0.25]
    kc, vc = attention_setup(ops, 16, nkv, d, dv, page, torch.float32)
    table = torch.tensor([[1, 2, 3]], dtype=torch.int32, device=DEV)
    batch, total = batch_tensors([(0, 0, T)])
    cos, sin = torch.empty(T, 2, device=DEV), torch.empty(T, 2, device=DEV)
    ops.rope_table(cos, sin, batch["positions"], torch.tensor(freqs, device=DEV))
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=batch["positions"], token_req=batch["token_req"], slots=batch["slots"],
                 table=table, page_size=page, num_pages=kc.shape[0])
    rows = qkv.to(DEV)
    ops.qk_norm_rope_kv_write(rows, kc, vc, cos, sin, rot_dim=4, interleaved=True, kv_slot=kv_slot,
                              nh=nh, nkv=nkv, d=d, dv=dv)
    rows = rows.cpu()
    for t in range(T):
        assert abs(rows[t, 0] - math.cos(0.5 * t)) < 1e-6 and abs(rows[t, 1] - math.sin(0.5 * t)) < 1e-6
        assert rows[t, 2:d].abs().max() == 0
        assert torch.equal(rows[t, 2 * d:], qkv[t, 2 * d:])
        page_id, off = 1 + t // page, t % page
        assert torch.equal(kc[page_id, 0, off].cpu(), rows[t, d: 2 * d])
        assert torch.equal(vc[page_id, 0, :, off].cpu(), qkv[t, 2 * d:])


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("T", [5, 40])  # few tokens: a block a token; many: a wave a head and tiled values
def test_head_norm_and_rotation_in_both_pairings(ops, interleaved, T):
    """The rewritten q and k rows and the cache after the kernel, against the norm and rotation
    written out here: pairs of neighbours, or pairs half the rotated width apart."""
    nh, nkv, d, dv, rot, page = 3, 2, 32, 16, 16, 8
    qkv = rnd(T, (nh + nkv) * d + nkv * dv, seed=T)
    gq, gk = rnd(d, seed=1) * 0.3 + 1, rnd(d, seed=2) * 0.3 + 1
    freqs = torch.tensor([0.7 ** i for i in range(rot // 2)], dtype=torch.float64)
    heads = qkv[:, : (nh + nkv) * d].double().view(T, nh + nkv, d)
    gains = torch.cat([gq.double().expand(nh, d), gk.double().expand(nkv, d)])
    normed = plain.rms_unit(heads, 1e-5) * gains
    ang = torch.arange(T, dtype=torch.float64)[:, None] * freqs
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    want = normed.clone()
    if interleaved:
        u, v = normed[..., 0:rot:2], normed[..., 1:rot:2]
        want[..., 0:rot:2], want[..., 1:rot:2] = u * c - v * s, v * c + u * s
    else:
        u, v = normed[..., : rot // 2], normed[..., rot // 2: rot]
        want[..., : rot // 2], want[..., rot // 2: rot] = u * c - v * s, v * c + u * s
    kc, vc = attention_setup(ops, T + 16, nkv, d, dv, page, torch.float32)
    table = torch.tensor([[4, 2, 7, 1, 3, 5, 6]], dtype=torch.int32, device=DEV)
    batch, total = batch_tensors([(0, 0, T)])
    cos, sin = torch.empty(T, rot // 2, device=DEV), torch.empty(T, rot // 2, device=DEV)
    ops.rope_table(cos, sin, batch["positions"], freqs.float().to(DEV))
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=batch["positions"], token_req=batch["token_req"], slots=batch["slots"],
                 table=table, page_size=page, num_pages=kc.shape[0])
    rows = qkv.to(DEV)
    ops.qk_norm_rope_kv_write(rows, kc, vc, cos, sin, rot_dim=rot, interleaved=interleaved, kv_slot=kv_slot,
                              nh=nh, nkv=nkv, d=d, dv=dv, q_gain=gq.to(DEV), k_gain=gk.to(DEV), eps=1e-5)
    close(rows[:, : (nh + nkv) * d].view(T, nh + nkv, d), want, 2e-5, 1e-5)
    assert torch.equal(rows[:, (nh + nkv) * d:].cpu(), qkv[:, (nh + nkv) * d:])
    pages = table[0].tolist()
    for t in range(T):
        pg, off = pages[t // page], t % page
        close(kc[pg, :, off], want[t, nh:], 2e-5, 1e-5)
        assert torch.equal(vc[pg, :, :, off].cpu(), qkv[t, (nh + nkv) * d:].view(nkv, dv))
