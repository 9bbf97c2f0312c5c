"""Nonetar on the GPU: every mechanism's kernel alone against the plain functions of oracle/nonetar.py, then the engine
(scheduler commit, pages, state slots, run_portions) against the oracle run on each request's whole token list."""

import math

import pytest
import torch

from nonetar_cases import (aligned_config, attention_only_config, engine_config, mixed_config, odd_config, plain_config,
                           random_checkpoint, row_error, row_errors, ssm_only_config)
from oracle import nonetar as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64
F32_TOL, BF16_TOL = 2e-4, 6e-2          # engine logits against the float64 oracle (row_error)
SAME_TOL = 2e-5                         # fp32 engine against itself under another schedule


def _tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def _steps(pieces, slot=0, past=0):
    """Single-request step arrays for consecutive pieces: (start, count, cu_q, past_lens, state_slots, seq_of_token)."""
    at = 0
    for n in pieces:
        yield at, n, _i32([0, n]), _i32([past + at]), _i32([slot]), _i32([0] * n)
        at += n


def _close(got, want, tol):
    scale = float(want.abs().max()) + 1e-30
    assert float((got.double().cpu() - want.double()).abs().max()) <= tol * scale, \
        float((got.double().cpu() - want.double()).abs().max()) / scale


# ------------------------------------------------------------------------------------------------ rows and streams
@pytest.mark.parametrize("width", [6, 7, 96])
def test_embedding_with_sinusoidal_positions(width):
    from byox_vllm_amd import kernels
    torch.manual_seed(0)
    table = torch.randn(11, width)
    ids = torch.tensor([3, 0, 10, 3, 7])
    pos = torch.tensor([0, 1, 777, 4095, 12])
    freq = torch.tensor([math.pow(10000.0, -2.0 * i / width) for i in range((width + 1) // 2)], dtype=F64, device=DEV)
    got = kernels.embed_sinusoid(ids.to(DEV), pos.to(DEV), table.to(DEV), freq, 3)
    want = table[ids].double() + O.sinusoid(4096, width)[pos]
    for s in range(3):
        _close(got[:, s], want, 2e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S", [1, 2, 3, 5])
def test_stream_norm_folds_the_previous_output_in_and_gathers(dtype, S):
    from byox_vllm_amd import kernels
    torch.manual_seed(S)
    T, width, eps = 9, 70, 1e-5
    x = torch.randn(T, S, width)
    delta = torch.randn(T, width + 3)[:, :width]              # a row stride that is not the width
    prev = torch.cat([torch.randn(S), torch.randn(S), torch.randn(S * S)])
    hin = torch.randn(S)
    w = (0.1 * torch.randn(width)).to(dtype)
    mix, out_w = prev[2 * S:].view(S, S).double(), prev[S:2 * S].double()
    new = torch.einsum("st,nsw->ntw", mix, x.double()) + out_w[None, :, None] * delta.double()[:, None, :]
    u = torch.einsum("s,nsw->nw", hin.double(), new)
    want = O.rms(u, eps) * (1.0 + w.double())
    xd = x.to(DEV)
    dd = torch.randn(T, width + 3, device=DEV)
    dd[:, :width] = delta.to(DEV)
    got = kernels.hc_norm(xd, w.to(DEV), eps, hc_in=hin.to(DEV), delta=dd[:, :width], hc_prev=prev.to(DEV))
    _close(got.float(), want, 1e-5 if dtype == torch.float32 else 1e-2)
    _close(xd, new, 1e-6)                                     # the streams took the update
    # fp32 output for a consumer that goes on in fp32; gathered rows leave the streams alone; the plain sum of streams
    xd = x.to(DEV)
    rows = _i32([4, 0, 8])
    got = kernels.hc_norm(xd, w.to(DEV), eps, delta=dd[:, :width], hc_prev=prev.to(DEV), rows_idx=rows,
                          out_dtype=torch.float32)
    want = (O.rms(new.sum(1), eps) * (1.0 + w.double()))[[4, 0, 8]]
    _close(got, want, 1e-5)
    assert torch.equal(xd.cpu(), x)
    # no connection numbers: the output is added to every stream
    got = kernels.hc_norm(xd, w.to(DEV), eps, delta=dd[:, :width], one_plus=False)
    _close(xd, x.double() + delta.double()[:, None, :], 1e-6)
    _close(got.float(), O.rms((x.double() + delta.double()[:, None, :]).sum(1), eps) * w.double(),
           1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("pieces", [[23], [1] * 23, [2, 2, 3, 16], [22, 1], [1, 22]])
def test_token_shift_carries_the_last_row_between_steps(pieces):
    from byox_vllm_amd import kernels
    torch.manual_seed(1)
    width = 37
    h, mu = torch.randn(23, width), torch.rand(width)
    want = O.token_shift(h.double(), mu.double())
    state = torch.full((3, width), 7.0, device=DEV)           # what an earlier request left in the slot must not show
    got = torch.cat([kernels.token_shift(h[a:a + n].to(DEV), mu.to(DEV), state, cu, past, slots, seq_of)
                     for a, n, cu, past, slots, seq_of in _steps(pieces, slot=1)])
    _close(got, want, 1e-6)
    assert torch.equal(state[1].cpu(), h[-1]) and float(state[0].min()) == 7.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_rms_norm(dtype):
    from byox_vllm_amd import kernels
    torch.manual_seed(2)
    x, w = torch.randn(5, 60), torch.randn(60).to(dtype)
    for groups in (1, 3, 4, 60):
        want = O.rms(x.double().view(5, groups, -1), 1e-5).reshape(5, 60) * w.double()
        got = kernels.group_rms_norm_f32(x.to(DEV), w.to(DEV), groups, 1e-5)
        _close(got.float(), want, 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [3, 100])
def test_linear_elementwise_epilogues(dtype, M):
    from byox_vllm_amd import kernels
    torch.manual_seed(3)
    K, N = 72, 50
    x, w = torch.randn(M, K).to(dtype), (torch.randn(N, K) * K ** -0.5).to(dtype)
    p, q = torch.tensor(0.3, dtype=F64), torch.tensor(-0.4, dtype=F64)
    coef = torch.stack([O.softplus(p), 0.5 + O.softplus(q)]).float().to(DEV)
    z = x.double() @ w.double().T
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got = kernels.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32, epilogue=kernels.EPI_ACT, act=kernels.ACT_XIELU,
                         gate=coef)
    _close(got, O.xielu(z, p, q), tol)
    got = kernels.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32, epilogue=kernels.EPI_ACT, act=kernels.ACT_SCALE,
                         cap=0.37)
    _close(got, 0.37 * z, tol)
    got = kernels.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32, epilogue=kernels.EPI_ACT, act=kernels.ACT_GELU_TANH)
    _close(got, O.gelu_tanh(z), tol)


def test_xielu_halves_meet_at_zero():
    z = torch.tensor([-1e-9, 0.0, 1e-9], dtype=F64)
    y = O.xielu(z, torch.tensor(0.7, dtype=F64), torch.tensor(0.2, dtype=F64))
    assert float(y[1]) == 0.0 and abs(float(y[2] - y[0]) / 2e-9 - 0.5) < 1e-6


# ------------------------------------------------------------------------------------------------ convolution, recurrences
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
@pytest.mark.parametrize("pieces", [[30], [1] * 30, [2, 1, 3, 24], [3, 27], [29, 1]])
def test_causal_convolution_in_pieces(taps, pieces):
    from byox_vllm_amd import kernels
    torch.manual_seed(taps)
    C = 70
    x, w, b, xb = torch.randn(30, C + 5), torch.randn(C, taps), torch.randn(C), torch.randn(C)
    # the inputs' own bias is added by the kernel (the product that made x has no epilogue); the slot keeps x + bias
    want = O.silu(O.causal_conv(x[:, 2:2 + C].double() + xb.double(), w.double(), b.double()))
    state = torch.full((2, taps - 1, C), 5.0, device=DEV)
    xd = x.to(DEV)
    got = torch.cat([kernels.causal_conv(xd[a:a + n, 2:2 + C], w.to(DEV), b.to(DEV), state, cu, past, slots, seq_of, act=1,
                                         x_bias=xb.to(DEV))[0]
                     for a, n, cu, past, slots, seq_of in _steps(pieces, slot=1)])
    _close(got, want, 1e-5)
    if taps > 1:
        assert torch.equal(state[1].cpu(), x[30 - (taps - 1):, 2:2 + C] + xb)


def test_causal_convolution_batch_of_unequal_requests_and_both_outputs():
    from byox_vllm_amd import kernels
    torch.manual_seed(9)
    C, taps = 33, 4
    w, b = torch.randn(C, taps).bfloat16(), torch.randn(C).bfloat16()
    xs = [torch.randn(n, C) for n in (7, 1, 2, 12)]
    want = [O.causal_conv(x.double(), w.double(), b.double()) for x in xs]
    state = torch.zeros(5, taps - 1, C, device=DEV)
    # first step: 5 / 1 / 1 / 3 tokens of the four requests, second step the rest of those that have more
    first, second = [5, 1, 1, 3], [2, 0, 1, 9]
    for step, counts, past in ((0, first, [0, 0, 0, 0]), (1, second, first)):
        live = [i for i, n in enumerate(counts) if n]
        rows = torch.cat([xs[i][past[i]:past[i] + counts[i]] for i in live]).to(DEV)
        cu = _i32([0] + torch.tensor([counts[i] for i in live]).cumsum(0).tolist())
        seq_of = _i32([k for k, i in enumerate(live) for _ in range(counts[i])])
        f32, t16 = kernels.causal_conv(rows, w.to(DEV), b.to(DEV), state, cu, _i32([past[i] for i in live]),
                                       _i32([i + 1 for i in live]), seq_of, want_t=True)
        expect = torch.cat([want[i][past[i]:past[i] + counts[i]] for i in live])
        _close(f32, expect, 1e-5)
        assert torch.equal(t16.cpu(), f32.cpu().bfloat16())


def _rglru_inputs(T, C, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(T, C, generator=g), torch.randn(T, 2 * C, generator=g), torch.randn(T, C, generator=g),
            torch.randn(C, generator=g))


def _rglru_plain(u, gates, y, lam, bw):
    T, C = u.shape
    gb = gates.double().view(T, C // bw, 2, bw)
    S = O.gated_linear_recurrence(u.double(), gb[:, :, 0].reshape(T, C), gb[:, :, 1].reshape(T, C), lam.double())
    return S * O.gelu_tanh(y.double())


@pytest.mark.parametrize("C,bw", [(70, 14), (36, 36), (256, 64)])
@pytest.mark.parametrize("pieces", [[40], [1] * 40, [2, 2, 35, 1]])
def test_gated_linear_recurrence_in_pieces(C, bw, pieces):
    from byox_vllm_amd import kernels
    u, gates, y, lam = _rglru_inputs(40, C, C)
    want = 0.7 * _rglru_plain(u, gates, y, lam, bw)
    state = torch.full((3, C), 9.0, device=DEV)
    out = torch.zeros(40, C + 4, device=DEV)
    ud, gd, yd = u.to(DEV), gates.to(DEV), y.to(DEV)
    for a, n, cu, past, slots, _ in _steps(pieces, slot=2):
        kernels.rglru_scan(ud[a:a + n], gd[a:a + n], yd[a:a + n], lam.to(DEV), state, cu, past, slots, bw,
                           out[a:a + n, 4:], out_scale=0.7)
    _close(out[:, 4:], want, 1e-5)
    assert float(out[:, :4].abs().max()) == 0.0


def test_gated_linear_recurrence_keeps_an_old_input_under_a_slow_decay():
    """One channel is given a decay close to one and a single large input 300 tokens back: it must still be there, and
    its neighbour with a fast decay must have lost it."""
    from byox_vllm_amd import kernels
    T, C = 320, 64
    u, gates, y, lam = torch.zeros(T, C), torch.zeros(T, 2 * C), torch.ones(T, C), torch.zeros(C)
    u[10] = 100.0
    lam[0], lam[1] = -12.0, 3.0
    want = _rglru_plain(u, gates, y, lam, C)
    assert abs(float(want[-1, 0])) > 0.01 and abs(float(want[-1, 1])) < 1e-30
    state = torch.zeros(1, C, device=DEV)
    out = torch.zeros(T, C, device=DEV)
    for a, n, cu, past, slots, _ in _steps([100, 1, 1, 218], slot=0):
        kernels.rglru_scan(u[a:a + n].to(DEV), gates[a:a + n].to(DEV), y[a:a + n].to(DEV), lam.to(DEV), state, cu, past,
                           slots, C, out[a:a + n])
    _close(out[-1, :2], want[-1, :2], 1e-4)
    _close(out, want, 1e-4)


def _ssd_inputs(T, H, G, P, N, seed):
    g = torch.Generator().manual_seed(seed)
    xbc = torch.randn(T, H * P + 2 * G * N, generator=g)
    return (xbc, torch.randn(T, H * P, generator=g), torch.randn(T, H, generator=g), torch.randn(H, generator=g) * 0.5,
            torch.randn(H, generator=g) * 0.5 - 1.0, torch.randn(H, generator=g))


def _ssd_plain(xbc, z, dt, dt_bias, A_log, D, H, G, P, N):
    T = xbc.shape[0]
    x = xbc[:, :H * P].double().view(T, H, P)
    B = xbc[:, H * P:H * P + G * N].double().view(T, G, N).repeat_interleave(H // G, 1)
    C = xbc[:, H * P + G * N:].double().view(T, G, N).repeat_interleave(H // G, 1)
    y = O.ssd_scan(x, B, C, O.softplus(dt.double() + dt_bias.double()), A_log.double(), D.double())
    return y.reshape(T, H * P) * O.silu(z.double())


@pytest.mark.parametrize("H,G,P,N", [(4, 1, 16, 24), (6, 3, 8, 12), (2, 2, 10, 12), (1, 1, 64, 128), (3, 1, 130, 5)])
@pytest.mark.parametrize("pieces", [[36], [1] * 36, [2, 30, 1, 3]])
def test_state_space_scan_in_pieces(H, G, P, N, pieces):
    from byox_vllm_amd import kernels
    xbc, z, dt, dt_bias, A_log, D = _ssd_inputs(36, H, G, P, N, H * 10 + N)
    want = _ssd_plain(xbc, z, dt, dt_bias, A_log, D, H, G, P, N)
    state = torch.full((2, H, N, P), 3.0, device=DEV)
    got = torch.cat([kernels.ssd_scan(xbc[a:a + n].to(DEV), z[a:a + n].to(DEV), dt[a:a + n].to(DEV), dt_bias.to(DEV),
                                      A_log.to(DEV), D.to(DEV), state, cu, past, slots, H, G, N, P)
                     for a, n, cu, past, slots, _ in _steps(pieces, slot=1)])
    _close(got, want, 2e-5)


@pytest.mark.parametrize("pieces", [[700], [300, 400], [257, 3, 440], [40, 660]])
def test_state_space_scan_long_prompts_are_walked_in_parallel_runs(pieces):
    """From 256 tokens per request on, a prompt is cut into runs whose end states meet through a workspace: same
    numbers as the plain walk, whatever the cut, also beside a short request in the same launch."""
    from byox_vllm_amd import kernels
    H, G, P, N = 3, 1, 16, 24
    xbc, z, dt, dt_bias, A_log, D = _ssd_inputs(700, H, G, P, N, 5)
    short = _ssd_inputs(5, H, G, P, N, 6)[:3]
    want = _ssd_plain(xbc, z, dt, dt_bias, A_log, D, H, G, P, N)
    want_short = _ssd_plain(*short, dt_bias, A_log, D, H, G, P, N)
    state = torch.full((3, H, N, P), 3.0, device=DEV)
    params = [t.to(DEV) for t in (dt_bias, A_log, D)]
    got, at = [], 0
    for k, n in enumerate(pieces):
        rows = [xbc[at:at + n], z[at:at + n], dt[at:at + n]]
        beside = k == 0                                   # the short request rides along in the first step
        if beside:
            rows = [torch.cat([s_, r]) for s_, r in zip(short, rows)]
        cu = _i32([0, 5, 5 + n] if beside else [0, n])
        out = kernels.ssd_scan(*[r.to(DEV) for r in rows], *params, state, cu, _i32([0, at] if beside else [at]),
                               _i32([2, 1] if beside else [1]), H, G, N, P, max_q=n)
        if beside:
            _close(out[:5], want_short, 2e-5)
            out = out[5:]
        got.append(out)
        at += n
    _close(torch.cat(got), want, 5e-5)


def test_state_space_scan_batch_and_reused_slot():
    """Two requests side by side, then a third one in the slot the first has left: it must start from zero."""
    from byox_vllm_amd import kernels
    H, G, P, N = 4, 2, 8, 16
    a, b, c = (_ssd_inputs(n, H, G, P, N, s) for n, s in ((9, 1), (4, 2), (6, 3)))
    params = _ssd_inputs(1, H, G, P, N, 7)[3:]
    plain = [_ssd_plain(*r[:3], *params, H, G, P, N) for r in (a, b, c)]
    state = torch.zeros(3, H, N, P, device=DEV)
    dev = [p.to(DEV) for p in params]

    def run(reqs, slots, past):
        rows = [torch.cat([r[k] for r in reqs]).to(DEV) for k in range(3)]
        cu = _i32([0] + torch.tensor([r[0].shape[0] for r in reqs]).cumsum(0).tolist())
        return kernels.ssd_scan(*rows, *dev, state, cu, _i32(past), _i32(slots), H, G, N, P)
    _close(run([a, b], [2, 0], [0, 0]), torch.cat(plain[:2]), 2e-5)
    _close(run([c], [2], [0]), plain[2], 2e-5)


# ------------------------------------------------------------------------------------------------ attention
def _attention_plain(q, k, v, H, G, scale, temp, softcap, window, eps, qn, kn):
    """Whole-sequence result from raw projections: [T, H * dv] in float64."""
    T = q.shape[0]
    d, dv = q.shape[1] // H, v.shape[1] // G
    qh = O.rms(q.double().view(T, H, d), eps) * qn.double()
    kh = O.rms(k.double().view(T, G, d), eps) * kn.double()
    kh, vh = kh.repeat_interleave(H // G, 1), v.double().view(T, G, dv).repeat_interleave(H // G, 1)
    return O.windowed_attention(qh, kh, vh, scale, temp.double(), softcap, window).reshape(T, H * dv)


def _paged_attention(proj, offs, pieces, H, G, d, dv, scale, temp, softcap, window, eps, qn, kn, dtype, block, seed=0,
                     out_scale=1.0):
    """The two kernels over one request cut into ``pieces``, on scattered pages."""
    from byox_vllm_amd import kernels
    T = proj.shape[0]
    nblocks = -(-T // block)
    g = torch.Generator().manual_seed(seed)
    pages = torch.randperm(nblocks + 3, generator=g)[:nblocks].tolist()
    cache = torch.full(((nblocks + 3) * block, G * (d + dv)), float("nan"), dtype=dtype, device=DEV)
    table = _i32([pages])
    out = torch.zeros(T, H * dv + 2, dtype=dtype, device=DEV)
    pd = proj.to(DEV)
    for a, n, cu, past, _, seq_of in _steps(pieces):
        slots = _i32([pages[p // block] * block + p % block for p in range(a, a + n)])
        q = kernels.qk_norm_store(pd[a:a + n], offs, qn.to(DEV).to(dtype), kn.to(DEV).to(dtype), temp.to(DEV).to(dtype),
                                  scale, eps, slots, cache, H, G, d, dv)
        kernels.window_attn(q, cache, table, cu, past, seq_of, n, H, G, d, dv, block, window, softcap, out[a:a + n, 2:],
                            out_scale)
    assert float(out[:, :2].float().abs().max()) == 0.0
    return out[:, 2:].float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,window,block", [(6, 2, 16, 24, 9, 16), (1, 1, 20, 12, 5, 16), (3, 1, 12, 6, 0, 32),
                                                   (4, 4, 64, 32, 70, 64), (8, 2, 32, 16, 16, 16), (2, 1, 128, 64, 33, 16)])
def test_window_attention_prompt_pieces_and_single_tokens(dtype, H, G, d, dv, window, block):
    torch.manual_seed(H * 100 + d)
    T, eps = 90, 1e-5
    proj = torch.randn(T, 3 + H * d + G * d + G * dv)
    offs = (3, 3 + H * d, 3 + H * d + G * d)
    qn, kn = (1.0 + 0.2 * torch.randn(d)).bfloat16().float(), (1.0 + 0.2 * torch.randn(d)).bfloat16().float()
    temp = (0.5 + torch.rand(H)).bfloat16().float()
    q, k, v = proj[:, 3:offs[1]], proj[:, offs[1]:offs[2]], proj[:, offs[2]:]
    for softcap in (None, 2.0):
        want = 1.3 * _attention_plain(q, k, v, H, G, 0.4, temp, softcap, window, eps, qn, kn)
        for pieces in ([T], [50] + [1] * 40, [2, 3, 16, 1, 17, 31, 2, 18]):
            got = _paged_attention(proj, offs, pieces, H, G, d, dv, 0.4, temp, softcap, window, eps, qn, kn, dtype, block,
                                   out_scale=1.3)
            _close(got, want, 2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pieces", [[200], [120, 80], [199, 1], [150] + [1] * 50, [64, 64, 64, 8]])
def test_window_attention_edges_stand_out(pieces, dtype):
    """Random keys would hide a window that is one token off.  Here every key is orthogonal to the last query except
    two: the one just inside the window and the one just outside carry large, different values.  The result must be
    the inside key's value and show nothing of the outside key's; the same for a far key under an unbounded window."""
    H = G = 1
    d, dv, T, eps, block = 16, 8, 200, 1e-6, 64
    for window, inside, outside in ((70, T - 70, T - 71), (64, T - 64, T - 65), (1, T - 1, T - 2), (0, 0, None)):
        q, k, v = torch.zeros(T, d), torch.zeros(T, d), torch.zeros(T, dv)
        k[:, 1] = 1.0                                   # every key is the unit vector e1 after its norm ...
        q[-1, 0] = 1.0                                  # ... and the last query e0: score 0
        k[inside] = 0.0
        k[inside, 0] = 1.0                              # the inside key matches the query
        v[inside, 0] = 5.0
        if outside is not None:
            k[outside] = 0.0
            k[outside, 0] = 1.0
            v[outside, 1] = 7.0
        proj = torch.cat([q, k, v], 1)
        ones, temp = torch.ones(d), torch.ones(H)
        scale = 40.0 * d ** -0.5 + (T * 2.0 ** -8 if window == 0 else 0.0)     # dwarfs the distance penalty
        want = _attention_plain(q, k, v, H, G, scale, temp, None, window, eps, ones, ones)
        assert abs(float(want[-1, 0]) - 5.0) < 1e-3 and abs(float(want[-1, 1])) < 1e-9
        got = _paged_attention(proj, (0, d, 2 * d), pieces, H, G, d, dv, scale, temp, None, window, eps, ones, ones, dtype,
                               block, seed=window)
        assert abs(float(got[-1, 0]) - 5.0) < 0.05 and abs(float(got[-1, 1])) < 1e-6, (window, got[-1, :2])


def test_distance_penalty_and_soft_cap_are_applied_in_this_order():
    """Two equal keys at different distances: only the distance term separates them, by slope * distance, and it is
    taken off AFTER the cap (a capped score cannot hide it)."""
    H, d, dv, T, eps = 2, 8, 4, 6, 1e-6
    q, k, v = torch.zeros(T, H * d), torch.zeros(T, d), torch.zeros(T, dv)
    q[:, 0] = q[:, d] = 1.0
    k[:, 0] = 1.0
    v[:, 0] = torch.arange(T).float()
    ones, temp = torch.ones(d), torch.tensor([1.0, 0.5])
    for softcap in (None, 0.5):
        want = _attention_plain(q, k, v, H, 1, 3.0, temp, softcap, 4, eps, ones, ones)
        slope = torch.tensor([2.0 ** -4, 2.0 ** -8], dtype=F64)
        for h in range(H):
            wts = torch.softmax(-slope[h] * torch.arange(4, dtype=F64), 0)        # keys at distances 0..3 from the last query
            assert abs(float(want[-1, h * dv]) - float((wts * torch.tensor([5.0, 4.0, 3.0, 2.0], dtype=F64)).sum())) < 1e-9
        got = _paged_attention(torch.cat([q, k, v], 1), (0, H * d, H * d + d), [4, 1, 1], H, 1, d, dv, 3.0, temp, softcap, 4,
                               eps, ones, ones, torch.float32, 16)
        _close(got, want, 1e-5)


def test_window_attention_batch_of_unequal_requests():
    """A prompt piece, a single decoded token with a long past and a two-token request in one launch."""
    from byox_vllm_amd import kernels
    torch.manual_seed(4)
    H, G, d, dv, window, block, eps = 4, 2, 16, 8, 20, 16, 1e-5
    lens, past = [37, 65, 2], [0, 64, 0]                  # request 1 already holds 64 tokens
    offs = (0, H * d, H * d + G * d)
    projs = [torch.randn(n, H * d + G * d + G * dv) for n in lens]
    ones, temp = torch.ones(d), torch.ones(H)
    want = [_attention_plain(p[:, :offs[1]], p[:, offs[1]:offs[2]], p[:, offs[2]:], H, G, 0.3, temp, 4.0, window, eps, ones, ones)
            for p in projs]
    cache = torch.zeros(12 * block, G * (d + dv), device=DEV)
    tables = _i32([[3, 7, 9, 0, 0], [5, 1, 2, 4, 11], [8, 0, 0, 0, 0]])
    row = lambda r, p: int(tables[r, p // block]) * block + p % block       # noqa: E731
    # request 1's first 64 tokens in a step of its own
    q = kernels.qk_norm_store(projs[1][:64].to(DEV), offs, ones.to(DEV), ones.to(DEV), temp.to(DEV), 0.3, eps,
                              _i32([row(1, p) for p in range(64)]), cache, H, G, d, dv)
    out = torch.zeros(64, H * dv, device=DEV)
    kernels.window_attn(q, cache, tables[1:2].contiguous(), _i32([0, 64]), _i32([0]), _i32([0] * 64), 64, H, G, d, dv, block,
                        window, 4.0, out)
    _close(out, want[1][:64], 2e-5)
    rows = torch.cat([projs[0], projs[1][64:], projs[2]]).to(DEV)
    slots = _i32([row(0, p) for p in range(37)] + [row(1, 64)] + [row(2, p) for p in range(2)])
    q = kernels.qk_norm_store(rows, offs, ones.to(DEV), ones.to(DEV), temp.to(DEV), 0.3, eps, slots, cache, H, G, d, dv)
    out = torch.zeros(40, H * dv, device=DEV)
    kernels.window_attn(q, cache, tables, _i32([0, 37, 38, 40]), _i32(past), _i32([0] * 37 + [1] + [2] * 2), 37, H, G, d, dv,
                        block, window, 4.0, out)
    _close(out, torch.cat([want[0], want[1][64:], want[2]]), 2e-5)


# ------------------------------------------------------------------------------------------------ the engine
class Engine:
    """ModelRunner + Scheduler of one configuration, replaying schedules of (request name, token count) steps."""

    def __init__(self, cfg_json, weights, dtype, blocks=16, slots=4, block_size=16):
        from byox_vllm_amd.engine.model_runner import ModelRunner
        from byox_vllm_amd.engine.scheduler import Scheduler
        self.config = engine_config(cfg_json, weights, dtype, blocks=blocks, slots=slots, block_size=block_size)
        self.runner = ModelRunner(self.config, 0, None)
        self.scheduler = Scheduler(self.config)
        self.block_size = block_size

    def replay(self, requests: dict, schedule: list):
        """requests: name -> token list; schedule: steps of [(name, count)].  Logits of every position, per request.
        A request ends (and gives back pages and slot) with the step that brings its last token."""
        from byox_vllm_amd.engine.sequence import Sequence
        live, at, out = {}, {n: 0 for n in requests}, {n: [] for n in requests}
        for step in schedule:
            plan = []
            for name, count in step:
                piece = requests[name][at[name]: at[name] + count]
                if name not in live:
                    live[name] = Sequence(piece, self.block_size)
                    self.scheduler.add(live[name])
                else:
                    live[name].extend_tokens(piece)
                plan.append((live[name], count))
                at[name] += count
            self.scheduler.commit(plan)
            logits = self.runner.run_portions(plan, want=[list(range(c)) for _, c in plan]).cpu()
            self.scheduler.advance(plan, [None] * len(plan))
            row = 0
            for name, count in step:
                out[name].append(logits[row: row + count])
                row += count
                if at[name] == len(requests[name]):
                    self.scheduler.finish(live.pop(name))
        return {n: torch.cat(v) for n, v in out.items()}


CASES = {"mixed": mixed_config, "odd": odd_config, "plain": plain_config, "aligned": aligned_config,
         "ssm_only": ssm_only_config, "attention_only": attention_only_config}


@pytest.fixture(scope="module", params=[(n, dt) for n in CASES for dt in (torch.float32, torch.bfloat16)
                                        if dt == torch.float32 or n not in ("ssm_only",)],
                ids=lambda p: f"{p[0]}-{str(p[1])[6:]}")
def setup(request):
    name, dtype = request.param
    cfg = CASES[name]()
    weights = random_checkpoint(cfg, seed=11)
    torch.manual_seed(99)
    reqs = {"a": torch.randint(0, cfg["vocab"], (83,)).tolist(), "b": torch.randint(0, cfg["vocab"], (31,)).tolist(),
            "c": torch.randint(0, cfg["vocab"], (2,)).tolist(), "d": torch.randint(0, cfg["vocab"], (50,)).tolist()}
    want = {n: O.forward(cfg, weights, t).float() for n, t in reqs.items()}
    engine = Engine(cfg, weights, dtype, blocks=12, slots=3)
    whole = engine.replay(reqs, [[(n, len(t))] for n, t in reqs.items()])
    return cfg, weights, dtype, reqs, want, engine, whole


def _check(setup, got):
    cfg, weights, dtype, reqs, want, engine, whole = setup
    for n in got:
        assert row_error(got[n], want[n]) < _tol(dtype), (n, row_error(got[n], want[n]))
        if dtype == torch.float32:
            assert row_error(got[n], whole[n]) < SAME_TOL, n


def test_whole_prompts_match_the_oracle(setup):
    _check(setup, setup[6])


def test_every_layer_matches_the_oracle(setup):
    """The sum of the streams after every layer, for one request in one step (fp32 only: it is the sharp comparison)."""
    cfg, weights, dtype, reqs, want, engine, whole = setup
    if dtype != torch.float32:
        pytest.skip("layer by layer in fp32 only")
    from byox_vllm_amd.engine.sequence import Sequence
    trace, plain = [], []
    O.forward(cfg, weights, reqs["b"], trace=plain)
    model = engine.runner.model
    forward = model.forward
    model.forward = lambda ids, pos: forward(ids, pos, trace=trace)
    try:
        seq = Sequence(reqs["b"], engine.block_size)
        engine.scheduler.add(seq)
        plan = [(seq, len(reqs["b"]))]
        engine.scheduler.commit(plan)
        engine.runner.run_portions(plan, want=[[0]])
        engine.scheduler.finish(seq)
    finally:
        model.forward = forward
    assert len(trace) == len(plain) == len(cfg["layers"])
    for i, (got, ref) in enumerate(zip(trace, plain)):
        _close(got, ref, 2e-5)


def test_prompt_then_token_by_token(setup):
    reqs = setup[3]
    # the decoded stretch is longer than every window and crosses page borders
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", 20)]] + [[("a", 1)]] * 63))
    _check(setup, setup[5].replay({"b": reqs["b"]}, [[("b", 1)]] * 31))           # from the very first token on


def test_portions_of_many_sizes(setup):
    reqs = setup[3]
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", n)] for n in (2, 2, 3, 9, 16, 1, 17, 2, 15, 14, 2)]))
    _check(setup, setup[5].replay({"d": reqs["d"]}, [[("d", n)] for n in (15, 1, 16, 2, 16)]))


def test_mixed_batches_reuse_pages_and_slots(setup):
    """Three slots, twelve pages of sixteen tokens: four requests only fit because the finished ones give theirs back.
    Prompt pieces run beside single tokens; requests sit out steps."""
    reqs = setup[3]
    schedule = [[("a", 30), ("b", 5)], [("a", 1), ("b", 20), ("c", 2)], [("a", 2), ("b", 1)], [("b", 1), ("d", 7), ("a", 1)],
                [("a", 40), ("d", 1), ("b", 4)], [("d", 30)], [("a", 1), ("d", 1)], [("a", 8), ("d", 11)]]
    _check(setup, setup[5].replay(reqs, schedule))
    # the same requests again, in slots and pages that the first pass has used
    _check(setup, setup[5].replay(reqs, [[("d", 50), ("c", 1)], [("c", 1), ("b", 31)], [("a", 83)]]))


def test_greedy_generation_through_the_engine(setup):
    """LLM.generate (scheduler's own portion policy, sampler at temperature 0) against the oracle's greedy run."""
    cfg, weights, dtype, reqs, want, engine, whole = setup
    from byox_vllm_amd import LLM, SamplingParams
    conf = engine_config(cfg, weights, dtype, blocks=12, slots=3)
    llm = LLM("synthetic", hf_config=conf.hf_config, state_dict=weights, kvcache_block_size=16, num_kvcache_blocks=12,
              max_num_seqs=3, num_state_slots=3, enforce_eager=True, max_num_batched_tokens=48, max_model_len=1 << 20)
    prompts = [reqs["b"], reqs["c"], reqs["d"][:20], reqs["a"][:40]]
    steps = 12
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True), use_tqdm=False)
    llm._exit()
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for k, tok in enumerate(out["token_ids"]):
            logits = O.forward(cfg, weights, tokens)[-1]
            best = logits.max().item()
            # the engine's choice is the oracle's argmax, or lies inside the rounding of the engine's dtype
            assert best - logits[tok].item() <= (1e-3 if dtype == torch.float32 else 0.25), (k, tok)
            tokens.append(tok)
        assert len(out["token_ids"]) == steps


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps replayed from hipGraphs (padded batches, the spare state slot, one staging copy) give the tokens of
    the eager engine, step after step, with prompt portions running eagerly between the replays."""
    from byox_vllm_amd import LLM, SamplingParams
    cfg = mixed_config()
    weights = random_checkpoint(cfg, seed=21)
    torch.manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab"], (n,)).tolist() for n in (37, 3, 18, 25, 9)]
    params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in (30, 41, 12, 25, 33)]
    outs = []
    for eager in (True, False):
        conf = engine_config(cfg, weights, dtype, blocks=24, slots=4)
        llm = LLM("synthetic", hf_config=conf.hf_config, state_dict=weights, kvcache_block_size=16, num_kvcache_blocks=24,
                  max_num_seqs=4, num_state_slots=4, enforce_eager=eager, max_num_batched_tokens=32, max_model_len=128)
        assert bool(llm.model_runner.graphs) == (not eager)
        outs.append([o["token_ids"] for o in llm.generate(prompts, params, use_tqdm=False)])
        llm._exit()
    assert outs[0] == outs[1]
    assert [len(t) for t in outs[0]] == [30, 41, 12, 25, 33]


def test_command_line_generation_and_trace_replay_from_a_model_folder(tmp_path):
    """A model folder (config.json + model.safetensors in bf16) through the two command-line entry points, each in a
    process of its own: `python -m byox_vllm_amd generate` against the oracle's greedy continuation, bin/trace_run
    against the oracle's logits for a replayed schedule with pieces, a pause and a request that ends early."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = aligned_config()
    weights = random_checkpoint(cfg, seed=31)
    model = tmp_path / "model"
    model.mkdir()
    with open(model / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, str(model / "model.safetensors"))
    torch.manual_seed(3)
    a = torch.randint(0, cfg["vocab"], (70,)).tolist()
    b = torch.randint(0, cfg["vocab"], (9,)).tolist()

    run = subprocess.run([sys.executable, "-m", "byox_vllm_amd", "generate", "--model", str(model), "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, b)), "--max-tokens", "6", "--block-size", "16", "--eager"],
                         cwd=root, capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-3000:]
    line = json.loads([ln for ln in run.stdout.splitlines() if ln.startswith("{")][0])
    tokens = list(b)
    for tok in line["token_ids"]:
        logits = O.forward(cfg, weights, tokens)[-1]
        assert logits.max().item() - logits[tok].item() <= 1e-3
        tokens.append(tok)
    assert len(line["token_ids"]) == 6

    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[40:41], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[41:], "want": [0, 28]}, {"id": "c", "tokens": b, "want": [8]}], "end": ["a", "c"]}]
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        out = tmp_path / ("out_" + dtype)
        run = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", dtype, "--out", str(out),
                              "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root,
                             capture_output=True, text=True, timeout=600)
        assert run.returncode == 0, run.stderr[-3000:]
        assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
        wa, wb = O.forward(cfg, weights, a).float(), O.forward(cfg, weights, b).float()
        expect = {0: wa[[0, 39]], 1: wa[[40]], 2: wb[[8]], 3: torch.cat([wa[[41, 69]], wb[[8]]])}
        for i, want in expect.items():
            got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert got.shape == want.shape and row_error(got, want) < tol, (dtype, i)
    assert row_errors(wa, wa).max() == 0
