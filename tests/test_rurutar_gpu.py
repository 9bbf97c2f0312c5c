"""Rurutar on the GPU: every mechanism's kernel alone against plain PyTorch, then the engine (scheduler commit, pages,
state slots, run_portions) against oracle/rurutar.py run on each request's whole token list."""

import math

import pytest
import torch

from oracle import rurutar as O
from rurutar_cases import aligned_config, assert_rows_close, engine_config, mixed_config, odd_config, row_error

pytestmark = pytest.mark.gpu
DEV = "cuda"
F32_TOL, BF16_TOL = 2e-4, 6e-2          # engine logits against the float64 oracle (row_error)
SAME_TOL = 2e-5                         # fp32 engine against itself under another schedule


def _tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


# ------------------------------------------------------------------------------------------------ nv_linear
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (70, 130, 100), (3, 64, 256), (65, 16, 24), (130, 3, 40)])
def test_linear_any_shape(dtype, M, N, K):
    from byox_vllm_amd import kernels
    torch.manual_seed(M * 1000 + N)
    x, w, b = torch.randn(M, K).to(dtype), torch.randn(N, K).to(dtype), torch.randn(N).to(dtype)
    want = x.double() @ w.double().T + b.double()
    got = kernels.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=torch.float32).cpu()
    tol = 1e-5 if dtype == torch.float32 else 1e-5          # bf16 operands are exact, accumulation is fp32
    assert torch.allclose(got.double(), want, rtol=tol, atol=tol * K ** 0.5)
    got16 = kernels.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=torch.bfloat16).cpu()
    assert torch.allclose(got16.double(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_strided_input_and_epilogues(dtype):
    from byox_vllm_amd import kernels
    torch.manual_seed(1)
    M, K, N = 37, 44, 21
    wide = torch.randn(M, K + 13).to(dtype)
    x = wide[:, 5:5 + K]
    w = torch.randn(2 * N, K).to(dtype)
    g, u = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    for act, fn in ((kernels.ACT_SILU, O.silu), (kernels.ACT_GELU_TANH, O.gelu_tanh)):
        got = kernels.linear(wide.to(DEV)[:, 5:5 + K], w.to(DEV), epilogue=kernels.EPI_GLU, act=act,
                             out_dtype=torch.float32).cpu()
        assert torch.allclose(got.double(), fn(g) * u, rtol=1e-4, atol=1e-4)
    got = kernels.linear(wide.to(DEV)[:, 5:5 + K], w.to(DEV), epilogue=kernels.EPI_SOFTCAP, cap=3.0,
                         out_dtype=torch.float32).cpu()
    assert torch.allclose(got.double(), 3.0 * torch.tanh(torch.cat([g, u], 1) / 3.0), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_per_head_batches_and_row_gate(dtype):
    from byox_vllm_amd import kernels
    torch.manual_seed(2)
    T, H, K, N = 19, 3, 20, 10
    x = torch.randn(T, H * (K + 4)).to(dtype)          # per head K used columns followed by 4 unused ones
    w = torch.randn(H, N, K).to(dtype)
    gate = torch.randn(T, H + 2)
    want = torch.stack([x.double().view(T, H, K + 4)[:, h, :K] @ w[h].double().T for h in range(H)], 1)
    want = want * torch.sigmoid(gate.double()[:, 2:, None])
    out = torch.zeros(T, H * N, dtype=torch.float32, device=DEV)
    gd = gate.to(DEV)
    kernels.linear(x.to(DEV), w.to(DEV), out=out, out_dtype=torch.float32, batch=H, a_batch_stride=K + 4,
                   w_batch_stride=N * K, out_batch_stride=N, n=N, epilogue=kernels.EPI_ROW_GATE, gate=gd[:, 2:],
                   gate_stride=gd.stride(0))
    assert torch.allclose(out.cpu().double().view(T, H, N), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_groups_over_gathered_rows(dtype):
    """One weight per group, groups of unequal size (one empty, one larger than a tile), rows gathered by index."""
    from byox_vllm_amd import kernels
    torch.manual_seed(3)
    T, K, N, sizes = 50, 24, 9, [0, 70, 3, 27]
    E, total = len(sizes), sum(sizes)
    x, w = torch.randn(T, K).to(dtype), torch.randn(E, N, K).to(dtype)
    rows = torch.randint(0, T, (total,), dtype=torch.int32)
    offsets = torch.tensor([0] + torch.tensor(sizes).cumsum(0).tolist(), dtype=torch.int32)
    got = kernels.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32, rows=total, a_rows=rows.to(DEV), batch=E,
                         w_batch_stride=N * K, group_offsets=offsets.to(DEV), max_group_rows=max(sizes)).cpu()
    for e in range(E):
        lo, hi = offsets[e], offsets[e + 1]
        want = x.double()[rows[lo:hi].long()] @ w[e].double().T
        assert torch.allclose(got[lo:hi].double(), want, rtol=1e-4, atol=1e-4), e


# ------------------------------------------------------------------------------------------------ row kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dynamic_tanh_add_and_gather(dtype):
    from byox_vllm_amd import kernels
    torch.manual_seed(4)
    T, n = 11, 52
    x, delta = torch.randn(T, n) * 2, torch.randn(T, n)
    w, b, alpha = torch.randn(n).to(dtype), torch.randn(n).to(dtype), torch.tensor([0.7])
    xd = x.to(DEV).clone()
    got = kernels.dyt_norm(xd, alpha.to(DEV), w.to(DEV), b.to(DEV), delta=delta.to(DEV)).cpu()
    s = (x + delta).double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(xd.cpu(), x + delta)                       # the residual was updated in place
    assert torch.allclose(got.double(), O.dynamic_tanh(s, w.double(), b.double(), 0.7), rtol=tol, atol=tol)
    idx = torch.tensor([9, 0, 3], dtype=torch.int32)
    xd = x.to(DEV).clone()
    got = kernels.dyt_norm(xd, alpha.to(DEV), w.to(DEV), b.to(DEV), delta=delta.to(DEV), rows_idx=idx.to(DEV)).cpu()
    assert torch.equal(xd.cpu(), x)                                  # gathered rows leave the residual alone
    assert torch.allclose(got.double(), O.dynamic_tanh(s[idx.long()], w.double(), b.double(), 0.7), rtol=tol, atol=tol)


def test_rms_norm_of_a_column_slice_and_scaled_embedding():
    from byox_vllm_amd import kernels
    torch.manual_seed(5)
    wide, w = torch.randn(9, 70), torch.randn(33)
    got = kernels.rms_norm_f32(wide.to(DEV)[:, 20:53], w.to(DEV), 1e-5).cpu()
    assert torch.allclose(got.double(), O.rms_norm(wide[:, 20:53].double(), w.double(), 1e-5), rtol=1e-5, atol=1e-5)
    table = torch.randn(13, 20).to(torch.bfloat16)
    ids = torch.tensor([12, 0, 5, 5], dtype=torch.int64)
    got = kernels.embed_scale(ids.to(DEV), table.to(DEV), 0.25).cpu()
    assert torch.equal(got, table[ids].float() * 0.25)


# ------------------------------------------------------------------------------------------------ gated linear attention
def _gla_inputs(T, H, d, dv, seed, decay_logit=2.0):
    g = torch.Generator().manual_seed(seed)
    proj = torch.randn(T, 2 * H * d + 2 * H * dv + 3, generator=g)        # q | k | 3 unused | v | g
    z = decay_logit + torch.randn(T, H * d, generator=g)
    return proj, z, (0, H * d, 2 * H * d + 3, 2 * H * d + 3 + H * dv)


def _gla_oracle(proj, z, offs, H, d, dv, tau, norm_w, eps):
    T = proj.shape[0]
    q = proj[:, offs[0]: offs[0] + H * d].double().view(T, H, d) / math.sqrt(d)
    k = proj[:, offs[1]: offs[1] + H * d].double().view(T, H, d)
    v = proj[:, offs[2]: offs[2] + H * dv].double().view(T, H, dv)
    gate = proj[:, offs[3]: offs[3] + H * dv].double()
    o = O.gla_recurrence(q, k, v, torch.sigmoid(z.double()).pow(1 / tau).view(T, H, d))
    return O.rms_norm(o, norm_w.double(), eps).reshape(T, H * dv) * O.silu(gate)


def _gla_run(proj, z, offs, pieces, slot, state, H, d, dv, tau, norm_w, eps):
    """One request stepped through ``pieces`` (token counts) in state slot ``slot``."""
    from byox_vllm_amd import kernels
    outs, at = [], 0
    for n in pieces:
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
        outs.append(kernels.gla_recurrent(proj[at:at + n].to(DEV), offs, z[at:at + n].to(DEV), state, i32([0, n]),
                                          i32([at]), i32([slot]), norm_w.to(DEV), H, d, dv, tau, d ** -0.5, eps).cpu())
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("H,d,dv", [(2, 16, 24), (1, 20, 12), (3, 8, 40), (2, 64, 64), (1, 130, 8)])
def test_gla_pieces_equal_whole_and_oracle(H, d, dv):
    T, tau, eps = 37, 5.0, 1e-5
    proj, z, offs = _gla_inputs(T, H, d, dv, seed=H * 100 + d)
    norm_w = torch.randn(dv)
    want = _gla_oracle(proj, z, offs, H, d, dv, tau, norm_w, eps)
    state = torch.full((3, H, d, dv), float("nan"), device=DEV)         # slots hold rubbish until a request starts
    whole = _gla_run(proj, z, offs, [T], 1, state, H, d, dv, tau, norm_w, eps)
    assert torch.allclose(whole.double(), want, rtol=2e-4, atol=2e-4)
    for pieces in ([2] + [1] * 35, [5, 2, 13, 2, 15], [1] * T):
        got = _gla_run(proj, z, offs, pieces, 2, state, H, d, dv, tau, norm_w, eps)      # slot 2 is used again each time
        assert torch.allclose(got, whole, rtol=1e-5, atol=1e-5), pieces


def test_gla_far_key_survives_hundreds_of_tokens():
    """Decay close to one: a key written at token 3 is what token 400's query finds.  The value read back must be the
    far token's value scaled by the accumulated decay, through a prompt piece followed by single tokens."""
    H, d, dv, T, tau = 1, 8, 8, 401, 64.0
    proj = torch.zeros(T, 2 * d + 2 * dv)
    z = torch.full((T, d), 6.0)
    offs = (0, d, 2 * d, 2 * d + dv)
    proj[3, d] = 5.0                       # key channel 0 at token 3
    proj[3, 2 * d: 2 * d + dv] = torch.arange(1, dv + 1).float()
    proj[400, 0] = 4.0                     # query channel 0 at the last token
    proj[:, 2 * d + dv:] = 1.0             # gates
    norm_w = torch.ones(dv)
    want = _gla_oracle(proj, z, offs, H, d, dv, tau, norm_w, 1e-6)
    state = torch.zeros(1, H, d, dv, device=DEV)
    got = _gla_run(proj, z, offs, [300] + [1] * 101, 0, state, H, d, dv, tau, norm_w, 1e-6)
    assert want[400].abs().max() > 0.1                                   # the far key is visible in the oracle
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-5)


def test_gla_batch_of_unequal_requests():
    from byox_vllm_amd import kernels
    H, d, dv, tau, eps = 2, 16, 24, 8.0, 1e-5
    lens, pasts = [5, 1, 9], [0, 4, 0]
    norm_w = torch.randn(dv)
    state = torch.zeros(4, H, d, dv, device=DEV)
    runs = [_gla_inputs(p + n, H, d, dv, seed=10 + i) for i, (n, p) in enumerate(zip(lens, pasts))]
    alone = [_gla_run(pr, z, offs, [p, n] if p else [n], 3, state, H, d, dv, tau, norm_w, eps)[p:]
             for (pr, z, offs), n, p in zip(runs, lens, pasts)]
    # request 1 first computes its 4 earlier tokens into slot 0; then all three run as one batch in slots 2, 0, 1
    pr, z, offs = runs[1]
    _gla_run(pr[:4], z[:4], offs, [4], 0, state, H, d, dv, tau, norm_w, eps)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    proj = torch.cat([r[0][p:] for r, p in zip(runs, pasts)]).to(DEV)
    zz = torch.cat([r[1][p:] for r, p in zip(runs, pasts)]).to(DEV)
    got = kernels.gla_recurrent(proj, offs, zz, state, i32([0, 5, 6, 15]), i32(pasts), i32([2, 0, 1]), norm_w.to(DEV),
                                H, d, dv, tau, d ** -0.5, eps).cpu()
    assert torch.allclose(got, torch.cat(alone), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------------ latent attention
def _window_attention_plain(qa, rows, R, scale, window):
    """qa [T, H, R + r] against cache rows [T, R + r] of the same request; float64."""
    T, H, _ = qa.shape
    out = torch.zeros(T, H, R, dtype=torch.float64)
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        s = torch.einsum("hd,jd->hj", qa[i].double(), rows[lo:i + 1].double()) * scale
        out[i] = torch.softmax(s, -1) @ rows[lo:i + 1, :R].double()
    return out


def _paged(rows, block, num_blocks, seed):
    """Scatter a request's cache rows over shuffled pages -> (cache, block table)."""
    g = torch.Generator().manual_seed(seed)
    need = -(-rows.shape[0] // block)
    table = torch.randperm(num_blocks, generator=g)[:need].to(torch.int32)
    cache = torch.full((num_blocks * block, rows.shape[1]), 99.0, dtype=rows.dtype)
    for t in range(rows.shape[0]):
        cache[table[t // block] * block + t % block] = rows[t]
    return cache, table


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,R,r,window,block", [(3, 40, 8, 9, 16), (1, 20, 6, 5, 16), (5, 12, 2, 0, 32), (2, 200, 16, 70, 64),
                                                # ranks that are multiples of 16: the matrix-core kernel in bf16
                                                (6, 64, 8, 33, 16), (16, 32, 8, 5, 16), (2, 256, 32, 0, 32),
                                                (20, 48, 16, 64, 64), (1, 16, 0, 3, 16), (4, 512, 32, 40, 64)])
def test_latent_attention_prompt_pieces_and_single_tokens(dtype, H, R, r, window, block):
    from byox_vllm_amd import kernels
    torch.manual_seed(H * 10 + R)
    T = 150
    rows = torch.randn(T, R + r).to(dtype)
    qa = torch.randn(T, H, R + r)
    scale = 0.5 / math.sqrt(R + r)
    want = _window_attention_plain(qa, rows.float(), R, scale, window)
    cache, table = _paged(rows, block, 12, seed=R)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    tables = torch.full((2, 12), -1, dtype=torch.int32)
    tables[1, : table.numel()] = table                                  # the request is the batch's second row
    outs, at = [], 0
    for n in [70, 2, 3, 60] + [1] * 15:                                 # pieces cut inside pages and windows
        got = kernels.latent_attn(qa[at:at + n].contiguous().to(DEV), cache.to(DEV), tables.to(DEV), i32([0, 0, n]),
                                  i32([0, at]), i32([1] * n), H, R, r, block, window, scale)
        outs.append(got.cpu().float().view(n, H, R))
        at += n
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert torch.allclose(torch.cat(outs).double(), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype,R", [(torch.float32, 8), (torch.bfloat16, 16), (torch.bfloat16, 8)])
@pytest.mark.parametrize("pieces", [[200], [120, 80], [199, 1], [150] + [1] * 50])
def test_latent_attention_window_edges_stand_out(pieces, dtype, R):
    """Scores are zero except for one loud key per probed token: exactly window - 1 tokens back (the last one seen) or
    exactly window tokens back (the first one not seen); tokens 36 and 37 share the loud key 0, the sequence's first
    token.  A seen loud key takes all the weight; an unseen one leaves the plain mean over the window."""
    from byox_vllm_amd import kernels
    H, r, window, block, T = 2, 8, 37, 16, 200
    rows = torch.zeros(T, R + r)
    rows[:, :R] = torch.arange(T).float()[:, None] / 256                 # latent j identifies token j (exact in bf16)
    qa = torch.zeros(T, H, R + r)
    probes = [(199, True), (150, True), (100, False), (36, True), (37, False)]   # (token, loud key inside its window?)
    for i, _ in probes:
        qa[i, :, R] = 1.0                                                # queries look at the first rotated channel
    for i, inside in probes:
        rows[i - window + 1 if inside else i - window, R] = 60.0         # one loud key per probe
    cache, table = _paged(rows.to(dtype), block, 16, seed=1)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    outs, at = [], 0
    for n in pieces:
        got = kernels.latent_attn(qa[at:at + n].contiguous().to(DEV), cache.to(DEV), table.view(1, -1).to(DEV),
                                  i32([0, n]), i32([at]), i32([0] * n), H, R, r, block, window, 1.0)
        outs.append(got.cpu().float().view(n, H, R))
        at += n
    got = torch.cat(outs)
    want = _window_attention_plain(qa, rows, R, 1.0, window)
    tol = 1e-5 if dtype == torch.float32 else 4e-3                       # the output is rounded to the cache's dtype
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=tol)
    for i, inside in probes:
        if inside:   # the loud key is seen and takes all the weight
            assert abs(got[i, 0, 0].item() - (i - window + 1) / 256) < 4e-3, i
        else:        # the loud key lies one token outside: the answer is the plain mean over the window
            mean = sum(range(i - window + 1, i + 1)) / window / 256
            assert abs(got[i, 0, 0].item() - mean) < 4e-3, i


def test_latent_kv_store_and_query_rotation():
    from byox_vllm_amd import kernels
    from byox_vllm_amd.layers.rotary_embedding import scaled_inv_freq
    from rurutar_cases import SCALING
    torch.manual_seed(7)
    T, R, r, H, d = 9, 20, 6, 2, 5
    for scaling in (None, SCALING):
        inv_freq, gain = scaled_inv_freq(r, 500.0, scaling)
        pos = torch.tensor([0, 1, 2, 40, 41, 1000, 3, 4, 5], dtype=torch.int64)
        cos, sin = O.rotary_tables(1001, r, 500.0, scaling)
        kv, w = torch.randn(T, R + r + 3), torch.randn(R)
        cache = torch.zeros(32, R + r, device=DEV)
        slots = torch.tensor([5, 6, 7, 31, 0, 1, -1, 9, 10], dtype=torch.int32)
        kernels.latent_kv_store(kv.to(DEV)[:, 3:], w.to(DEV), pos.to(DEV), inv_freq.to(DEV), gain, slots.to(DEV), cache,
                                R, r, r, 1e-5)
        want_c = O.rms_norm(kv[:, 3:3 + R].double(), w.double(), 1e-5)
        want_k = O.rotate(kv[:, 3 + R:].double(), cos[pos], sin[pos], r)
        for t, s in enumerate(slots.tolist()):
            if s >= 0:
                assert torch.allclose(cache[s].cpu().double(), torch.cat([want_c[t], want_k[t]]), rtol=1e-4, atol=1e-4), t
        assert cache[2].abs().sum() == 0                                 # a negative slot writes nothing
        q = torch.randn(T, H * (d + r))
        qa = torch.zeros(T, H * (R + r), device=DEV)
        kernels.latent_q_rope(q.to(DEV), pos.to(DEV), inv_freq.to(DEV), gain, qa, H, d, r, r, R)
        want_q = O.rotate(q.double().view(T, H, d + r)[..., d:], cos[pos], sin[pos], r)
        assert torch.allclose(qa.cpu().double().view(T, H, R + r)[..., R:], want_q, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------------------------------------ mixture of experts
@pytest.mark.parametrize("E,top", [(5, 2), (3, 1), (12, 4), (4, 4)])
def test_moe_route_sort_combine(E, top):
    from byox_vllm_amd import kernels
    torch.manual_seed(E)
    T, width = 45, 28
    logits = torch.randn(T, E + 1)
    idx, wt = kernels.moe_route(logits.to(DEV), E, top)
    chosen, weights = O.route(logits[:, :E].double(), top)
    assert torch.equal(idx.cpu().long(), chosen)
    assert torch.allclose(wt.cpu().double(), weights, rtol=1e-5, atol=1e-6)
    offsets, sorted_token, slot_of = kernels.moe_sort(idx, E)
    offsets, sorted_token, slot_of = offsets.cpu(), sorted_token.cpu(), slot_of.cpu()
    assert offsets[0] == 0 and offsets[-1] == T * top
    assert sorted(slot_of.flatten().tolist()) == list(range(T * top))
    for t in range(T):
        for j in range(top):
            s = slot_of[t, j]
            assert sorted_token[s] == t and offsets[idx[t, j]] <= s < offsets[idx[t, j] + 1]
    y, shared = torch.randn(T * top, width), torch.randn(T, width)
    got = kernels.moe_combine(y.to(DEV), slot_of.to(DEV), wt, shared.to(DEV), logits.to(DEV)[:, E:]).cpu()
    want = (weights[:, :, None] * y.double()[slot_of.long()]).sum(1) + torch.sigmoid(logits[:, E:].double()) * shared.double()
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-5)


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


CASES = {"mixed": (mixed_config, 8), "odd": (odd_config, 5), "aligned": (aligned_config, 16)}


@pytest.fixture(scope="module", params=[("mixed", torch.float32), ("mixed", torch.bfloat16), ("odd", torch.float32),
                                        ("odd", torch.bfloat16), ("aligned", torch.float32), ("aligned", torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1])[6:]}")
def setup(request):
    name, dtype = request.param
    make, decay_rank = CASES[name]
    cfg = make()
    weights = O.random_checkpoint(cfg, seed=11, decay_rank=decay_rank)
    torch.manual_seed(99)
    reqs = {"a": torch.randint(0, cfg["vocab"], (83,)).tolist(), "b": torch.randint(0, cfg["vocab"], (31,)).tolist(),
            "c": torch.randint(0, cfg["vocab"], (2,)).tolist(), "d": torch.randint(0, cfg["vocab"], (50,)).tolist()}
    want = {n: O.forward(t, weights, cfg).float() for n, t in reqs.items()}
    engine = Engine(cfg, weights, dtype, blocks=12, slots=3)
    whole = engine.replay(reqs, [[(n, len(t))] for n, t in reqs.items()])
    return cfg, weights, dtype, reqs, want, engine, whole


def test_whole_prompts_match_the_oracle(setup):
    cfg, weights, dtype, reqs, want, engine, whole = setup
    for n in reqs:
        assert_rows_close(whole[n], want[n], _tol(dtype), dtype == torch.float32, n)


def _check(setup, got):
    cfg, weights, dtype, reqs, want, engine, whole = setup
    for n in got:
        assert_rows_close(got[n], want[n], _tol(dtype), dtype == torch.float32, n)
        if dtype == torch.float32:
            assert row_error(got[n], whole[n]) < SAME_TOL, n


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
    # the same requests again, in slots and pages that the first round has used
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
            logits = O.forward(tokens, weights, cfg)[-1]
            best = logits.max().item()
            # the engine's choice is the oracle's argmax, or lies inside the rounding of the engine's dtype
            assert best - logits[tok].item() <= (1e-3 if dtype == torch.float32 else 0.25), (k, tok)
            tokens.append(tok)
        assert len(out["token_ids"]) == steps


def test_fp32_sampler_argmax_and_temperature():
    from byox_vllm_amd import kernels
    torch.manual_seed(8)
    logits = torch.randn(6, 301)
    logits[2, 17] = logits[2, 200] = 9.0                                  # a tie goes to the lower index
    got = kernels.sample_f32(logits.to(DEV), torch.zeros(6, device=DEV)).cpu()
    want = logits.argmax(-1)
    want[2] = 17
    assert torch.equal(got, want)
    # with a temperature the draws follow softmax(logits / T): frequencies of a 3-way distribution over many rows
    rows = torch.tensor([[2.0, 1.0, 0.0]]).repeat(4000, 1)
    draws = kernels.sample_f32(rows.to(DEV), torch.full((4000,), 0.5, device=DEV), seed=5).cpu()
    freq = torch.bincount(draws, minlength=3).double() / 4000
    assert torch.allclose(freq, torch.softmax(torch.tensor([4.0, 2.0, 0.0]).double(), 0), atol=0.03)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps replayed from hipGraphs (padded batches, the spare state slot, one staging copy) give the tokens of
    the eager engine, step after step, with prompt portions running eagerly between the replays."""
    from byox_vllm_amd import LLM, SamplingParams
    cfg = mixed_config()
    weights = O.random_checkpoint(cfg, seed=21, decay_rank=8)
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
    weights = O.random_checkpoint(cfg, seed=31, decay_rank=16)
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
        logits = O.forward(tokens, weights, cfg)[-1]
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
        wa, wb = O.forward(a, weights, cfg).float(), O.forward(b, weights, cfg).float()
        expect = {0: wa[[0, 39]], 1: wa[[40]], 2: wb[[8]], 3: torch.cat([wa[[41, 69]], wb[[8]]])}
        for i, want in expect.items():
            got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert got.shape == want.shape and row_error(got, want) < tol, (dtype, i)


@pytest.mark.parametrize("M,N,K", [(256, 128, 32), (300, 200, 72), (1000, 72, 256), (513, 130, 40), (65, 40, 64), (130, 16, 512)])
def test_linear_many_rows_go_through_the_tiled_kernel(M, N, K):
    """From 65 rows of 16-byte-aligned bf16 on, nv_linear stages its operands through LDS: plain, gated, soft-capped,
    with bias, with row and column tails and a K that is no multiple of the K-block."""
    from byox_vllm_amd import kernels
    torch.manual_seed(M + N)
    x, w, b = (torch.randn(M, K) / 4).bfloat16(), torch.randn(2 * N, K).bfloat16(), torch.randn(N).bfloat16()
    xd, wd = x.to(DEV), w.to(DEV)
    want = x.double() @ w[:N].double().T + b.double()
    got = kernels.linear(xd, wd[:N], b.to(DEV), out_dtype=torch.float32).cpu()
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-4)
    g, u = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    got = kernels.linear(xd, wd, epilogue=kernels.EPI_GLU, act=kernels.ACT_GELU_TANH, out_dtype=torch.float32).cpu()
    assert torch.allclose(got.double(), O.gelu_tanh(g) * u, rtol=1e-4, atol=1e-4)
    got = kernels.linear(xd, wd[:N], epilogue=kernels.EPI_SOFTCAP, cap=2.0).cpu()
    assert torch.allclose(got.double(), 2.0 * torch.tanh(g / 2.0), rtol=2e-2, atol=2e-2)


def test_linear_many_rows_groups_batches_and_gates():
    from byox_vllm_amd import kernels
    torch.manual_seed(12)
    T, K, N, sizes = 400, 48, 40, [0, 700, 3, 129, 260]
    E, total = len(sizes), sum(sizes)
    x, w = (torch.randn(T, K) / 4).bfloat16(), torch.randn(E, 2 * N, K).bfloat16()
    rows = torch.randint(0, T, (total,), dtype=torch.int32)
    offsets = torch.tensor([0] + torch.tensor(sizes).cumsum(0).tolist(), dtype=torch.int32)
    got = kernels.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32, rows=total, a_rows=rows.to(DEV), batch=E,
                         w_batch_stride=2 * N * K, group_offsets=offsets.to(DEV), max_group_rows=max(sizes),
                         epilogue=kernels.EPI_GLU).cpu()
    for e in range(E):
        lo, hi = offsets[e], offsets[e + 1]
        xe = x.double()[rows[lo:hi].long()]
        want = O.silu(xe @ w[e, :N].double().T) * (xe @ w[e, N:].double().T)
        assert torch.allclose(got[lo:hi].double(), want, rtol=1e-4, atol=1e-4), e
    H, Kh, Nh = 3, 24, 20
    xh, wh, gate = (torch.randn(T, H * Kh) / 4).bfloat16(), torch.randn(H, Nh, Kh).bfloat16(), torch.randn(T, H)
    want = torch.stack([xh.double().view(T, H, Kh)[:, h] @ wh[h].double().T for h in range(H)], 1)
    want = want * torch.sigmoid(gate.double()[:, :, None])
    out = torch.zeros(T, H * Nh, dtype=torch.float32, device=DEV)
    gd = gate.to(DEV)
    kernels.linear(xh.to(DEV), wh.to(DEV), out=out, out_dtype=torch.float32, batch=H, a_batch_stride=Kh,
                   w_batch_stride=Nh * Kh, out_batch_stride=Nh, n=Nh, epilogue=kernels.EPI_ROW_GATE, gate=gd,
                   gate_stride=gd.stride(0))
    assert torch.allclose(out.cpu().double().view(T, H, Nh), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 40, 256), (8, 130, 1000), (16, 64, 2048), (5, 7, 300), (17, 40, 512), (64, 72, 260),
                                   (33, 130, 1024)])
def test_linear_few_rows_split_k_over_the_wavefronts(dtype, M, N, K):
    """Up to 64 rows and K >= 256: one 16-column tile per workgroup with K split over its wavefronts; plain, gated,
    grouped over gathered rows."""
    from byox_vllm_amd import kernels
    torch.manual_seed(M * 7 + N)
    x, w, b = (torch.randn(M, K) / 8).to(dtype), torch.randn(2 * N, K).to(dtype), torch.randn(N).to(dtype)
    xd, wd = x.to(DEV), w.to(DEV)
    g, u = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    got = kernels.linear(xd, wd[:N], b.to(DEV), out_dtype=torch.float32).cpu()
    assert torch.allclose(got.double(), g + b.double(), rtol=1e-4, atol=1e-4)
    got = kernels.linear(xd, wd, epilogue=kernels.EPI_GLU, out_dtype=torch.float32).cpu()
    assert torch.allclose(got.double(), O.silu(g) * u, rtol=1e-4, atol=1e-4)
    E, sizes = 3, [M, 0, max(1, M // 2)]
    we = torch.randn(E, N, K).to(dtype)
    rows = torch.randint(0, M, (sum(sizes),), dtype=torch.int32)
    offsets = torch.tensor([0, sizes[0], sizes[0], sum(sizes)], dtype=torch.int32)
    got = kernels.linear(xd, we.to(DEV), out_dtype=torch.float32, rows=sum(sizes), a_rows=rows.to(DEV), batch=E,
                         w_batch_stride=N * K, group_offsets=offsets.to(DEV), max_group_rows=M).cpu()
    for e in range(E):
        lo, hi = offsets[e], offsets[e + 1]
        assert torch.allclose(got[lo:hi].double(), x.double()[rows[lo:hi].long()] @ we[e].double().T, rtol=1e-4, atol=1e-4)
