"""Plain, slow restatement of the Nonetar design in float64 PyTorch on the CPU: one function per mechanism, whole
sequences only, no cache, no batching, nothing shared with byox_vllm_amd.  Tests compare the engine (portions, pages,
state slots, mixed batches) with these functions run on each request's full token list.

Weights are a dict keyed by the checkpoint's tensor names; ``cfg`` is the config.json dict."""

import math

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


def xielu(z, p, q):
    """Quadratic above zero, an exponential tail below; both halves meet at 0 with slope 1/2."""
    ap, an = softplus(p), 0.5 + softplus(q)
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)


def rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def sinusoid(T, width):
    """[T, width]: pairs (sin, cos) of position * 10000^(-2i / width)."""
    e = torch.arange(width)
    freq = 10000.0 ** (-2.0 * (e // 2).to(F) / width)
    angle = torch.arange(T, dtype=F)[:, None] * freq[None, :]
    return torch.where(e % 2 == 0, angle.sin(), angle.cos())


def token_shift(h, mu):
    """Every token moves towards its predecessor (zeros before the first) by the per-channel fraction mu."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last tap multiplies the current token), zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F), x], 0)
    out = b.expand(T, -1).clone()
    for j in range(taps):
        out += pad[j:j + T] * w[:, j]
    return out


def windowed_attention(q, k, v, scale, temp, softcap, window):
    """q, k [T, H, d] (k already repeated to H heads), v [T, H, dv] -> [T, H, dv].  Score of query i on key j:
    cap(q.k * scale * temp_h) - slope_h (i - j), keys with 0 <= i - j < window."""
    T, H, _ = q.shape
    s = torch.einsum("ihd,jhd->hij", q, k) * scale * temp[:, None, None]
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    slope = 2.0 ** (-8.0 * (torch.arange(H, dtype=F) + 1) / H)
    s = s - slope[:, None, None] * (i - j).to(F)
    seen = (j <= i) if not window else ((j <= i) & (i - j < window))
    s = s.masked_fill(~seen, -math.inf)
    return torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), v)


def attention_branch(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q = rms(q, eps) * W[p + "q.norm"]
    k = rms(k, eps) * W[p + "k.norm"]
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    window = int((m.get("mask") or {}).get("size", 0))
    o = windowed_attention(q, k, v, m["scale"], W[p + "temp"], m.get("softcap"), window)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def gated_linear_recurrence(u, gr, gi, lam):
    """u, gr, gi [T, C]: a_t = exp(-8 sigmoid(gr) softplus(lam)); S_t = a_t S_(t-1) + sqrt(1 - a_t^2) sigmoid(gi) u."""
    log_a = -8.0 * torch.sigmoid(gr) * softplus(lam)
    a, b = log_a.exp(), torch.sqrt(-torch.expm1(2.0 * log_a)) * torch.sigmoid(gi) * u
    S, out = torch.zeros_like(u[0]), []
    for t in range(u.shape[0]):
        S = a[t] * S + b[t]
        out.append(S)
    return torch.stack(out)


def recurrent_branch(h, W, p, m):
    T, C, nb = h.shape[0], m["width"], m["blocks"]
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = causal_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    ub = u.view(T, nb, C // nb)
    gr = torch.einsum("tbi,boi->tbo", ub, W[p + "ra"]) + W[p + "ra.b"]
    gi = torch.einsum("tbi,boi->tbo", ub, W[p + "ri"]) + W[p + "ri.b"]
    S = gated_linear_recurrence(u, gr.reshape(T, C), gi.reshape(T, C), W[p + "lam"])
    return (S * y) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    return (m["left_scale"] * attention_branch(h, W, p + "left.", m["left"], eps)
            + m["right_scale"] * recurrent_branch(h, W, p + "right.", m["right"]))


def ssd_scan(x, B, C, dt, A_log, D):
    """x [T, H, P], B, C [T, H, N] (already per head), dt [T, H]: S_t = exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x."""
    T, H, P = x.shape
    S = torch.zeros(H, B.shape[-1], P, dtype=F)
    out = []
    for t in range(T):
        decay = torch.exp(-torch.exp(A_log) * dt[t])
        S = decay[:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        out.append(torch.einsum("hnp,hn->hp", S, C[t]) + D[:, None] * x[t])
    return torch.stack(out)


def mamba2_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, 1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, 1)
    dt = softplus(dt + W[p + "dt_bias"])
    y = ssd_scan(x, B, C, dt, W[p + "A_log"], W[p + "D"]).reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def feed_forward(h, W, p):
    a = W[p + "act"]
    return xielu(h @ W[p + "up"].T, a[0], a[1]) @ W[p + "down"].T


def forward(cfg, W, tokens, trace=None):
    """Token ids of one sequence -> logits [T, vocab].  ``trace`` collects the sum of the streams after every layer."""
    W = {k: v.to(F) for k, v in W.items()}
    eps, S = cfg["norm"]["eps"], int(cfg.get("streams", 1))
    T = len(tokens)
    x0 = W["embed"][torch.tensor(tokens)] + sinusoid(T, cfg["width"])
    xs = [x0.clone() for _ in range(S)]

    def sublayer(xs, hc, norm_w, fn):
        if hc + "in" in W:
            u = sum(W[hc + "in"][s] * xs[s] for s in range(S))
            y = fn(rms(u, eps) * (1.0 + norm_w))
            return [sum(W[hc + "mix"][s, t] * xs[s] for s in range(S)) + W[hc + "out"][t] * y for t in range(S)]
        return [xs[0] + fn(rms(xs[0], eps) * (1.0 + norm_w))]

    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."

        def mixer(h, p=p, layer=layer):
            if p + "shift" in W:
                h = token_shift(h, W[p + "shift"])
            if layer["type"] == "parallel":
                return parallel_mixer(h, W, p + "mix.", layer["mixer"], eps)
            if layer["type"] == "mamba2":
                return mamba2_mixer(h, W, p + "mix.", layer["mixer"], eps)
            raise ValueError(layer["type"])
        xs = sublayer(xs, p + "hc1.", W[p + "norm1"], mixer)
        if layer.get("mlp"):
            xs = sublayer(xs, p + "hc2.", W[p + "norm2"], lambda h, p=p: feed_forward(h, W, p + "mlp."))
        if trace is not None:
            trace.append(sum(xs))
    x = rms(sum(xs), eps) * (1.0 + W["final.norm"])
    return (x @ W["head"].T) * cfg.get("logit_scale", 1.0)
