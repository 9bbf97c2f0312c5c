"""Plain, slow restatement of the Rurutar design in float64 PyTorch on the CPU: one function per mechanism, whole
sequences only, no cache, no batching, nothing shared with byox_vllm_amd.  Tests compare the engine (portions, pages,
state slots, mixed batches) with these functions run on each request's full token list.

Weights are a dict keyed by the checkpoint's tensor names; ``cfg`` is the config.json dict."""

import math

import torch

F = torch.float64


def dynamic_tanh(x, weight, bias, alpha):
    return torch.tanh(alpha * x) * weight + bias


def rms_norm(x, weight, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotary_tables(num_positions, dims, base, scaling=None):
    """cos / sin [positions, dims/2] of the 'rotate half' layout, with the optional ramped frequency scaling."""
    idx = torch.arange(dims // 2, dtype=F)
    freq = base ** (-2.0 * idx / dims)
    gain = 1.0
    if scaling:
        def where(turns):
            return dims * math.log(scaling["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        first = max(math.floor(where(scaling["fast"])), 0)
        last = min(math.ceil(where(scaling["slow"])), dims - 1)
        blend = ((idx - first) / max(last - first, 0.001)).clamp(0, 1)
        freq = blend * freq / scaling["factor"] + (1 - blend) * freq
        gain = 1.0 + 0.1 * math.log(scaling["factor"])
    angle = torch.arange(num_positions, dtype=F)[:, None] * freq[None, :]
    return gain * angle.cos(), gain * angle.sin()


def rotate(x, cos, sin, dims):
    """x [T, ..., n]: the first ``dims`` entries rotated (entry i with entry i + dims/2), the rest unchanged."""
    half = dims // 2
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos.reshape(shape), sin.reshape(shape)
    a, b, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)


def gla_recurrence(q, k, v, decay):
    """q, k, decay [T, H, d], v [T, H, dv] -> o [T, H, dv]; the state starts at zero."""
    T, H, d = q.shape
    state = torch.zeros(H, d, v.shape[-1], dtype=F)
    out = []
    for t in range(T):
        state = decay[t].unsqueeze(-1) * state + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append((state * q[t].unsqueeze(-1)).sum(1))
    return torch.stack(out)


def gla_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, d) / math.sqrt(d)
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, d)
    o = rms_norm(gla_recurrence(q, k, v, decay), W[p + "norm"], eps).reshape(T, H * dv)
    return (o * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def window_softmax_attention(q_plain, q_rot, k_plain, k_rot, v, scale, window):
    """q_plain [T, H, d], q_rot [T, H, r], k_plain [T, H, d], k_rot [T, r], v [T, H, dv]; token i sees j with
    0 <= i - j < window (window 0: all earlier tokens and itself)."""
    T = q_plain.shape[0]
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * scale
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (j <= i) & ((i - j < window) if window else True)
    weights = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
    return torch.einsum("hij,jhv->ihv", weights, v)


def latent_mixer(h, W, p, m, eps, shared_kv):
    """``shared_kv``: dict layer index -> (latent, rotated key part) of the layers run so far; updated in place by
    layers that project their own."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    dims = rot.get("dims", r)
    cos, sin = rotary_tables(T, dims, rot.get("base", 10000.0), rot.get("scaling"))
    q = (rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps) @ W[p + "uq"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], cos, sin, dims)
    if m.get("kv_from") is not None:
        latent, k_rot = shared_kv[m["kv_from"]]
    else:
        kv = h @ W[p + "dkv"].T
        latent, k_rot = rms_norm(kv[:, :R], W[p + "dkv.norm"], eps), rotate(kv[:, R:], cos, sin, dims)
        shared_kv[m["_index"]] = (latent, k_rot)
    k_plain = (latent @ W[p + "uk"].T).view(T, H, d)
    v = (latent @ W[p + "uv"].T).view(T, H, dv)
    o = window_softmax_attention(q_plain, q_rot, k_plain, k_rot, v, m["scale"], (m.get("mask") or {}).get("size", 0))
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (o * gate.unsqueeze(-1)).reshape(T, H * dv) @ W[p + "o"].T


def gated_unit(h, W, p, act):
    return (act(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(logits, top):
    """-> (chosen experts [T, top], their weights: softmax over the chosen logits only)."""
    values, chosen = torch.topk(logits, top, dim=-1)
    return chosen, torch.softmax(values, dim=-1)


def mixture(h, W, p, m):
    chosen, weights = route(h @ W[p + "router"].T, m["router"]["top"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            out[t] += w * gated_unit(h[t:t + 1], W, f"{p}e{e}.", silu)[0]
    if m.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * gated_unit(h, W, p + "shared.", silu)
    return out


def forward(tokens, weights, cfg, layers_out=None):
    """Token ids of one request -> logits [T, vocab] (float64)."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    shared_kv = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = dynamic_tanh(x, W[p + "norm1"], W[p + "norm1.b"], W[p + "norm1.alpha"])
        if layer["type"] == "gla":
            x = x + gla_mixer(h, W, p + "mix.", layer["mixer"], eps)
        else:
            x = x + latent_mixer(h, W, p + "mix.", dict(layer["mixer"], _index=i), eps, shared_kv)
        if layer.get("mlp"):
            h = dynamic_tanh(x, W[p + "norm2"], W[p + "norm2.b"], W[p + "norm2.alpha"])
            if layer["mlp"]["kind"] == "dense":
                x = x + gated_unit(h, W, p + "mlp.", gelu_tanh)
            else:
                x = x + mixture(h, W, p + "mlp.", layer["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    h = dynamic_tanh(x, W["final.norm"], W["final.norm.b"], W["final.norm.alpha"])
    logits = h @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def random_checkpoint(cfg, seed=0, decay_rank=8, dtype=torch.bfloat16):
    """Random weights under the checkpoint's tensor names, drawn so that activations stay of order one; values are
    exactly representable in ``dtype`` (they are returned in it)."""
    g = torch.Generator().manual_seed(seed)
    width, out = cfg["width"], {}

    def mat(rows, cols, gain=1.0):
        return (torch.randn(rows, cols, generator=g) * gain / math.sqrt(cols)).to(dtype)

    def norm(name, n=None):
        n = n or width
        out[name] = (1.0 + 0.2 * torch.randn(n, generator=g)).to(dtype)
        out[name + ".b"] = (0.1 * torch.randn(n, generator=g)).to(dtype)
        out[name + ".alpha"] = torch.tensor(0.5 + 0.5 * torch.rand((), generator=g).item()).to(dtype)

    out["embed"] = torch.randn(cfg["vocab"], width, generator=g).to(dtype)
    out["head"] = mat(cfg["vocab"], width, 4.0)
    norm("final.norm")
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1")
        if layer["type"] == "gla":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            for name, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                out[p + "mix." + name] = mat(rows, width, 1.5)
            out[p + "mix.a1"] = mat(decay_rank, width)
            out[p + "mix.a2"] = mat(H * d, decay_rank, 2.0)
            out[p + "mix.a2.b"] = (2.0 + torch.randn(H * d, generator=g)).to(dtype)
            out[p + "mix.norm"] = (1.0 + 0.2 * torch.randn(dv, generator=g)).to(dtype)
            out[p + "mix.o"] = mat(width, H * dv)
        else:
            H, d, r, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out[p + "mix.dq"] = mat(Q, width)
            out[p + "mix.dq.norm"] = (1.0 + 0.2 * torch.randn(Q, generator=g)).to(dtype)
            out[p + "mix.uq"] = mat(H * (d + r), Q, 2.0)
            if m.get("kv_from") is None:
                out[p + "mix.dkv"] = mat(R + r, width, 2.0)
                out[p + "mix.dkv.norm"] = (1.0 + 0.2 * torch.randn(R, generator=g)).to(dtype)
            out[p + "mix.uk"] = mat(H * d, R, 2.0)
            out[p + "mix.uv"] = mat(H * dv, R)
            out[p + "mix.g"] = mat(H, width)
            out[p + "mix.o"] = mat(width, H * dv)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        norm(p + "norm2")
        if mlp["kind"] == "dense":
            units = [(p + "mlp.", mlp["ff"])]
        else:
            units = [(f"{p}mlp.e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            out[p + "mlp.router"] = mat(mlp["router"]["experts"], width, 3.0)
            if mlp.get("shared"):
                units.append((p + "mlp.shared.", mlp["shared"]["ff"]))
                out[p + "mlp.shared.sg"] = mat(1, width)
        for q, ff in units:
            out[q + "gate"], out[q + "up"], out[q + "down"] = mat(ff, width, 1.5), mat(ff, width, 1.5), mat(width, ff)
    return out
