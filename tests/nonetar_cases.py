"""Small Nonetar configurations, random checkpoints and helpers shared by the host and GPU tests.  Sizes are deliberately
awkward: several query heads per key head, head counts that are no powers of two, key, value and state sizes that all
differ, widths that are no multiples of 8, one stream and several, one gate block and several, convolutions of two to
five taps, a window shorter than a page and one longer than every prompt, layers without a feed-forward."""

import copy

import torch


def parallel(heads, kv_heads, dim, vdim, window, rec_width, blocks, taps, softcap=30.0, scale=None, left_scale=0.8,
             right_scale=1.1):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
            "softcap": softcap}
    if window:
        left["mask"] = {"size": window}
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale,
                                          "right": {"width": rec_width, "blocks": blocks, "conv": taps},
                                          "right_scale": right_scale}}


def mamba2(heads, groups, vdim, state, taps, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "groups": groups, "vdim": vdim, "state": state, "conv": taps,
                                        "norm_groups": norm_groups}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, layers, streams=2, logit_scale=0.5, eps=1e-5):
    cfg = {"architecture": "Nonetar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
           "layers": [dict(copy.deepcopy(mixer), mlp=mlp) for mixer, mlp in layers]}
    if streams:
        cfg["streams"] = streams
    return cfg


def mixed_config():
    """Three streams; three query heads per key head; a window shorter than a page; one gate block; a layer without a
    feed-forward; state-space layers with one group and with several."""
    return config(160, 96, [
        (parallel(6, 2, 16, 24, 9, 80, 5, 3), dense(72)),
        (mamba2(4, 1, 16, 24, 4, 1), dense(40)),
        (parallel(4, 4, 8, 40, 40, 48, 1, 2, softcap=None, left_scale=1.2, right_scale=0.7), None),
        (mamba2(6, 3, 8, 12, 2, 3), dense(56)),
    ], streams=3)


def odd_config():
    """Nothing is a multiple of 8; one stream with learned connections; the state-space layer comes first; one head; a
    window longer than every prompt; five taps."""
    return config(77, 100, [
        (mamba2(2, 2, 10, 12, 5, 4), dense(36)),
        (parallel(1, 1, 20, 12, 5, 36, 3, 4, scale=0.3), dense(52)),
        (parallel(3, 1, 12, 6, 64, 20, 2, 3, softcap=8.0), None),
    ], streams=1, logit_scale=1.0)


def plain_config():
    """No 'streams' entry: the ordinary residual sum, no connection tensors in the checkpoint; no window at all."""
    return config(64, 48, [
        (parallel(2, 1, 8, 8, 0, 16, 2, 2), dense(24)),
        (mamba2(3, 1, 8, 4, 3, 1), None),
    ], streams=None, logit_scale=2.0)


def ssm_only_config():
    """No layer owns cache rows: the page pool stays empty-handed while block tables still grow."""
    return config(50, 40, [(mamba2(2, 1, 8, 16, 4, 2), dense(24)), (mamba2(5, 5, 4, 4, 3, 1), None)], streams=2)


def attention_only_config():
    """Only parallel layers, none with a feed-forward; eight query heads on one key/value head."""
    return config(90, 64, [(parallel(8, 1, 8, 16, 7, 24, 3, 3), None), (parallel(2, 2, 24, 8, 100, 40, 1, 2, softcap=None), None)],
                  streams=2, logit_scale=1.5)


def aligned_config():
    """Sizes in multiples of 16 and 32, where the 16-bit engine takes its matrix-core kernels; a window of exactly one
    page."""
    return config(256, 128, [
        (parallel(4, 2, 32, 16, 16, 64, 2, 4), dense(96)),
        (mamba2(4, 2, 16, 32, 3, 2), dense(64)),
        (parallel(8, 8, 16, 16, 33, 32, 4, 4), None),
    ], streams=4)


def random_checkpoint(cfg, seed=0):
    """Random weights keyed by checkpoint names, rounded to bf16 so that every dtype of the engine loads the same numbers."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def rand(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16)

    def matrix(out, inp, gain=1.0):
        return rand(out, inp, std=gain * inp ** -0.5)
    width, S = cfg["width"], cfg.get("streams")
    W["embed"] = rand(cfg["vocab"], width)
    W["head"] = matrix(cfg["vocab"], width, 2.0)
    W["final.norm"] = rand(width, std=0.1)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        W[p + "norm1"] = rand(width, std=0.1)
        W[p + "shift"] = torch.rand(width, generator=g).to(torch.bfloat16)
        subs = ["hc1"] + (["hc2"] if layer["mlp"] else [])
        if S:
            for hc in subs:
                W[p + hc + ".in"] = rand(S, std=0.2, mean=1.0 / S)
                W[p + hc + ".out"] = rand(S, std=0.3, mean=1.0)
                W[p + hc + ".mix"] = (torch.eye(S) + 0.2 * torch.randn(S, S, generator=g)).to(torch.bfloat16)
        if layer["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, d, dv, C, nb = a["heads"], a["kv_heads"], a["dim"], a["vdim"], r["width"], r["blocks"]
            q = p + "mix.left."
            for name, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                W[q + name] = matrix(rows, width, 1.5)
                W[q + name + ".b"] = rand(rows, std=0.2)
            W[q + "q.norm"], W[q + "k.norm"] = rand(d, std=0.2, mean=1.5), rand(d, std=0.2, mean=1.5)
            W[q + "temp"] = (0.5 + torch.rand(H, generator=g)).to(torch.bfloat16)
            W[q + "o"] = matrix(width, H * dv)
            q = p + "mix.right."
            for name in ("y", "x"):
                W[q + name] = matrix(C, width)
                W[q + name + ".b"] = rand(C, std=0.2)
            W[q + "conv"], W[q + "conv.b"] = rand(C, r["conv"], std=0.5), rand(C, std=0.1)
            for name in ("ra", "ri"):
                W[q + name] = rand(nb, C // nb, C // nb, std=(C // nb) ** -0.5)
                W[q + name + ".b"] = rand(nb, C // nb, std=0.5)
            W[q + "lam"] = rand(C, std=1.0, mean=-1.0)
            W[q + "o"] = matrix(width, C)
        else:
            H, G, P, N = m["heads"], m["groups"], m["vdim"], m["state"]
            inner, q = H * P, p + "mix."
            W[q + "in"] = matrix(2 * inner + 2 * G * N + H, width)
            W[q + "conv"], W[q + "conv.b"] = rand(inner + 2 * G * N, m["conv"], std=0.5), rand(inner + 2 * G * N, std=0.1)
            W[q + "dt_bias"] = rand(H, std=0.5)
            W[q + "A_log"] = rand(H, std=0.5, mean=-1.0)
            W[q + "D"] = rand(H, std=0.2, mean=1.0)
            W[q + "norm"] = rand(inner, std=0.2, mean=1.0)
            W[q + "o"] = matrix(width, inner)
        if layer["mlp"]:
            ff = layer["mlp"]["ff"]
            W[p + "norm2"] = rand(width, std=0.1)
            W[p + "mlp.up"], W[p + "mlp.down"] = matrix(ff, width), matrix(width, ff)
            W[p + "mlp.act"] = rand(2, std=0.5)
    return W


def engine_config(cfg_json, weights, dtype, blocks=16, slots=4, block_size=16, **kw):
    """The engine's Config for an in-memory checkpoint of one of the configurations above."""
    from byox_vllm_amd.config import Config
    from byox_vllm_amd.models.nonetar import nonetar_config
    hf = nonetar_config(cfg_json, dtype=dtype)
    return Config("synthetic", hf_config=hf, state_dict=weights, kvcache_block_size=block_size, num_kvcache_blocks=blocks,
                  max_num_seqs=slots, num_state_slots=slots, enforce_eager=True, max_num_batched_tokens=1 << 20,
                  max_model_len=1 << 20, **kw)


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per-row error: difference with its mean taken off, root mean square over the vocabulary, relative to the root
    mean square of the expected logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    scale = want.double().pow(2).mean().sqrt()
    return d.pow(2).mean(-1).sqrt() / scale


def row_error(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errors(got, want).max())
