"""Small Rurutar configurations and helpers shared by the host and GPU tests.  Sizes are deliberately awkward: head
counts that are no powers of two, key and value sizes that differ, widths that are no multiples of 8, one expert per
token, a layer without a feed-forward, a layer that borrows another layer's cache rows."""

import copy

import torch

SCALING = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, base=10000.0, scaling=None, kv_from=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "mask": {"size": window}, "rot": {"base": base, "dims": rot_dim},
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if scaling:
        m["rot"]["scaling"] = scaling
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def gla(heads, dim, vdim, tau):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared_ff=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff}
    return m


def config(vocab, width, layers, softcap=20.0, scale=0.7, eps=1e-5):
    return {"architecture": "Rurutar", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "logit_softcap": softcap,
            "layers": [dict(copy.deepcopy(mixer), mlp=mlp) for mixer, mlp in layers]}


def mixed_config():
    """Latent attention first, two recurrent layers (one without a feed-forward), a layer on borrowed cache rows."""
    return config(160, 96, [
        (latent(3, 16, 8, 24, 40, 48, window=9, scaling=SCALING, scale=0.2), moe(5, 2, 40, shared_ff=56)),
        (gla(2, 16, 24, 8.0), dense(72)),
        (gla(3, 8, 40, 4.0), None),
        (latent(5, 8, 8, 16, 40, 24, window=17, scaling=SCALING, kv_from=0), moe(3, 1, 24)),
    ])


def odd_config():
    """Nothing is a multiple of 8; one head; no soft cap; no frequency scaling; the recurrent layer comes first."""
    return config(77, 100, [
        (gla(1, 20, 12, 3.0), moe(4, 3, 36, shared_ff=20)),
        (latent(1, 12, 6, 10, 20, 28, window=5, base=500.0), dense(52)),
        (latent(2, 4, 2, 6, 12, 10, window=64), None),
    ], softcap=None, scale=1.0)


def aligned_config():
    """Sizes in multiples of 16 and 32, where the 16-bit engine takes its matrix-core kernels; dense feed-forwards only,
    so that 16-bit runs have no routing decisions to flip."""
    return config(256, 128, [
        (latent(6, 16, 8, 16, 32, 24, window=11, scaling=SCALING), dense(96)),
        (gla(2, 32, 64, 6.0), dense(64)),
        (latent(3, 32, 8, 32, 32, 48, window=40, scaling=SCALING, kv_from=0), None),
    ], softcap=15.0)


def engine_config(cfg_json, weights, dtype, blocks=16, slots=4, block_size=16, decay_rank=None, **kw):
    """The engine's Config for an in-memory checkpoint of one of the configurations above."""
    from byox_vllm_amd.config import Config
    from byox_vllm_amd.models.rurutar import rurutar_config
    shapes = {k: list(v.shape) for k, v in weights.items()}
    hf = rurutar_config(cfg_json, shapes, dtype=dtype)
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


def assert_rows_close(got, want, tol, exact_routing: bool, what=""):
    """Every row within ``tol``.  In 16-bit runs a router logit of random weights can lie closer to its neighbour than
    the rounding of the router's input, and the token then takes another expert than the float64 oracle: there (not
    ``exact_routing``) a twentieth of the rows may differ, and the typical row must be well inside the tolerance."""
    err = row_errors(got, want)
    if exact_routing:
        assert float(err.max()) < tol, (what, float(err.max()))
    else:
        assert float((err > tol).double().mean()) <= 0.05 and float(err.median()) < tol / 2, \
            (what, float(err.max()), float(err.median()), float((err > tol).double().mean()))
