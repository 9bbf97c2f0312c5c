"""Host side of the Nonetar integration on the CPU: registry and configuration, checkpoint names and merged layouts, the
cache and state specifications the engine sizes its pools from, and the oracle's own consistency."""

import json

import pytest
import torch

from nonetar_cases import (aligned_config, attention_only_config, mixed_config, odd_config, plain_config,
                           random_checkpoint, ssm_only_config)
from oracle import nonetar as O

F64 = torch.float64


def test_registry_and_configuration():
    from byox_vllm_amd.models import registry
    from byox_vllm_amd.models.nonetar import nonetar_config
    assert registry.model_class({"architecture": "Nonetar"}).__name__ == "NonetarForCausalLM"
    cfg = mixed_config()
    hf = registry.read_config(cfg, None)
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers, hf.streams) == (160, 96, 4, 3)
    assert hf.connections and hf.logit_scale == 0.5 and hf.norm_eps == 1e-5
    plain = nonetar_config(plain_config())
    assert plain.streams == 1 and not plain.connections and plain.logit_scale == 2.0
    hf.layers[0]["mixer"]["left"]["heads"] = 99                     # the given dict is left as it was
    assert cfg["layers"][0]["mixer"]["left"]["heads"] == 6


def test_config_from_a_model_folder(tmp_path):
    from safetensors.torch import save_file

    from byox_vllm_amd.config import Config
    cfg = odd_config()
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in random_checkpoint(cfg, 1).items()}, str(tmp_path / "model.safetensors"))
    c = Config(str(tmp_path), dtype="float32", kvcache_block_size=32, max_num_seqs=3)
    assert c.portioned and c.num_state_slots == 3 and c.hf_config.dtype == torch.float32
    assert c.hf_config.layers[1]["mixer"]["right"]["blocks"] == 3


def test_a_model_without_attention_owns_no_pages_and_one_without_state_space_layers_still_has_slots():
    from byox_vllm_amd.models.nonetar import NonetarForCausalLM, nonetar_config
    ssm = NonetarForCausalLM(nonetar_config(ssm_only_config(), dtype=torch.float32))
    assert ssm.page_layers() == [] and len(ssm.state_layers()) == 6
    att = NonetarForCausalLM(nonetar_config(attention_only_config(), dtype=torch.float32))
    assert [m.page_spec()["width"] for m in att.page_layers()] == [1 * (8 + 16), 2 * (24 + 8)]
    assert len(att.state_layers()) == 6


@pytest.mark.parametrize("make", [mixed_config, odd_config, plain_config, aligned_config])
def test_every_checkpoint_tensor_has_a_parameter_and_every_parameter_a_tensor(make):
    """Builds the model on the CPU (parameters only; nothing is launched) and loads a random checkpoint through the
    framework's loader: every tensor finds its place, merged parameters are filled completely."""
    from byox_vllm_amd.models.nonetar import NonetarForCausalLM, nonetar_config
    from byox_vllm_amd.utils.loader import load_state_dict_packed
    cfg = make()
    weights = {k: v.float() for k, v in random_checkpoint(cfg, seed=2).items()}
    hf = nonetar_config(cfg, dtype=torch.float32)
    model = NonetarForCausalLM(hf)
    for name, p in model.named_parameters():
        if not (name.endswith(".hc") and not hf.connections):
            p.data.fill_(float("nan"))
    load_state_dict_packed(model, weights, hf)
    for name, p in model.named_parameters():
        assert not torch.isnan(p).any(), name
    assert all(model.checkpoint_target(k) is not None for k in weights)
    assert model.checkpoint_target("l0.mix.nothing") is None and model.checkpoint_target("l99.norm1") is None
    layer = next(l for l in model.layers if l.kind == "parallel")
    i = list(model.layers).index(layer)
    m, p = cfg["layers"][i]["mixer"], f"l{i}.mix."
    mix = layer.mix
    H, G, d, dv, C = [m["left"][k] for k in ("heads", "kv_heads", "dim", "vdim")] + [m["right"]["width"]]
    # one input projection: q | k | v | y | x rows, biases alike
    assert torch.equal(mix.inp.weight.data[mix.at["k"]:mix.at["k"] + G * d], weights[p + "left.k"])
    assert torch.equal(mix.inp.bias.data[mix.at["x"]:mix.at["x"] + C], weights[p + "right.x.b"])
    assert mix.inp.weight.shape[0] == H * d + G * d + G * dv + 2 * C
    # one output projection over [attention | recurrence] columns
    assert torch.equal(mix.o.weight.data[:, :H * dv], weights[p + "left.o"])
    assert torch.equal(mix.o.weight.data[:, H * dv:], weights[p + "right.o"])
    # gate rows per block: recurrence gate, then input gate
    bw = C // m["right"]["blocks"]
    assert torch.equal(mix.rec.gates.data[-1, :bw], weights[p + "right.ra"][-1])
    assert torch.equal(mix.rec.gates.data[0, bw:], weights[p + "right.ri"][0])
    assert torch.equal(mix.rec.gates_bias.data[:, bw:], weights[p + "right.ri.b"])
    if hf.connections:
        S = hf.streams
        hc = layer.norm1.hc.data
        assert torch.equal(hc[:S], weights[f"l{i}.hc1.in"]) and torch.equal(hc[S:2 * S], weights[f"l{i}.hc1.out"])
        assert torch.equal(hc[2 * S:].view(S, S), weights[f"l{i}.hc1.mix"])
    # a layer without a feed-forward has no second norm, and tensors addressed to one are dropped, not misplaced
    bare = [j for j, l in enumerate(model.layers) if l.mlp is None]
    for j in bare:
        assert model.layers[j].norm2 is None and model.checkpoint_target(f"l{j}.norm2") == (None, None)


def test_pools_are_sized_from_the_layers_own_specifications():
    from byox_vllm_amd.models.nonetar import NonetarForCausalLM, nonetar_config
    cfg = mixed_config()
    model = NonetarForCausalLM(nonetar_config(cfg, dtype=torch.float32))
    pages = [m.page_spec()["width"] for m in model.page_layers()]
    assert pages == [2 * (16 + 24), 4 * (8 + 40)]                    # key/value heads x (key + value size)
    shapes = [tuple(m.state_spec()["shape"]) for m in model.state_layers()]
    assert shapes == [(96,), (2, 80), (80,),                         # shift, conv inputs (taps - 1), recurrence
                      (96,), (3, 4 * 16 + 2 * 24), (4, 24, 16),      # shift, conv over x | B | C, heads x state x value
                      (96,), (1, 48), (48,),
                      (96,), (1, 6 * 8 + 2 * 3 * 12), (6, 12, 8)]
    assert "streams" in model.kernel_sources and "scan" in model.kernel_sources and "window_attn" in model.kernel_sources


# ------------------------------------------------------------------------------------------------ the oracle itself
def test_oracle_prefix_property_and_position_zero():
    """Causality: the logits of a prefix do not change when tokens follow; the first token sees zeros behind it."""
    cfg = mixed_config()
    W = random_checkpoint(cfg, 5)
    torch.manual_seed(1)
    tokens = torch.randint(0, cfg["vocab"], (30,)).tolist()
    full, part = O.forward(cfg, W, tokens), O.forward(cfg, W, tokens[:17])
    assert torch.allclose(full[:17], part, atol=1e-10)
    assert torch.allclose(O.forward(cfg, W, tokens[:1])[0], full[0], atol=1e-10)


def test_oracle_mechanisms_against_closed_forms():
    # sinusoid: position 0 is (0, 1) pairs; entry pairs share a frequency
    s = O.sinusoid(3, 6)
    assert torch.equal(s[0], torch.tensor([0.0, 1.0] * 3, dtype=F64))
    assert abs(float(s[2, 2]) - torch.sin(torch.tensor(2.0 * 10000.0 ** (-2 / 6), dtype=F64)).item()) < 1e-12
    # token shift: mu = 1 gives the previous row, mu = 0 the row itself
    h = torch.arange(12, dtype=F64).view(4, 3)
    assert torch.equal(O.token_shift(h, torch.ones(3, dtype=F64))[1:], h[:-1]) and torch.equal(O.token_shift(h, torch.zeros(3, dtype=F64)), h)
    # convolution: the last tap is the current token's
    x = torch.randn(5, 2, dtype=F64)
    w = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=F64)
    y = O.causal_conv(x, w, torch.zeros(2, dtype=F64))
    assert torch.equal(y[:, 0], x[:, 0]) and torch.equal(y[2:, 1], x[:-2, 1]) and float(y[:2, 1].abs().max()) == 0.0
    # state-space scan against the unrolled sum  y_t = sum_s (prod_{s<r<=t} decay_r) dt_s (C_t . B_s) x_s + D x_t
    T, H, P, N = 6, 2, 3, 4
    xs, B, C, dt = torch.randn(T, H, P, dtype=F64), torch.randn(T, H, N, dtype=F64), torch.randn(T, H, N, dtype=F64), torch.rand(T, H, dtype=F64)
    A_log, D = torch.randn(H, dtype=F64), torch.randn(H, dtype=F64)
    y = O.ssd_scan(xs, B, C, dt, A_log, D)
    t, hd = 4, 1
    total = D[hd] * xs[t, hd]
    for s_ in range(t + 1):
        decay = torch.exp(-torch.exp(A_log[hd]) * dt[s_ + 1:t + 1, hd].sum())
        total = total + decay * dt[s_, hd] * (C[t, hd] @ B[s_, hd]) * xs[s_, hd]
    assert torch.allclose(y[t, hd], total, atol=1e-12)
    # gated recurrence: the state's variance is preserved for unit-variance inputs (a^2 + (1 - a^2) = 1) - here the
    # deterministic part: constant input 1 with an open input gate converges to sqrt((1 - a^2)) / (1 - a)
    u = torch.ones(400, 1, dtype=F64)
    S = O.gated_linear_recurrence(u, torch.zeros(400, 1, dtype=F64), torch.full((400, 1), 50.0, dtype=F64), torch.zeros(1, dtype=F64))
    a = torch.exp(torch.tensor(-8.0 * 0.5 * 0.6931471805599453, dtype=F64))
    assert abs(float(S[-1, 0]) - float(torch.sqrt(1 - a * a) / (1 - a))) < 1e-9
