"""Host side of the Rurutar integration on the CPU: registry and configuration, checkpoint names, the portion
scheduler with pages and state slots, the integer arrays of a portioned step, and the oracle's own consistency."""

import json
import math
import os
import struct

import pytest
import torch

from oracle import rurutar as O
from rurutar_cases import SCALING, engine_config, mixed_config, odd_config

from byox_vllm_amd.engine.block_manager import BlockManager, StateSlotManager
from byox_vllm_amd.engine.scheduler import Scheduler
from byox_vllm_amd.engine.sequence import Sequence, SequenceStatus


# ------------------------------------------------------------------------------------------------ registry, config
def test_registry_resolves_architectures():
    from types import SimpleNamespace

    from byox_vllm_amd.models import registry
    assert registry.architecture_of({"architecture": "Rurutar"}) == "Rurutar"
    assert registry.architecture_of({"architectures": ["Qwen2ForCausalLM"]}) == "Qwen2ForCausalLM"
    assert registry.architecture_of(SimpleNamespace(hidden_size=8)) == registry.DEFAULT      # synthetic Qwen shapes
    assert registry.model_class({"architecture": "Rurutar"}).__name__ == "RurutarForCausalLM"
    assert registry.model_class({"architectures": ["Qwen3ForCausalLM"]}).__name__ == "Qwen3ForCausalLM"


def _write_safetensors(path, tensors):
    header, blob = {}, b""
    for name, t in tensors.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": {torch.bfloat16: "BF16", torch.float32: "F32"}[t.dtype], "shape": list(t.shape),
                        "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    head = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)) + head + blob)


def test_config_from_a_model_folder_reads_sizes_from_json_and_tensor_shapes(tmp_path):
    from byox_vllm_amd.config import Config
    cfg = mixed_config()
    weights = O.random_checkpoint(cfg, seed=1, decay_rank=7)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    _write_safetensors(tmp_path / "model.safetensors", weights)
    c = Config(str(tmp_path), dtype="float32", kvcache_block_size=32, max_num_seqs=3)
    hf = c.hf_config
    assert c.portioned and c.num_state_slots == 3 and hf.dtype == torch.float32
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers) == (160, 96, 4)
    assert hf.layers[1]["mixer"]["decay_rank"] == 7                  # not in config.json: the shape of the tensor
    assert hf.embedding_scale == 0.7 and hf.logit_softcap == 20.0 and hf.norm_eps == 1e-5
    # the given configuration object is left as it was
    assert "decay_rank" not in cfg["layers"][1]["mixer"]


@pytest.mark.parametrize("make", [mixed_config, odd_config])
def test_every_checkpoint_tensor_has_a_parameter_and_every_parameter_a_tensor(make):
    """Builds the model on the CPU (parameters only; nothing is launched) and loads a random checkpoint through the
    framework's loader: every tensor finds its place, merged and stacked parameters are filled completely."""
    from byox_vllm_amd.models.rurutar import RurutarForCausalLM, rurutar_config
    from byox_vllm_amd.utils.loader import load_state_dict_packed
    cfg = make()
    weights = O.random_checkpoint(cfg, seed=2, decay_rank=6, dtype=torch.float32)
    hf = rurutar_config(cfg, {k: list(v.shape) for k, v in weights.items()}, dtype=torch.float32)
    model = RurutarForCausalLM(hf)
    for p in model.parameters():
        p.data.fill_(float("nan"))
    load_state_dict_packed(model, weights, hf)
    for name, p in model.named_parameters():
        assert not torch.isnan(p).any(), name
    # spot checks of the layouts the kernels assume
    if make is mixed_config:
        mix = model.layers[0].mix
        H, d, R = 3, 16, 40
        assert torch.equal(mix.uk_t.data[1], weights["l0.mix.uk"].view(H, d, R)[1].T)
        at = mix.down.offset("dkv")
        assert torch.equal(mix.down.weight.data[at: at + R + 8], weights["l0.mix.dkv"])
        assert not model.layers[3].mix.own_kv and model.layers[3].mix.kv_source is mix
        assert "dkv" not in model.layers[3].mix.down.row_of
        mlp = model.layers[0].mlp
        assert torch.equal(mlp.gate_up.data[4, 40:], weights["l0.mlp.e4.up"])
        assert torch.equal(mlp.router.weight.data[5], weights["l0.mlp.shared.sg"][0])
        assert model.layers[2].mlp is None and model.layers[2].norm2 is None
        assert [m.state_spec()["shape"] for m in model.state_layers()] == [(2, 16, 24), (3, 8, 40)]
        assert [m.page_spec()["width"] for m in model.page_layers()] == [48]
    assert model.checkpoint_target("l0.mix.nonsense") is None


def test_scaled_frequencies_match_the_oracle_tables():
    from byox_vllm_amd.layers.rotary_embedding import scaled_inv_freq
    for dims, base, scaling in ((8, 10000.0, SCALING), (6, 500.0, None), (32, 50000.0, {"factor": 16.0, "original": 256,
                                                                                        "fast": 16.0, "slow": 2.0})):
        inv_freq, gain = scaled_inv_freq(dims, base, scaling)
        cos, sin = O.rotary_tables(50, dims, base, scaling)
        angle = torch.arange(50, dtype=torch.float64)[:, None] * inv_freq.double()[None, :]
        assert torch.allclose(gain * angle.cos(), cos, atol=1e-5) and torch.allclose(gain * angle.sin(), sin, atol=1e-5)
    plain, gain = scaled_inv_freq(8, 10000.0, None)
    scaled, _ = scaled_inv_freq(8, 10000.0, SCALING)
    assert gain == 1.0 and scaled[0] == plain[0] and math.isclose(float(scaled[-1]), float(plain[-1]) / 4.0, rel_tol=1e-6)


# ------------------------------------------------------------------------------------------------ oracle consistency
def test_oracle_absorbed_queries_equal_explicit_keys_and_values():
    """The identity the product's latent attention rests on, on the oracle's own functions: folding W_uk into the query
    and applying W_uv after the weighted sum of latents gives what explicit per-head keys and values give."""
    torch.manual_seed(0)
    T, H, d, r, dv, R, window = 12, 2, 5, 4, 3, 7, 4
    qp, qr = torch.randn(T, H, d, dtype=torch.float64), torch.randn(T, H, r, dtype=torch.float64)
    c, kr = torch.randn(T, R, dtype=torch.float64), torch.randn(T, r, dtype=torch.float64)
    uk, uv = torch.randn(H * d, R, dtype=torch.float64), torch.randn(H * dv, R, dtype=torch.float64)
    want = O.window_softmax_attention(qp, qr, (c @ uk.T).view(T, H, d), kr, (c @ uv.T).view(T, H, dv), 0.3, window)
    q_abs = torch.einsum("thd,hdr->thr", qp, uk.view(H, d, R))
    for i in range(T):
        lo = max(0, i - window + 1)
        for h in range(H):
            s = (c[lo:i + 1] @ q_abs[i, h] + kr[lo:i + 1] @ qr[i, h]) * 0.3
            mixed = torch.softmax(s, 0) @ c[lo:i + 1]
            assert torch.allclose(uv.view(H, dv, R)[h] @ mixed, want[i, h], atol=1e-12)


def test_oracle_is_causal_and_windows_forget():
    cfg = odd_config()
    weights = O.random_checkpoint(cfg, seed=3, decay_rank=4)
    torch.manual_seed(1)
    tokens = torch.randint(0, cfg["vocab"], (20,)).tolist()
    full = O.forward(tokens, weights, cfg)
    assert torch.allclose(O.forward(tokens[:11], weights, cfg), full[:11], atol=1e-9)      # later tokens change nothing


# ------------------------------------------------------------------------------------------------ pages and slots
def test_block_manager_extend_grows_page_by_page_and_returns_everything():
    bm = BlockManager(6, 16)
    a, b = Sequence(list(range(40)), 16), Sequence(list(range(5)), 16)
    assert bm.blocks_short(a, 17) == 2
    bm.extend(a, 17)
    assert len(a.block_table) == 2
    bm.extend(a, 32)
    assert len(a.block_table) == 2                                   # still covered
    bm.extend(b, 5)
    bm.extend(a, 40)
    assert len(a.block_table) == 3 and len(bm.free_block_ids) == 2 and not set(a.block_table) & set(b.block_table)
    with pytest.raises(RuntimeError):
        bm.extend(b, 16 * 4)                                          # three more pages, two free
    a.num_computed_tokens = 40
    bm.deallocate(a)
    assert a.block_table == [] and a.num_computed_tokens == 0 and len(bm.free_block_ids) == 5
    bm.extend(b, 16 * 4)                                              # fits now, in pages that a has used
    assert len(bm.free_block_ids) == 2


def test_state_slots_are_handed_out_and_taken_back():
    sm = StateSlotManager(2)
    a, b, c = (Sequence([1], 16) for _ in range(3))
    sm.allocate(a)
    sm.allocate(b)
    assert {a.state_slot, b.state_slot} == {0, 1} and not sm.can_allocate()
    with pytest.raises(RuntimeError):
        sm.allocate(c)
    sm.release(a)
    sm.release(a)                                                     # a second release is harmless
    sm.allocate(c)
    assert c.state_slot == 0 and a.state_slot == -1


def _scheduler(blocks=8, slots=2, budget=32, max_seqs=4, block_size=16):
    from types import SimpleNamespace
    return Scheduler(SimpleNamespace(max_num_seqs=max_seqs, max_num_batched_tokens=budget, eos=-1,
                                     num_kvcache_blocks=blocks, kvcache_block_size=block_size, portioned=True,
                                     num_state_slots=slots))


def test_commit_admits_grows_tables_and_finish_returns_slots():
    s = _scheduler()
    a, b = Sequence(list(range(50)), 16), Sequence(list(range(3)), 16)
    s.add(a)
    s.add(b)
    s.commit([(a, 20), (b, 3)])
    assert a.status is SequenceStatus.RUNNING and a.state_slot >= 0 and len(a.block_table) == 2 and not s.waiting
    s.advance([(a, 20), (b, 3)], [None, None])
    assert a.num_computed_tokens == 20 and b.num_computed_tokens == 3 and b.num_tokens == 3       # nothing was sampled
    s.commit([(a, 13)])
    assert len(a.block_table) == 3
    with pytest.raises(AssertionError):
        s.commit([(b, 1)])                                            # b has no token left to run
    c = Sequence([7], 16)
    s.add(c)
    with pytest.raises(RuntimeError):
        s.commit([(c, 1)])                                            # both slots are taken
    s.finish(b)
    s.commit([(c, 1)])
    assert c.state_slot == 0 or c.state_slot == 1


def test_own_policy_decodes_first_cuts_prompts_to_the_budget_and_finishes():
    s = _scheduler(blocks=8, slots=2, budget=32)
    a, b, c = Sequence(list(range(40)), 16), Sequence(list(range(10)), 16), Sequence(list(range(4)), 16)
    for seq in (a, b, c):
        seq.max_tokens, seq.ignore_eos = 2, True
        s.add(seq)
    plan = s.schedule_portions()
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 32)]      # the budget cuts the first prompt
    s.advance(plan, [None])
    plan = s.schedule_portions()
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 8), (b.seq_id, 10)] and list(s.waiting) == [c]   # two slots
    assert s.advance(plan, [5, 6]) == []                              # both prompts end: one token each
    assert a.num_tokens == 41 and b.token_ids[-1] == 6
    plan = s.schedule_portions()
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 1), (b.seq_id, 1)]
    done = s.advance(plan, [1, 2])
    assert done == [a, b] and a.state_slot == -1 and a.block_table == []
    plan = s.schedule_portions()                                      # the freed slots admit the third request
    assert [(q.seq_id, n) for q, n in plan] == [(c.seq_id, 4)]
    s.advance(plan, [9])
    s.advance(s.schedule_portions(), [9])
    assert s.is_finished() and len(s.block_manager.free_block_ids) == 8 and len(s.state_slots.free) == 2


def test_own_policy_preempts_the_youngest_when_pages_run_out():
    s = _scheduler(blocks=3, slots=3, budget=64)
    a, b = Sequence(list(range(16)), 16), Sequence(list(range(30)), 16)
    for seq in (a, b):
        seq.max_tokens, seq.ignore_eos = 8, True
        s.add(seq)
    plan = s.schedule_portions()
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 16), (b.seq_id, 30)]
    s.advance(plan, [1, 1])
    plan = s.schedule_portions()                                      # a needs a second page; b holds the other two
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 1)]
    assert b.status is SequenceStatus.WAITING and b.num_computed_tokens == 0 and b.state_slot == -1
    assert list(s.waiting) == [b]


def test_portion_step_arrays(monkeypatch):
    """The integers run_portions hands to the kernels, with the model replaced by a recorder."""
    from byox_vllm_amd.engine.model_runner import ModelRunner
    from byox_vllm_amd.utils.context import get_context
    runner = ModelRunner.__new__(ModelRunner)
    runner.block_size, runner.device = 16, torch.device("cpu")
    seen = {}

    class Recorder:
        def __call__(self, ids, pos):
            ctx = get_context()
            seen.update(ids=ids.tolist(), pos=pos.tolist(), cu=ctx.cu_seqlens_q.tolist(), past=ctx.past_lens.tolist(),
                        slots=ctx.slot_mapping.tolist(), states=ctx.state_slots.tolist(), owner=ctx.seq_of_token.tolist(),
                        tables=ctx.block_tables.tolist())
            return "state"

        def compute_logits(self, state, rows, out_dtype):
            seen["rows"] = rows.tolist()
            return torch.zeros(len(seen["rows"]), 4)
    runner.model = Recorder()
    monkeypatch.setattr(torch.cuda, "current_stream", lambda: type("S", (), {"synchronize": lambda self: None})())
    a, b = Sequence(list(range(100, 140)), 16), Sequence([7, 8, 9], 16)
    a.block_table, a.num_computed_tokens, a.state_slot = [5, 2, 9], 30, 1
    b.block_table, b.num_computed_tokens, b.state_slot = [4], 0, 0
    out = runner.run_portions([(a, 4), (b, 3)], want=[[0, 3], [2]])
    assert out.shape == (3, 4)
    assert seen["ids"] == [130, 131, 132, 133, 7, 8, 9] and seen["pos"] == [30, 31, 32, 33, 0, 1, 2]
    assert seen["slots"] == [2 * 16 + 14, 2 * 16 + 15, 9 * 16, 9 * 16 + 1, 64, 65, 66]     # token 32 opens the third page
    assert seen["cu"] == [0, 4, 7] and seen["past"] == [30, 0] and seen["states"] == [1, 0]
    assert seen["owner"] == [0, 0, 0, 0, 1, 1, 1] and seen["tables"] == [[5, 2, 9], [4, -1, -1]]
    assert seen["rows"] == [0, 3, 6]


def test_trace_runner_refuses_models_without_portions(tmp_path, capsys):
    """The replay entry point answers with exit code 3 for a model family that cannot step through portions."""
    from byox_vllm_amd import trace
    with open(tmp_path / "config.json", "w") as f:
        json.dump({"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "num_attention_heads": 4,
                   "num_key_value_heads": 2, "num_hidden_layers": 1, "intermediate_size": 128, "vocab_size": 100,
                   "max_position_embeddings": 1 << 30, "rms_norm_eps": 1e-6, "hidden_act": "silu"}, f)
    code = trace.main(["--model", str(tmp_path), "--dtype", "bfloat16", "--out", str(tmp_path / "o"), "--max-tokens", "64"])
    assert code == 3


def test_engine_config_helper_marks_the_model_portioned():
    cfg = odd_config()
    c = engine_config(cfg, O.random_checkpoint(cfg, seed=4, decay_rank=5), torch.bfloat16)
    assert c.portioned and c.hf_config.layers[0]["mixer"]["decay_rank"] == 5 and os.path.basename(c.model) == "synthetic"


def test_own_policy_says_so_when_the_pool_cannot_hold_one_request():
    s = _scheduler(blocks=2, slots=1, budget=64)
    a = Sequence(list(range(40)), 16)
    a.max_tokens, a.ignore_eos = 4, True
    s.add(a)
    plan = s.schedule_portions()
    assert [(q.seq_id, n) for q, n in plan] == [(a.seq_id, 32)]      # what two pages hold
    s.advance(plan, [None])
    with pytest.raises(RuntimeError):
        s.schedule_portions()                                         # the third page does not exist
