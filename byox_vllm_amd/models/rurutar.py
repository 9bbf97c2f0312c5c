"""Rurutar: a decoder-only language model whose layers alternate freely between two mixers - gated linear attention
(a recurrent fp32 state per request, layers/gla.py) and sliding-window latent attention (a paged cache of low-rank
latents, optionally shared between layers, layers/latent_attention.py) - with Dynamic Tanh in place of the usual norms
(layers/dyt.py), dense GELU or mixture-of-experts SiLU feed-forwards (layers/moe.py), a scaled embedding and a
soft-capped head.

The residual stream is fp32 from the embedding to the final norm.  Each block is pre-norm,
x <- x + mixer(norm1(x)); x <- x + ff(norm2(x)), and every residual add is fused into the norm that follows it.

config.json: {"architecture": "Rurutar", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, "logit_softcap",
"layers": [{"type": "gla" | "latent_attention", "mixer": {...}, "mlp": {...} | null}]}.  Sizes the configuration does not
name (the rank of the decay projection) are taken from the checkpoint's tensor shapes.  Checkpoint tensor names:
'embed', 'head', 'final.norm[.b|.alpha]', 'l<i>.norm1|norm2[.b|.alpha]', 'l<i>.mix.<name>', 'l<i>.mlp.<name>'.

The model steps through portions: any mixture of prompt pieces and single decoded tokens in one batch, each request
continuing from its pages and its state slot (engine/model_runner.py run_portions)."""

import json
import os
import re
import struct
from types import SimpleNamespace

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.dyt import DynamicTanh
from byox_vllm_amd.layers.gla import GatedLinearAttention
from byox_vllm_amd.layers.latent_attention import LatentAttention
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.layers.moe import GatedMLP, MixtureOfExperts


def _safetensors_shapes(path: str) -> dict:
    """name -> shape from the headers of the safetensors files under ``path`` (8-byte length, then JSON)."""
    shapes = {}
    for file in sorted(os.listdir(path)) if path and os.path.isdir(path) else []:
        if file.endswith(".safetensors"):
            with open(os.path.join(path, file), "rb") as f:
                (n,) = struct.unpack("<Q", f.read(8))
                header = json.loads(f.read(n))
            shapes.update({k: v["shape"] for k, v in header.items() if k != "__metadata__"})
    return shapes


def rurutar_config(raw: dict, shapes: dict | None = None, dtype=torch.bfloat16):
    """config.json contents (+ tensor shapes) -> the configuration object the engine and the model read."""
    shapes = shapes or {}
    layers = []
    for i, layer in enumerate(raw["layers"]):
        layer = json.loads(json.dumps(layer))           # deep copy
        mixer = layer["mixer"]
        if layer["type"] == "gla" and "decay_rank" not in mixer:
            mixer["decay_rank"] = shapes.get(f"l{i}.mix.a1", [16])[0]
        layers.append(layer)
    return SimpleNamespace(
        architecture="Rurutar", vocab_size=raw["vocab"], hidden_size=raw["width"],
        embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
        norm_eps=float((raw.get("norm") or {}).get("eps", 1e-6)), logit_softcap=raw.get("logit_softcap"),
        layers=layers, num_hidden_layers=len(layers), max_position_embeddings=1 << 30, dtype=dtype,
        tie_word_embeddings=False)


class RurutarLayer(nn.Module):
    def __init__(self, cfg, spec: dict, earlier: list):
        super().__init__()
        width, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.norm1 = DynamicTanh(width)
        if self.kind == "gla":
            self.mix = GatedLinearAttention(width, m["heads"], m["dim"], m["vdim"], m["decay_rank"], m["tau"], eps)
        elif self.kind == "latent_attention":
            rot = m.get("rot") or {}
            source = earlier[m["kv_from"]].mix if m.get("kv_from") is not None else None
            self.mix = LatentAttention(width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"],
                                       float(m["scale"]), int((m.get("mask") or {}).get("size", 0)),
                                       int(rot.get("dims", m["rot_dim"])), float(rot.get("base", 10000.0)),
                                       rot.get("scaling"), eps, kv_source=source)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.norm2 = self.mlp = None
        if mlp:
            self.norm2 = DynamicTanh(width)
            if mlp["kind"] == "dense":
                self.mlp = GatedMLP(width, mlp["ff"], "gelu_tanh")
            elif mlp["kind"] == "moe":
                shared = mlp.get("shared")
                self.mlp = MixtureOfExperts(width, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"],
                                            "silu", shared["ff"] if shared else None)
            else:
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")

    def forward(self, x, delta, positions):
        """x: fp32 residual (updated in place); delta: what the previous sublayer still owes it -> the same pair."""
        h = self.norm1(x, delta)
        delta = self.mix(h, positions) if self.kind == "latent_attention" else self.mix(h)
        if self.mlp is not None:
            delta = self.mlp(self.norm2(x, delta))
        return delta


class RurutarForCausalLM(nn.Module):
    portioned = True          # steps through ModelRunner.run_portions: prompt pieces and decoded tokens in one batch
    prefix_cache = False      # a recurrent state cannot be rebuilt from cached pages
    kernel_sources = ("linear", "rowops", "gla", "latent_attn", "moe", "misc", "gemm_lt")     # csrc files this model launches

    @staticmethod
    def config_from_json(raw: dict, path: str | None):
        return rurutar_config(raw, _safetensors_shapes(path) if path else None)

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size), requires_grad=False)
        self.layers = nn.ModuleList()
        for spec in cfg.layers:
            self.layers.append(RurutarLayer(cfg, spec, list(self.layers)))
        self.final_norm = DynamicTanh(cfg.hidden_size)
        self.head = DenseLinear(cfg.hidden_size, cfg.vocab_size)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace: list | None = None):
        """-> (fp32 residual [T, width], the last sublayer's output still to be added).  ``trace`` collects the residual
        after every layer (a debugging aid: it adds the pending output eagerly)."""
        x = kernels.embed_scale(input_ids, self.embed.data, self.cfg.embedding_scale)
        delta = None
        for layer in self.layers:
            delta = layer(x, delta, positions)
            if trace is not None:
                x += delta
                delta = None
                trace.append(x.clone())
        return x, delta

    def compute_logits(self, state, rows_idx=None, out_dtype=torch.float32):
        """Final norm on the wanted rows, head, soft cap -> logits [rows, vocab]."""
        x, delta = state
        if rows_idx is None:
            rows_idx = torch.arange(x.size(0), dtype=torch.int32, device=x.device)
        h = self.final_norm(x, delta, rows_idx)
        cap = self.cfg.logit_softcap
        if cap:
            return self.head(h, out_dtype=out_dtype, epilogue=kernels.EPI_SOFTCAP, cap=float(cap))
        return self.head(h, out_dtype=out_dtype)

    def finalize(self, quantization=None) -> None:
        assert quantization is None, "Rurutar runs unquantised"

    # ------------------------------------------------------------------ cache and state
    def page_layers(self):
        """Mixers that own rows of the paged cache."""
        return [l.mix for l in self.layers if l.kind == "latent_attention" and l.mix.own_kv]

    def state_layers(self):
        """Mixers that own a per-request recurrent state."""
        return [l.mix for l in self.layers if l.kind == "gla"]

    # ------------------------------------------------------------------ checkpoint names
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")

    def checkpoint_target(self, name: str):
        """Checkpoint tensor name -> (parameter path, shard id or None); None for a name this model does not own."""
        if name == "embed":
            return "embed", None
        if name == "head":
            return "head.weight", None
        if name.startswith("final.norm"):
            return "final_norm." + self._norm_part(name[len("final.norm"):]), None
        m = self._LAYER.match(name)
        if not m:
            return None
        i, rest = int(m.group(1)), m.group(2)
        base = f"layers.{i}."
        layer = self.layers[i]
        for norm in ("norm1", "norm2"):
            if rest == norm or rest.startswith(norm + "."):
                if getattr(layer, norm) is None:
                    return None, None          # a layer without a feed-forward has no second norm to feed
                return base + norm + "." + self._norm_part(rest[len(norm):]), None
        part, _, leaf = rest.partition(".")
        if part == "mix":
            if layer.kind == "gla":
                table = {"q": ("qkvg.weight", "q"), "k": ("qkvg.weight", "k"), "v": ("qkvg.weight", "v"),
                         "g": ("qkvg.weight", "g"), "a1": ("a1.weight", None), "a2": ("a2.weight", None),
                         "a2.b": ("a2.bias", None), "norm": ("norm", None), "o": ("o.weight", None)}
            else:
                table = {"dq": ("down.weight", "dq"), "dkv": ("down.weight", "dkv"), "g": ("down.weight", "g"),
                         "dq.norm": ("dq_norm", None), "dkv.norm": ("dkv_norm", None), "uq": ("uq.weight", None),
                         "uk": ("uk_t", None), "uv": ("uv.weight", None), "o": ("o.weight", None)}
            if leaf in table:
                return base + "mix." + table[leaf][0], table[leaf][1]
            return None
        if part == "mlp":
            if isinstance(layer.mlp, GatedMLP):
                table = {"gate": ("gate_up.weight", "gate"), "up": ("gate_up.weight", "up"), "down": ("down.weight", None)}
                return (base + "mlp." + table[leaf][0], table[leaf][1]) if leaf in table else None
            e = re.match(r"^e(\d+)\.(gate|up|down)$", leaf)
            if e:
                if e.group(2) == "down":
                    return base + "mlp.down", int(e.group(1))
                return base + "mlp.gate_up", (int(e.group(1)), e.group(2))
            table = {"router": ("router.weight", "router"), "shared.sg": ("router.weight", "sg"),
                     "shared.gate": ("shared.gate_up.weight", "gate"), "shared.up": ("shared.gate_up.weight", "up"),
                     "shared.down": ("shared.down.weight", None)}
            return (base + "mlp." + table[leaf][0], table[leaf][1]) if leaf in table else None
        return None

    @staticmethod
    def _norm_part(suffix: str) -> str:
        return {"": "weight", ".b": "b", ".alpha": "alpha"}[suffix]
