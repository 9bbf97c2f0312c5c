"""Nonetar: a decoder-only language model whose residual is a set of fp32 streams (layers/hyper.py) and whose layers
choose between two mixers:

* ``parallel``: two branches reading the same input side by side - softmax attention over a sliding window with
  normalised queries and keys, a per-head temperature, a soft cap and a linear distance penalty
  (layers/window_attention.py), and a real-gated linear recurrent unit behind a short convolution (layers/rglru.py) -
  summed with fixed weights.  Both branches share one input projection (q | k | v | y | x rows, with biases) and one
  output projection over their concatenated results (the branch weights are applied to the fp32 results before they
  are rounded for that product);
* ``mamba2``: a selective state-space mixer (layers/mamba2.py).

Every mixer reads its norm's output through a token shift (layers/hyper.py).  Feed-forwards are one up-projection with the
xIELU activation (layers/mlp.py) or absent.  The embedding adds sinusoidal positions; the head multiplies by a constant.

config.json: {"architecture": "Nonetar", "vocab", "width", "streams", "norm": {"eps"}, "logit_scale",
"layers": [{"type": "parallel" | "mamba2", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}]}.
Checkpoint tensor names: 'embed', 'head', 'final.norm', 'l<i>.norm1|norm2', 'l<i>.shift', 'l<i>.hc1|hc2.in|out|mix',
'l<i>.mix.<name>', 'l<i>.mlp.up|down|act'.

The model steps through portions: any mixture of prompt pieces and single decoded tokens in one batch, each request
continuing from its pages and its state slot (engine/model_runner.py run_portions)."""

import json
import math
import re
from types import SimpleNamespace

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.hyper import StreamNorm, TokenShift
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.layers.mamba2 import Mamba2Mixer
from byox_vllm_amd.layers.mlp import UnaryMLP
from byox_vllm_amd.layers.rglru import RealGatedLRU
from byox_vllm_amd.layers.window_attention import WindowAttention


def nonetar_config(raw: dict, dtype=torch.bfloat16):
    """config.json contents -> the configuration object the engine and the model read."""
    layers = json.loads(json.dumps(raw["layers"]))           # deep copy
    return SimpleNamespace(
        architecture="Nonetar", vocab_size=raw["vocab"], hidden_size=raw["width"],
        streams=int(raw.get("streams") or 1), connections="streams" in raw,
        norm_eps=float((raw.get("norm") or {}).get("eps", 1e-6)), logit_scale=float(raw.get("logit_scale", 1.0)),
        layers=layers, num_hidden_layers=len(layers), max_position_embeddings=1 << 30, dtype=dtype,
        tie_word_embeddings=False)


class ParallelMixer(nn.Module):
    """Window attention and a gated linear recurrence over the same input; result = a * attention + b * recurrence."""

    def __init__(self, width: int, m: dict, eps: float):
        super().__init__()
        left, right = m["left"], m["right"]
        self.left_scale, self.right_scale = float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))
        self.attn = WindowAttention(left["heads"], left.get("kv_heads", left["heads"]), left["dim"], left["vdim"],
                                    left["scale"], int((left.get("mask") or {}).get("size", 0)), left.get("softcap"), eps)
        self.rec = RealGatedLRU(right["width"], right["blocks"], right["conv"])
        sizes = dict(self.attn.sizes(), y=right["width"], x=right["width"])
        self.inp = DenseLinear(width, bias=True, shards=sizes)
        self.at = {name: self.inp.offset(name) for name in sizes}
        self.attn_cols, self.rec_cols = left["heads"] * left["vdim"], right["width"]
        # [W_o of the attention | W_o of the recurrence] over the concatenated branch outputs
        self.o = DenseLinear(self.attn_cols + self.rec_cols, width)
        self.o.weight.weight_loader = self._load_o

    def _load_o(self, param, tensor, side: str):
        at, n = (0, self.attn_cols) if side == "left" else (self.attn_cols, self.rec_cols)
        assert tensor.shape == (param.shape[0], n)
        param.data[:, at:at + n].copy_(tensor)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        # the biases are added where the projection is consumed: the product needs no epilogue and a prompt's rows go
        # through the engine's plain many-row route
        bias = self.inp.bias.data
        proj = kernels.linear(h, self.inp.weight.data, out_dtype=torch.float32)
        both = torch.empty(h.size(0), self.attn_cols + self.rec_cols, dtype=h.dtype, device=h.device)
        self.attn(proj, (self.at["q"], self.at["k"], self.at["v"]), both, self.left_scale, bias=bias)
        c, ax, ay = self.rec_cols, self.at["x"], self.at["y"]
        self.rec(proj[:, ax:ax + c], proj[:, ay:ay + c], both[:, self.attn_cols:], self.right_scale,
                 x_bias=bias[ax:ax + c], y_bias=bias[ay:ay + c])
        return self.o(both, out_dtype=torch.float32)


class NonetarLayer(nn.Module):
    def __init__(self, cfg, spec: dict):
        super().__init__()
        width, eps, m, S = cfg.hidden_size, cfg.norm_eps, spec["mixer"], cfg.streams
        self.kind = spec["type"]
        self.norm1 = StreamNorm(width, S, eps, cfg.connections)
        self.shift = TokenShift(width)
        if self.kind == "parallel":
            self.mix = ParallelMixer(width, m, eps)
        elif self.kind == "mamba2":
            self.mix = Mamba2Mixer(width, m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"], eps)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.norm2 = self.mlp = None
        if mlp:
            if mlp["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            self.norm2 = StreamNorm(width, S, eps, cfg.connections)
            self.mlp = UnaryMLP(width, mlp["ff"], "xielu")

    def forward(self, x, pending):
        """x: fp32 streams [T, S, width] (updated in place); pending: (what the previous sublayer still owes them, its
        norm) -> the same pair for this layer's last sublayer."""
        h = self.shift(self.norm1(x, pending, out_dtype=torch.float32))
        pending = (self.mix(h), self.norm1)
        if self.mlp is not None:
            pending = (self.mlp(self.norm2(x, pending)), self.norm2)
        return pending


class NonetarForCausalLM(nn.Module):
    portioned = True          # steps through ModelRunner.run_portions: prompt pieces and decoded tokens in one batch
    prefix_cache = False      # a recurrent state cannot be rebuilt from cached pages
    kernel_sources = ("linear", "rowops", "streams", "window_attn", "scan", "misc", "gemm_lt")   # csrc files launched

    @staticmethod
    def config_from_json(raw: dict, path: str | None):
        return nonetar_config(raw)

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size), requires_grad=False)
        self.layers = nn.ModuleList(NonetarLayer(cfg, spec) for spec in cfg.layers)
        self.final_norm = StreamNorm(cfg.hidden_size, cfg.streams, cfg.norm_eps, connections=False)
        self.head = DenseLinear(cfg.hidden_size, cfg.vocab_size)
        # 10000^(-2i / width) in float64: the kernel forms position * frequency in double
        width = cfg.hidden_size
        freq = [math.pow(10000.0, -2.0 * i / width) for i in range((width + 1) // 2)]
        self.register_buffer("inv_freq", torch.tensor(freq, dtype=torch.float64), persistent=False)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace: list | None = None):
        """-> (fp32 streams [T, S, width], what the last sublayer still owes them).  ``trace`` collects the sum of the
        streams after every layer (a debugging aid: it folds the pending output in eagerly)."""
        x = kernels.embed_sinusoid(input_ids, positions, self.embed.data, self.inv_freq, self.cfg.streams)
        pending = None
        for layer in self.layers:
            pending = layer(x, pending)
            if trace is not None:
                self.final_norm(x, pending)          # run for its side effect: the streams take the pending output
                pending = None
                trace.append(x.sum(1))
        return x, pending

    def compute_logits(self, state, rows_idx=None, out_dtype=torch.float32):
        """Final norm over the sum of the streams on the wanted rows, head, constant factor -> logits [rows, vocab]."""
        x, pending = state
        if rows_idx is None:
            rows_idx = torch.arange(x.size(0), dtype=torch.int32, device=x.device)
        h = self.final_norm(x, pending, rows_idx)
        return self.head(h, out_dtype=out_dtype, epilogue=kernels.EPI_ACT, act=kernels.ACT_SCALE, cap=self.cfg.logit_scale)

    def finalize(self, quantization=None) -> None:
        assert quantization is None, "Nonetar runs unquantised"
        for layer in self.layers:
            if layer.mlp is not None:
                layer.mlp.finalize()

    # ------------------------------------------------------------------ cache and state
    def page_layers(self):
        """Modules that own rows of the paged cache."""
        return [l.mix.attn for l in self.layers if l.kind == "parallel"]

    def state_layers(self):
        """Modules that own a piece of a request's state slot."""
        out = []
        for l in self.layers:
            out.append(l.shift)
            out.extend(l.mix.rec.state_modules() if l.kind == "parallel" else l.mix.state_modules())
        return out

    # ------------------------------------------------------------------ checkpoint names
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _PARALLEL = {"left.q": ("inp.weight", "q"), "left.q.b": ("inp.bias", "q"), "left.k": ("inp.weight", "k"),
                 "left.k.b": ("inp.bias", "k"), "left.v": ("inp.weight", "v"), "left.v.b": ("inp.bias", "v"),
                 "left.q.norm": ("attn.q_norm", None), "left.k.norm": ("attn.k_norm", None),
                 "left.temp": ("attn.temp", None), "left.o": ("o.weight", "left"),
                 "right.y": ("inp.weight", "y"), "right.y.b": ("inp.bias", "y"), "right.x": ("inp.weight", "x"),
                 "right.x.b": ("inp.bias", "x"), "right.conv": ("rec.conv.weight", None),
                 "right.conv.b": ("rec.conv.bias", None), "right.ra": ("rec.gates", "a"),
                 "right.ra.b": ("rec.gates_bias", "a"), "right.ri": ("rec.gates", "i"),
                 "right.ri.b": ("rec.gates_bias", "i"), "right.lam": ("rec.lam", None), "right.o": ("o.weight", "right")}
    _MAMBA2 = {"in": ("inp.weight", None), "conv": ("conv.weight", None), "conv.b": ("conv.bias", None),
               "dt_bias": ("dt_bias", None), "A_log": ("A_log", None), "D": ("D", None), "norm": ("norm", None),
               "o": ("o.weight", None)}

    def checkpoint_target(self, name: str):
        """Checkpoint tensor name -> (parameter path, shard id or None); None for a name this model does not own."""
        if name == "embed":
            return "embed", None
        if name == "head":
            return "head.weight", None
        if name == "final.norm":
            return "final_norm.weight", None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None
        i, rest = int(m.group(1)), m.group(2)
        base = f"layers.{i}."
        layer = self.layers[i]
        if rest == "norm1":
            return base + "norm1.weight", None
        if rest == "shift":
            return base + "shift.mu", None
        part, _, leaf = rest.partition(".")
        if part == "hc1" and leaf in ("in", "out", "mix"):
            return base + "norm1.hc", leaf
        if rest == "norm2" or part in ("hc2", "mlp"):
            if layer.mlp is None:
                return None, None          # a layer without a feed-forward has no second sublayer to feed
            if rest == "norm2":
                return base + "norm2.weight", None
            if part == "hc2":
                return (base + "norm2.hc", leaf) if leaf in ("in", "out", "mix") else None
            table = {"up": "up.weight", "down": "down.weight", "act": "act_params"}
            return (base + "mlp." + table[leaf], None) if leaf in table else None
        if part == "mix":
            table = self._PARALLEL if layer.kind == "parallel" else self._MAMBA2
            return (base + "mix." + table[leaf][0], table[leaf][1]) if leaf in table else None
        return None
