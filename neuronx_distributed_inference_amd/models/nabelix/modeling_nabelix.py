"""Nabelix for MI355X: a hybrid decoder whose every layer runs a windowed
softmax attention and a gated delta-rule recurrence side by side.

Layer: ``x += mixer(h)`` with ``h = LN(x) + shortconv(LN(x))`` (bias-free
LayerNorm, residual causal short convolution with carried tail), then an
optional ``x += W_down(gelu_tanh(W_gate n) * W_up n)`` with ``n = LN(x)``.
The 'parallel' mixer is ``left_scale * attention(h) + right_scale *
delta_rule(h)``:

- left: :class:`DistanceBiasWindowAttention` — GQA without rotation,
  log-distance score penalty, sliding window plus kept first tokens,
  sigmoid output gate, separate key and value head sizes;
- right: :class:`GatedDeltaRule` — matrix-state linear recurrence with
  per-key-channel decay, short-conv + SiLU on q/k/v, unit-norm q/k.

A span of layers may be repeated with shared weights ("loop"); every run
has its own KV pages and recurrent state, and every repeated pass re-adds
the embedding output before its first layer. Output: LayerNorm, tied
embedding head, tanh soft cap.

Engine integration: the residual stream is fp32 (norm statistics, attention
scores, decays and recurrent state are fp32 in the kernels; projections run
in the engine dtype). KV lives in the paged block cache with per-run
(kv_heads, k_dim, v_dim) shapes; convolution tails and delta-rule state
live in the cache manager's RecurrentStateManager, indexed by the engine's
seq_ids. One set of kernels serves prefill portions, decode tokens and
mixed batches — each token carries its position, pad tokens carry -1.
All ten projections that read ``h`` are one fused GEMM.
"""

from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.config import InferenceConfig
from neuronx_distributed_inference_amd.models.hybrid_base import HybridDecoderModel
from neuronx_distributed_inference_amd.models.model_base import CausalLMBase
from neuronx_distributed_inference_amd.modules.attention.distance_bias import (
    DistanceBiasWindowAttention,
)
from neuronx_distributed_inference_amd.modules.conv import CausalShortConv
from neuronx_distributed_inference_amd.modules.linear_recurrence import GatedDeltaRule
from neuronx_distributed_inference_amd.modules.mlp import GatedMLP
from neuronx_distributed_inference_amd.modules.norm import LayerNorm
from neuronx_distributed_inference_amd.ops import seqmix
from neuronx_distributed_inference_amd.parallel.layers import (
    ColumnParallelLinear,
    RowParallelLinear,
)


class NabelixInferenceConfig(InferenceConfig):
    """Reads the checkpoint's ``config.json`` as is (keys: architecture,
    width, vocab, layers[], loop, canon.taps, norm.eps, logit_softcap) and
    derives the generic attribute names the engine uses."""

    def get_required_attributes(self) -> List[str]:
        return ["width", "vocab", "layers", "norm"]

    def add_derived_config(self):
        if not hasattr(self, "layers"):
            return
        self.hidden_size = self.width
        self.vocab_size = self.vocab
        self.num_hidden_layers = len(self.layers)
        self.tie_word_embeddings = True
        if not getattr(self, "loop", None):
            self.loop = {"start": 0, "stop": 0, "times": 1}
        if not getattr(self, "canon", None):
            self.canon = {"taps": 1}
        if not hasattr(self, "logit_softcap"):
            self.logit_softcap = None
        for lc in self.layers:
            if lc.get("type") != "parallel":
                raise ValueError(f"unknown Nabelix layer type {lc.get('type')!r}")
            kind = (lc.get("mlp") or {}).get("kind", "dense")
            if kind != "dense":
                raise ValueError(f"unknown Nabelix feed-forward kind {kind!r}")
        ec = self.neuron_config
        if ec.tp_degree != 1:
            raise ValueError("Nabelix runs with tp_degree=1")
        # KV is paged; recurrent state has one slot per batch row
        ec.is_block_kv_layout = True

    @classmethod
    def from_hf_config(cls, model_path: str, neuron_config=None, **overrides):
        """Sizes that config.json leaves to the tensors' shapes (the ranks
        of the two-stage decay and gate projections) are read from the
        checkpoint header."""
        import json
        import os

        with open(os.path.join(model_path, "config.json")) as f:
            hf = json.load(f)
        hf.update(overrides)
        ckpt = os.path.join(model_path, "model.safetensors")
        if os.path.exists(ckpt):
            from safetensors import safe_open

            with safe_open(ckpt, framework="pt") as st:
                names = set(st.keys())

                def shape(name):
                    return st.get_slice(name).get_shape() if name in names else None

                emb = shape("embed")
                if emb:
                    hf.setdefault("vocab", emb[0])
                    hf.setdefault("width", emb[1])
                c0 = shape("l0.canon1")
                if c0 and not hf.get("canon"):
                    hf["canon"] = {"taps": c0[1]}
                for i, lc in enumerate(hf["layers"]):
                    rc = lc["mixer"]["right"]
                    rc["decay_rank"] = shape(f"l{i}.mix.right.a1")[0]
                    rc["gate_rank"] = shape(f"l{i}.mix.right.g1")[0]
                    # sizes the file may leave to the tensors
                    cv = shape(f"l{i}.mix.right.q.conv")
                    if cv and "conv" not in rc:
                        rc["conv"] = cv[1]
                    gate = shape(f"l{i}.mlp.gate")
                    if gate and isinstance(lc.get("mlp"), dict) and "ff" not in lc["mlp"]:
                        lc["mlp"]["ff"] = gate[0]
        return cls(neuron_config=neuron_config, **hf)

    def run_order(self) -> List[int]:
        """Layer index of every layer run, in execution order."""
        lp = self.loop
        n = len(self.layers)
        order = list(range(lp["start"]))
        for _ in range(lp["times"]):
            order += list(range(lp["start"], lp["stop"]))
        return order + list(range(lp["stop"], n))

    def pass_starts(self) -> List[int]:
        """Run indices that open a repeated pass after the first."""
        lp = self.loop
        span = lp["stop"] - lp["start"]
        if span <= 0:
            return []
        return [lp["start"] + t * span for t in range(1, lp["times"])]


class NabelixParallelMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        lc, rc = mc["left"], mc["right"]
        self.left_scale = float(mc["left_scale"])
        self.right_scale = float(mc["right_scale"])
        self.left = DistanceBiasWindowAttention(
            lc["heads"], lc["kv_heads"], lc["dim"], lc["vdim"], lc["scale"],
            lc["mask"]["size"], lc["mask"].get("keep_first", 0))
        self.decay_rank = int(rc["decay_rank"])
        self.gate_rank = int(rc["gate_rank"])
        self.right = GatedDeltaRule(
            rc["heads"], rc["kv_heads"], rc["dim"], rc["vdim"], rc["conv"],
            self.decay_rank, self.gate_rank, eps, dtype)
        # one GEMM for every projection that reads the layer input
        H, G, Dk, Dv = lc["heads"], lc["kv_heads"], lc["dim"], lc["vdim"]
        self.splits = [H * Dk, G * Dk, G * Dv, H * Dv,        # left q k v gate
                       self.right.qkv_channels, rc["heads"],  # right q|k|v, beta
                       self.decay_rank + self.gate_rank]      # low-rank first stages
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.left_o = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)
        self.right_o = RowParallelLinear(rc["heads"] * rc["vdim"], width, dtype=dtype,
                                         tp_degree=1)

    def forward(self, h, kv_mgr, run_idx: int, step):
        y = self.in_proj(h)
        lq, lk, lv, lg, rqkv, rb, rag = torch.split(y, self.splits, dim=-1)
        left = self.left(lq, lk, lv, kv_mgr, run_idx, step, gate=lg)
        right = self.right(rqkv, rb, rag, kv_mgr.state, f"run{run_idx}", step)
        return self.left_o(left), self.right_o(right)


class NabelixLayer(nn.Module):
    def __init__(self, config: NabelixInferenceConfig, layer_idx: int):
        super().__init__()
        ec = config.neuron_config
        lc = config.layers[layer_idx]
        eps = config.norm["eps"]
        W = config.width
        self.out_dtype = ec.torch_dtype
        self.norm1 = LayerNorm(W, eps=eps)
        self.canon = CausalShortConv(W, config.canon["taps"], residual=True)
        self.mixer = NabelixParallelMixer(W, lc["mixer"], eps, ec.torch_dtype)
        self.mlp = None
        if lc.get("mlp"):
            self.norm2 = LayerNorm(W, eps=eps)
            self.mlp = GatedMLP(W, lc["mlp"]["ff"], tp_degree=1, dtype=ec.torch_dtype,
                                hidden_act="gelu_pytorch_tanh", fused_gate_up=True)
            self.mlp.act_mul_fused = seqmix.gelu_tanh_mul_fused

    def kv_shape(self):
        return self.mixer.left.kv_shape()

    def state_shapes(self) -> Dict[str, tuple]:
        out = {"canon": self.canon.state_shape()}
        out.update(self.mixer.right.state_shapes())
        return out

    def forward(self, x, kv_mgr, run_idx: int):
        step = kv_mgr.step
        hn = seqmix.layer_norm(x, self.norm1.weight, self.norm1.eps, torch.float32)
        h = self.canon(hn, kv_mgr.state.get(f"run{run_idx}.canon"), step,
                       out_dtype=self.out_dtype)
        left, right = self.mixer(h, kv_mgr, run_idx, step)
        seqmix.residual_add(x, left, self.mixer.left_scale, right, self.mixer.right_scale)
        if self.mlp is not None:
            n = seqmix.layer_norm(x, self.norm2.weight, self.norm2.eps, self.out_dtype)
            seqmix.residual_add(x, self.mlp(n))
        return x


class _FinalNorm(LayerNorm):
    def __init__(self, width, eps, out_dtype):
        super().__init__(width, eps=eps)
        self.out_dtype = out_dtype

    def forward(self, x, residual=None):
        return seqmix.layer_norm(x, self.weight, self.eps, self.out_dtype)


class NabelixModel(HybridDecoderModel):
    def build_layers(self, config) -> nn.ModuleList:
        return nn.ModuleList(NabelixLayer(config, i) for i in range(len(config.layers)))

    def build_norm(self, config) -> nn.Module:
        return _FinalNorm(config.width, config.norm["eps"], config.neuron_config.torch_dtype)

    def run_order(self, config):
        self._pass_starts = set(config.pass_starts())
        return config.run_order()

    def before_layer_run(self, run_idx, h, h_embed):
        if run_idx == 0:
            return h.clone()          # layers update the stream in place
        if run_idx in self._pass_starts:
            return seqmix.residual_add(h, h_embed)
        return h

    def finalize_logits(self, logits):
        cap = self.config.logit_softcap
        return seqmix.softcap(logits, float(cap)) if cap else logits.float()


class NabelixForCausalLM(CausalLMBase):
    _model_cls = NabelixModel
    _config_cls = NabelixInferenceConfig

    @staticmethod
    def convert_hf_to_native_state_dict(sd: Dict[str, torch.Tensor], config) -> Dict[str, torch.Tensor]:
        dt = config.neuron_config.torch_dtype
        out: Dict[str, torch.Tensor] = {}

        def w(name):                       # projection weights: engine dtype
            return sd[name].to(dt)

        def f(name):                       # 32-bit parameters
            return sd[name].float()

        out["embed_tokens.weight"] = w("embed")
        out["lm_head.weight"] = out["embed_tokens.weight"].clone()   # saved shards may not alias
        out["norm.weight"] = f("final.norm")
        for i, lc in enumerate(config.layers):
            s, d = f"l{i}.", f"layers.{i}."
            out[d + "norm1.weight"] = f(s + "norm1")
            out[d + "canon.weight"] = f(s + "canon1")
            L, R = s + "mix.left.", s + "mix.right."
            out[d + "mixer.in_proj.weight"] = torch.cat(
                [w(L + "q"), w(L + "k"), w(L + "v"), w(L + "g"),
                 w(R + "q"), w(R + "k"), w(R + "v"), w(R + "b"),
                 w(R + "a1"), w(R + "g1")], dim=0)
            out[d + "mixer.left.r1"] = f(L + "r1")
            out[d + "mixer.left.r2"] = f(L + "r2")
            out[d + "mixer.left_o.weight"] = w(L + "o")
            out[d + "mixer.right_o.weight"] = w(R + "o")
            out[d + "mixer.right.conv.weight"] = torch.cat(
                [f(R + "q.conv"), f(R + "k.conv"), f(R + "v.conv")], dim=0)
            out[d + "mixer.right.ag2.weight"] = GatedDeltaRule.block_diagonal(
                w(R + "a2"), w(R + "g2"))
            out[d + "mixer.right.A_log"] = f(R + "A_log")
            out[d + "mixer.right.dt_bias"] = f(R + "dt_bias")
            out[d + "mixer.right.norm_weight"] = f(R + "norm")
            if lc.get("mlp"):
                out[d + "norm2.weight"] = f(s + "norm2")
                out[d + "mlp.gate_up_proj.weight"] = torch.cat(
                    [w(s + "mlp.gate"), w(s + "mlp.up")], dim=0)
                out[d + "mlp.down_proj.weight"] = w(s + "mlp.down")
        return out
