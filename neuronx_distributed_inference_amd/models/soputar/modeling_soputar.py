"""Soputar for MI355X: a decoder whose layers each pick one of three token
mixers and normalise the sublayer OUTPUT.

Layer: ``x += norm1(mixer(x))`` then, when the layer has a feed-forward,
``x += norm2(ff(x))``; both sublayers read the stream itself and the norms
are RMS norms with weights stored around zero (scale ``1 + w``). The stream
is the embedding times a constant. Mixers, chosen per layer by ``type``:

- ``delta``: :class:`GatedDeltaRule` with one decay per head, a silu output
  gate and full-size decay/gate projections;
- ``attention``: :class:`NormedCappedAttention` — GQA without rotation,
  whole-projection q/k norm, query temperature, tanh score cap; a layer with
  ``kv_from`` borrows another attention layer's cached keys and values;
- ``latent_attention``: :class:`LatentSinkAttention` — low-rank latent KV
  with a shared rotated key part (interleaved rotary) and a softmax sink.

Feed-forward: ``W_down(g * sigmoid(1.702 g) * (u + 1))`` with ``g`` the gate
projection clamped from above and ``u`` the up projection clamped on both
sides. Output: the same one-plus RMS norm, then an untied head.

Engine integration (shared with the other hybrid decoders through
:class:`HybridDecoderModel`): fp32 residual stream, paged KV with per-layer
page shapes (a latent layer keeps one row per token and no value pages, a
borrowing layer none at all), convolution tails and delta-rule state in the
cache manager's recurrent-state slots, one set of kernels for prompt
portions, decoded tokens and mixed batches. Every projection that reads the
stream is one fused GEMM per mixer; the post-norm residual step is one
kernel that also emits the stream in the GEMM input dtype for the next
sublayer.
"""

from __future__ import annotations

import json
import os
from typing import Dict, List

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.config import InferenceConfig
from neuronx_distributed_inference_amd.models.hybrid_base import HybridDecoderModel
from neuronx_distributed_inference_amd.models.model_base import CausalLMBase
from neuronx_distributed_inference_amd.modules.attention.capped_attention import (
    NormedCappedAttention,
)
from neuronx_distributed_inference_amd.modules.attention.latent_attention import (
    LatentSinkAttention,
)
from neuronx_distributed_inference_amd.modules.linear_recurrence import GatedDeltaRule
from neuronx_distributed_inference_amd.modules.mlp import GatedMLP
from neuronx_distributed_inference_amd.modules.norm import StreamRMSNorm
from neuronx_distributed_inference_amd.parallel.layers import (
    ColumnParallelLinear,
    RowParallelLinear,
)

MIXER_TYPES = ("delta", "attention", "latent_attention")
GLU_ALPHA = 1.702          # fixed by the design; the clamp limit is per model


class SoputarInferenceConfig(InferenceConfig):
    """Reads the checkpoint's ``config.json`` as is (keys: architecture,
    width, vocab, embedding.scale, layers[], norm.eps) and derives the
    generic attribute names the engine uses."""

    def get_required_attributes(self) -> List[str]:
        return ["width", "vocab", "layers", "norm"]

    def add_derived_config(self):
        if not hasattr(self, "layers"):
            return
        if not getattr(self, "embedding", None):
            self.embedding = {"scale": 1.0}       # a file without the entry scales nothing
        self.hidden_size = self.width
        self.vocab_size = self.vocab
        self.num_hidden_layers = len(self.layers)
        self.tie_word_embeddings = False
        for i, lc in enumerate(self.layers):
            if lc.get("type") not in MIXER_TYPES:
                raise ValueError(f"unknown Soputar layer type {lc.get('type')!r}")
            fc = lc.get("mlp")
            if fc and fc.get("kind", "dense") != "dense":
                raise ValueError(f"unknown Soputar feed-forward kind {fc.get('kind')!r}")
            src = lc["mixer"].get("kv_from")
            if src is not None:
                sc = self.layers[src]
                if lc["type"] != "attention" or sc["type"] != "attention" or \
                        sc["mixer"].get("kv_from") is not None or src >= i:
                    raise ValueError(f"layer {i}: kv_from must name an earlier attention "
                                     "layer that owns its keys and values")
                for key in ("kv_heads", "dim", "vdim"):
                    if sc["mixer"][key] != lc["mixer"][key]:
                        raise ValueError(f"layer {i}: {key} differs from the lender's")
        ec = self.neuron_config
        if ec.tp_degree != 1:
            raise ValueError("Soputar runs with tp_degree=1")
        ec.is_block_kv_layout = True

    @classmethod
    def from_hf_config(cls, model_path: str, neuron_config=None, **overrides):
        """Sizes that config.json leaves out are taken from the tensors'
        shapes in the checkpoint header, where a shape determines them."""
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
                for i, lc in enumerate(hf["layers"]):
                    _fill_from_shapes(lc, lambda n, i=i: shape(f"l{i}.{n}"))
        return cls(neuron_config=neuron_config, **hf)


def _fill_from_shapes(lc: dict, shape):
    mc = lc["mixer"]
    fc = lc.get("mlp")
    if isinstance(fc, dict) and "ff" not in fc and shape("mlp.gate"):
        fc["ff"] = shape("mlp.gate")[0]
    if lc["type"] == "delta":
        if "conv" not in mc and shape("mix.q.conv"):
            mc["conv"] = shape("mix.q.conv")[1]
        if "heads" not in mc and shape("mix.A_log"):
            mc["heads"] = shape("mix.A_log")[0]
        if "vdim" not in mc and shape("mix.norm"):
            mc["vdim"] = shape("mix.norm")[0]
        if "dim" not in mc and "kv_heads" in mc and shape("mix.q"):
            mc["dim"] = shape("mix.q")[0] // mc["kv_heads"]
        if "kv_heads" not in mc and "dim" in mc and shape("mix.q"):
            mc["kv_heads"] = shape("mix.q")[0] // mc["dim"]
    elif lc["type"] == "attention":
        if "dim" not in mc and "heads" in mc and shape("mix.q"):
            mc["dim"] = shape("mix.q")[0] // mc["heads"]
        if "heads" not in mc and "dim" in mc and shape("mix.q"):
            mc["heads"] = shape("mix.q")[0] // mc["dim"]
        if "kv_heads" not in mc and "dim" in mc and shape("mix.k"):
            mc["kv_heads"] = shape("mix.k")[0] // mc["dim"]
        if "vdim" not in mc and "kv_heads" in mc and shape("mix.v"):
            mc["vdim"] = shape("mix.v")[0] // mc["kv_heads"]
    elif lc["type"] == "latent_attention":
        if "heads" not in mc and shape("mix.sink"):
            mc["heads"] = shape("mix.sink")[0]
        if "kv_rank" not in mc and shape("mix.dkv.norm"):
            mc["kv_rank"] = shape("mix.dkv.norm")[0]
        if "rot_dim" not in mc and "kv_rank" in mc and shape("mix.dkv"):
            mc["rot_dim"] = shape("mix.dkv")[0] - mc["kv_rank"]
        if "dim" not in mc and "heads" in mc and shape("mix.uk"):
            mc["dim"] = shape("mix.uk")[0] // mc["heads"]
        if "vdim" not in mc and "heads" in mc and shape("mix.uv"):
            mc["vdim"] = shape("mix.uv")[0] // mc["heads"]


# ----------------------------------------------------------------- mixers
class SoputarDeltaMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        self.core = GatedDeltaRule(H, G, D, Dv, mc["conv"], 0, 0, eps, dtype,
                                   decay_per_channel=False, gate_act="silu")
        # one GEMM for everything that reads the stream: q|k|v, gate, beta, decay
        self.splits = [self.core.qkv_channels, H * Dv, H, H]
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)

    def kv_shape(self):
        return None

    def state_shapes(self):
        return self.core.state_shapes()

    def forward(self, h, kv_mgr, run_idx: int, step):
        qkv, gate, beta, a = torch.split(self.in_proj(h), self.splits, dim=-1)
        y = self.core(qkv, beta, a, kv_mgr.state, f"run{run_idx}", step, gate=gate)
        return self.o_proj(y)

    @staticmethod
    def convert(sd, s, d, w, f, out):
        out[d + "in_proj.weight"] = torch.cat(
            [w(s + "q"), w(s + "k"), w(s + "v"), w(s + "g"), w(s + "b"), w(s + "a")], dim=0)
        out[d + "core.conv.weight"] = torch.cat(
            [f(s + "q.conv"), f(s + "k.conv"), f(s + "v.conv")], dim=0)
        out[d + "core.A_log"] = f(s + "A_log")
        out[d + "core.dt_bias"] = f(s + "dt_bias")
        out[d + "core.norm_weight"] = f(s + "norm")
        out[d + "o_proj.weight"] = w(s + "o")


class SoputarAttentionMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        self.source = mc.get("kv_from")
        qt = mc.get("q_temp")
        self.core = NormedCappedAttention(
            H, G, D, Dv, mc["scale"], eps, softcap=mc.get("softcap") or 0.0,
            q_temp=(qt["coef"], qt["every"]) if qt else None,
            owns_kv=self.source is None)
        self.splits = [H * D] + ([G * D, G * Dv] if self.source is None else [])
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)

    def kv_shape(self):
        return self.core.kv_shape()

    def state_shapes(self):
        return {}

    def forward(self, h, kv_mgr, run_idx: int, step):
        y = self.in_proj(h)
        if self.source is None:
            q, k, v = torch.split(y, self.splits, dim=-1)
        else:
            q, k, v = y, None, None
        return self.o_proj(self.core(q, k, v, kv_mgr, run_idx, step))

    @staticmethod
    def convert(sd, s, d, w, f, out):
        own = (s + "k") in sd
        out[d + "in_proj.weight"] = torch.cat(
            [w(s + "q"), w(s + "k"), w(s + "v")], dim=0) if own else w(s + "q")
        out[d + "core.q_norm"] = f(s + "q.norm")
        if own:
            out[d + "core.k_norm"] = f(s + "k.norm")
        out[d + "o_proj.weight"] = w(s + "o")


class SoputarLatentMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
        rot = mc.get("rot") or {}
        self.core = LatentSinkAttention(
            H, D, R, Dv, C, mc["scale"], eps, rot.get("base", 10000.0),
            rot.get("dims", R), dtype)
        self.splits = [H * (D + R), C + R]
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)

    def kv_shape(self):
        return self.core.kv_shape()

    def state_shapes(self):
        return {}

    def forward(self, h, kv_mgr, run_idx: int, step):
        q, dkv = torch.split(self.in_proj(h), self.splits, dim=-1)
        return self.o_proj(self.core(q, dkv, kv_mgr, run_idx, step))

    @staticmethod
    def convert(sd, s, d, w, f, out):
        out[d + "in_proj.weight"] = torch.cat([w(s + "q"), w(s + "dkv")], dim=0)
        out[d + "core.latent_norm.weight"] = f(s + "dkv.norm")
        H = sd[s + "sink"].shape[0]
        uk, uv = w(s + "uk"), w(s + "uv")
        C = uk.shape[1]
        out[d + "core.uk"] = uk.view(H, -1, C).contiguous()                   # (H, dim, C)
        out[d + "core.uv"] = uv.view(H, -1, C).contiguous()                   # (H, vdim, C)
        out[d + "core.sink"] = f(s + "sink")
        out[d + "o_proj.weight"] = w(s + "o")


_MIXERS = {"delta": SoputarDeltaMixer, "attention": SoputarAttentionMixer,
           "latent_attention": SoputarLatentMixer}


class SoputarLayer(nn.Module):
    def __init__(self, config: SoputarInferenceConfig, layer_idx: int):
        super().__init__()
        ec = config.neuron_config
        lc = config.layers[layer_idx]
        eps = config.norm["eps"]
        W = config.width
        self.dtype = ec.torch_dtype
        self.mixer = _MIXERS[lc["type"]](W, lc["mixer"], eps, ec.torch_dtype)
        self.norm1 = StreamRMSNorm(W, eps=eps, one_plus=True)
        self.mlp = None
        fc = lc.get("mlp")
        if fc:
            self.norm2 = StreamRMSNorm(W, eps=eps, one_plus=True)
            self.mlp = GatedMLP(W, fc["ff"], tp_degree=1, dtype=ec.torch_dtype,
                                hidden_act="clamped_swiglu", fused_gate_up=True,
                                act_limit=fc["limit"], act_alpha=GLU_ALPHA)

    def kv_shape(self):
        return self.mixer.kv_shape()

    def kv_source(self):
        return getattr(self.mixer, "source", None)

    def state_shapes(self) -> Dict[str, tuple]:
        return self.mixer.state_shapes()

    def forward(self, x, kv_mgr, run_idx: int):
        step = kv_mgr.step
        # the stream in the GEMM input dtype: left by the previous sublayer's
        # residual-norm kernel, or cast here for the first layer
        h = step.stream_copy if step.stream_copy is not None else x.to(self.dtype)
        h = self.norm1.add_into(x, self.mixer(h, kv_mgr, run_idx, step), self.dtype)
        if self.mlp is not None:
            h = self.norm2.add_into(x, self.mlp(h), self.dtype)
        step.stream_copy = h
        return x


class SoputarModel(HybridDecoderModel):
    def __init__(self, config):
        self.embed_scale = float(config.embedding["scale"])
        super().__init__(config)

    def build_layers(self, config) -> nn.ModuleList:
        return nn.ModuleList(SoputarLayer(config, i) for i in range(len(config.layers)))

    def build_norm(self, config) -> nn.Module:
        return StreamRMSNorm(config.width, eps=config.norm["eps"], one_plus=True,
                             out_dtype=config.neuron_config.torch_dtype)

    def begin_step(self, position_ids, seq_ids, block_table):
        block_table = super().begin_step(position_ids, seq_ids, block_table)
        self.kv_mgr.step.stream_copy = None
        return block_table

    def finalize_logits(self, logits):
        return logits.float()


class SoputarForCausalLM(CausalLMBase):
    _model_cls = SoputarModel
    _config_cls = SoputarInferenceConfig

    @staticmethod
    def convert_hf_to_native_state_dict(sd: Dict[str, torch.Tensor], config) -> Dict[str, torch.Tensor]:
        dt = config.neuron_config.torch_dtype
        out: Dict[str, torch.Tensor] = {}

        def w(name):                       # projection weights: engine dtype
            return sd[name].to(dt)

        def f(name):                       # 32-bit parameters
            return sd[name].float()

        out["embed_tokens.weight"] = w("embed")
        out["lm_head.weight"] = w("head")
        out["norm.weight"] = f("final.norm")
        for i, lc in enumerate(config.layers):
            s, d = f"l{i}.", f"layers.{i}."
            out[d + "norm1.weight"] = f(s + "norm1")
            _MIXERS[lc["type"]].convert(sd, s + "mix.", d + "mixer.", w, f, out)
            if lc.get("mlp"):
                out[d + "norm2.weight"] = f(s + "norm2")
                out[d + "mlp.gate_up_proj.weight"] = torch.cat(
                    [w(s + "mlp.gate"), w(s + "mlp.up")], dim=0)
                out[d + "mlp.down_proj.weight"] = w(s + "mlp.down")
        return out
