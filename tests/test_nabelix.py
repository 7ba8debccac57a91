"""Nabelix (windowed distance-bias attention + gated delta rule, side by
side) against the plain float64 oracle in ``nabelix_oracle.py``.

Every test builds its own small configuration and random weights. The
device-parametrized tests run the torch reference ops on the CPU and the
gfx950 kernels on the GPU (``-m gpu``) through the same engine code.
"""

import copy
import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nabelix_oracle as oracle  # noqa: E402

from neuronx_distributed_inference_amd.config import EngineConfig  # noqa: E402
from neuronx_distributed_inference_amd.models.nabelix.modeling_nabelix import (  # noqa: E402
    NabelixForCausalLM,
    NabelixInferenceConfig,
)
from neuronx_distributed_inference_amd.modules.attention.distance_bias import (  # noqa: E402
    DistanceBiasWindowAttention,
)
from neuronx_distributed_inference_amd.modules.conv import CausalShortConv  # noqa: E402
from neuronx_distributed_inference_amd.modules.kvcache.block_kv_cache_manager import (  # noqa: E402
    BlockKVCacheManager,
    generate_slot_mapping,
)
from neuronx_distributed_inference_amd.modules.linear_recurrence import GatedDeltaRule  # noqa: E402
from neuronx_distributed_inference_amd.ops import seqmix  # noqa: E402
from neuronx_distributed_inference_amd.serving import ServingEngine  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32 = torch.float32


# ---------------------------------------------------------------- builders
def left_cfg(heads=4, kv_heads=2, dim=8, vdim=16, size=6, keep=2, scale=0.3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale, "mask": {"size": size, "keep_first": keep}}


def right_cfg(heads=4, kv_heads=2, dim=8, vdim=4, conv=2, decay_rank=3, gate_rank=5):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "conv": conv, "decay_rank": decay_rank, "gate_rank": gate_rank}


def layer_cfg(left=None, right=None, ff=48, ls=1.3, rs=0.7):
    return {"type": "parallel",
            "mixer": {"left": left or left_cfg(), "right": right or right_cfg(),
                      "left_scale": ls, "right_scale": rs},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model_cfg(layers=None, width=32, vocab=40, taps=3, loop=None, softcap=12.0, eps=1e-5):
    layers = layers or [layer_cfg(), layer_cfg(), layer_cfg()]
    return {"architecture": "Nabelix", "width": width, "vocab": vocab,
            "layers": layers, "canon": {"taps": taps},
            "loop": loop or {"start": 1, "stop": 3, "times": 2},
            "norm": {"eps": eps}, "logit_softcap": softcap}


def varied_cfg():
    """Per-layer sizes differ; one layer has no feed-forward and no kept
    tokens; equal and unequal head counts / head sizes both occur."""
    return model_cfg(layers=[
        layer_cfg(left_cfg(4, 4, 8, 8, size=5, keep=0), right_cfg(2, 1, 16, 8, conv=3), ff=0),
        layer_cfg(left_cfg(6, 2, 4, 12, size=9, keep=3), right_cfg(3, 3, 4, 20, conv=4, decay_rank=2),
                  ff=24, ls=0.5, rs=2.0),
        layer_cfg(left_cfg(2, 1, 16, 4, size=64, keep=1), right_cfg(4, 2, 8, 8, conv=1), ff=40),
    ], width=24, vocab=33, taps=2, loop={"start": 0, "stop": 2, "times": 3}, softcap=7.5)


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors, values exactly representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    Wd = cfg["width"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def uni(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).bfloat16().float()

    def lin(o, i, gain=1.0):
        return rnd(o, i, std=gain / i ** 0.5)

    W["embed"] = rnd(cfg["vocab"], Wd)
    W["final.norm"] = (1 + rnd(Wd, std=0.1)).bfloat16().float()
    for i, lc in enumerate(cfg["layers"]):
        p = "l%d." % i
        W[p + "norm1"] = (1 + rnd(Wd, std=0.1)).bfloat16().float()
        W[p + "canon1"] = rnd(Wd, cfg["canon"]["taps"], std=0.4)
        L, R = lc["mixer"]["left"], lc["mixer"]["right"]
        a = p + "mix.left."
        W[a + "q"] = lin(L["heads"] * L["dim"], Wd, 2.0)
        W[a + "k"] = lin(L["kv_heads"] * L["dim"], Wd, 2.0)
        W[a + "v"] = lin(L["kv_heads"] * L["vdim"], Wd)
        W[a + "g"] = lin(L["heads"] * L["vdim"], Wd)
        W[a + "o"] = lin(Wd, L["heads"] * L["vdim"])
        W[a + "r1"] = uni(L["heads"], 0.2, 1.5)
        W[a + "r2"] = uni(L["heads"], 0.1, 2.0)
        b = p + "mix.right."
        for n, ch in (("q", R["kv_heads"] * R["dim"]), ("k", R["kv_heads"] * R["dim"]),
                      ("v", R["heads"] * R["vdim"])):
            W[b + n] = lin(ch, Wd, 2.0)
            W[b + n + ".conv"] = rnd(ch, R["conv"], std=0.6)
        W[b + "b"] = lin(R["heads"], Wd)
        W[b + "A_log"] = uni(R["heads"], -1.0, 0.5)
        W[b + "norm"] = (1 + rnd(R["vdim"], std=0.1)).bfloat16().float()
        W[b + "a1"] = lin(R["decay_rank"], Wd)
        W[b + "a2"] = lin(R["heads"] * R["dim"], R["decay_rank"])
        W[b + "dt_bias"] = rnd(R["heads"] * R["dim"])
        W[b + "g1"] = lin(R["gate_rank"], Wd)
        W[b + "g2"] = lin(R["heads"] * R["vdim"], R["gate_rank"])
        W[b + "o"] = lin(Wd, R["heads"] * R["vdim"])
        if lc["mlp"]:
            W[p + "norm2"] = (1 + rnd(Wd, std=0.1)).bfloat16().float()
            W[p + "mlp.gate"] = lin(lc["mlp"]["ff"], Wd)
            W[p + "mlp.up"] = lin(lc["mlp"]["ff"], Wd)
            W[p + "mlp.down"] = lin(Wd, lc["mlp"]["ff"])
    return W


def make_engine(cfg, W, device="cpu", dtype="float32", slots=3, page=4, pages=40,
                max_len=96, **engine_kw):
    ec = EngineConfig(batch_size=slots, max_batch_size=slots, kv_cache_batch_size=slots,
                      seq_len=max_len, max_length=max_len, torch_dtype=dtype, tp_degree=1,
                      is_block_kv_layout=True, pa_block_size=page, pa_num_blocks=pages,
                      enable_hip_graphs=False)
    config = NabelixInferenceConfig(neuron_config=ec, **copy.deepcopy(cfg))
    model = NabelixForCausalLM(config)
    sd = NabelixForCausalLM.convert_hf_to_native_state_dict(W, config)
    missing, unexpected = model.model.load_state_dict(sd, strict=False)
    assert not unexpected and all(m.startswith("kv_mgr.") for m in missing), (missing, unexpected)
    model = model.to(device).eval()
    engine_kw.setdefault("capture_decode", False)
    engine_kw.setdefault("async_depth", 1)
    return ServingEngine(model, max_slots=slots, **engine_kw)


def feed(engine, tokens, cuts):
    """One request alone, fed in portions of the given sizes; logits (T, V)."""
    req = engine.admit()
    out, at = [], 0
    for n in cuts:
        lg = engine.forced_step([(req, torch.tensor(tokens[at:at + n]))])
        out.append(lg[0, :n].float().cpu())
        at += n
    assert at == len(tokens)
    engine.release(req)
    return torch.cat(out)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def close(got, want, tol, rtol=0.0):
    """|got - want| <= tol + rtol * |want| everywhere."""
    excess = ((got.double() - want.double()).abs() - rtol * want.double().abs()).max().item()
    assert excess < tol, excess


# ----------------------------------------------------- mechanisms, alone
@pytest.mark.parametrize("device", DEVICES)
def test_layer_norm_op(device):
    torch.manual_seed(1)
    x = torch.randn(7, 37) * 3 + 1.5
    w = torch.randn(37)
    got = seqmix.layer_norm(x.to(device), w.to(device), 1e-3, F32).cpu()
    close(got, oracle.layer_norm(x.double(), w.double(), 1e-3), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("ff", [12, 16, 40])          # scalar and 8-wide kernel paths
def test_gelu_mul_and_residual_ops(device, ff):
    torch.manual_seed(16)
    gu = torch.randn(5, 2 * ff) * 2
    want = oracle.gelu_tanh(gu[:, :ff].double()) * gu[:, ff:].double()
    close(seqmix.gelu_tanh_mul_fused(gu.to(device)).cpu(), want, 1e-5)
    x, a, b = torch.randn(3, 7), torch.randn(3, 7), torch.randn(3, 7)
    got = seqmix.residual_add(x.clone().to(device), a.to(device), 1.25, b.to(device), 0.5).cpu()
    close(got, x.double() + 1.25 * a.double() + 0.5 * b.double(), 1e-5)
    lg = torch.randn(4, 9) * 40
    close(seqmix.softcap(lg.to(device), 30.0).cpu(), 30.0 * torch.tanh(lg.double() / 30.0), 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("act,residual", [("none", True), ("silu", False)])
@pytest.mark.parametrize("C", [10, 16])               # per-element and 8-channel tiled kernels
def test_short_conv_portions_and_slots(device, taps, act, residual, C):
    """Two sequences in different slots fed in unequal portions (down to one
    token) against the whole-sequence convolution."""
    torch.manual_seed(2)
    T = 17
    conv = CausalShortConv(C, taps, activation=act, residual=residual)
    conv.weight.data = torch.randn(C, taps)
    conv = conv.to(device)
    xs = [torch.randn(T, C), torch.randn(T - 4, C)]
    want = []
    for x in xs:
        y = oracle.causal_conv(x.double(), conv.weight.double().cpu())
        if act == "silu":
            y = torch.nn.functional.silu(y)
        want.append(y + x.double() if residual else y)
    tail = torch.randn(3, max(taps - 1, 0), C).to(device)   # dirty: start must read as zeros
    slots = [2, 0]
    cuts = [[5, 1, 2, 9], [1, 3, 1, 8]]
    got = [[], []]
    at = [0, 0]
    for step_i in range(4):
        n = [cuts[0][step_i], cuts[1][step_i]]
        L = max(n)
        x = torch.zeros(2, L, C)
        pos = torch.full((2, L), -1)
        for b in range(2):
            x[b, :n[b]] = xs[b][at[b]:at[b] + n[b]]
            pos[b, :n[b]] = torch.arange(at[b], at[b] + n[b])
        st = seqmix.StepLayout(pos.to(device), torch.tensor(slots).to(device))
        y = conv(x.to(device), tail, st).cpu()
        for b in range(2):
            got[b].append(y[b, :n[b]])
            at[b] += n[b]
    for b in range(2):
        close(torch.cat(got[b]), want[b], 1e-5)


def _attention_alone(device, L, T, spikes, page=4, cuts=None, dtype=F32, tol=2e-5, rtol=0.0):
    """Attention core on its own paged cache. `spikes`: (query i, key j) pairs
    whose score is made to dominate if (and only if) the mask lets it."""
    torch.manual_seed(3)
    Wd = 12
    H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    h = torch.randn(T, Wd).double()
    W = {"q": torch.randn(H * D, Wd) * 0.3, "k": torch.randn(G * D, Wd) * 0.3,
         "v": torch.randn(G * Dv, Wd), "g": torch.randn(H * Dv, Wd),
         "o": torch.eye(H * Dv), "r1": torch.rand(H) + 0.2, "r2": torch.rand(H) + 0.1}
    W = {k: v.double() for k, v in W.items()}
    q = (h @ W["q"].T).view(T, H, D)
    k = (h @ W["k"].T).view(T, G, D)
    for i, j in spikes:                       # make key j stand out for query i
        d = torch.zeros(D, dtype=torch.float64)
        d[(i + j) % D] = 1.0
        k[j] += 6.0 * d
        q[i] += 6.0 * d
    v = h @ W["v"].T
    gate = h @ W["g"].T
    if dtype != F32:      # both sides see the values the kernel is given
        q, k, v, gate = (t.to(dtype).double() for t in (q, k, v, gate))
    # oracle with the same (spiked) q/k: feed them through identity projections
    hq = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v, gate], 1)
    o0, o1, o2 = H * D, H * D + G * D, H * D + G * D + G * Dv
    Wo = {"p.q": torch.eye(hq.shape[1])[:o0], "p.k": torch.eye(hq.shape[1])[o0:o1],
          "p.v": torch.eye(hq.shape[1])[o1:o2], "p.g": torch.eye(hq.shape[1])[o2:],
          "p.o": W["o"], "p.r1": W["r1"], "p.r2": W["r2"]}
    Wo = {kk: vv.double() for kk, vv in Wo.items()}
    want = oracle.biased_window_attention(hq, Wo, "p.", L)

    att = DistanceBiasWindowAttention(H, G, D, Dv, L["scale"], L["mask"]["size"],
                                      L["mask"]["keep_first"])
    att.r1.data, att.r2.data = W["r1"].float(), W["r2"].float()
    att = att.to(device)
    nblk = (T + page - 1) // page
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=nblk + 3, block_size=page, dtype=dtype,
                              tp_degree=1, layer_kv_shapes=[(G, D, Dv)]).to(device)
    perm = torch.randperm(nblk + 3)[:nblk]              # scattered pages
    bt = perm.view(1, nblk).to(device)
    got, at = [], 0
    for n in cuts or [T]:
        pos = torch.arange(at, at + n).view(1, n).to(device)
        mgr.set_step_context(bt, generate_slot_mapping(bt, pos, page))
        st = seqmix.StepLayout(pos, torch.zeros(1, dtype=torch.long, device=device))
        sl = slice(at, at + n)
        y = att(q[sl].reshape(1, n, -1).to(device, dtype), k[sl].reshape(1, n, -1).to(device, dtype),
                v[sl].view(1, n, -1).to(device, dtype), mgr, 0, st,
                gate=gate[sl].view(1, n, -1).to(device, dtype))
        got.append(y[0].float().cpu())
        at += n
    close(torch.cat(got), want, tol, rtol)


EDGE = left_cfg(heads=4, kv_heads=2, dim=8, vdim=16, size=7, keep=3, scale=0.5)
# query 20: window covers 14..20, kept 0..2. Inside/outside each edge, a far
# key, page borders (page 4: keys 15|16), and the very first tokens
EDGE_SPIKES = [(20, 14), (21, 14), (22, 2), (23, 3), (24, 0), (25, 16), (26, 15),
               (19, 19), (2, 0), (1, 1), (30, 10), (29, 23)]


@pytest.mark.parametrize("device", DEVICES)
def test_attention_edges_prompt(device):
    _attention_alone(device, EDGE, 33, EDGE_SPIKES)


@pytest.mark.parametrize("device", DEVICES)
def test_attention_edges_decoded(device):
    _attention_alone(device, EDGE, 33, EDGE_SPIKES, cuts=[5] + [1] * 28)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [
    left_cfg(2, 2, 4, 4, size=3, keep=0), left_cfg(6, 1, 12, 20, size=70, keep=5),
    left_cfg(3, 3, 5, 7, size=1, keep=1), left_cfg(2, 1, 8, 130, size=8, keep=9)])
def test_attention_other_shapes(device, L):
    _attention_alone(device, L, 23, [(22, 3), (12, 5)], page=8, cuts=[2, 7, 1, 13])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [100] + [1] * 50])
def test_attention_far_keys_among_many(device, cuts):
    """150 tokens: a kept first token 145 positions back, the first token
    that is NOT kept, and the keys on both sides of the window's far edge,
    each made to dominate its query's scores if the mask lets it."""
    L = left_cfg(2, 1, 8, 8, size=40, keep=5, scale=0.5)
    spikes = [(149, 4), (148, 5), (147, 108), (146, 106), (120, 0), (110, 70), (109, 70)]
    _attention_alone(device, L, 150, spikes, page=16, cuts=cuts)


@pytest.mark.gpu
def test_attention_bf16_long_window_gpu():
    L = left_cfg(8, 2, 64, 128, size=200, keep=20, scale=0.1)
    _attention_alone("cuda", L, 300, [(290, 91), (290, 90), (299, 19)], page=64,
                     cuts=[150, 1, 1, 148], dtype=torch.bfloat16, tol=0.01, rtol=0.01)


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (left_cfg(4, 2, 64, 64, size=7, keep=3, scale=0.5), None),
    (left_cfg(4, 2, 64, 64, size=7, keep=3, scale=0.5), [5, 9, 2, 17]),
    (left_cfg(8, 1, 128, 64, size=40, keep=0, scale=0.3), [3, 30]),
    (left_cfg(2, 2, 64, 128, size=100, keep=6, scale=0.3), [33]),
    (left_cfg(16, 1, 128, 128, size=20, keep=2, scale=0.2), [20, 13]),
    (left_cfg(6, 2, 32, 128, size=9, keep=4, scale=0.4), [2, 31]),
    (left_cfg(5, 1, 64, 32, size=12, keep=1, scale=0.4), [16, 16, 1]),
])
def test_attention_edges_bf16_matrix_path_gpu(L, cuts):
    """bf16 prompt portions with common head shapes take the matrix-core
    kernel: same spiked edges (window, kept-first, page border, far)."""
    _attention_alone("cuda", L, 33, EDGE_SPIKES, page=8, cuts=cuts,
                     dtype=torch.bfloat16, tol=0.01, rtol=0.01)


def _delta_alone(device, R, T, cuts, slots=(1,), eps=1e-4):
    torch.manual_seed(4)
    Wd = 10
    H, G, D, Dv = R["heads"], R["kv_heads"], R["dim"], R["vdim"]
    h = torch.randn(T, Wd).double()
    W = {"q": torch.randn(G * D, Wd), "k": torch.randn(G * D, Wd), "v": torch.randn(H * Dv, Wd),
         "q.conv": torch.randn(G * D, R["conv"]) * 0.6, "k.conv": torch.randn(G * D, R["conv"]) * 0.6,
         "v.conv": torch.randn(H * Dv, R["conv"]) * 0.6, "b": torch.randn(H, Wd),
         "A_log": torch.rand(H) - 1.0, "norm": torch.rand(Dv) + 0.5,
         "a1": torch.randn(R["decay_rank"], Wd), "a2": torch.randn(H * D, R["decay_rank"]),
         "dt_bias": torch.randn(H * D), "g1": torch.randn(R["gate_rank"], Wd),
         "g2": torch.randn(H * Dv, R["gate_rank"]), "o": torch.eye(H * Dv)}
    W = {"p." + k: v.double() for k, v in W.items()}
    want = oracle.gated_delta_rule(h, W, "p.", R, eps)

    mod = GatedDeltaRule(H, G, D, Dv, R["conv"], R["decay_rank"], R["gate_rank"], eps, F32)
    mod.conv.weight.data = torch.cat([W["p.q.conv"], W["p.k.conv"], W["p.v.conv"]]).float()
    mod.ag2.weight.data = GatedDeltaRule.block_diagonal(W["p.a2"].float(), W["p.g2"].float())
    mod.A_log.data, mod.dt_bias.data = W["p.A_log"].float(), W["p.dt_bias"].float()
    mod.norm_weight.data = W["p.norm"].float()
    mod = mod.to(device)
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=1, block_size=4, dtype=F32, tp_degree=1,
                              state_slots=3)
    for name, shape in mod.state_shapes().items():
        mgr.state.register("x." + name, shape)
    mgr = mgr.to(device)
    for t in mgr.state.tensors.values():        # dirty slots: a start must not read them
        t.data.normal_()
    qkv = torch.cat([h @ W["p.q"].T, h @ W["p.k"].T, h @ W["p.v"].T], 1).float()
    beta = (h @ W["p.b"].T).float()
    aglow = torch.cat([h @ W["p.a1"].T, h @ W["p.g1"].T], 1).float()
    got, at = [], 0
    for n in cuts:
        sl = slice(at, at + n)
        pos = torch.arange(at, at + n).view(1, n).to(device)
        st = seqmix.StepLayout(pos, torch.tensor(list(slots)).to(device))
        y = mod(qkv[sl][None].to(device), beta[sl][None].to(device), aglow[sl][None].to(device),
                mgr.state, "x", st)
        got.append(y[0].float().cpu())
        at += n
    close(torch.cat(got), want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R", [
    right_cfg(), right_cfg(2, 2, 4, 4, conv=1), right_cfg(3, 1, 12, 70, conv=4),
    right_cfg(2, 1, 40, 6, conv=3), right_cfg(1, 1, 100, 66, conv=2)])
def test_delta_rule_portions(device, R):
    _delta_alone(device, R, 27, [27])
    _delta_alone(device, R, 27, [9, 1, 1, 2, 11, 3])


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_long_decode(device):
    _delta_alone(device, right_cfg(), 90, [3] + [1] * 87)


# ------------------------------------------------------------ whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [model_cfg, varied_cfg])
def test_prefill_decode_portions_match_oracle(device, make):
    cfg = make()
    W = make_weights(cfg, seed=5)
    toks = tokens_for(cfg, 41, seed=6)
    want = oracle.forward(toks, W, cfg)
    eng = make_engine(cfg, W, device)
    whole = feed(eng, toks, [41])
    close(whole, want, 3e-4)
    stepwise = feed(eng, toks, [1] * 41)                 # token by token from the start
    close(stepwise, want, 3e-4)
    portions = feed(eng, toks, [2, 5, 2, 1, 9, 3, 2, 16, 1])
    close(portions, want, 3e-4)
    decoded = feed(eng, toks, [11] + [1] * 30)           # decodes far past every window
    close(decoded, want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_per_run(device):
    """The stream after every layer run (looped layers count each time)."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=7)
    toks = tokens_for(cfg, 9, seed=8)
    _, streams = oracle.forward(toks, W, cfg, want_streams=True)
    eng = make_engine(cfg, W, device)
    dm = eng.model.model
    seen = []
    orig = dm.before_layer_run

    def spy(ri, h, h0):
        if ri > 0:
            seen.append(h.detach().clone().cpu())
        return orig(ri, h, h0)

    dm.before_layer_run = spy
    feed(eng, toks, [9])
    assert len(seen) == streams.shape[0] - 1 == 4
    for r, s in enumerate(seen):
        close(s[0], streams[r], 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reuse(device):
    """Unequal requests side by side (portions beside single tokens, one
    request pausing) equal each request alone; slots and pages are handed
    back and used again with stale contents."""
    cfg = varied_cfg()
    W = make_weights(cfg, seed=9)
    seqs = {n: tokens_for(cfg, L, seed=10 + i)
            for i, (n, L) in enumerate([("a", 30), ("b", 7), ("c", 19), ("d", 26), ("e", 12)])}
    want = {n: oracle.forward(t, W, cfg) for n, t in seqs.items()}
    eng = make_engine(cfg, W, device, slots=3, page=4, pages=18, max_len=32)
    plan = [                                   # (name, count) per step
        [("a", 6), ("b", 1), ("c", 2)],
        [("a", 1), ("b", 3), ("c", 9)],
        [("a", 11), ("c", 1)],                 # b pauses
        [("a", 1), ("b", 3), ("c", 7)],        # b, c end
        [("a", 1), ("d", 13), ("e", 2)],       # d, e take the freed slots/pages
        [("a", 10), ("d", 1), ("e", 1)],       # a ends
        [("d", 12), ("e", 9)],
    ]
    live, at, got = {}, {n: 0 for n in seqs}, {n: [] for n in seqs}
    for step in plan:
        parts = []
        for n, c in step:
            if n not in live:
                live[n] = eng.admit()
            parts.append((live[n], torch.tensor(seqs[n][at[n]:at[n] + c])))
        lg = eng.forced_step(parts)
        for i, (n, c) in enumerate(step):
            got[n].append(lg[i, :c].float().cpu())
            at[n] += c
            if at[n] == len(seqs[n]):
                eng.release(live.pop(n))
    assert not live and eng.allocator.available() == 18 and len(eng.free_slots) == 3
    for n in seqs:
        close(torch.cat(got[n]), want[n], 3e-4)


def _oracle_greedy(cfg, W, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(oracle.forward(toks, W, cfg)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(chunk_size=4), dict(chunk_size=4, mixed_chunking=True)])
def test_greedy_generation_through_scheduler(device, kw):
    """Queue -> slots -> (chunked / mixed) prefill -> batched decode; more
    requests than slots, so slots and pages are recycled."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=11)
    prompts = [tokens_for(cfg, n, seed=20 + n) for n in (9, 5, 14, 6)]
    want = [_oracle_greedy(cfg, W, p, 7) for p in prompts]
    eng = make_engine(cfg, W, device, slots=2, page=4, pages=14, max_len=28, **kw)
    rids = [eng.add_request(torch.tensor(p), max_new_tokens=7) for p in prompts]
    out = eng.run()
    assert [out[r] for r in rids] == want


@pytest.mark.gpu
def test_greedy_generation_captured_decode_gpu():
    """The engine's default GPU configuration: hipGraph-captured decode."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=11)
    prompts = [tokens_for(cfg, n, seed=20 + n) for n in (9, 5, 14, 6)]
    want = [_oracle_greedy(cfg, W, p, 7) for p in prompts]
    eng = make_engine(cfg, W, "cuda", slots=2, page=4, pages=14, max_len=28,
                      capture_decode=True, async_depth=2)
    rids = [eng.add_request(torch.tensor(p), max_new_tokens=7) for p in prompts]
    out = eng.run()
    assert [out[r] for r in rids] == want


@pytest.mark.gpu
def test_bfloat16_serving_precision_gpu():
    """bf16 projections, fp32 stream/scores/state: close to the oracle and
    independent of how the prompt is cut, beyond rounding."""
    cfg = model_cfg(layers=[layer_cfg(left_cfg(4, 2, 32, 64, size=24, keep=4, scale=0.15),
                                      right_cfg(4, 2, 32, 64, conv=4, decay_rank=8, gate_rank=8),
                                      ff=128)] * 2,
                    width=128, vocab=96, taps=4, loop={"start": 0, "stop": 1, "times": 2})
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, seed=13)
    want = oracle.forward(toks, W, cfg)
    eng = make_engine(cfg, W, "cuda", dtype="bfloat16", page=16, pages=12, max_len=96)
    a = feed(eng, toks, [80])
    b = feed(eng, toks, [7, 30, 2, 1, 1, 39])
    scale = want.std().item()
    assert (a.double() - want).std().item() < 0.05 * scale
    assert (b.double() - want).std().item() < 0.05 * scale
    assert (a - b).double().std().item() < 0.05 * scale


def test_checkpoint_folder_and_schedule_replay(tmp_path):
    """config.json + model.safetensors on disk -> registry lookup by the
    config's architecture -> schedule replay writes the wanted logits."""
    from safetensors.torch import save_file

    from neuronx_distributed_inference_amd import trace_replay
    from neuronx_distributed_inference_amd.registry import model_type_from_config

    cfg = varied_cfg()
    W = make_weights(cfg, seed=14)
    disk = copy.deepcopy(cfg)
    for lc in disk["layers"]:                  # ranks are the tensors' business
        del lc["mixer"]["right"]["decay_rank"], lc["mixer"]["right"]["gate_rank"]
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(disk))
    save_file({k: (v.bfloat16() if v.dim() >= 1 else v) for k, v in W.items()},
              str(mdir / "model.safetensors"))
    assert model_type_from_config(str(mdir)) == "nabelix"
    a, b = tokens_for(cfg, 21, 30), tokens_for(cfg, 9, 31)
    lines = [
        {"step": 0, "entries": [{"id": "x", "tokens": a[:8], "want": [0, 7]}], "end": []},
        {"step": 1, "entries": [{"id": "x", "tokens": a[8:20], "want": []},
                                {"id": "y", "tokens": b[:1], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "y", "tokens": b[1:], "want": [7]},
                                {"id": "x", "tokens": a[20:], "want": [0]}], "end": ["x", "y"]},
    ]
    out = tmp_path / "out"
    out.mkdir()
    eng = trace_replay.build_engine(str(mdir), "float32", 128, device=torch.device("cpu"))
    said = []
    trace_replay.replay(eng, [json.dumps(x) for x in lines], str(out), said.append)
    assert said == ["done 0", "done 1", "done 2"]
    wa, wb = oracle.forward(a, W, cfg), oracle.forward(b, W, cfg)
    import numpy as np

    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
    close(g0, wa[[0, 7]], 3e-4)
    close(g1, wb[[0]], 3e-4)
    close(g2, torch.stack([wb[8], wa[20]]), 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_generate_adapter(device):
    """The plain generate() entry point (no page table passed: the model
    lays its slots out linearly over the page pool)."""
    from neuronx_distributed_inference_amd.utils.hf_adapter import (
        GenerationConfig,
        HuggingFaceGenerationAdapter,
    )

    cfg = model_cfg()
    W = make_weights(cfg, seed=15)
    prompts = [tokens_for(cfg, 8, seed=40), tokens_for(cfg, 8, seed=41)]
    want = [_oracle_greedy(cfg, W, p, 6) for p in prompts]
    eng = make_engine(cfg, W, device, slots=2, page=4, pages=16, max_len=32)
    model = eng.model
    out = HuggingFaceGenerationAdapter(model).generate(
        torch.tensor(prompts, device=device),
        generation_config=GenerationConfig(max_new_tokens=6))
    assert out[:, 8:].tolist() == want
