"""Soputar (post-norm decoder mixing gated-delta-rule, capped GQA and latent
sink-attention layers) against the plain float64 oracle in
``soputar_oracle.py``.

Every test builds its own small configuration and weights. The
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
import soputar_oracle as oracle  # noqa: E402

from neuronx_distributed_inference_amd.config import EngineConfig  # noqa: E402
from neuronx_distributed_inference_amd.models.soputar.modeling_soputar import (  # noqa: E402
    SoputarForCausalLM,
    SoputarInferenceConfig,
)
from neuronx_distributed_inference_amd.modules.attention.capped_attention import (  # noqa: E402
    NormedCappedAttention,
)
from neuronx_distributed_inference_amd.modules.attention.latent_attention import (  # noqa: E402
    LatentSinkAttention,
)
from neuronx_distributed_inference_amd.modules.kvcache.block_kv_cache_manager import (  # noqa: E402
    BlockKVCacheManager,
    generate_slot_mapping,
)
from neuronx_distributed_inference_amd.modules.linear_recurrence import GatedDeltaRule  # noqa: E402
from neuronx_distributed_inference_amd.ops import ref, seqmix  # noqa: E402
from neuronx_distributed_inference_amd.serving import ServingEngine  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32 = torch.float32
BF16 = torch.bfloat16
EPS = 1e-5


# ---------------------------------------------------------------- builders
def delta_cfg(heads=4, kv_heads=2, dim=8, vdim=4, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def attn_cfg(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.4, softcap=5.0, coef=0.7, every=4,
             kv_from=None):
    mc = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        mc["softcap"] = softcap
    if every:
        mc["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        mc["kv_from"] = kv_from
    return mc


def latent_cfg(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=10, scale=0.3, base=50.0, dims=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
            "scale": scale, "rot": {"base": base, "dims": dims or rot_dim}}


def layer(kind, mixer, ff=24, limit=0.8):
    return {"type": kind, "mixer": mixer,
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def model_cfg(layers=None, width=16, vocab=37, scale=3.0):
    layers = layers or [
        layer("attention", attn_cfg()),
        layer("delta", delta_cfg()),
        layer("attention", attn_cfg(kv_from=0)),
        layer("latent_attention", latent_cfg()),
    ]
    return {"architecture": "Soputar", "width": width, "vocab": vocab,
            "embedding": {"scale": scale}, "norm": {"eps": EPS}, "layers": layers}


def varied_cfg():
    """Other sizes and another order: one KV head, heads == KV heads, sizes
    that are no powers of two, a layer without feed-forward, no cap and no
    temperature, a borrowing layer two layers after its lender, two latent
    layers, rotation on a part of the rotated channels only."""
    return model_cfg(layers=[
        layer("delta", delta_cfg(3, 1, 12, 10, conv=2), ff=0),
        layer("latent_attention", latent_cfg(2, 6, 8, 10, 12, scale=0.5, base=9.0, dims=4), ff=20),
        layer("attention", attn_cfg(3, 3, 6, 5, scale=0.7, softcap=0.0, every=0), ff=12,
              limit=0.3),
        layer("delta", delta_cfg(2, 2, 5, 7, conv=4)),
        layer("attention", attn_cfg(3, 3, 6, 5, scale=0.2, softcap=2.0, coef=1.5, every=3,
                                    kv_from=2), ff=0),
        layer("latent_attention", latent_cfg(4, 4, 2, 3, 5, scale=0.9), ff=16, limit=2.0),
    ], width=24, vocab=29, scale=0.7)


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
    W["head"] = lin(cfg["vocab"], Wd)
    W["final.norm"] = rnd(Wd, std=0.2)
    for i, lc in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = p + "mix."
        mc = lc["mixer"]
        W[p + "norm1"] = rnd(Wd, std=0.2)
        if lc["type"] == "delta":
            H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            for n, ch in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                W[m + n] = lin(ch, Wd, 2.0)
                W[m + n + ".conv"] = rnd(ch, mc["conv"], std=0.6)
            W[m + "b"] = lin(H, Wd)
            W[m + "a"] = lin(H, Wd)
            W[m + "A_log"] = uni(H, -1.0, 0.5)
            W[m + "dt_bias"] = rnd(H)
            W[m + "norm"] = (1 + rnd(Dv, std=0.1)).bfloat16().float()
            W[m + "g"] = lin(H * Dv, Wd, 2.0)
            W[m + "o"] = lin(Wd, H * Dv)
        elif lc["type"] == "attention":
            H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            W[m + "q"] = lin(H * D, Wd)
            W[m + "q.norm"] = (1 + rnd(H * D, std=0.3)).bfloat16().float()
            if mc.get("kv_from") is None:
                W[m + "k"] = lin(G * D, Wd)
                W[m + "k.norm"] = (1 + rnd(G * D, std=0.3)).bfloat16().float()
                W[m + "v"] = lin(G * Dv, Wd)
            W[m + "o"] = lin(Wd, H * Dv)
        else:
            H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
            W[m + "q"] = lin(H * (D + R), Wd, 2.0)
            W[m + "dkv"] = lin(C + R, Wd, 2.0)
            W[m + "dkv.norm"] = (1 + rnd(C, std=0.3)).bfloat16().float()
            W[m + "uk"] = lin(H * D, C, 2.0)
            W[m + "uv"] = lin(H * Dv, C)
            W[m + "sink"] = rnd(H, std=1.5)
            W[m + "o"] = lin(Wd, H * Dv)
        if lc["mlp"]:
            W[p + "norm2"] = rnd(Wd, std=0.2)
            W[p + "mlp.gate"] = lin(lc["mlp"]["ff"], Wd, 2.0)
            W[p + "mlp.up"] = lin(lc["mlp"]["ff"], Wd, 2.0)
            W[p + "mlp.down"] = lin(Wd, lc["mlp"]["ff"])
    return W


def make_engine(cfg, W, device="cpu", dtype="float32", slots=3, page=4, pages=40,
                max_len=96, **engine_kw):
    ec = EngineConfig(batch_size=slots, max_batch_size=slots, kv_cache_batch_size=slots,
                      seq_len=max_len, max_length=max_len, torch_dtype=dtype, tp_degree=1,
                      is_block_kv_layout=True, pa_block_size=page, pa_num_blocks=pages,
                      enable_hip_graphs=False)
    config = SoputarInferenceConfig(neuron_config=ec, **copy.deepcopy(cfg))
    model = SoputarForCausalLM(config)
    sd = SoputarForCausalLM.convert_hf_to_native_state_dict(W, config)
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


# ------------------------------------------------------------ elementwise ops
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("one_plus", [False, True])
@pytest.mark.parametrize("total,lo,n", [(50, 7, 20), (64, 8, 32)])   # scalar / 16-byte kernels
def test_rms_norm_ops(device, one_plus, total, lo, n):
    torch.manual_seed(0)
    wide = torch.randn(2, 5, total) * 3
    w = torch.randn(n) * 0.3
    x = wide[..., lo:lo + n]                              # a column slice, read in place
    want = oracle.rms(x.double(), EPS) * ((1 + w.double()) if one_plus else w.double())
    got = seqmix.rms_norm(x.to(device), w.to(device), EPS, one_plus, out_dtype=F32)
    close(got.cpu(), want, 1e-5)
    buf = torch.zeros(2, 5, n + 12, device=device)        # ... and written into a slice
    seqmix.rms_norm(wide.to(device)[..., lo:lo + n], w.to(device), EPS, one_plus,
                    out=buf[..., 4:4 + n])
    close(buf[..., 4:4 + n].cpu(), want, 1e-5)
    assert float(buf[..., :4].abs().sum() + buf[..., 4 + n:].abs().sum()) == 0.0
    # the post-norm residual step
    stream = torch.randn(2, 5, n)
    y = torch.randn(2, 5, n) * 4
    want = stream.double() + oracle.rms(y.double(), EPS) * (
        (1 + w.double()) if one_plus else w.double())
    s = stream.clone().to(device)
    cp = seqmix.add_rms_norm(s, y.to(device), w.to(device), EPS, one_plus, F32)
    close(s.cpu(), want, 1e-5)
    close(cp.cpu(), want, 1e-5)


@pytest.mark.gpu
def test_add_rms_norm_bf16_copy_gpu():
    torch.manual_seed(1)
    stream, y, w = torch.randn(7, 96), (torch.randn(7, 96) * 2).bfloat16(), torch.randn(96) * 0.2
    want = stream.double() + oracle.rms(y.double(), EPS) * (1 + w.double())
    s = stream.clone().cuda()
    cp = seqmix.add_rms_norm(s, y.cuda(), w.cuda(), EPS, True, BF16)
    close(s.cpu(), want, 1e-5)
    assert cp.dtype == BF16 and torch.equal(cp.cpu(), s.cpu().bfloat16())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C,dims", [(6, 6), (10, 4), (16, 16)])
def test_rotate_interleaved_op(device, C, dims):
    from neuronx_distributed_inference_amd.modules.rope import interleaved_inv_freq

    torch.manual_seed(2)
    B, S, N = 2, 5, 3
    wide = torch.randn(B, S, N, C + 5)
    x = wide[..., 5:]
    pos = torch.tensor([[900, 901, 902, 903, 904], [0, 1, 2, -1, -1]])
    st = seqmix.StepLayout(pos.to(device), torch.tensor([0, 1]).to(device))
    inv = interleaved_inv_freq(100.0, dims)
    got = seqmix.rotate_interleaved(x.to(device), st, inv.to(device), out_dtype=F32).cpu()
    for b in range(B):
        n = int((pos[b] >= 0).sum())
        want = oracle.rotate_pairs(x[b, :n].double(), pos[b, :n], 100.0, dims)
        close(got[b, :n], want, 2e-4)      # fp32 angles near position 900
    out = torch.zeros(B, S, N, C + 3, device=device)
    seqmix.rotate_interleaved(x.to(device), st, inv.to(device), out=out[..., 3:])
    assert torch.equal(out[..., 3:].cpu()[0], got[0])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("ff", [12, 16, 40])          # scalar and 8-wide kernel paths
def test_clamped_glu_op(device, ff):
    torch.manual_seed(3)
    gu = torch.randn(9, 2 * ff) * 2
    g, u = gu[:, :ff].double(), gu[:, ff:].double()
    for limit in (0.5, 3.0):
        gc, uc = g.clamp(max=limit), u.clamp(-limit, limit)
        want = gc * torch.sigmoid(1.702 * gc) * (uc + 1)
        close(seqmix.clamped_glu_fused(gu.to(device), limit).cpu(), want, 1e-5)


# ------------------------------------------------------------ capped attention
def _capped_alone(device, L, T, spikes, page=4, cuts=None, dtype=F32, tol=2e-5, gain=6.0):
    """Attention core on its own paged cache. `spikes`: (query i, key j) pairs
    whose score is made to stand out, so a lost or misplaced key shows."""
    torch.manual_seed(3)
    Wd = 12
    H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    h = torch.randn(T, Wd).double()
    q = h @ (torch.randn(H * D, Wd).double() * 0.3).T
    k = h @ (torch.randn(G * D, Wd).double() * 0.3).T
    v = h @ torch.randn(G * Dv, Wd).double().T
    for i, j in spikes:
        d = torch.zeros(G * D, dtype=torch.float64)
        d[(i + j) % D::D] = 1.0                   # the same channel in every head
        k[j] += gain * d
        q[i] += gain * d.view(G, D)[:1].repeat(H, 1).reshape(-1)
    qn, kn = (1 + 0.3 * torch.randn(H * D)).double(), (1 + 0.3 * torch.randn(G * D)).double()
    if dtype != F32:      # both sides see the values the kernel is given
        q, k, v = (t.to(dtype).double() for t in (q, k, v))
    hq = torch.cat([q, k, v], 1)
    o0, o1 = H * D, H * D + G * D
    eye = torch.eye(hq.shape[1], dtype=torch.float64)
    Wo = {"p.q": eye[:o0], "p.k": eye[o0:o1], "p.v": eye[o1:], "p.q.norm": qn, "p.k.norm": kn,
          "p.o": torch.eye(H * Dv, dtype=torch.float64)}
    kv = oracle.attention_keys_values(hq, Wo, "p.", L, EPS)
    want = oracle.attention_mixer(hq, Wo, "p.", L, EPS, kv)

    qt = L.get("q_temp")
    att = NormedCappedAttention(H, G, D, Dv, L["scale"], EPS, L.get("softcap", 0.0),
                                (qt["coef"], qt["every"]) if qt else None)
    att.q_norm.data, att.k_norm.data = qn.float(), kn.float()
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
        y = att(q[sl].view(1, n, -1).to(device, dtype), k[sl].view(1, n, -1).to(device, dtype),
                v[sl].view(1, n, -1).to(device, dtype), mgr, 0, st)
        got.append(y[0].float().cpu())
        at += n
    got = torch.cat(got)
    if dtype == F32:
        close(got, want, tol)
    else:
        assert (got.double() - want).std().item() < tol * want.std().item()


# temperature steps where floor((p+1)/every) changes: with every=4 between
# positions 2|3, 6|7, ...; page 4: keys 15|16 sit on a page border
CAP = attn_cfg(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.5, softcap=4.0, coef=0.9, every=4)
CAP_SPIKES = [(20, 0), (21, 1), (22, 15), (23, 16), (24, 24), (3, 0), (2, 2), (0, 0),
              (30, 7), (31, 28), (7, 3), (6, 4)]


@pytest.mark.parametrize("device", DEVICES)
def test_capped_attention_prompt(device):
    _capped_alone(device, CAP, 33, CAP_SPIKES)


@pytest.mark.parametrize("device", DEVICES)
def test_capped_attention_decoded_and_portions(device):
    _capped_alone(device, CAP, 33, CAP_SPIKES, cuts=[2, 3, 11] + [1] * 17)
    _capped_alone(device, CAP, 33, CAP_SPIKES, cuts=[1] * 5 + [2, 2, 9, 15])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [
    attn_cfg(3, 3, 5, 3, softcap=0.0, every=0), attn_cfg(6, 1, 16, 8, every=1, coef=0.2),
    attn_cfg(2, 2, 12, 20, softcap=30.0, every=0), attn_cfg(8, 2, 4, 70, softcap=1.0, every=7),
    attn_cfg(2, 1, 24, 40, scale=0.2)])
def test_capped_attention_other_shapes(device, L):
    _capped_alone(device, L, 21, [(20, 0), (12, 7), (5, 5)])
    _capped_alone(device, L, 21, [(20, 0), (12, 7), (5, 5)], cuts=[6, 1, 1, 5, 8], page=8)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [300] + [1] * 40])
def test_capped_attention_far_key_among_hundreds(device, cuts):
    L = attn_cfg(2, 1, 8, 8, scale=0.6, softcap=50.0, every=48, coef=0.4)
    _capped_alone(device, L, 340, [(339, 1), (320, 2), (310, 255), (301, 256), (338, 46),
                                   (337, 47), (336, 48)], page=16, cuts=cuts, tol=5e-5, gain=9.0)


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (attn_cfg(4, 2, 32, 64, scale=0.15, softcap=8.0, every=16), None),
    (attn_cfg(6, 6, 40, 56, scale=0.12, softcap=15.0, every=32), [70, 3, 1, 56]),  # padded tiles
    (attn_cfg(4, 1, 64, 80, scale=0.1, softcap=0.0, every=0), [2, 64, 64]),
    (attn_cfg(2, 2, 128, 128, scale=0.08), [1, 129]),
    (attn_cfg(4, 2, 40, 24, scale=0.15), None),
    (attn_cfg(3, 1, 20, 12, scale=0.2), [5, 120, 1, 1, 1, 1, 1]),   # no 16-byte lines: vector kernel
])
def test_capped_attention_bf16_matrix_path_gpu(L, cuts):
    _capped_alone("cuda", L, 130, [(129, 0), (100, 63), (101, 64), (64, 64), (90, 1)],
                  page=16, cuts=cuts, dtype=BF16, tol=0.02, gain=3.0)


# ------------------------------------------------------------ latent attention
def _latent_alone(device, L, T, cuts=None, page=4, dtype=F32, tol=3e-5, sink=None, spikes=(),
                  fresh=False):
    torch.manual_seed(5)
    Wd = 14
    H, D, R, Dv, C = L["heads"], L["dim"], L["rot_dim"], L["vdim"], L["kv_rank"]
    h = torch.randn(T, Wd).double()
    q = h @ (torch.randn(H * (D + R), Wd).double() * 0.4).T
    dkv = h @ (torch.randn(C + R, Wd).double() * 0.6).T
    for i, j in spikes:                       # through the shared rotated part
        dkv[j, C:] *= 5.0
        q.view(T, H, D + R)[i, :, D:] *= 5.0
    if dtype != F32:
        q, dkv = q.to(dtype).double(), dkv.to(dtype).double()
    hq = torch.cat([q, dkv], 1)
    eye = torch.eye(hq.shape[1], dtype=torch.float64)
    W = {"p.q": eye[:H * (D + R)], "p.dkv": eye[H * (D + R):],
         "p.dkv.norm": (1 + 0.3 * torch.randn(C)).double(),
         "p.uk": torch.randn(H * D, C).double().bfloat16().double() * 0.5,
         "p.uv": torch.randn(H * Dv, C).double().bfloat16().double() * 0.5,
         "p.sink": torch.randn(H).double() if sink is None else torch.full((H,), sink).double(),
         "p.o": torch.eye(H * Dv, dtype=torch.float64)}
    want = oracle.latent_mixer(hq, W, "p.", L, EPS)

    att = LatentSinkAttention(H, D, R, Dv, C, L["scale"], EPS, L["rot"]["base"],
                              L["rot"]["dims"], dtype)
    att.latent_norm.weight.data = W["p.dkv.norm"].float()
    att.uk.data = W["p.uk"].view(H, D, C).to(dtype)
    att.uv.data = W["p.uv"].view(H, Dv, C).to(dtype)
    att.sink.data = W["p.sink"].float()
    att = att.to(device)
    nblk = (T + page - 1) // page
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=nblk + 2, block_size=page, dtype=dtype,
                              tp_degree=1, layer_kv_shapes=[att.kv_shape()]).to(device)
    assert mgr.v_caches[0].numel() == 0                 # one row per token, no value pages
    mgr.k_caches[0].data.normal_()                      # stale pages
    perm = torch.randperm(nblk + 2)[:nblk]
    bt = perm.view(1, nblk).to(device)
    got, at = [], 0
    for n in cuts or [T]:
        pos = torch.arange(at, at + n).view(1, n).to(device)
        mgr.set_step_context(bt, generate_slot_mapping(bt, pos, page))
        st = seqmix.StepLayout(pos, torch.zeros(1, dtype=torch.long, device=device))
        st.fresh = fresh and at == 0          # whole-prompt form for the first portion
        sl = slice(at, at + n)
        y = att(q[sl].view(1, n, -1).to(device, dtype), dkv[sl].view(1, n, -1).to(device, dtype),
                mgr, 0, st)
        got.append(y[0].float().cpu())
        at += n
    got = torch.cat(got)
    if dtype == F32:
        close(got, want, tol)
    else:
        assert (got.double() - want).std().item() < tol * want.std().item()
    return got


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [latent_cfg(), latent_cfg(2, 6, 8, 10, 12, base=9.0, dims=4),
                               latent_cfg(5, 4, 2, 3, 5), latent_cfg(1, 16, 16, 24, 40)])
def test_latent_attention_portions(device, L):
    _latent_alone(device, L, 26)
    _latent_alone(device, L, 26, cuts=[1, 2, 7, 1, 1, 1, 13])
    _latent_alone(device, L, 26, cuts=[3] + [1] * 23, page=8)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [latent_cfg(), latent_cfg(2, 6, 8, 10, 12, base=9.0, dims=4)])
def test_latent_attention_whole_prompt_form(device, L):
    """A prompt taken in the expanded form, then continued from the cache
    rows it left (absorbed form): both equal the oracle."""
    _latent_alone(device, L, 26, fresh=True)
    _latent_alone(device, L, 26, cuts=[17, 1, 1, 7], fresh=True)


@pytest.mark.parametrize("device", DEVICES)
def test_latent_attention_sink_counts_once(device):
    """A dominant sink empties the output, an absent one (-> -inf) leaves a
    plain softmax; the first token alone shares its weight with the sink."""
    L = latent_cfg()
    big = _latent_alone(device, L, 9, sink=30.0)
    none = _latent_alone(device, L, 9, sink=-80.0)
    assert big.abs().max() < 1e-6 < none.abs().max()
    _latent_alone(device, L, 1, sink=0.5)
    _latent_alone(device, L, 9, cuts=[1] * 9, sink=2.0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [250] + [1] * 30])
def test_latent_attention_far_keys_and_positions(device, cuts):
    L = latent_cfg(2, 8, 8, 6, 12, scale=0.4, base=10000.0)
    _latent_alone(device, L, 280, cuts=cuts, page=16, tol=1e-4,
                  spikes=[(279, 0), (270, 3), (260, 127), (251, 128)])


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (latent_cfg(4, 32, 16, 32, 64, scale=0.1), None),
    (latent_cfg(6, 24, 8, 40, 72, scale=0.1), [3, 60, 1, 66]),       # 80-wide rows, padded
    (latent_cfg(2, 64, 32, 64, 96, scale=0.08, dims=16), [64, 66]),
    # wide rows: 32-key tiles, values split over workgroups, also when decoding
    (latent_cfg(8, 32, 32, 48, 224, scale=0.1), [70, 50] + [1] * 10),
    (latent_cfg(16, 64, 64, 64, 512, scale=0.07), [100] + [1] * 30),
    (latent_cfg(4, 16, 8, 16, 200, scale=0.1), [129, 1]),        # few heads: decode on the vector path
    (latent_cfg(3, 12, 6, 10, 20, scale=0.2), [100, 29, 1]),     # 26-wide rows: vector kernel
])
def test_latent_attention_bf16_matrix_path_gpu(L, cuts):
    _latent_alone("cuda", L, 130, cuts=cuts, page=16, dtype=BF16, tol=0.03)
    _latent_alone("cuda", L, 130, cuts=[100] + [1] * 30, page=16, dtype=BF16, tol=0.03, fresh=True)


@pytest.mark.gpu
def test_latent_attention_wide_rows_float32_gpu():
    """32-bit steps never take the matrix-core kernels: 520-wide rows on the
    vector kernel (its merge area needs more than the default LDS)."""
    L = latent_cfg(2, 8, 8, 8, 512, scale=0.3)
    _latent_alone("cuda", L, 40, cuts=[30, 5] + [1] * 5, page=8, tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("L", [latent_cfg(16, 64, 64, 64, 512, scale=0.07),
                               latent_cfg(20, 32, 32, 48, 224, scale=0.1)])
def test_latent_attention_decode_key_splits_gpu(L):
    """Long contexts split a decoded token's keys over several workgroups
    whose partial softmaxes are merged (sink included once)."""
    _latent_alone("cuda", L, 420, cuts=[400] + [1] * 20, page=16, dtype=BF16, tol=0.03)
    _latent_alone("cuda", L, 300, cuts=[290] + [1] * 10, page=16, dtype=BF16, tol=0.03, sink=3.0)


# ------------------------------------------------------------------ delta rule
def _delta_alone(device, R, T, cuts, slots=(1,)):
    torch.manual_seed(4)
    Wd = 10
    H, G, D, Dv = R["heads"], R["kv_heads"], R["dim"], R["vdim"]
    h = torch.randn(T, Wd).double()
    W = {"q": torch.randn(G * D, Wd), "k": torch.randn(G * D, Wd), "v": torch.randn(H * Dv, Wd),
         "q.conv": torch.randn(G * D, R["conv"]) * 0.6, "k.conv": torch.randn(G * D, R["conv"]) * 0.6,
         "v.conv": torch.randn(H * Dv, R["conv"]) * 0.6, "b": torch.randn(H, Wd),
         "a": torch.randn(H, Wd), "A_log": torch.rand(H) - 1.0, "dt_bias": torch.randn(H),
         "norm": torch.rand(Dv) + 0.5, "g": torch.randn(H * Dv, Wd), "o": torch.eye(H * Dv)}
    W = {"p." + k: v.double() for k, v in W.items()}
    want = oracle.delta_mixer(h, W, "p.", R, EPS)

    mod = GatedDeltaRule(H, G, D, Dv, R["conv"], 0, 0, EPS, F32, decay_per_channel=False,
                         gate_act="silu")
    mod.conv.weight.data = torch.cat([W["p.q.conv"], W["p.k.conv"], W["p.v.conv"]]).float()
    mod.A_log.data, mod.dt_bias.data = W["p.A_log"].float(), W["p.dt_bias"].float()
    mod.norm_weight.data = W["p.norm"].float()
    mod = mod.to(device)
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=1, block_size=4, dtype=F32, tp_degree=1,
                              state_slots=3, layer_kv_shapes=[None])
    for name, shape in mod.state_shapes().items():
        mgr.state.register("x." + name, shape)
    mgr = mgr.to(device)
    for t in mgr.state.tensors.values():        # dirty slots: a start must not read them
        t.data.normal_()
    qkv = torch.cat([h @ W["p.q"].T, h @ W["p.k"].T, h @ W["p.v"].T], 1).float()
    beta, a, gate = ((h @ W["p." + n].T).float() for n in ("b", "a", "g"))
    got, at = [], 0
    for n in cuts:
        sl = slice(at, at + n)
        pos = torch.arange(at, at + n).view(1, n).to(device)
        st = seqmix.StepLayout(pos, torch.tensor(list(slots)).to(device))
        y = mod(qkv[sl][None].to(device), beta[sl][None].to(device), a[sl][None].to(device),
                mgr.state, "x", st, gate=gate[sl][None].to(device))
        got.append(y[0].float().cpu())
        at += n
    close(torch.cat(got), want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R", [
    delta_cfg(), delta_cfg(2, 2, 4, 4, conv=1), delta_cfg(3, 1, 12, 70, conv=4),
    delta_cfg(2, 1, 40, 6, conv=2), delta_cfg(1, 1, 100, 66, conv=2), delta_cfg(2, 2, 1, 3)])
def test_delta_rule_portions(device, R):
    _delta_alone(device, R, 27, [27])
    _delta_alone(device, R, 27, [9, 1, 1, 2, 11, 3])
    _delta_alone(device, R, 27, [2] * 13 + [1])


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_long_decode(device):
    _delta_alone(device, delta_cfg(), 90, [3] + [1] * 87)


# ------------------------------------------------------------ whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [model_cfg, varied_cfg])
def test_prefill_decode_portions_match_oracle(device, make):
    cfg = make()
    W = make_weights(cfg, seed=5)
    toks = tokens_for(cfg, 41, seed=6)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, device)
    close(feed(eng, toks, [41]), want, 3e-4)
    close(feed(eng, toks, [1] * 41), want, 3e-4)          # token by token from the start
    close(feed(eng, toks, [2, 5, 2, 1, 9, 3, 2, 16, 1]), want, 3e-4)
    close(feed(eng, toks, [2] * 20 + [1]), want, 3e-4)
    close(feed(eng, toks, [11] + [1] * 30), want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make,tol", [(model_cfg, 3e-5), (varied_cfg, 1e-3)])
def test_residual_stream_per_layer(device, make, tol):
    """The stream after every layer. (The second configuration normalises
    read-outs that nearly cancel in its first tokens, which magnifies fp32
    rounding; its bound is looser for that reason only.)"""
    cfg = make()
    W = make_weights(cfg, seed=7)
    toks = tokens_for(cfg, 9, seed=8)
    _, streams = oracle.forward(cfg, W, toks, return_layers=True)
    eng = make_engine(cfg, W, device)
    dm = eng.model.model
    seen = []
    hooks = [l.register_forward_hook(lambda m, a, out: seen.append(out.detach().clone().cpu()))
             for l in dm.layers]
    feed(eng, toks, [9])
    for hk in hooks:
        hk.remove()
    assert len(seen) == streams.shape[0] == len(cfg["layers"])
    for r, s in enumerate(seen):
        close(s[0], streams[r], tol)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reuse(device):
    """Unequal requests side by side (portions beside single tokens, one
    request pausing) equal each request alone; slots and pages are handed
    back and used again with stale contents."""
    cfg = varied_cfg()
    W = make_weights(cfg, seed=9)
    seqs = {n: tokens_for(cfg, L, seed=10 + i)
            for i, (n, L) in enumerate([("a", 30), ("b", 7), ("c", 19), ("d", 26), ("e", 12)])}
    want = {n: oracle.forward(cfg, W, t) for n, t in seqs.items()}
    eng = make_engine(cfg, W, device, slots=3, page=4, pages=18, max_len=32)
    for t in eng.kv_mgr.state.tensors.values():
        t.data.normal_()
    for t in list(eng.kv_mgr.k_caches) + list(eng.kv_mgr.v_caches):
        t.data.normal_()
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


def test_borrowed_keys_are_the_lenders():
    """The borrowing layer reads what the lender cached: changing the
    lender's key weights changes the borrower's output, and the borrower
    owns no pages."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=16)
    eng = make_engine(cfg, W)
    mgr = eng.kv_mgr
    assert mgr.k_caches[2].numel() == 0 and mgr.get_cache(2)[0] is mgr.get_cache(0)[0]
    assert mgr.k_caches[1].numel() == 0                       # the recurrent layer
    toks = tokens_for(cfg, 12, seed=17)
    close(feed(eng, toks, [5, 7]), oracle.forward(cfg, W, toks), 3e-4)


def _oracle_greedy(cfg, W, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(oracle.forward(cfg, W, toks)[-1].argmax()))
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
    cfg = model_cfg(layers=[
        layer("latent_attention", latent_cfg(4, 32, 16, 48, 64, scale=0.12), ff=128),
        layer("delta", delta_cfg(4, 2, 32, 64, conv=4), ff=128),
        layer("attention", attn_cfg(4, 2, 32, 64, scale=0.15, softcap=10.0, every=16), ff=128),
        layer("attention", attn_cfg(4, 2, 32, 64, scale=0.15, softcap=10.0, every=16, kv_from=2),
              ff=128),
    ], width=128, vocab=96, scale=8.0)
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, seed=13)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, "cuda", dtype="bfloat16", page=16, pages=12, max_len=96)
    a = feed(eng, toks, [80])
    b = feed(eng, toks, [7, 30, 2, 1, 1, 39])
    scale = want.std().item()
    assert (a.double() - want).std().item() < 0.05 * scale
    assert (b.double() - want).std().item() < 0.05 * scale
    assert (a - b).double().std().item() < 0.05 * scale


def test_checkpoint_folder_and_schedule_replay(tmp_path):
    """config.json + model.safetensors on disk -> registry lookup by the
    config's architecture -> schedule replay writes the wanted logits. Sizes
    the file leaves out come from the tensors' shapes."""
    from safetensors.torch import save_file

    from neuronx_distributed_inference_amd import trace_replay
    from neuronx_distributed_inference_amd.registry import model_type_from_config

    cfg = varied_cfg()
    W = make_weights(cfg, seed=14)
    disk = copy.deepcopy(cfg)
    del disk["vocab"], disk["width"]
    for lc in disk["layers"]:
        if lc["mlp"]:
            del lc["mlp"]["ff"]
        if lc["type"] == "delta":
            del lc["mixer"]["conv"], lc["mixer"]["vdim"]
        if lc["type"] == "latent_attention":
            del lc["mixer"]["kv_rank"], lc["mixer"]["vdim"]
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(disk))
    save_file({k: v.bfloat16() for k, v in W.items()}, str(mdir / "model.safetensors"))
    assert model_type_from_config(str(mdir)) == "soputar"
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
    wa, wb = oracle.forward(cfg, W, a), oracle.forward(cfg, W, b)
    import numpy as np

    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
    close(g0, wa[[0, 7]], 3e-4)
    close(g1, wb[[0]], 3e-4)
    close(g2, torch.stack([wb[8], wa[20]]), 3e-4)


def test_command_line_generation(tmp_path, capsys):
    """inference_demo --model-type soputar: checkpoint folder -> compile ->
    load -> greedy generation, the same path as every other family."""
    from safetensors.torch import save_file

    from neuronx_distributed_inference_amd.inference_demo import main

    cfg = model_cfg()
    W = make_weights(cfg, seed=3)
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16() for k, v in W.items()}, str(mdir / "model.safetensors"))
    prompt = tokens_for(cfg, 9, seed=1)
    rc = main(["--model-type", "soputar", "run", "--model-path", str(mdir),
               "--compiled-model-path", str(tmp_path / "compiled"),
               "--prompt-ids", json.dumps([prompt]), "--max-new-tokens", "6",
               "--torch-dtype", "float32", "--on-cpu", "--seq-len", "32",
               "--max-context-length", "16"])
    assert rc == 0
    printed = [json.loads(l) for l in capsys.readouterr().out.splitlines() if l.startswith("[[")]
    assert printed and printed[-1][0] == prompt + _oracle_greedy(cfg, W, prompt, 6)


def test_config_rejects_what_it_does_not_know():
    cfg = model_cfg()
    bad = copy.deepcopy(cfg)
    bad["layers"][1]["type"] = "window"
    with pytest.raises(ValueError):
        SoputarInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)
    bad = copy.deepcopy(cfg)
    bad["layers"][0]["mlp"]["kind"] = "experts"
    with pytest.raises(ValueError):
        SoputarInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)
    bad = copy.deepcopy(cfg)
    bad["layers"][2]["mixer"]["kv_from"] = 1          # a delta layer lends nothing
    with pytest.raises(ValueError):
        SoputarInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)


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
    out = HuggingFaceGenerationAdapter(eng.model).generate(
        torch.tensor(prompts, device=device),
        generation_config=GenerationConfig(max_new_tokens=6))
    assert out[:, 8:].tolist() == want
