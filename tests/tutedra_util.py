"""Helpers of the Tutedra tests: small configurations, random checkpoints in the design's tensor names, and engines on
the CPU stand-ins or on the HIP layers.  The replay driver and the error measure are the Buvalix tests'."""
import math

import torch

import nanovllm_amd  # noqa: F401
from buvalix_util import paged_context, rel_err, replay  # noqa: F401
from nanovllm_amd.engine.llm_engine import LLMEngine
from nanovllm_amd.model.tutedra import TutedraConfig, TutedraForCausalLM
from oracle import ref_tutedra, ref_tutedra_modules


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=12, groups=3, keep=2, shared=10):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if groups:
        m["router"]["groups"] = {"count": groups, "keep": keep}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def mlstm_layer(heads=3, dim=10, vdim=6, cap=9.0, mlp="default"):
    return {"type": "mlstm", "mlp": dense() if mlp == "default" else mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def hgrn2_layer(heads=2, dim=12, vdim=9, mlp="default"):
    return {"type": "hgrn2", "mlp": moe() if mlp == "default" else mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def attention_layer(heads=6, kv_heads=2, dim=12, conv=4, rot_dims=8, base=300.0, scaling="default", scale=None, mlp="default"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale or 1.4 / math.sqrt(dim)}
    if conv:
        m["conv"] = conv
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling == "default":
            scaling = {"factor": 6.0, "low": 1.0, "high": 3.0, "original": 40}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "attention", "mlp": dense(24) if mlp == "default" else mlp, "mixer": m}


def config(layers, vocab=83, width=36, eps=1e-5, buckets=29, mul_prev=13, mul_cur=5):
    cfg = {"architecture": "Tutedra", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if buckets:
        cfg["embedding"] = {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}
    return cfg


def random_checkpoint(cfg: dict, seed: int, dtype=torch.bfloat16, scales=True, shift=True, correction=True) -> dict:
    """Tensors by checkpoint name, stored in bfloat16 like a file (so every dtype sees the same values).  `scales`,
    `shift`, `correction`: whether the checkpoint has column scales, a token shift, a selection bias."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0, mean=0.0: (torch.randn(*s, generator=g) * std + mean).to(dtype)
    lin = lambda o, i, gain=1.0: rn(o, i, std=gain / math.sqrt(i))
    t = {"embed": rn(V, W, std=0.7), "final.norm": rn(W, std=0.1)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        t["bigram"] = rn(bg["buckets"] + 1, W, std=0.7)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = rn(W, std=0.1)
        if scales:
            t[p + "ls1"] = rn(W, std=0.2, mean=0.8)
        if shift:
            t[p + "shift"] = torch.rand(W, generator=g).to(dtype)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        q = p + "mix."
        if L["type"] == "mlstm":
            t[q + "q"], t[q + "k"], t[q + "v"], t[q + "g"] = lin(H * D, W, 1.5), lin(H * D, W, 1.5), lin(H * Dv, W), lin(H * Dv, W)
            t[q + "i"], t[q + "f"] = lin(H, W, 2.0), lin(H, W, 2.0)
            t[q + "i.b"], t[q + "f.b"] = rn(H, std=1.0), rn(H, std=1.0, mean=3.0)
            t[q + "norm"], t[q + "o"] = rn(H * Dv, std=0.1, mean=1.0), lin(W, H * Dv)
        elif L["type"] == "hgrn2":
            t[q + "q"], t[q + "f"], t[q + "v"] = lin(H * D, W, 1.5), lin(H * D, W, 1.5), lin(H * Dv, W)
            t[q + "f.b"], t[q + "lower"] = rn(H * D, std=1.0, mean=1.0), (torch.rand(H * D, generator=g) * 0.9).to(dtype)
            t[q + "norm"], t[q + "o"] = rn(Dv, std=0.1, mean=1.0), lin(W, H * Dv)
        else:
            G = m["kv_heads"]
            t[q + "q"], t[q + "k"], t[q + "o"] = lin(H * D, W, 2.0), lin(G * D, W, 2.0), lin(W, H * D)
            t[q + "q.norm"], t[q + "k.norm"] = rn(D, std=0.2, mean=1.0), rn(D, std=0.2, mean=1.0)
            if m.get("conv"):
                t[q + "q.conv"], t[q + "k.conv"] = rn(H * D, m["conv"], std=0.5), rn(G * D, m["conv"], std=0.5)
        mlp = L["mlp"]
        if mlp is None:
            continue
        t[p + "norm2"] = rn(W, std=0.1)
        if scales:
            t[p + "ls2"] = rn(W, std=0.2, mean=0.8)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            t[q + "up"], t[q + "down"], t[q + "act"] = lin(mlp["ff"], W, 1.5), lin(W, mlp["ff"]), rn(4, std=0.6)
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            t[q + "router"] = lin(E, W, 2.0)
            if correction:
                t[q + "correction"] = rn(E, std=0.3)
            for e in range(E):
                t[f"{q}e{e}.up"], t[f"{q}e{e}.down"] = lin(ff, W, 2.0), lin(W, ff)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                t[q + "shared.up"], t[q + "shared.down"], t[q + "shared.sg"] = lin(sf, W, 2.0), lin(W, sf), lin(1, W, 2.0)
    return t


def make_engine(cfg: dict, tensors: dict, device: str, dtype=torch.float32, block_size=4, num_blocks=64, max_seqs=4, **kw):
    layers = ref_tutedra_modules if device == "cpu" else None
    model = TutedraForCausalLM(TutedraConfig.from_dict(cfg), layers=layers, dtype=dtype, device=device)
    model.load_tensors(tensors)
    return LLMEngine(model, model.config, block_size=block_size, num_kvcache_blocks=num_blocks, device=device,
                     max_num_seqs=max_seqs, dtype=dtype, **kw)


def oracle_logits(cfg: dict, tensors: dict, tokens, dtype=torch.float32):
    return ref_tutedra.forward(cfg, tensors, tokens, dtype)[0]


def layer_namespace(device: str):
    """The layer classes the model would use on this device: eager stand-ins on the CPU, HIP-backed on the GPU."""
    if device == "cpu":
        return ref_tutedra_modules
    from nanovllm_amd.model.tutedra import _default_layers
    return _default_layers()
