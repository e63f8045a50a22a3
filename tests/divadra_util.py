"""Helpers of the Divadra tests: small configurations, random checkpoints in the design's tensor names, and engines on
the CPU stand-ins or on the HIP layers.  The replay driver and the error measure are the Buvalix tests'."""
import math

import torch

import nanovllm_amd  # noqa: F401
from buvalix_util import paged_context, rel_err, replay  # noqa: F401
from nanovllm_amd.engine.llm_engine import LLMEngine
from nanovllm_amd.model.divadra import DivadraConfig, DivadraForCausalLM
from oracle import ref_divadra, ref_divadra_modules


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def mamba_layer(heads=4, vdim=6, state=10, groups=2, norm_groups=3, conv=4, mlp="default"):
    return {"type": "mamba2", "mlp": dense() if mlp == "default" else mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}}


def parallel_layer(heads=6, kv_heads=3, dim=10, vdim=8, chunk=7, rot_dims=6, base=300.0, r_heads=3, r_dim=12, mlp="default"):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.9 / math.sqrt(dim),
            "mask": {"size": chunk}, "rot": {"dims": rot_dims, "base": base}}
    return {"type": "parallel", "mlp": moe() if mlp == "default" else mlp,
            "mixer": {"left": left, "right": {"heads": r_heads, "dim": r_dim}}}


def config(layers, vocab=83, width=36, eps=1e-5, taps=3, buckets=29, mul_prev=31, mul_cur=5):
    cfg = {"architecture": "Divadra", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if taps:
        cfg["canon"] = {"taps": taps}
    if buckets:
        cfg["embedding"] = {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}
    return cfg


def random_checkpoint(cfg: dict, seed: int, rank: int = 4, dtype=torch.bfloat16) -> dict:
    """Tensors by checkpoint name, stored in bfloat16 like a file (so every dtype sees the same values)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0, mean=0.0: (torch.randn(*s, generator=g) * std + mean).to(dtype)
    lin = lambda o, i, gain=1.0: rn(o, i, std=gain / math.sqrt(i))
    t = {"embed": rn(V, W, std=0.7), "embed.norm": rn(W, std=0.1, mean=1.0), "head": lin(V, W),
         "final.norm": rn(W, std=0.1, mean=1.0)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        t["bigram"] = rn(bg["buckets"] + 1, W, std=0.7)
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = rn(W, std=0.1, mean=1.0)
        if taps:
            t[p + "canon1"] = rn(W, taps, std=0.4)
        if L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            t[p + "mix.in"] = lin(2 * inner + 2 * G * N + H, W, 1.5)
            t[p + "mix.conv"], t[p + "mix.conv.b"] = rn(ch, m["conv"], std=0.5), rn(ch, std=0.3)
            t[p + "mix.dt_bias"], t[p + "mix.A_log"], t[p + "mix.D"] = rn(H, std=1.0), rn(H, std=0.7, mean=-1.0), rn(H)
            t[p + "mix.norm"], t[p + "mix.o"] = rn(inner, std=0.1, mean=1.0), lin(W, inner)
        else:
            a, r = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            t[q + "q"], t[q + "k"], t[q + "v"], t[q + "o"] = lin(H * D, W, 2.0), lin(G * D, W, 2.0), lin(G * Dv, W), lin(W, H * Dv)
            t[q + "q.norm"], t[q + "k.norm"] = rn(H * D, std=0.2, mean=1.0), rn(G * D, std=0.2, mean=1.0)
            t[q + "pb"], t[q + "out"] = rn(H, std=1.0, mean=-1.0), rn(W, std=0.1, mean=1.0)
            q, n = p + "mix.right.", r["heads"] * r["dim"]
            for s in ("r", "k", "v", "g", "w"):
                t[q + "mu." + s] = (torch.rand(W, generator=g)).to(dtype)
            for s in ("r", "k", "v", "g"):
                t[q + s] = lin(n, W, 1.5)
            t[q + "w1"], t[q + "w2"], t[q + "w0"] = lin(rank, W, 2.0), lin(n, rank, 2.0), rn(n, std=1.0, mean=-2.0)
            t[q + "u"], t[q + "norm"] = rn(r["heads"], r["dim"], std=0.5), rn(n, std=0.1, mean=1.0)
            t[q + "o"], t[q + "out"] = lin(W, n), rn(W, std=0.1, mean=1.0)
        mlp = L["mlp"]
        if mlp is None:
            continue
        t[p + "norm2"] = rn(W, std=0.1, mean=1.0)
        if taps:
            t[p + "canon2"] = rn(W, taps, std=0.4)
        if mlp["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = lin(mlp["ff"], W, 1.5), lin(W, mlp["ff"])
        else:
            E, top, ff = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            t[p + "mlp.table"] = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
            for e in range(E):
                q = f"{p}mlp.e{e}."
                t[q + "gate"], t[q + "up"], t[q + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)
    return t


def make_engine(cfg: dict, tensors: dict, device: str, dtype=torch.float32, block_size=4, num_blocks=64, max_seqs=4, **kw):
    layers = ref_divadra_modules if device == "cpu" else None
    model = DivadraForCausalLM(DivadraConfig.from_dict(cfg), layers=layers, dtype=dtype, device=device)
    model.load_tensors(tensors)
    return LLMEngine(model, model.config, block_size=block_size, num_kvcache_blocks=num_blocks, device=device,
                     max_num_seqs=max_seqs, dtype=dtype, **kw)


def oracle_logits(cfg: dict, tensors: dict, tokens, dtype=torch.float32):
    return ref_divadra.forward(cfg, tensors, tokens, dtype)[0]


def layer_namespace(device: str):
    """The layer classes the model would use on this device: eager stand-ins on the CPU, HIP-backed on the GPU."""
    if device == "cpu":
        return ref_divadra_modules
    from nanovllm_amd.model.divadra import _default_layers
    return _default_layers()
