#!/usr/bin/env python3
"""Tutedra beside Benarax (the closest existing model with a full-size record: fp32 stream, input convolutions, a
recurrent and an attention mixer, routed experts) at equal sizes, random weights: every kernel of the design next to the
like kernel, with its HBM or MFMA rate, and prefill / decode throughput of whole models through the engine.
`python bench.py --tutedra` prints the record as one JSON line.  Every step names itself on stderr before it uses the
GPU."""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import nanovllm_amd as nv  # noqa: E402
from nanovllm_amd import ops  # noqa: E402
from nanovllm_amd.engine.llm_engine import LLMEngine  # noqa: E402
from nanovllm_amd.engine.sequence import SamplingParams  # noqa: E402
from nanovllm_amd.layers import delta_rule, gated_memory, general_delta, moe, sequential_stream, tied_attention  # noqa: E402
from nanovllm_amd.model.tutedra import TutedraConfig, TutedraForCausalLM  # noqa: E402
from tools.benarax_bench import benarax_config, random_benarax  # noqa: E402
from tools.buvalix_bench import paged, rate, timed  # noqa: E402


def note(what):
    print("tutedra_bench: " + what, file=sys.stderr, flush=True)


def kernel_records(dev):
    out = {}
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s, dtype=bf: torch.randn(*s, generator=g, device=dev).to(dtype)
    W, bs = 2048, 256
    for name, T in (("prefill_8192_tokens", 8192), ("decode_256_tokens", 256)):
        note("stream kernels, " + name)
        rec = {}
        x, a, b, parts = rn(T, W, dtype=torch.float32), rn(T, W), rn(T, W + 1), rn(T, 4, W, dtype=torch.float32)
        w, ls = rn(W, dtype=torch.float32), rn(W, dtype=torch.float32)
        t = timed(lambda: ops.stream_boundary_scaled(x, add=a, col_scale=ls, norm=w, eps=1e-5, out_dtype=bf))
        rec["stream_boundary_scaled (mixer -> scaled into the stream -> norm bf16)"] = rate(t, nbytes=T * W * (8 + 2 + 2))
        t = timed(lambda: ops.stream_boundary_scaled(x, gated=(b[:, :W], b[:, W]), parts=parts, col_scale=ls, norm=w, eps=1e-5,
                                                     out_dtype=bf, want_f32=True))
        rec["stream_boundary_scaled (4 expert parts + gated shared expert -> stream -> norm fp32 + bf16)"] = \
            rate(t, nbytes=T * W * (8 + 2 + 16 + 6))
        t = timed(lambda: ops.stream_boundary(x, add=a, add_parts=parts, mult=0.5, norm=w, groups=4, eps=1e-5, out_dtype=bf, want_f32=True))
        rec["like: stream_boundary (mixer + 4 expert parts -> stream -> grouped norm, fp32 + bf16)"] = rate(t, nbytes=T * W * (8 + 2 + 16 + 6))
        y = rn(T, 4 * W)
        act = sequential_stream.PolyNorm(1e-5, device=dev)
        with torch.no_grad():
            act.coef.copy_(torch.tensor([0.5, 0.3, 0.2, 0.1]))
        rec["poly_norm (ff 8192; the row is read twice, the second time from cache)"] = rate(timed(lambda: act(y)), nbytes=T * 4 * W * 4)
        rec["like: gelu_tanh_and_mul (ff 4096)"] = rate(timed(lambda: ops.gelu_tanh_and_mul(y)), nbytes=T * 4 * W * 3)
        out[name] = rec

    H, D, taps = 16, 128, 4
    for name, n_qs in (("prefill_4x2048", [2048] * 4), ("decode_256_seqs", [1] * 256)):
        note("recurrent kernels, " + name)
        n_ks = [n + 100 for n in n_qs]
        ctx, pos, _ = paged(n_qs, n_ks, bs, dev)
        T, B = sum(n_qs), len(n_qs)
        nv.set_context(ctx)
        rec = {}
        cell = gated_memory.MatrixLSTMMemory(H, D, D, 20.0, 1e-5, device=dev)
        cache = {"state": torch.zeros(B, H, D, D, device=dev), "normaliser": torch.zeros(B, H, D, device=dev),
                 "maximum": torch.zeros(B, H, device=dev)}
        q, k, v = rn(T, H, D), rn(T, H, D), rn(T, H, D)
        fr, gr, ar = rn(T, H * D), rn(T, H * D), rn(T, H * D)
        pre = rn(T, 2 * H, dtype=torch.float32)
        t = timed(lambda: cell(q, k, v, pre, gr, cache), iters=5)
        rec["mlstm_memory (16 heads 128 x 128)"] = dict(rate(t, nbytes=T * 5 * H * D * 2 + 2 * B * H * D * D * 4), tokens_per_s=round(T / t))
        cell2 = gated_memory.GatedWriteMemory(H, D, D, 1e-5, device=dev)
        t = timed(lambda: cell2(q, fr.view(T, H, D), v, cache), iters=5)
        rec["gated_write_memory (16 heads 128 x 128)"] = dict(rate(t, nbytes=T * 4 * H * D * 2 + 2 * B * H * D * D * 4), tokens_per_s=round(T / t))
        rule = general_delta.GeneralDeltaRule(H, D, 1e-5, device=dev)
        st = torch.zeros(B, H, D, D, device=dev)
        t = timed(lambda: rule(q, k, v, fr, ar, gr, st), iters=5)
        rec["like: general_delta_rule"] = dict(rate(t, nbytes=T * 7 * H * D * 2 + 2 * B * H * D * D * 4), tokens_per_s=round(T / t))
        ch = (16 + 8) * 128
        xb = rn(T, ch)
        conv = tied_attention.ShortConv(ch, taps, device=dev)
        cs = torch.zeros(B, taps - 1, ch, device=dev, dtype=bf)
        rec["causal_conv without activation over q | k (the like kernel with its activation switched off)"] = \
            rate(timed(lambda: conv(xb, cs)), nbytes=T * ch * 4)
        conv3 = delta_rule.ShortConvSilu(ch, taps, device=dev)
        rec["like: causal_conv_silu"] = rate(timed(lambda: conv3(xb, cs)), nbytes=T * ch * 4)
        nv.set_context(None)
        out["recurrent " + name] = rec

    Hq, G, Dh = 16, 8, 128
    cases = {"prefill_4x2048": ([2048] * 4, [2048] * 4), "chunk_512_over_8192": ([512], [8192]),
             "decode_256_seqs_ctx_513_768": ([1] * 256, torch.randint(513, 769, (256,), generator=torch.Generator().manual_seed(1)).tolist()),
             "decode_8_seqs_ctx_8192": ([1] * 8, [8192] * 8)}
    for name, (n_qs, n_ks) in cases.items():
        note("attention kernels, " + name)
        ctx, pos, nb = paged(n_qs, n_ks, bs, dev)
        T = sum(n_qs)
        nv.set_context(ctx)
        att = tied_attention.KeyTiedAttention(Hq, G, Dh, Dh ** -0.5, 1e-5, 64, 1e4, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192},
                                              device=dev)
        q, k, v = rn(T, Hq, Dh), rn(T, G, Dh), rn(T, G, Dh)
        kc, vc = rn(nb, bs, G, Dh), rn(nb, bs, G, Dh)
        rec = {}
        t = timed(lambda: ops.head_norm_rope_store(pos, q, k, att.q_norm, att.k_norm, 1e-5, att.freq, 64, ctx.slot_mapping, kc, vc))
        rec["head_norm_rope_store (per-head norms, rotary on 64 of 128, prepared and raw keys scattered)"] = \
            rate(t, nbytes=T * (2 * Hq + 3 * G) * Dh * 2)
        inv = torch.ones(Dh // 2, device=dev)
        t = timed(lambda: ops.qk_prep_store(pos, q, k, v, ctx.slot_mapping, kc, vc, inv, Dh))
        rec["like: qk_prep_store"] = rate(t, nbytes=T * (Hq + 2 * G) * Dh * 4)
        full = sum(nq * (nk - nq) + nq * (nq + 1) // 2 for nq, nk in zip(n_qs, n_ks))
        singles = int(max(n_qs) == 1)
        t = timed(lambda: ops.attn_scoremod_paged(q, kc, vc, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables, Dh ** -0.5, 0.0,
                                                  None, None, max(n_qs), max(n_ks), singles), iters=5)
        rec["attention (the like kernel itself: attn_scoremod with every modifier off)"] = rate(
            t, nbytes=(sum(n_ks) * G * Dh * 4 + T * Hq * Dh * 4) if singles else None, flops=None if singles else 4 * Dh * Hq * full)
        nv.set_context(None)
        out["attention " + name] = rec

    E, top, ff = 32, 4, 1024
    up, gu, dn = rn(E, ff, W) * 0.02, rn(E, 2 * ff, W) * 0.02, rn(E, W, ff) * 0.02
    router = moe.GroupedSigmoidRouter(E, top, 4, 2, device=dev)
    ex, like = moe.SquaredReluExperts(), moe.MoEExperts(top, 7.0)
    for name, T in (("prefill_8192_tokens", 8192), ("decode_256_tokens", 256), ("decode_16_tokens", 16)):
        note("expert kernels, " + name)
        h, lg = rn(T, W), rn(T, E, dtype=torch.float32)
        rec = {"moe_route_grouped (32 experts, 4 groups, 2 kept, top 4)": rate(timed(lambda: router(lg)), nbytes=T * (E * 4 + top * 8))}
        ids, wts = router(lg)
        flops = 2 * T * top * 2 * ff * W
        wbytes = min(E, T * top) * 2 * ff * W * 2
        rec["squared-ReLU experts (32 experts, top 4, ff 1024; up and down)"] = rate(
            timed(lambda: ex(h, ids, wts, up, dn), iters=5), nbytes=wbytes + T * W * (2 + 4 * top), flops=flops)
        rec["like: routed gated experts (gate, up and down behind a softmax router)"] = rate(
            timed(lambda: like(h, lg, gu, dn), iters=5), nbytes=wbytes * 3 // 2 + T * W * (2 + 4 * top), flops=flops * 3 // 2)
        out["feed-forward " + name] = rec
    return out


def tutedra_config(width, n_groups, vocab, experts=32, top=4, ff=1024):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top, "groups": {"count": 4, "keep": 2}}, "expert": {"ff": ff},
           "shared": {"ff": ff}}
    att = {"heads": 16, "kv_heads": 8, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "conv": 4,
           "rot": {"dims": 64, "base": 1e4, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 2048}}}
    group = [{"type": "mlstm", "mlp": mlp, "mixer": {"heads": 16, "dim": 128, "vdim": 128, "gate_cap": 20.0}},
             {"type": "attention", "mlp": {"kind": "dense", "ff": 4096}, "mixer": att},
             {"type": "hgrn2", "mlp": mlp, "mixer": {"heads": 16, "dim": 128, "vdim": 128}},
             {"type": "attention", "mlp": mlp, "mixer": att}]
    return {"architecture": "Tutedra", "layers": group * n_groups, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width,
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 131, "mul_cur": 3}}}


def random_tutedra(cfg_dict, dev, dtype):
    cfg = TutedraConfig.from_dict(cfg_dict)
    model = TutedraForCausalLM(cfg, dtype=dtype, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name and "cell" not in name and "attn" not in name:
                p.zero_()                                   # one-plus weights
            elif p.dim() >= 2 and "mu" not in name:
                p.copy_((torch.randn(p.shape, generator=g, device=dev) * (0.5 if "conv" in name else 0.02)).to(p.dtype))
            elif "norm" in name or name.endswith(("ls1", "ls2")):
                p.fill_(1.0)
            elif "lower" in name or "mu" in name:
                p.copy_(torch.rand(p.shape, generator=g, device=dev) * 0.9)
            elif "f_bias" in name:
                p.fill_(3.0)
            elif "coef" in name:
                p.copy_(torch.tensor([0.5, 0.3, 0.2, 0.0], device=dev))
            else:
                p.copy_((torch.randn(p.shape, generator=g, device=dev) * 0.1).to(p.dtype))
    model.finalize()
    return model, cfg


def model_records(dev, width=2048, n_groups=2, vocab=32000, batch=32, prompt_len=1024, out_len=64):
    out = {"shape": dict(width=width, layers=4 * n_groups, vocab=vocab, batch=batch, prompt_len=prompt_len, out_len=out_len,
                         block_size=256, tutedra="mlstm (16 heads 128 x 128) / attention (16/8 x 128, 4 taps, rotary 64) / hgrn2 "
                         "(16 heads 128 x 128) / attention; 32 squared-ReLU experts in 4 groups, top 4, ff 1024, plus a shared expert "
                         "ff 1024, and dense ff 4096 with the polynomial activation in one layer of four",
                         benarax="16 heads; 32 experts, top 4, ff 1024 (active ff 4096); latent 128 + 32")}
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, vocab, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    warm = [torch.randint(0, vocab, (prompt_len,), generator=g).tolist() for _ in range(2)]
    blocks = batch * (-(-(prompt_len + out_len) // 256)) + 8

    def measure(engine):
        engine.generate(warm, SamplingParams(0.0, 4))
        torch.cuda.synchronize()
        _, m = engine.generate(prompts, SamplingParams(0.0, out_len))
        s = m.summary()
        prefill = sum(t for t, _, only in m.step_times if not only)
        return {"prefill_tok_per_s": round(batch * prompt_len / prefill), "decode_tok_per_s": round(s["decode_only_tok_per_s"]),
                "mean_tpot_ms": round(s["mean_tpot_ms"], 3), "output_tok_per_s": round(s["output_tok_per_s"])}

    note("model: tutedra")
    model, cfg = random_tutedra(tutedra_config(width, n_groups, vocab), dev, torch.bfloat16)
    eng = LLMEngine(model, cfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, max_num_seqs=batch, long_prefill_token_threshold=0)
    out["tutedra"] = measure(eng)
    del eng, model
    torch.cuda.empty_cache()
    note("model: benarax")
    model, cfg = random_benarax(benarax_config(width, n_groups, vocab), dev, torch.bfloat16)
    eng = LLMEngine(model, cfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, max_num_seqs=batch, long_prefill_token_threshold=0)
    out["like: benarax (same width and depth; 32 experts, top 4 in every layer)"] = measure(eng)
    return out


def run(device="cuda:0", kernels=True, models=True):
    rec = {"metric": "tutedra_vs_like_model", "rooflines": {"hbm_TB_s": 8.0, "mfma_bf16_PFLOP_s": 2.5},
           "data": "synthetic", "dtype": "bf16"}
    if kernels:
        rec["kernels"] = kernel_records(device)
    if models:
        rec["models"] = model_records(device)
    return rec


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-models", action="store_true")
    a = ap.parse_args()
    print(json.dumps(run(kernels=not a.no_kernels, models=not a.no_models)))
