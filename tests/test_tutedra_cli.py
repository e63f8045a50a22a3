"""Tutedra from a checkpoint directory: config.json -> registry -> model, *.safetensors -> parameters, and the two
command-line programs.  CPU: the registry and loader with the eager stand-in layers.  gpu: bin/trace_run and
bin/generate as child processes on a small random checkpoint, against the plain oracle."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from conftest import ROOT
from nanovllm_amd.engine.llm_engine import LLMEngine
from nanovllm_amd.model import registry
from oracle import ref_tutedra_modules
from tutedra_util import attention_layer, config, dense, hgrn2_layer, mlstm_layer, moe, oracle_logits, random_checkpoint, rel_err

CFG = config([attention_layer(heads=4, kv_heads=2, dim=16, conv=3, rot_dims=8, mlp=moe(experts=6, top=3, ff=16, groups=3, keep=2, shared=24)),
              mlstm_layer(heads=2, dim=16, vdim=8, mlp=dense(48)), hgrn2_layer(mlp=None)], vocab=61, width=40, buckets=17)


def write_checkpoint(path, cfg, seed):
    ck = random_checkpoint(cfg, seed)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in ck.items()}, os.path.join(path, "model.safetensors"))
    return ck


def test_registry_builds_and_loads_a_checkpoint_directory(tmp_path):
    ck = write_checkpoint(str(tmp_path), CFG, seed=1)
    assert registry.architecture_of(registry.read_config(str(tmp_path))) == "Tutedra"
    model, cfg = registry.build_model(str(tmp_path), dtype=torch.float32, device="cpu", layers=ref_tutedra_modules)
    assert cfg.hidden_size == CFG["width"] and cfg.bigram_buckets == 17
    assert model.layers[0].mlp.up.shape == (6, 16, 40) and model.layers[0].mlp.shared_in.weight.shape == (25, 40)
    assert model.layers[0].mix.conv.weight.shape == (96, 3) and model.layers[1].mix.gates.shape == (4, 40)
    assert model.layers[2].norm2 is None and model.layers[2].mlp is None
    torch.testing.assert_close(model.layers[1].norm1.applied, 1.0 + ck["l1.norm1"].float())
    # the previous token; then per layer: the shift's carried row and the mixer's caches
    kinds = [type(s).__name__ for s in model.cache_specs()]
    assert kinds == ["SlotStateSpec"] + ["SlotStateSpec", "PagedKVSpec", "SlotStateSpec"] + ["SlotStateSpec"] * 4
    eng = LLMEngine(model, cfg, block_size=4, num_kvcache_blocks=16, device="cpu", max_num_seqs=2, dtype=torch.float32)
    toks = list(range(3, 30))
    got = eng.replay_step([("a", toks, list(range(len(toks))))], ["a"])
    assert rel_err(got, oracle_logits(CFG, ck, toks)) < 5e-5
    for gone in ("l0.mix.q.conv", "l0.mlp.e4.up", "l0.mlp.router", "l0.mlp.shared.sg", "l1.mix.f", "l1.mix.i.b", "l1.mlp.act",
                 "l2.mix.lower", "bigram", "final.norm"):
        with pytest.raises(KeyError):
            model.load_tensors({k: v for k, v in ck.items() if k != gone})
    with pytest.raises(KeyError):
        model.load_tensors({**ck, "l2.norm2": torch.zeros(40)})             # a layer without feed-forward has no second norm
    with pytest.raises(ValueError):
        model.load_tensors({**ck, "l0.mlp.e0.up": torch.zeros(17, 40)})
    make = registry._REGISTRY["Tutedra"].make_config
    for bad in ({**CFG, "layers": [{**CFG["layers"][0], "type": "no_such_mixer"}]},
                {**CFG, "layers": [{**CFG["layers"][1], "mlp": {"kind": "no_such_kind"}}]},
                {**CFG, "layers": [attention_layer(heads=3, kv_heads=2)]}, {**CFG, "layers": [attention_layer(rot_dims=14)]},
                {**CFG, "layers": [mlstm_layer(cap=0.0)]}, {**CFG, "layers": [hgrn2_layer(mlp=moe(experts=6, top=5, groups=3, keep=2))]},
                {**CFG, "layers": [hgrn2_layer(mlp=moe(experts=7, groups=3))]}):
        with pytest.raises(ValueError):
            make(bad)
    bad = attention_layer()
    bad["mixer"]["vdim"] = 7
    with pytest.raises(ValueError):
        make({**CFG, "layers": [bad]})                                      # values are read from the keys


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_replays_steps_and_writes_logits(tmp_path, dtype):
    model_dir, out_dir = str(tmp_path / "model"), str(tmp_path / "out")
    ck = write_checkpoint(model_dir, CFG, seed=2)
    a, b = list(range(5, 45)), [7, 7, 9, 11, 2, 60, 33]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[17:19], "want": []}, {"id": "b", "tokens": b[:6], "want": [5]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[6:], "want": [0]}, {"id": "a", "tokens": a[19:], "want": [20, 0]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [6]}], "end": ["c"]},      # reuses a's pages and slot
    ]
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", out_dir,
                        "--max-tokens", "128", "--block-size", "16", "--max-seqs", "2"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    V = CFG["vocab"]
    la, lb = oracle_logits(CFG, ck, a), oracle_logits(CFG, ck, b)
    want = {0: [("a", 0), ("a", 16)], 1: [("b", 5)], 2: [("b", 6), ("a", 19 + 20), ("a", 19)], 3: [("b", 6)]}
    ref = {"a": la, "b": lb}
    bound = 5e-5 if dtype == "float32" else 3 * max(rel_err(oracle_logits(CFG, ck, a, torch.bfloat16), la),
                                                    rel_err(oracle_logits(CFG, ck, b, torch.bfloat16), lb))
    for n, rows in want.items():
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{n}.f32"), dtype="<f4").reshape(-1, V).copy())
        assert got.shape[0] == len(rows)
        scale = la.pow(2).mean().sqrt()
        for g, (i, at) in zip(got, rows):
            d = g - ref[i][at]
            assert ((d - d.mean()).pow(2).mean().sqrt() / scale).item() < bound, (n, dtype)


@pytest.mark.gpu
def test_generate_program_matches_the_oracle_greedy(tmp_path):
    model_dir = str(tmp_path / "model")
    ck = write_checkpoint(model_dir, CFG, seed=3)
    prompt = [4, 8, 15, 16, 23, 42]
    p = subprocess.run([os.path.join(ROOT, "bin", "generate"), "--model", model_dir, "--dtype", "float32", "--prompt-ids",
                        ",".join(map(str, prompt)), "--max-tokens", "6", "--block-size", "16", "--max-seqs", "2", "--num-blocks", "8"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    out = json.loads(p.stdout.splitlines()[0])
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(oracle_logits(CFG, ck, seq)[-1].argmax()))
    assert out["token_ids"] == seq[len(prompt):]


def test_a_model_can_be_loaded_again_with_other_optional_tensors():
    cfg = config([mlstm_layer(mlp=moe())])
    from tutedra_util import make_engine
    full, bare = random_checkpoint(cfg, 5), random_checkpoint(cfg, 5, scales=False, shift=False, correction=False)
    eng = make_engine(cfg, bare, "cpu")
    layer = eng.runner.model.layers[0]
    assert layer.ls1 is None and layer.ls2 is None and layer.shift is None and layer.mlp.router.correction is None
    toks = list(range(2, 21))
    got = eng.replay_step([("a", toks, list(range(len(toks))))], ["a"])
    assert rel_err(got, oracle_logits(cfg, bare, toks)) < 5e-5
    eng.runner.model.load_tensors(full)
    assert layer.ls1 is not None and layer.shift is not None and layer.mlp.router.correction is not None
    got = eng.replay_step([("b", toks, list(range(len(toks))))], ["b"])
    assert rel_err(got, oracle_logits(cfg, full, toks)) < 5e-5
