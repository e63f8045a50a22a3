"""Tutedra: a pre-norm decoder with a float32 residual stream that starts from a token embedding plus a hashed bigram
embedding (not normed), one-plus RMS norms, a per-column scale on every sublayer's output, a token shift in front of every
mixer, three kinds of mixer chosen per layer, and a dense or routed feed-forward.

  * `mlstm`      a matrix memory with exponential input / forget gates (soft-capped pre-activations, the forget gate a
                 log-sigmoid), a normaliser vector and a running maximum that keeps the exponentials bounded; the
                 read-out is normalised per head, weighted, gated by sigmoid(W_g h) and projected;
  * `hgrn2`      a gated linear recurrence without keys: the forget gate f (bounded below per channel) decays the
                 memory and 1 - f is what is written; read with silu(W_q h); normalised per head;
  * `attention`  grouped-query softmax attention whose values are its keys as the short convolution behind the q / k
                 projections leaves them; q and k are then RMS-normed per head and rotated on their first dimensions
                 with wavelength-rescaled frequencies;
  * feed-forward `dense`: down(polynorm(up h));  `moe`: squared-ReLU experts chosen by sigmoid scores plus a selection
                 bias within the best groups of experts, weighted by the plain scores, plus a shared expert behind a
                 per-token sigmoid gate;  absent where the config says null.

Per layer:  h = norm1(x);  h <- h + (h_prev - h) * shift;  x += ls1 * mixer(h);  x += ls2 * ff(norm2(x)).

Per sequence the engine's state slots carry: the previous token id (bigram hash), every layer's previous norm output
(token shift), and per mixer the recurrent state (memory, normaliser, running maximum) or the last inputs of the
convolution; the attention caches prepared keys and raw keys (its values) in the engine's paged KV cache.

Every size and constant comes from config.json (`TutedraConfig.from_dict`); which optional tensors a checkpoint has
(column scales, shift, selection bias) is read from the checkpoint.  The model is built from the package's layers
(`layers=` swaps in stand-ins, as for the other models); the matrix products are torch's.  What the design keeps in 32
bits is kept there also when the model runs in bfloat16: the residual stream, norms, rotary angles, scores and weights,
router scores, and both recurrences with their gates (the gate pre-activations of the matrix memory are a float32
product).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.cache_spec import PagedKVSpec, SlotStateSpec
from ..utils.cache_context import get_context
from .buvalix import _FusedInputs, _linear


# ------------------------------------------------------------------------------------------------ configuration
@dataclass
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass
class GatedWriteConfig:
    heads: int
    dim: int
    vdim: int


@dataclass
class TiedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    conv: int                   # taps of the convolution behind q / k; 0: none
    rot_dims: int               # 0: no rotary
    rot_base: float
    rot_scaling: dict | None    # factor, low, high, original


@dataclass
class FeedForwardConfig:
    kind: str                   # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    shared_ff: int = 0          # 0: no shared expert


@dataclass
class TutedraLayerConfig:
    kind: str                   # "mlstm" | "hgrn2" | "attention"
    mixer: object
    mlp: FeedForwardConfig | None


@dataclass
class TutedraConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    bigram_buckets: int         # 0: no bigram table
    bigram_mul_prev: int
    bigram_mul_cur: int
    layers: list = field(default_factory=list)
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None      # the design has no position table: no bound

    @classmethod
    def from_dict(cls, d: dict) -> "TutedraConfig":
        layers = []
        for L in d["layers"]:
            m, kind = L["mixer"], L["type"]
            if kind == "mlstm":
                mc = MatrixMemoryConfig(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]))
                if mc.gate_cap <= 0:
                    raise ValueError("mlstm: gate_cap must be positive")
            elif kind == "hgrn2":
                mc = GatedWriteConfig(int(m["heads"]), int(m["dim"]), int(m["vdim"]))
            elif kind == "attention":
                rot = m.get("rot") or {}
                mc = TiedAttentionConfig(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                                         scale=float(m["scale"]), conv=int(m.get("conv") or 0),
                                         rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                         rot_scaling=rot.get("scaling") or None)
                if int(m.get("vdim", mc.dim)) != mc.dim:
                    raise ValueError("attention: values are read from the keys, so vdim must equal dim")
                if mc.heads % mc.kv_heads or mc.rot_dims % 2 or mc.rot_dims > mc.dim:
                    raise ValueError("attention: kv_heads must divide heads; rot.dims even and at most dim")
            else:
                raise ValueError(f"unknown layer type {kind!r}")
            mlp = L.get("mlp")
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    mlp = FeedForwardConfig("dense", int(mlp["ff"]))
                elif mlp.get("kind") == "moe":
                    r = mlp["router"]
                    g = r.get("groups") or {}
                    mlp = FeedForwardConfig("moe", int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]),
                                            int(g.get("count", 1)), int(g.get("keep", g.get("count", 1))),
                                            int((mlp.get("shared") or {}).get("ff", 0)))
                    if mlp.experts % mlp.groups or not 1 <= mlp.keep_groups <= mlp.groups \
                            or not 1 <= mlp.top <= mlp.keep_groups * (mlp.experts // mlp.groups):
                        raise ValueError("router: groups must divide the experts and the kept groups must hold `top` experts")
                else:
                    raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(TutedraLayerConfig(kind, mc, mlp))
        bg = (d.get("embedding") or {}).get("bigram") or {}
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   bigram_buckets=int(bg.get("buckets", 0)), bigram_mul_prev=int(bg.get("mul_prev", 0)),
                   bigram_mul_cur=int(bg.get("mul_cur", 0)), layers=layers, eos_token_id=d.get("eos_token_id"))


def _default_layers():
    from ..layers import gated_memory, linear_memory, moe, parallel_stream, sequential_stream, tied_attention

    class _L:
        HashedBigramEmbedding = parallel_stream.HashedBigramEmbedding
        ReluSquared = parallel_stream.ReluSquared
        stream_boundary_scaled = staticmethod(sequential_stream.stream_boundary_scaled)
        OnePlusNorm = sequential_stream.OnePlusNorm
        PolyNorm = sequential_stream.PolyNorm
        TokenShiftMix = linear_memory.TokenShiftMix
        MatrixLSTMMemory = gated_memory.MatrixLSTMMemory
        GatedWriteMemory = gated_memory.GatedWriteMemory
        ShortConv = tied_attention.ShortConv
        KeyTiedAttention = tied_attention.KeyTiedAttention
        GroupedSigmoidRouter = moe.GroupedSigmoidRouter
        SquaredReluExperts = moe.SquaredReluExperts
    return _L


# ------------------------------------------------------------------------------------------------ mixers
class TutedraMatrixMemory(nn.Module, _FusedInputs):
    _inputs = ("q", "k", "v", "g")

    def __init__(self, m: MatrixMemoryConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m = m
        qk, vv = m.heads * m.dim, m.heads * m.vdim
        self.q = _linear(width, qk, False, dtype, device)
        self.k = _linear(width, qk, False, dtype, device)
        self.v = _linear(width, vv, False, dtype, device)
        self.g = _linear(width, vv, False, dtype, device)
        self.o = _linear(vv, width, False, dtype, device)
        # input-gate rows, then forget-gate rows: a float32 product (the gates enter exponentials)
        self.gates = nn.Parameter(torch.zeros(2 * m.heads, width, dtype=torch.float32, device=device))
        self.cell = L.MatrixLSTMMemory(m.heads, m.dim, m.vdim, m.gate_cap, eps, device=device)

    def cache_specs(self):
        return [SlotStateSpec(self.cell.state_shapes())]

    def names(self, p, t):
        n = {p + x: t + x + ".weight" for x in ("q", "k", "v", "g", "o")}
        n.update({p + "i.b": t + "cell.i_bias", p + "f.b": t + "cell.f_bias", p + "norm": t + "cell.norm_weight"})
        return n

    def place(self, p, take):
        H = self.m.heads
        for j, name in enumerate(("i", "f")):
            t = take(p + name)
            if t.shape != (H, self.gates.shape[1]):
                raise ValueError(f"{p}{name}: shape {tuple(t.shape)} does not match the configuration")
            self.gates[j * H:(j + 1) * H].copy_(t)

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, h, positions, caches):
        m = self.m
        q, k, v, g = self._project(h, self._inputs)
        pre = F.linear(h.float(), self.gates)
        o = self.cell(q.unflatten(1, (m.heads, m.dim)), k.unflatten(1, (m.heads, m.dim)), v.unflatten(1, (m.heads, m.vdim)),
                      pre, g, caches[0])
        return self.o(o)


class TutedraGatedWrite(nn.Module, _FusedInputs):
    _inputs = ("q", "f", "v")

    def __init__(self, m: GatedWriteConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m = m
        qk, vv = m.heads * m.dim, m.heads * m.vdim
        self.q = _linear(width, qk, False, dtype, device)
        self.f = _linear(width, qk, False, dtype, device)
        self.v = _linear(width, vv, False, dtype, device)
        self.o = _linear(vv, width, False, dtype, device)
        self.cell = L.GatedWriteMemory(m.heads, m.dim, m.vdim, eps, device=device)

    def cache_specs(self):
        return [SlotStateSpec(self.cell.state_shapes())]

    def names(self, p, t):
        n = {p + x: t + x + ".weight" for x in ("q", "f", "v", "o")}
        n.update({p + "f.b": t + "cell.f_bias", p + "lower": t + "cell.lower", p + "norm": t + "cell.norm_weight"})
        return n

    def place(self, p, take):
        pass

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, h, positions, caches):
        m = self.m
        q, f, v = self._project(h, self._inputs)
        o = self.cell(q.unflatten(1, (m.heads, m.dim)), f.unflatten(1, (m.heads, m.dim)), v.unflatten(1, (m.heads, m.vdim)),
                      caches[0])
        return self.o(o)


class TutedraAttention(nn.Module, _FusedInputs):
    _inputs = ("q", "k")

    def __init__(self, m: TiedAttentionConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m = m
        self.q = _linear(width, m.heads * m.dim, False, dtype, device)
        self.k = _linear(width, m.kv_heads * m.dim, False, dtype, device)
        self.o = _linear(m.heads * m.dim, width, False, dtype, device)
        self.channels = (m.heads + m.kv_heads) * m.dim
        self.conv = L.ShortConv(self.channels, m.conv, device=device) if m.conv else None      # q | k channels in one launch
        self.attn = L.KeyTiedAttention(m.heads, m.kv_heads, m.dim, m.scale, eps, m.rot_dims, m.rot_base, m.rot_scaling,
                                       device=device)

    def cache_specs(self):
        specs = [PagedKVSpec(self.m.kv_heads, self.m.dim, self.m.dim)]
        if self.conv is not None:
            specs.append(SlotStateSpec({"conv": ((self.m.conv - 1, self.channels), None)}))
        return specs

    def names(self, p, t):
        n = {p + x: t + x + ".weight" for x in ("q", "k", "o")}
        n.update({p + "q.norm": t + "attn.q_norm", p + "k.norm": t + "attn.k_norm"})
        return n

    def place(self, p, take):
        if self.conv is not None:
            nq = self.m.heads * self.m.dim
            for name, rows in (("q.conv", slice(0, nq)), ("k.conv", slice(nq, self.channels))):
                t = take(p + name)
                if t.shape != self.conv.weight[rows].shape:
                    raise ValueError(f"{p}{name}: shape {tuple(t.shape)} does not match the configuration")
                self.conv.weight[rows].copy_(t)

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, h, positions, caches):
        m = self.m
        nq = m.heads * m.dim
        w = getattr(self, "_fused_w", None)
        if w is not None and w.device == h.device and w.dtype == h.dtype:
            qk = F.linear(h, w)                                    # [q | k] rows of one product
        else:
            qk = torch.cat(self._project(h, self._inputs), dim=1)
        if self.conv is not None:
            qk = self.conv(qk, caches[1]["conv"])
        o = self.attn(qk[:, :nq].unflatten(1, (m.heads, m.dim)), qk[:, nq:].unflatten(1, (m.kv_heads, m.dim)), positions,
                      caches[0][0], caches[0][1])
        return self.o(o)


# ------------------------------------------------------------------------------------------------ feed-forward
class TutedraDenseFF(nn.Module):
    def __init__(self, c: FeedForwardConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.up = _linear(width, c.ff, False, dtype, device)
        self.down = _linear(c.ff, width, False, dtype, device)
        self.act = L.PolyNorm(eps, device=device)

    def forward(self, h, h32):
        """Returns the keyword arguments of the stream boundary that adds this sublayer's output."""
        return dict(add=self.down(self.act(self.up(h))))


class TutedraMoE(nn.Module):
    def __init__(self, c: FeedForwardConfig, width: int, L, dtype, device):
        super().__init__()
        self.c = c
        self.router_weight = nn.Parameter(torch.zeros(c.experts, width, dtype=torch.float32, device=device))
        self.router = L.GroupedSigmoidRouter(c.experts, c.top, c.groups, c.keep_groups, device=device)
        self.up = nn.Parameter(torch.zeros(c.experts, c.ff, width, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.zeros(c.experts, width, c.ff, dtype=dtype, device=device))
        self.experts = L.SquaredReluExperts()
        if c.shared_ff:
            # the shared expert's up rows and its gate row as one product
            self.shared_in = _linear(width, c.shared_ff + 1, False, dtype, device)
            self.shared_down = _linear(c.shared_ff, width, False, dtype, device)
            self.shared_act = L.ReluSquared()

    def forward(self, h, h32):
        ids, weights = self.router(F.linear(h32 if h32 is not None else h, self.router_weight))
        out = dict(parts=self.experts(h, ids, weights, self.up, self.down))
        if self.c.shared_ff:
            z = self.shared_in(h)
            out["gated"] = (self.shared_down(self.shared_act(z[:, :self.c.shared_ff])), z[:, self.c.shared_ff])
        return out


class TutedraLayer(nn.Module):
    def __init__(self, lc: TutedraLayerConfig, cfg: TutedraConfig, L, dtype, device):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.norm_eps
        f32 = dict(dtype=torch.float32, device=device)
        self.norm1 = L.OnePlusNorm(W, device=device)
        self.shift = L.TokenShiftMix(1, W, device=device)          # dropped when the checkpoint has no shift
        self.ls1 = nn.Parameter(torch.ones(W, **f32))              # column scales: dropped when the checkpoint has none
        if lc.kind == "mlstm":
            self.mix = TutedraMatrixMemory(lc.mixer, W, eps, L, dtype, device)
        elif lc.kind == "hgrn2":
            self.mix = TutedraGatedWrite(lc.mixer, W, eps, L, dtype, device)
        else:
            self.mix = TutedraAttention(lc.mixer, W, eps, L, dtype, device)
        if lc.mlp is None:
            self.mlp = self.norm2 = self.ls2 = None
        else:
            self.norm2 = L.OnePlusNorm(W, device=device)
            self.ls2 = nn.Parameter(torch.ones(W, **f32))
            self.mlp = TutedraDenseFF(lc.mlp, W, eps, L, dtype, device) if lc.mlp.kind == "dense" \
                else TutedraMoE(lc.mlp, W, L, dtype, device)


class TutedraForCausalLM(nn.Module):
    #: the in-tree library this model's layers need (`nanovllm_amd._lib.build(target)`)
    kernel_library = "mixers"
    #: a cached prompt prefix cannot be taken over: the carried state at its end is not kept
    prefix_caching = False

    def __init__(self, cfg: TutedraConfig, layers=None, dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        L = layers if layers is not None else _default_layers()
        self.config, self.dtype, self._L = cfg, dtype, L
        self.embed = L.HashedBigramEmbedding(cfg.vocab_size, cfg.hidden_size, cfg.bigram_buckets, cfg.bigram_mul_prev,
                                             cfg.bigram_mul_cur, cfg.norm_eps, dtype=dtype, device=device, normed=False)
        self.layers = nn.ModuleList(TutedraLayer(lc, cfg, L, dtype, device) for lc in cfg.layers)
        self.final_norm = L.OnePlusNorm(cfg.hidden_size, device=device)
        self._caches = None

    # ---- weights ----------------------------------------------------------------------------------------
    def checkpoint_names(self) -> dict[str, str]:
        """checkpoint tensor name -> parameter name of this module tree (gates, convolutions, experts and the shared
        expert are placed separately; column scales, shift and selection bias only where the checkpoint has them)."""
        names = {"embed": "embed.weight", "final.norm": "final_norm.weight"}
        if self.embed.bigram is not None:
            names["bigram"] = "embed.bigram"
        for i, layer in enumerate(self.layers):
            p, t = f"l{i}.", f"layers.{i}."
            names[p + "norm1"] = t + "norm1.weight"
            names.update(layer.mix.names(p + "mix.", t + "mix."))
            if layer.mlp is not None:
                names[p + "norm2"] = t + "norm2.weight"
            if isinstance(layer.mlp, TutedraDenseFF):
                names.update({p + "mlp.up": t + "mlp.up.weight", p + "mlp.down": t + "mlp.down.weight",
                              p + "mlp.act": t + "mlp.act.coef"})
            elif isinstance(layer.mlp, TutedraMoE):
                names[p + "mlp.router"] = t + "mlp.router_weight"
                if layer.mlp.c.shared_ff:
                    names[p + "mlp.shared.down"] = t + "mlp.shared_down.weight"
        return names

    def load_tensors(self, tensors: dict[str, torch.Tensor]) -> None:
        """Copy checkpoint tensors (by checkpoint name) into the parameters.  The experts of a layer are stacked into
        [experts, rows, cols] tensors, the two convolutions of an attention into one over [q | k] channels, the two gate
        projections of a matrix memory into one float32 product, the shared expert's gate row under its up rows."""
        names = self.checkpoint_names()
        params = dict(self.named_parameters())
        seen = set()

        def take(name):
            if name not in tensors:
                raise KeyError(f"checkpoint lacks {name}")
            seen.add(name)
            return tensors[name]

        with torch.no_grad():
            W = self.config.hidden_size
            for i, layer in enumerate(self.layers):
                p = f"l{i}."
                layer.mix.place(p + "mix.", take)
                dev = layer.norm1.weight.device
                for name in ("ls1", "ls2"):
                    if name == "ls2" and layer.mlp is None:
                        continue
                    if p + name in tensors:
                        if getattr(layer, name) is None:
                            setattr(layer, name, nn.Parameter(torch.ones(W, dtype=torch.float32, device=dev)))
                        getattr(layer, name).copy_(take(p + name).reshape(W))
                    else:
                        setattr(layer, name, None)
                if p + "shift" in tensors:
                    if layer.shift is None:
                        layer.shift = self._L.TokenShiftMix(1, W, device=dev)
                    layer.shift.mu[0].copy_(take(p + "shift").reshape(W))
                else:
                    layer.shift = None
                if isinstance(layer.mlp, TutedraMoE):
                    mlp, c = layer.mlp, layer.mlp.c
                    if p + "mlp.correction" in tensors:
                        if mlp.router.correction is None:
                            mlp.router.correction = nn.Parameter(torch.zeros(c.experts, dtype=torch.float32, device=dev))
                        mlp.router.correction.copy_(take(p + "mlp.correction").reshape(c.experts))
                    else:
                        mlp.router.correction = None
                    for e in range(c.experts):
                        up, dn = take(f"{p}mlp.e{e}.up"), take(f"{p}mlp.e{e}.down")
                        if up.shape != mlp.up.shape[1:] or dn.shape != mlp.down.shape[1:]:
                            raise ValueError(f"{p}mlp.e{e}.*: expert shapes do not match the configuration")
                        mlp.up[e].copy_(up)
                        mlp.down[e].copy_(dn)
                    if c.shared_ff:
                        up, sg = take(p + "mlp.shared.up"), take(p + "mlp.shared.sg")
                        if up.shape != (c.shared_ff, W) or sg.numel() != W:
                            raise ValueError(f"{p}mlp.shared.*: shapes do not match the configuration")
                        mlp.shared_in.weight[:c.shared_ff].copy_(up)
                        mlp.shared_in.weight[c.shared_ff].copy_(sg.reshape(W))
            for ck, pn in names.items():
                t, prm = take(ck), params[pn]
                if t.shape != prm.shape:
                    raise ValueError(f"{ck}: checkpoint shape {tuple(t.shape)} != parameter {tuple(prm.shape)}")
                prm.copy_(t)
        extra = sorted(set(tensors) - seen)
        if extra:
            raise KeyError(f"checkpoint has tensors the model does not know, e.g. {extra[:3]}")
        self.finalize()

    def finalize(self) -> "TutedraForCausalLM":
        for layer in self.layers:
            layer.mix.finalize()
            layer.norm1.finalize()
            if layer.norm2 is not None:
                layer.norm2.finalize()
        self.final_norm.finalize()
        return self

    # ---- caches -------------------------------------------------------------------------------------------
    def cache_specs(self) -> list:
        """The previous token id first; then per layer the previous norm output (token shift) and the mixer's caches
        (state slots, or a paged KV cache and the convolution's carried inputs)."""
        cfg = self.config
        specs = [SlotStateSpec({"token": ((), torch.int64)})]
        for layer in self.layers:
            specs.append(SlotStateSpec({"prev": ((cfg.hidden_size,), None)}))
            specs.extend(layer.mix.cache_specs())
        return specs

    def bind_caches(self, caches: list) -> None:
        self._prev_token = caches[0]["token"]
        at, bound = 1, []
        for layer in self.layers:
            n = len(layer.mix.cache_specs())
            bound.append((caches[at]["prev"], caches[at + 1:at + 1 + n]))
            at += 1 + n
        assert at == len(caches)
        self._caches = bound

    # ---- forward ------------------------------------------------------------------------------------------
    def forward(self, input_ids, positions, logits_rows=None, streams: list | None = None):
        """Returns float32 logits [T or len(logits_rows), vocab].  streams: a list that receives the residual stream
        after every layer."""
        if self._caches is None:
            raise RuntimeError("caches are not bound: the model runs through the engine's cache and state manager")
        cfg, L, dt = self.config, self._L, self.dtype
        eps = cfg.norm_eps
        ctx = get_context()
        boundary = L.stream_boundary_scaled
        x = self.embed(input_ids, positions, self._prev_token)
        _, h = boundary(x, norm=self.layers[0].norm1.applied, eps=eps, out_dtype=dt)
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            ctx.layer_idx = i
            prev, caches = self._caches[i]
            if layer.shift is not None:
                h = layer.shift(h, prev)[0]
            y = layer.mix(h, positions, caches)
            nxt = (self.layers[i + 1].norm1 if i < last else self.final_norm).applied
            # behind the last mixer only the asked rows go on: the caches and states of this step are complete
            cut = i == last and logits_rows is not None and streams is None
            if layer.mlp is None:
                if cut:
                    x, y, logits_rows = x[logits_rows], y[logits_rows], None
                _, h = boundary(x, add=y, col_scale=layer.ls1, norm=nxt, eps=eps, out_dtype=dt)
            else:
                # a router reads the norm in float32 (in a float32 model that is h itself)
                h32, h = boundary(x, add=y, col_scale=layer.ls1, norm=layer.norm2.applied, eps=eps, out_dtype=dt,
                                  want_f32=isinstance(layer.mlp, TutedraMoE) and dt != torch.float32)
                if cut:
                    h32 = h32[logits_rows] if h32 is not None else None
                    x, h, logits_rows = x[logits_rows], h[logits_rows], None
                _, h = boundary(x, col_scale=layer.ls2, norm=nxt, eps=eps, out_dtype=dt, **layer.mlp(h, h32))
            if streams is not None:
                streams.append(x.clone())
        if logits_rows is not None:
            h = h[logits_rows]
        return F.linear(h, self.embed.weight).float()
