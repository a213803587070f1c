"""Dogidra: a decoder over an fp32 residual stream whose layers put a
windowed attention with pooled far blocks and a minimal gated recurrent unit
side by side, followed by a routed feed-forward of ungated squared-relu
experts; every sublayer reads a layer norm of the stream that has passed a
short causal convolution over time, and a span of the layers runs several
times in a row with the same weights.

With ln(x; w, b) = (x - mean) / sqrt(var + eps) * w + b and c(h) = h +
conv(h) (causal, per channel, `taps` taps) a layer does
    x <- x + a_l * attention(c1(ln(x; w1, b1))) + a_r * mingru(c1(...))
    x <- x + ff(c2(ln(x; w2, b2)))                (layers with a feed-forward)
The embedding output is x0 = embed[token] * scale. Layers [start, stop) of
`loop` run `times` times; every pass begins with x <- W_in [x; x0] and owns
its caches and states, so the stack has one cache entry per layer RUN.
Logits are embed ln(x; w_f, b_f) (the unscaled embedding table).

Per layer run the GPU work is: boundary kernel (add the previous sublayer's
outputs to the stream in fp32, layer norm, input convolution) -> one GEMM
over q|k|v of the attention half and z|x|g of the recurrent half -> rotary +
whole-projection norms + cache append, pooled-block means, attention |
recurrence scan -> output GEMMs -> boundary kernel -> router kernel ->
experts (+ shared expert) -> the next run's boundary kernel.

Numerics: the stream, layer norms and their convolutions, router,
attention scores / weights, rotary angles and the recurrence with its gates
are fp32; projections and activations run in the serving dtype.

config.json layout read here: architecture, vocab, width, norm{eps},
embedding{scale}, canon{taps}, loop{start, stop, times}, layers[i] = {type,
mixer{left{heads, kv_heads, dim, vdim, scale, softcap, mask{size, pool},
rot{base, dims, scaling{factor, original, fast, slow}}}, right{width},
left_scale, right_scale}, mlp{kind, expert{ff}, router{experts, top, scale},
shared{ff}}|null}. Checkpoint names: embed, loop.in, final.norm(.b),
l<i>.norm1(.b) / norm2(.b) / canon1 / canon2, l<i>.mix.left.{q, k, v, q.norm,
k.norm, o}, l<i>.mix.right.{z, z.b, x, x.b, g, o}, l<i>.mlp.{router,
correction, e<j>.up, e<j>.down, shared.up, shared.down}.
"""

from __future__ import annotations

import json
import os
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from production_stack_amd import ops
from production_stack_amd.engine.config import (
    LayerSpec,
    MixerSpec,
    MlpSpec,
    ModelConfig,
)
from production_stack_amd.engine.models.ffn import SparseMoE
from production_stack_amd.engine.models.mixers import build_mixer
from production_stack_amd.ops import gemm_policy

ARCHITECTURE = "Dogidra"

# positions a rotary table is built for unless the engine asks for more
DEFAULT_MAX_POSITION = 8192


# ---------------------------------------------------------------------------
# configuration
# ---------------------------------------------------------------------------
def _attention_spec(m: dict) -> MixerSpec:
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    sc = rot.get("scaling")
    mask = m.get("mask") or {}
    return MixerSpec(
        kind="attention", heads=int(m["heads"]), dim=int(m["dim"]),
        kv_heads=int(m.get("kv_heads", m["heads"])),
        vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
        window=int(mask.get("size", 0)),
        window_pool=int(mask.get("pool", 0)) if mask.get("size") else 0,
        softcap=float(m.get("softcap") or 0.0),
        rope=dims > 0, rot_dims=dims, rot_layout="half",
        rot_base=float(rot.get("base", 10000.0)),
        rot_scaling=((float(sc["factor"]), float(sc["original"]),
                      float(sc["fast"]), float(sc["slow"])) if sc else None),
        qk_norm_all=True)


def _mixer_spec(kind: str, m: dict) -> MixerSpec:
    if kind != "parallel":
        raise ValueError(f"unknown layer type {kind!r}")
    left = _attention_spec(m["left"])
    right = MixerSpec(kind="mingru", heads=1, dim=1,
                      vdim=int(m["right"]["width"]), rope=False)
    return MixerSpec(
        kind="pair", heads=left.heads, dim=left.dim, rope=False, left=left,
        right=right, combine="weighted",
        left_scale=float(m.get("left_scale", 1.0)),
        right_scale=float(m.get("right_scale", 1.0)))


def _mlp_spec(m: Optional[dict]) -> Optional[MlpSpec]:
    if m is None:
        return None
    if m.get("kind", "moe") != "moe":
        raise ValueError(f"unknown mlp kind {m['kind']!r}")
    r = m["router"]
    return MlpSpec(
        kind="moe", ff=int(m["expert"]["ff"]), act="relu2", gated=False,
        experts=int(r["experts"]), top=int(r["top"]), score="sigmoid",
        renormalize=False, weight_on_input=False,
        shared_ff=int((m.get("shared") or {}).get("ff", 0)),
        shared_gate=False, correction=True,
        route_scale=float(r.get("scale", 1.0)))


def config_from_json(cfg: dict, name: str = "dogidra") -> ModelConfig:
    taps = int((cfg.get("canon") or {}).get("taps", 0))
    specs: List[LayerSpec] = [
        LayerSpec(mixer=_mixer_spec(layer["type"], layer["mixer"]),
                  mlp=_mlp_spec(layer.get("mlp")), parallel=False,
                  norm="layer", input_conv=taps)
        for layer in cfg["layers"]]
    loop = cfg.get("loop")
    if loop:
        loop = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        if not 0 <= loop[0] <= loop[1] <= len(specs) or loop[2] < 1:
            raise ValueError(f"bad loop {loop} for {len(specs)} layers")
    att = [s.mixer.left for s in specs]
    ffs = [max(s.mlp.ff, s.mlp.shared_ff) for s in specs
           if s.mlp is not None]
    return ModelConfig(
        name=name, family="dogidra", hidden_size=int(cfg["width"]),
        num_layers=len(specs),
        num_q_heads=max([m.heads for m in att], default=1),
        num_kv_heads=max([m.kv_heads for m in att], default=1),
        head_dim=max([m.dim for m in att], default=1),
        intermediate_size=max(ffs, default=0), vocab_size=int(cfg["vocab"]),
        max_position=int(cfg.get("max_position", DEFAULT_MAX_POSITION)),
        rms_norm_eps=float(cfg["norm"]["eps"]), layer_specs=specs,
        embedding_scale=float((cfg.get("embedding") or {}).get("scale",
                                                               1.0)),
        loop=loop, tie_word_embeddings=True,
        # no BOS/EOS convention in this design: never stop on a token id
        bos_token_id=0, eos_token_id=-1)


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    return config_from_json(cfg, name=os.path.basename(
        os.path.normpath(path)) or "dogidra")


def layer_runs(n_layers: int, loop: Optional[tuple]):
    """[(layer index, a pass begins here)] in execution order."""
    if not loop:
        return [(i, False) for i in range(n_layers)]
    a, b, times = loop
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    runs += [(i, False) for i in range(b, n_layers)]
    return runs


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------
class DogidraLayer(nn.Module):
    def __init__(self, width: int, spec: LayerSpec, eps: float,
                 dtype: torch.dtype, max_pos: int) -> None:
        super().__init__()
        if spec.parallel or spec.norm != "layer":
            raise NotImplementedError(
                "sequential sublayers behind layer norms only")
        self.spec = spec
        self.width = width
        f32 = torch.float32
        K = spec.input_conv
        self.norm1 = nn.Parameter(torch.empty(width, dtype=f32))
        self.norm1_b = nn.Parameter(torch.empty(width, dtype=f32))
        self.conv1 = (nn.Parameter(torch.empty(width, K, dtype=f32))
                      if K else None)
        self.mixer = build_mixer(width, spec.mixer, eps, dtype, max_pos)
        self.mlp = None
        self.norm2 = self.norm2_b = self.conv2 = None
        if spec.mlp is not None:
            if spec.mlp.kind != "moe":
                raise NotImplementedError("routed feed-forwards only")
            self.norm2 = nn.Parameter(torch.empty(width, dtype=f32))
            self.norm2_b = nn.Parameter(torch.empty(width, dtype=f32))
            self.conv2 = (nn.Parameter(torch.empty(width, K, dtype=f32))
                          if K else None)
            self.mlp = SparseMoE(width, spec.mlp, dtype)

    def cache_shape(self):
        """mixer cache, then the convolution tails of both sublayers."""
        parts = [self.mixer.cache_shape()]
        K = self.spec.input_conv
        if K:
            parts.append(("slots", (K - 1, self.width), torch.float32))
            if self.mlp is not None:
                parts.append(("slots", (K - 1, self.width), torch.float32))
        return ("multi", parts)


class DogidraForCausalLM(nn.Module):
    # per-step metadata this family needs from the runner
    needs_seq_meta = True
    # single-token steps route through the all-experts path (router and
    # weighted sum are kernels, no host read), so they replay a hipGraph
    supports_decode_graph = True

    def __init__(self, cfg: ModelConfig, tp: int = 1, pp_rank: int = 0,
                 pp_size: int = 1, dtype: torch.dtype = torch.bfloat16
                 ) -> None:
        super().__init__()
        if tp != 1 or pp_size != 1:
            raise NotImplementedError(
                "Dogidra runs on one GPU per replica (no TP/PP sharding of "
                "the recurrent state yet)")
        self.cfg = cfg
        self.tp = 1
        self.dtype = dtype
        W = cfg.hidden_size
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                              dtype=dtype))
        self.layers = nn.ModuleList(
            DogidraLayer(W, spec, cfg.rms_norm_eps, dtype, cfg.max_position)
            for spec in cfg.layer_specs)
        self.runs = layer_runs(len(self.layers), cfg.loop)
        # x <- W_in [x; x0] at the start of every pass
        self.loop_in = (nn.Parameter(torch.empty(W, 2 * W, dtype=dtype))
                        if cfg.loop else None)
        self.final_norm = nn.Parameter(torch.empty(W, dtype=torch.float32))
        self.final_norm_b = nn.Parameter(torch.empty(W,
                                                     dtype=torch.float32))
        # optional debugging tap: called with (run index, fp32 residual
        # stream after that layer run)
        self.residual_hook = None

    # ---- cache geometry ------------------------------------------------
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def cache_shapes(self):
        """One entry per layer run: a looped layer owns a cache and state
        for every pass."""
        return [self.layers[i].cache_shape() for i, _ in self.runs]

    def _flat_shapes(self):
        def walk(d):
            if d[0] == "multi":
                for c in d[1]:
                    yield from walk(c)
            else:
                yield d
        for d in self.cache_shapes():
            yield from walk(d)

    def kv_bytes_per_block(self, block_size: int) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        n = 0
        for d in self._flat_shapes():
            if d[0] == "kv":
                n += d[1] * block_size * (d[2] + d[3]) * esz
            elif d[0] == "kvpool":
                rows = block_size + (block_size + d[4] - 1) // d[4]
                n += d[1] * rows * (d[2] + d[3]) * esz
        return n

    def state_bytes_per_seq(self) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        n = 0
        for d in self._flat_shapes():
            if d[0] == "slots":
                e = 1
                for s in d[1]:
                    e *= s
                n += e * (4 if d[2] == torch.float32 else esz)
        return n

    def gemm_weights(self):
        """One weight per distinct projection shape of the stack (for the
        per-shape GEMM choice at decode batch sizes)."""
        seen, out = set(), []
        for layer in self.layers:
            mx = layer.mixer
            cands = [mx.fuse()[0], mx.left.out_weight, mx.right.out_weight]
            if layer.mlp is not None and layer.mlp.shared is not None:
                cands += [layer.mlp.fused_in(), layer.mlp.shared.down]
            for w in cands:
                if w is not None and w.dim() == 2 and w.is_contiguous() \
                        and tuple(w.shape) not in seen:
                    seen.add(tuple(w.shape))
                    out.append(w)
        return out

    # ---- weights -------------------------------------------------------
    @torch.no_grad()
    def random_init(self, seed: int = 0) -> None:
        dev = self.embed.device
        gen = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            last = name.rsplit(".", 1)[-1]
            if last in ("norm1", "norm2", "final_norm", "q_norm", "k_norm"):
                p.normal_(1.0, 0.1, generator=gen)
            elif last in ("norm1_b", "norm2_b", "final_norm_b"):
                p.normal_(0.0, 0.1, generator=gen)
            elif last in ("z_bias", "x_bias"):
                p.normal_(0.0, 0.5, generator=gen)
            elif last == "correction":
                p.normal_(0.0, 0.01, generator=gen)
            elif last in ("conv1", "conv2"):
                p.normal_(0.0, 0.3, generator=gen)
            elif last == "embed":
                p.normal_(0.0, 1.0 / max(self.cfg.embedding_scale, 1.0),
                          generator=gen)
            elif last == "loop_in":
                p.normal_(0.0, (0.5 / self.cfg.hidden_size) ** 0.5,
                          generator=gen)
            else:
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
        self._drop_fused()

    def _drop_fused(self) -> None:
        for layer in self.layers:
            layer.mixer._fused = None
            if layer.mlp is not None:
                layer.mlp._fused_in = None

    @torch.no_grad()
    def load_weights(self, path: str) -> None:
        from safetensors import safe_open

        f = safe_open(os.path.join(path, "model.safetensors"),
                      framework="pt", device="cpu")

        def check(t, param, name):
            if t.numel() != param.numel() or (
                    t.dim() == param.dim()
                    and tuple(t.shape) != tuple(param.shape)):
                raise ValueError(
                    f"{name}: checkpoint shape {tuple(t.shape)} != "
                    f"{tuple(param.shape)}")

        def put(param, name):
            t = f.get_tensor(name)
            check(t, param, name)
            param.copy_(t.to(param.dtype).view(param.shape))

        def cat(param, names):
            t = torch.cat([f.get_tensor(n) for n in names], dim=0)
            check(t, param, names)
            param.copy_(t.to(param.dtype))

        put(self.embed, "embed")
        if self.loop_in is not None:
            put(self.loop_in, "loop.in")
        put(self.final_norm, "final.norm")
        put(self.final_norm_b, "final.norm.b")
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            put(layer.norm1, pre + "norm1")
            put(layer.norm1_b, pre + "norm1.b")
            if layer.conv1 is not None:
                put(layer.conv1, pre + "canon1")
            left, right = layer.mixer.left, layer.mixer.right
            lp, rp = pre + "mix.left.", pre + "mix.right."
            cat(left.qkv, [lp + "q", lp + "k", lp + "v"])
            put(left.q_norm, lp + "q.norm")
            put(left.k_norm, lp + "k.norm")
            put(left.out_weight, lp + "o")
            cat(right.in_proj, [rp + "z", rp + "x", rp + "g"])
            put(right.z_bias, rp + "z.b")
            put(right.x_bias, rp + "x.b")
            put(right.out_weight, rp + "o")
            ml, mp = layer.mlp, pre + "mlp."
            if ml is not None:
                put(layer.norm2, pre + "norm2")
                put(layer.norm2_b, pre + "norm2.b")
                if layer.conv2 is not None:
                    put(layer.conv2, pre + "canon2")
                put(ml.router, mp + "router")
                put(ml.correction, mp + "correction")
                for e in range(ml.spec.experts):
                    put(ml.experts_gate_up[e], f"{mp}e{e}.up")
                    put(ml.experts_down[e], f"{mp}e{e}.down")
                if ml.shared is not None:
                    put(ml.shared.gate_up, mp + "shared.up")
                    put(ml.shared.down, mp + "shared.down")
        self._drop_fused()

    # ---- forward -------------------------------------------------------
    def _inject(self, x: torch.Tensor, x0: torch.Tensor) -> torch.Tensor:
        """x <- W_in [x; x0]: a projection of the serving dtype whose result
        becomes the fp32 stream."""
        h = torch.cat([x, x0], dim=1).to(self.dtype)
        return gemm_policy.linear(h, self.loop_in).float()

    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, meta, caches,
                residual=None) -> torch.Tensor:
        cfg = self.cfg
        eps, dt = cfg.rms_norm_eps, self.dtype
        x0 = ops.embed_scale(token_ids, self.embed, cfg.embedding_scale)
        # the stream is updated in place; passes read x0 again
        x = x0.clone() if self.loop_in is not None else x0
        shared: dict = {}
        hook = self.residual_hook
        # steps of single tokens only: every expert over every row
        dense = True if getattr(meta, "num_prefill_tokens", None) == 0 \
            else None
        # sublayer outputs not yet added to the stream: (tensors, scales);
        # the next boundary kernel adds them in fp32
        pend, pend_s = [], []

        def flush():
            for d, s in zip(pend, pend_s):
                x.add_(d.float(), alpha=s)
            pend.clear()
            pend_s.clear()

        for n, ((i, begins), cache) in enumerate(zip(self.runs, caches)):
            layer = self.layers[i]
            K = layer.spec.input_conv
            if begins:
                flush()
                x = self._inject(x, x0)
            h = ops.add_layer_norm_conv32(
                x, pend, pend_s, layer.norm1, layer.norm1_b, eps,
                layer.conv1, cache[1] if K else None, meta.seq_rows, dt)
            mx = layer.mixer
            a, b = mx.forward_parts(h, meta, cache[0], shared)
            pend, pend_s = [a, b], [mx.spec.left_scale, mx.spec.right_scale]
            if layer.mlp is not None:
                h = ops.add_layer_norm_conv32(
                    x, pend, pend_s, layer.norm2, layer.norm2_b, eps,
                    layer.conv2, cache[2] if K else None, meta.seq_rows, dt)
                pend, pend_s = [layer.mlp(h, dense)], [1.0]
            if hook is not None:
                flush()
                hook(n, x)
        return ops.add_layer_norm_conv32(
            x, pend, pend_s, self.final_norm, self.final_norm_b, eps, None,
            None, meta.seq_rows, dt)

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.embed).float()
