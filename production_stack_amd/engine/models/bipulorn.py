"""Bipulorn: a decoder of sequential sublayers whose outputs are normalised
before they join the fp32 residual stream, with three kinds of mixers (a
sliding-window rotary attention and a state-space-duality recurrence side by
side; gated linear attention; a matrix-memory LSTM) and routed feed-forwards
with identity experts and a gated shared expert.

Per layer, with n(x; w) = x / sqrt(mean(x^2) + eps) * (1 + w):
    x <- x + ls1 * n(mixer(n(x; w1)); w1b)
    x <- x + ls2 * n(ff(n(x; w2)); w2b)            (layers with a feed-forward)
and logits = cap * tanh(head n(x; w_final) / cap).

At load time 1 + w is stored for the pre-norms and (1 + wb) * ls for the
post-norms, so a sublayer boundary is ONE kernel: normalise the sublayer's
output, add it to the stream, normalise the stream for the next sublayer
(ops.post_norm_add_norm32). Per layer the GPU work is
    mixer: one GEMM over all input projections (both halves of a pair), the
           mixer kernels (rotary + append + attention + gate | convolution +
           scan + grouped norm | scan), output GEMM(s), pair combine;
    boundary kernel; router + experts + shared expert; boundary kernel.

Numerics: residual stream, all norms, router, attention scores and weights,
decays / gates / step sizes and the recurrences with their states are fp32;
projections, convolutions and activations run in the serving dtype.

config.json layout read here: architecture, vocab, width, norm{eps},
logit_softcap, layers[i] = {type, mixer{...}, mlp{kind, expert{ff},
router{experts, identity, top, scale}, shared{ff}}|null}. Checkpoint names:
embed, head, final.norm, l<i>.norm1/norm1b/norm2/norm2b/ls1/ls2,
l<i>.mix.*, l<i>.mlp.*.
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

ARCHITECTURE = "Bipulorn"

# positions a rotary table is built for unless the engine asks for more
DEFAULT_MAX_POSITION = 8192

# the chosen experts' weights are divided by their sum plus this
ROUTE_RENORM_EPS = 1e-20


# ---------------------------------------------------------------------------
# configuration
# ---------------------------------------------------------------------------
def _attention_spec(m: dict) -> MixerSpec:
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    return MixerSpec(
        kind="attention", heads=m["heads"], dim=m["dim"],
        kv_heads=m.get("kv_heads", m["heads"]),
        vdim=m.get("vdim", m["dim"]), scale=float(m["scale"]),
        window=int((m.get("mask") or {}).get("size", 0)),
        rope=dims > 0, rot_dims=dims,
        rot_base=float(rot.get("base", 10000.0)),
        rot_factor=float((rot.get("scaling") or {}).get("factor", 1.0)),
        bias=True, out_bias=True, out_gate=True)


def _ssd_spec(m: dict) -> MixerSpec:
    return MixerSpec(
        kind="ssd", heads=m["heads"], dim=m["state"], state=m["state"],
        vdim=m["vdim"], groups=int(m.get("groups", 1)),
        norm_groups=int(m.get("norm_groups", 1)),
        conv=int(m.get("conv", 1)), rope=False)


def _mixer_spec(kind: str, m: dict, rank: int) -> MixerSpec:
    if kind == "parallel":
        left, right = _attention_spec(m["left"]), _ssd_spec(m["right"])
        return MixerSpec(kind="pair", heads=left.heads, dim=left.dim,
                         rope=False, left=left, right=right)
    if kind == "gla":
        return MixerSpec(
            kind="gla", heads=m["heads"], dim=m["dim"],
            vdim=m.get("vdim", m["dim"]), tau=float(m["tau"]),
            decay_rank=int(rank or m.get("decay_rank", 0)), rope=False)
    if kind == "mlstm":
        return MixerSpec(
            kind="mlstm", heads=m["heads"], dim=m["dim"],
            vdim=m.get("vdim", m["dim"]), gate_cap=float(m["gate_cap"]),
            rope=False)
    raise ValueError(f"unknown layer type {kind!r}")


def _mlp_spec(m: Optional[dict]) -> Optional[MlpSpec]:
    if m is None:
        return None
    if m.get("kind", "moe") != "moe":
        raise ValueError(f"unknown mlp kind {m['kind']!r}")
    r = m["router"]
    return MlpSpec(
        kind="moe", ff=int(m["expert"]["ff"]), act="silu",
        experts=int(r["experts"]), top=int(r["top"]), score="softmax",
        renormalize=True, weight_on_input=False,
        shared_ff=int((m.get("shared") or {}).get("ff", 0)),
        correction=True, identity=int(r.get("identity", 0)),
        route_scale=float(r.get("scale", 1.0)),
        renorm_eps=ROUTE_RENORM_EPS)


def config_from_json(cfg: dict, name: str = "bipulorn",
                     ranks: Optional[dict] = None) -> ModelConfig:
    """ranks: layer index -> rows of the low-rank decay projection of a
    gated-linear-attention layer (a tensor shape, not a config.json entry;
    the checkpoint reader passes them in, named configs carry them as
    mixer.decay_rank)."""
    specs: List[LayerSpec] = []
    for i, layer in enumerate(cfg["layers"]):
        specs.append(LayerSpec(
            mixer=_mixer_spec(layer["type"], layer["mixer"],
                              (ranks or {}).get(i, 0)),
            mlp=_mlp_spec(layer.get("mlp")), parallel=False,
            post_norm=True, layer_scale=True))
    att = [s.mixer.left for s in specs if s.mixer.kind == "pair"]
    ffs = [max(s.mlp.ff, s.mlp.shared_ff) for s in specs
           if s.mlp is not None]
    return ModelConfig(
        name=name, family="bipulorn", hidden_size=cfg["width"],
        num_layers=len(specs),
        num_q_heads=max([m.heads for m in att], default=1),
        num_kv_heads=max([m.kv_heads for m in att], default=1),
        head_dim=max([m.dim for m in att], default=1),
        intermediate_size=max(ffs, default=0), vocab_size=cfg["vocab"],
        max_position=int(cfg.get("max_position", DEFAULT_MAX_POSITION)),
        rms_norm_eps=float(cfg["norm"]["eps"]), layer_specs=specs,
        logit_softcap=float(cfg.get("logit_softcap") or 0.0),
        # no BOS/EOS convention in this design: never stop on a token id
        bos_token_id=0, eos_token_id=-1)


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    ranks: dict = {}
    st = os.path.join(path, "model.safetensors")
    if os.path.exists(st):
        from production_stack_amd.engine.weights import safetensors_header

        for key, info in safetensors_header(st).items():
            parts = key.split(".")
            if len(parts) == 3 and parts[1] == "mix" and parts[2] == "a1":
                ranks[int(parts[0][1:])] = int(info["shape"][0])
    return config_from_json(cfg, name=os.path.basename(
        os.path.normpath(path)) or "bipulorn", ranks=ranks)


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------
class BipulornLayer(nn.Module):
    def __init__(self, width: int, spec: LayerSpec, eps: float,
                 dtype: torch.dtype, max_pos: int) -> None:
        super().__init__()
        if spec.parallel or not spec.post_norm:
            raise NotImplementedError(
                "sequential sublayers with normalised outputs only")
        self.spec = spec
        f32 = torch.float32
        # pre-norm weights hold 1 + w; post-norm weights (1 + w) * scale
        self.norm1 = nn.Parameter(torch.empty(width, dtype=f32))
        self.post1 = nn.Parameter(torch.empty(width, dtype=f32))
        self.mixer = build_mixer(width, spec.mixer, eps, dtype, max_pos)
        self.mlp = None
        self.norm2 = self.post2 = None
        if spec.mlp is not None:
            if spec.mlp.kind != "moe":
                raise NotImplementedError("routed feed-forwards only")
            self.norm2 = nn.Parameter(torch.empty(width, dtype=f32))
            self.post2 = nn.Parameter(torch.empty(width, dtype=f32))
            self.mlp = SparseMoE(width, spec.mlp, dtype)


class BipulornForCausalLM(nn.Module):
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
                "Bipulorn runs on one GPU per replica (no TP/PP sharding of "
                "the recurrent state yet)")
        self.cfg = cfg
        self.tp = 1
        self.dtype = dtype
        W = cfg.hidden_size
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                              dtype=dtype))
        self.layers = nn.ModuleList(
            BipulornLayer(W, spec, cfg.rms_norm_eps, dtype,
                          cfg.max_position)
            for spec in cfg.layer_specs)
        self.final_norm = nn.Parameter(torch.empty(W, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))
        # optional debugging tap: called with (layer index, fp32 residual
        # stream after that layer)
        self.residual_hook = None

    # ---- cache geometry ------------------------------------------------
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def cache_shapes(self):
        return [layer.mixer.cache_shape() for layer in self.layers]

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
        return sum(d[1] * block_size * (d[2] + d[3]) * esz
                   for d in self._flat_shapes() if d[0] == "kv")

    def state_bytes_per_seq(self) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        n = 0
        for d in self._flat_shapes():
            if d[0] == "state":
                n += d[1] * d[2] * d[3] * 4
            elif d[0] == "slots":
                e = 1
                for s in d[1]:
                    e *= s
                n += e * (4 if d[2] == torch.float32 else esz)
        return n

    def gemm_weights(self):
        """One weight per distinct projection shape of the stack (for the
        per-shape GEMM choice at decode batch sizes)."""
        seen, out = set(), []

        def mixer_weights(mx):
            if mx.kind == "pair":
                yield mx.fuse()[0]
                for half in (mx.left, mx.right):
                    yield half.out_weight
                return
            yield from mx.in_params()
            yield getattr(mx, "a2", None)
            yield mx.out_weight

        for layer in self.layers:
            cands = list(mixer_weights(layer.mixer))
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
            if last in ("norm1", "norm2", "final_norm", "out_norm",
                        "left_norm", "right_norm"):
                p.normal_(1.0, 0.1, generator=gen)
            elif last in ("post1", "post2"):
                p.normal_(0.5, 0.05, generator=gen)
            elif last in ("a_bias", "i_bias", "dt_bias", "qkv_bias",
                          "out_bias", "conv_b"):
                p.normal_(0.0, 0.5, generator=gen)
            elif last == "f_bias":
                p.normal_(3.0, 0.5, generator=gen)
            elif last == "a_log":
                p.uniform_(-1.0, 1.0, generator=gen)
            elif last == "d_skip":
                p.normal_(1.0, 0.2, generator=gen)
            elif last == "correction":
                p.normal_(0.0, 0.01, generator=gen)
            elif last == "conv_w":
                p.normal_(0.0, 0.5, generator=gen)
            else:
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
        self._drop_fused()

    def _drop_fused(self) -> None:
        for layer in self.layers:
            if layer.mixer.kind == "pair":
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

        def cat(param, names, pad_rows: int = 0):
            ts = [f.get_tensor(n) for n in names]
            if pad_rows:
                ts.append(torch.zeros((pad_rows, *ts[0].shape[1:]),
                                      dtype=ts[0].dtype))
            t = torch.cat(ts, dim=0)
            check(t, param, names)
            param.copy_(t.to(param.dtype))

        def unit_offset(param, name):
            # the checkpoint holds the weight's offset from one
            t = f.get_tensor(name)
            check(t, param, name)
            param.copy_(1.0 + t.float())

        def post(param, norm_name, scale_name):
            t = 1.0 + f.get_tensor(norm_name).float()
            check(t, param, norm_name)
            param.copy_(t * f.get_tensor(scale_name).float())

        def attention(mx, mp):
            gate = mx.spec.out_gate
            cat(mx.qkv, [mp + n for n in
                         (("q", "k", "v", "g") if gate else ("q", "k", "v"))])
            if mx.qkv_bias is not None:
                cat(mx.qkv_bias, [mp + "q.b", mp + "k.b", mp + "v.b"],
                    pad_rows=mx.H * mx.DV if gate else 0)
            put(mx.out_weight, mp + "o")
            if mx.out_bias is not None:
                put(mx.out_bias, mp + "o.b")

        def ssd(mx, mp):
            put(mx.in_proj, mp + "in")
            put(mx.conv_w, mp + "conv")
            put(mx.conv_b, mp + "conv.b")
            put(mx.dt_bias, mp + "dt_bias")
            put(mx.a_log, mp + "A_log")
            put(mx.d_skip, mp + "D")
            put(mx.out_norm, mp + "norm")
            put(mx.out_weight, mp + "o")

        put(self.embed, "embed")
        put(self.lm_head, "head")
        unit_offset(self.final_norm, "final.norm")
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            unit_offset(layer.norm1, pre + "norm1")
            post(layer.post1, pre + "norm1b", pre + "ls1")
            mx, mp = layer.mixer, pre + "mix."
            if mx.kind == "pair":
                attention(mx.left, mp + "left.")
                ssd(mx.right, mp + "right.")
                put(mx.left_norm, mp + "left.out")
                put(mx.right_norm, mp + "right.out")
            elif mx.kind == "gla":
                cat(mx.in_proj, [mp + n for n in
                                 ("q", "k", "v", "g", "a1")])
                put(mx.a2, mp + "a2")
                put(mx.a_bias, mp + "a2.b")
                put(mx.out_norm, mp + "norm")
                put(mx.out_weight, mp + "o")
            elif mx.kind == "mlstm":
                cat(mx.in_proj, [mp + n for n in
                                 ("q", "k", "v", "g", "i", "f")])
                put(mx.i_bias, mp + "i.b")
                put(mx.f_bias, mp + "f.b")
                put(mx.out_norm, mp + "norm")
                put(mx.out_weight, mp + "o")
            else:
                raise ValueError(f"no loader for mixer kind {mx.kind!r}")
            ml, lp = layer.mlp, pre + "mlp."
            if ml is not None:
                unit_offset(layer.norm2, pre + "norm2")
                post(layer.post2, pre + "norm2b", pre + "ls2")
                put(ml.router, lp + "router")
                put(ml.correction, lp + "correction")
                for e in range(ml.spec.experts):
                    ep = f"{lp}e{e}."
                    cat(ml.experts_gate_up[e], [ep + "gate", ep + "up"])
                    put(ml.experts_down[e], ep + "down")
                if ml.shared is not None:
                    sp = lp + "shared."
                    cat(ml.shared.gate_up, [sp + "gate", sp + "up"])
                    put(ml.shared.down, sp + "down")
                    put(ml.shared_gate, sp + "sg")
        self._drop_fused()

    # ---- forward -------------------------------------------------------
    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, meta, caches,
                residual=None) -> torch.Tensor:
        cfg = self.cfg
        eps, dt = cfg.rms_norm_eps, self.dtype
        x = ops.embed_scale(token_ids, self.embed, 1.0)       # fp32 [T, W]
        layers = self.layers
        h = ops.add_rms_norm32(x, [], layers[0].norm1, eps, dt)
        shared: dict = {}
        hook = self.residual_hook
        # steps of single tokens only: every expert over every row
        dense = True if getattr(meta, "num_prefill_tokens", None) == 0 \
            else None
        for i, (layer, cache) in enumerate(zip(layers, caches)):
            mx = layer.mixer
            delta, w_post = mx.project(mx(h, meta, cache, shared)), \
                layer.post1
            if layer.mlp is not None:
                h = ops.post_norm_add_norm32(x, delta, w_post, layer.norm2,
                                             eps, dt)
                delta, w_post = layer.mlp(h, dense), layer.post2
            w_next = (layers[i + 1].norm1 if i + 1 < len(layers)
                      else self.final_norm)
            h = ops.post_norm_add_norm32(x, delta, w_post, w_next, eps, dt)
            if hook is not None:
                hook(i, x)
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.lm_head).float()
        cap = self.cfg.logit_softcap
        if cap > 0:
            logits = torch.tanh(logits.mul_(1.0 / cap)).mul_(cap)
        return logits
