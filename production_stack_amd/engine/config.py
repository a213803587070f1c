"""Engine configuration.

Mirrors the engine-flag surface the reference deploys through helm
(`vllm serve` argv assembled at reference helm/templates/
deployment-vllm-multi.yaml:127-221 — SURVEY.md section 2.9): model, dtype,
max-model-len, max-num-seqs, gpu-memory-utilization, enable-prefix-caching,
enable-chunked-prefill, kv-transfer role. Architecture definitions are local
(random-init weights by default: no network in the build environment).
"""

from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional


@dataclass
class MixerSpec:
    """One layer's token mixer.

    kind "attention": softmax attention over a paged KV cache. `chunk`
    restricts every query to keys of its own aligned block of positions
    (0 = plain causal), `window` to the trailing N keys (0 = off) with the
    first `keep_first` keys of the sequence staying visible behind it,
    `sink` adds a value-less key to the softmax denominator (score 0, or a
    learned per-head score with `learned_sink`), `softcap` squashes scores
    to cap * tanh(score / cap) (0 = off), `talking_heads` mixes the heads'
    scores with a learned [H, H] matrix before the softmax, `rope` applies
    the rotary position code, `bias` adds projection biases to q/k/v,
    `qk_norm` RMS-normalises every query and key head with a learned
    weight, `v_mix` blends the layer's values with those of the first
    `v_mix` layer of the stack (learned scalar weight).
    kind "latent_attention": keys and values of all heads are expanded from
    one cached latent of `kv_rank` entries per token; every head has `dim`
    position-free query/key entries and `rot_dim` rotated ones (the rotated
    key part is shared by the heads); `rot_dims` leading entries of the
    rotated part turn with base `rot_base`, interleaved pairs.
    kind "general_delta" / "channel_delta": gated delta-rule linear
    recurrences with a per-sequence fp32 state of heads x dim x vdim;
    `decay_rank` is the width of the low-rank decay projection
    (general_delta), `conv` the taps of the short causal convolution on
    q/k/v and `gate_rank` the width of the low-rank output gate
    (channel_delta).
    Attention with `rope` and `rot_dims` > 0 turns the first `rot_dims`
    entries of every query and key head (interleaved pairs, base
    `rot_base`, positions divided by `rot_factor`); `out_gate` multiplies
    the concatenated heads by sigmoid(W_g h), `out_bias` adds a bias to the
    output projection.
    kind "gla" / "ssd" / "mlstm": gated linear recurrences without a
    removal term (state heads x dim x vdim): "gla" decays every key channel
    by sigmoid(low-rank projection of width `decay_rank`)^(1/`tau`); "ssd"
    is the state-space-duality mixer (`state` = dim entries per head,
    keys/queries shared by `groups` groups, convolution of `conv` taps, one
    step size and decay per head, gated read-out normalised in
    `norm_groups` parts); "mlstm" has exponential input/forget gates capped
    at +-`gate_cap`, a running maximum and a normaliser.
    kind "pair": two mixers `left` and `right` read the same input; the
    result is the mean of their separately normalised outputs, or
    (`combine` "weighted") left_scale * left + right_scale * right.
    Attention options of the windowed kind: `window_pool` = P > 0 adds, for
    every block of P consecutive positions that lies wholly before a
    query's window, one key and value (the block's means as cached) to the
    softmax; `qk_norm_all` RMS-normalises the whole query (and key)
    projection at once, weights of that full size; `rot_layout` "half"
    pairs entry i with entry i + rot_dims/2 instead of its neighbour;
    `rot_scaling` = (factor, original length, fast turns, slow turns)
    blends every frequency between itself and itself / factor by where its
    number of turns over the original length falls, and scales cos/sin by
    0.1 ln(factor) + 1.
    kind "mingru": an element-wise gated recurrence over `vdim` channels
    (heads = 1) whose gate and candidate read the current token only:
    S <- (1 - z) S + z c, z = sigmoid(W_z h + b_z), c = u + 1/2 for
    u = W_x h + b_x >= 0 and sigmoid(u) below; read-out S silu(W_g h).
    """

    kind: str
    heads: int
    dim: int
    kv_heads: int = 0
    vdim: int = 0
    scale: float = 0.0
    chunk: int = 0
    window: int = 0
    sink: bool = False
    talking_heads: bool = False
    rope: bool = True
    decay_rank: int = 0
    keep_first: int = 0
    softcap: float = 0.0
    learned_sink: bool = False
    bias: bool = False
    qk_norm: bool = False
    v_mix: bool = False
    kv_rank: int = 0
    rot_dim: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    conv: int = 0
    gate_rank: int = 0
    rot_factor: float = 1.0
    out_gate: bool = False
    out_bias: bool = False
    state: int = 0
    groups: int = 0
    norm_groups: int = 1
    tau: float = 1.0
    gate_cap: float = 0.0
    left: Optional["MixerSpec"] = None
    right: Optional["MixerSpec"] = None
    window_pool: int = 0
    qk_norm_all: bool = False
    rot_layout: str = "interleaved"   # interleaved | half
    rot_scaling: Optional[tuple] = None
    combine: str = "norm_mean"        # norm_mean | weighted (pair)
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class MlpSpec:
    """One layer's feed-forward. kind "dense": gated MLP with `act`.
    kind "moe": `experts` small gated MLPs of width `ff`, `top` per token,
    routed by `score` ("softmax" | "sigmoid") with optional renormalised
    weights applied to the expert's output or (`weight_on_input`) input;
    an always-on shared expert of width `shared_ff` may be added, scaled by
    a per-token sigmoid gate. `correction`: a learned per-expert offset
    joins the scores for the choice only; `identity`: that many extra
    router outputs (after the experts) stand for experts that return their
    input; `route_scale` multiplies the final weights; `renorm_eps` is
    added to the sum the chosen weights are divided by. `gated` False:
    experts (and the shared expert) are down(act(up x)) without a gate
    branch; `shared_gate` False: the shared expert joins unscaled. act
    "relu2" is relu(z)^2."""

    kind: str
    ff: int
    act: str = "silu"          # silu | gelu_tanh | clamped_swish | relu2
    limit: float = 0.0
    experts: int = 0
    top: int = 0
    score: str = "softmax"
    renormalize: bool = True
    weight_on_input: bool = False
    shared_ff: int = 0
    shared_limit: float = 0.0
    correction: bool = False
    identity: int = 0
    route_scale: float = 1.0
    renorm_eps: float = 0.0
    gated: bool = True
    shared_gate: bool = True


@dataclass
class LayerSpec:
    mixer: MixerSpec
    mlp: Optional[MlpSpec]
    # True: mixer and feed-forward both read one norm's output and their
    # sum joins the residual; False: sequential pre-norm sublayers
    parallel: bool = False
    # the mixer's input is blended with the previous token's (learned
    # per-channel weight); the previous input is per-sequence state
    token_shift: bool = False
    # the layer hands on a learned weighted sum of the embedding output and
    # all layer results so far instead of its own result
    depth_average: bool = False
    # every sublayer's output is RMS-normalised (own weight) before it
    # joins the residual stream, and then scaled per channel (`layer_scale`)
    post_norm: bool = False
    layer_scale: bool = False
    # "rms" or "layer" (mean removed, weight and bias)
    norm: str = "rms"
    # taps of the causal per-channel convolution over time that every
    # sublayer's normed input h passes as h + conv(h) (0 = none); the last
    # taps - 1 normed inputs of both sublayers are per-sequence state
    input_conv: int = 0


@dataclass
class ModelConfig:
    name: str
    hidden_size: int
    num_layers: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rope_theta: float = 500000.0
    max_position: int = 8192
    rms_norm_eps: float = 1e-5
    bos_token_id: int = 1
    eos_token_id: int = 2
    # family knobs: Qwen2 uses qkv biases; Mistral attends over a sliding
    # window; small models often tie lm_head to the embedding
    qkv_bias: bool = False
    tie_word_embeddings: bool = False
    sliding_window: Optional[int] = None
    # Llama-3.1-style RoPE frequency scaling (None = off):
    # (factor, low_freq_factor, high_freq_factor, original_max_position)
    rope_scaling: Optional[tuple] = None
    # Mixtral-style sparse MoE MLP: num_experts > 0 replaces the dense
    # gate/up/down with per-expert projections + a top-k router
    num_experts: int = 0
    num_experts_per_tok: int = 2
    # model family: selects the model class in engine/models/registry.py
    family: str = "llama"
    # heterogeneous stacks (family != "llama"): one spec per layer; the
    # scalar head/ff fields above then hold the stack's maxima
    layer_specs: Optional[list] = None
    embedding_scale: float = 1.0
    # RMS norms of the stack normalise this many equal consecutive parts
    # of the vector separately
    norm_groups: int = 1
    # logits become cap * tanh(logits / cap) (0 = off)
    logit_softcap: float = 0.0
    # (start, stop, times): layers start .. stop-1 run `times` times in a
    # row with the same weights, every pass with a cache and state of its
    # own; each pass begins with x <- W_in [x; embedding output]
    loop: Optional[tuple] = None

    @property
    def has_recurrent_state(self) -> bool:
        return bool(self.layer_specs) and any(
            ls.mixer.kind not in ("attention", "latent_attention")
            or ls.token_shift or ls.input_conv > 1
            for ls in self.layer_specs)

    @property
    def q_size(self) -> int:
        return self.num_q_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim


# Named architectures (shapes follow the public HF configs for the Llama
# family; weights are random-init — see BASELINE.md: synthetic data /
# random-init weights).
ARCHITECTURES = {
    "llama-3-8b": ModelConfig(
        name="llama-3-8b",
        hidden_size=4096,
        num_layers=32,
        num_q_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=8192,
    ),
    "llama-3-70b": ModelConfig(
        name="llama-3-70b",
        hidden_size=8192,
        num_layers=80,
        num_q_heads=64,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=28672,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=8192,
    ),
    "llama-3.1-8b": ModelConfig(
        name="llama-3.1-8b",
        hidden_size=4096,
        num_layers=32,
        num_q_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=131072,
        rope_scaling=(8.0, 1.0, 4.0, 8192),
    ),
    "llama-3.1-70b": ModelConfig(
        name="llama-3.1-70b",
        hidden_size=8192,
        num_layers=80,
        num_q_heads=64,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=28672,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=131072,
        rope_scaling=(8.0, 1.0, 4.0, 8192),
    ),
    "llama-2-7b": ModelConfig(
        name="llama-2-7b",
        hidden_size=4096,
        num_layers=32,
        num_q_heads=32,
        num_kv_heads=32,
        head_dim=128,
        intermediate_size=11008,
        vocab_size=32000,
        rope_theta=10000.0,
        max_position=4096,
    ),
    "llama-2-13b": ModelConfig(
        name="llama-2-13b",
        hidden_size=5120,
        num_layers=40,
        num_q_heads=40,
        num_kv_heads=40,
        head_dim=128,
        intermediate_size=13824,
        vocab_size=32000,
        rope_theta=10000.0,
        max_position=4096,
    ),
    "llama-3.2-1b": ModelConfig(
        name="llama-3.2-1b",
        hidden_size=2048,
        num_layers=16,
        num_q_heads=32,
        num_kv_heads=8,
        head_dim=64,
        intermediate_size=8192,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=8192,
        tie_word_embeddings=True,
    ),
    "llama-3.2-3b": ModelConfig(
        name="llama-3.2-3b",
        hidden_size=3072,
        num_layers=28,
        num_q_heads=24,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=8192,
        vocab_size=128256,
        rope_theta=500000.0,
        max_position=8192,
        tie_word_embeddings=True,
    ),
    "qwen2-72b": ModelConfig(
        name="qwen2-72b",
        hidden_size=8192,
        num_layers=80,
        num_q_heads=64,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=29568,
        vocab_size=152064,
        rope_theta=1000000.0,
        max_position=32768,
        qkv_bias=True,
    ),
    "mistral-7b": ModelConfig(
        name="mistral-7b",
        hidden_size=4096,
        num_layers=32,
        num_q_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=32000,
        rope_theta=10000.0,
        max_position=32768,
        sliding_window=4096,
    ),

    "mixtral-8x7b": ModelConfig(
        name="mixtral-8x7b",
        hidden_size=4096,
        num_layers=32,
        num_q_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=32000,
        rope_theta=1e6,
        max_position=32768,
        num_experts=8,
        num_experts_per_tok=2,
    ),
    "tiny-mixtral": ModelConfig(
        name="tiny-mixtral",
        hidden_size=64,
        num_layers=2,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=16,
        intermediate_size=128,
        vocab_size=512,
        max_position=512,
        num_experts=4,
        num_experts_per_tok=2,
    ),
    "qwen2-7b": ModelConfig(
        name="qwen2-7b",
        hidden_size=3584,
        num_layers=28,
        num_q_heads=28,
        num_kv_heads=4,
        head_dim=128,
        intermediate_size=18944,
        vocab_size=152064,
        rope_theta=1000000.0,
        max_position=32768,
        qkv_bias=True,
    ),
    # Small config for tests (CPU-runnable).
    "tiny-llama": ModelConfig(
        name="tiny-llama",
        hidden_size=128,
        num_layers=2,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=32,
        intermediate_size=256,
        vocab_size=1024,
        rope_theta=10000.0,
        max_position=2048,
    ),
    "tiny-mistral": ModelConfig(
        name="tiny-mistral",
        hidden_size=128,
        num_layers=2,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=32,
        intermediate_size=256,
        vocab_size=1024,
        rope_theta=10000.0,
        max_position=2048,
        sliding_window=48,
    ),
    "tiny-qwen2": ModelConfig(
        name="tiny-qwen2",
        hidden_size=128,
        num_layers=2,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=32,
        intermediate_size=256,
        vocab_size=1024,
        rope_theta=10000.0,
        max_position=2048,
        qkv_bias=True,
        tie_word_embeddings=True,
    ),
    "mini-mistral": ModelConfig(
        name="mini-mistral",
        hidden_size=512,
        num_layers=4,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=1024,
        vocab_size=2048,
        rope_theta=10000.0,
        max_position=4096,
        sliding_window=64,
    ),
    # GPU-runnable small config with kernel-supported head_dim.
    "mini-mixtral": ModelConfig(
        name="mini-mixtral",
        hidden_size=512,
        num_layers=4,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=1024,
        vocab_size=2048,
        rope_theta=10000.0,
        max_position=4096,
        num_experts=4,
        num_experts_per_tok=2,
    ),
    "mini-llama": ModelConfig(
        name="mini-llama",
        hidden_size=512,
        num_layers=4,
        num_q_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=1024,
        vocab_size=2048,
        rope_theta=10000.0,
        max_position=4096,
    ),
}


def _nanurax_stack(
    name: str, width: int, vocab: int, n_layers: int, *, delta_heads: int,
    delta_dim: int, decay_rank: int, attn_heads: int, attn_kv: int,
    attn_dim: int, chunk: int, ff: int, experts: int, top: int,
    expert_ff: int, shared_ff: int, limit: float = 7.0,
) -> ModelConfig:
    """A Nanurax stack in the repeating order delta+dense, delta+routed,
    attention+dense, delta+routed (three recurrent layers per attention
    layer, every other feed-forward routed)."""
    pattern = [("general_delta", "dense"), ("general_delta", "moe"),
               ("attention", "dense"), ("general_delta", "moe")]
    specs = []
    for i in range(n_layers):
        mk, fk = pattern[i % len(pattern)]
        if mk == "attention":
            mixer = MixerSpec(
                kind="attention", heads=attn_heads, dim=attn_dim,
                kv_heads=attn_kv, vdim=attn_dim,
                scale=attn_dim ** -0.5, chunk=chunk, sink=True,
                talking_heads=True, rope=False)
        else:
            mixer = MixerSpec(kind="general_delta", heads=delta_heads,
                              dim=delta_dim, rope=False,
                              decay_rank=decay_rank)
        if fk == "dense":
            mlp = MlpSpec(kind="dense", ff=ff, act="gelu_tanh")
        else:
            mlp = MlpSpec(
                kind="moe", ff=expert_ff, act="clamped_swish", limit=limit,
                experts=experts, top=top, score="sigmoid",
                renormalize=False, weight_on_input=True,
                shared_ff=shared_ff, shared_limit=limit)
        specs.append(LayerSpec(mixer=mixer, mlp=mlp, parallel=True))
    return ModelConfig(
        name=name, family="nanurax", hidden_size=width,
        num_layers=n_layers, num_q_heads=attn_heads, num_kv_heads=attn_kv,
        head_dim=attn_dim, intermediate_size=ff, vocab_size=vocab,
        max_position=1 << 20, layer_specs=specs,
        embedding_scale=float(width) ** 0.5, bos_token_id=0,
        eos_token_id=-1)


ARCHITECTURES.update({
    # CPU-runnable test config
    "tiny-nanurax": _nanurax_stack(
        "tiny-nanurax", 96, 384, 4, delta_heads=3, delta_dim=32,
        decay_rank=8, attn_heads=6, attn_kv=3, attn_dim=16, chunk=40,
        ff=160, experts=5, top=2, expert_ff=32, shared_ff=64),
    # llama-3.2-1b-sized stack (same width, depth, dense ff and vocab)
    "nanurax-1b": _nanurax_stack(
        "nanurax-1b", 2048, 128256, 16, delta_heads=32, delta_dim=64,
        decay_rank=64, attn_heads=32, attn_kv=8, attn_dim=64, chunk=1024,
        ff=8192, experts=8, top=2, expert_ff=2048, shared_ff=2048),
    # llama-3-8b-sized layers (width 4096, head dim 128, ff 14336)
    "nanurax-8b": _nanurax_stack(
        "nanurax-8b", 4096, 128256, 32, delta_heads=32, delta_dim=128,
        decay_rank=64, attn_heads=32, attn_kv=8, attn_dim=128, chunk=2048,
        ff=14336, experts=8, top=2, expert_ff=3584, shared_ff=3584),
})


def _derusun_stack(
    name: str, width: int, vocab: int, n_layers: int, *, delta_heads: int,
    delta_kv: int, delta_dim: int, delta_vdim: int, conv: int, rank: int,
    attn_heads: int, attn_kv: int, attn_dim: int, window: int,
    keep_first: int, softcap: float, lat_heads: int, lat_dim: int,
    lat_rot: int, lat_vdim: int, kv_rank: int, ff: int, limit: float = 7.0,
    groups: int = 4,
) -> ModelConfig:
    """A Derusun stack in the repeating order channel-delta, windowed
    attention, channel-delta, latent attention; sequential sublayers, every
    layer with a dense clamped-swish feed-forward, token shift and
    depth-weighted streams; all windowed layers mix values."""
    specs = []
    for i in range(n_layers):
        k = i % 4
        if k in (0, 2):
            mixer = MixerSpec(
                kind="channel_delta", heads=delta_heads, kv_heads=delta_kv,
                dim=delta_dim, vdim=delta_vdim, conv=conv, decay_rank=rank,
                gate_rank=rank, rope=False)
        elif k == 1:
            mixer = MixerSpec(
                kind="attention", heads=attn_heads, kv_heads=attn_kv,
                dim=attn_dim, vdim=attn_dim, scale=attn_dim ** -0.5,
                window=window, keep_first=keep_first, softcap=softcap,
                sink=True, learned_sink=True, bias=True, qk_norm=True,
                v_mix=True, rope=False)
        else:
            mixer = MixerSpec(
                kind="latent_attention", heads=lat_heads, kv_heads=1,
                dim=lat_dim, vdim=lat_vdim, kv_rank=kv_rank,
                rot_dim=lat_rot, rot_dims=lat_rot, rot_base=1e6,
                scale=(lat_dim + lat_rot) ** -0.5, sink=True,
                learned_sink=True, rope=True)
        specs.append(LayerSpec(
            mixer=mixer,
            mlp=MlpSpec(kind="dense", ff=ff, act="clamped_swish",
                        limit=limit),
            parallel=False, token_shift=True, depth_average=True))
    return ModelConfig(
        name=name, family="derusun", hidden_size=width,
        num_layers=n_layers, num_q_heads=attn_heads, num_kv_heads=attn_kv,
        head_dim=attn_dim, intermediate_size=ff, vocab_size=vocab,
        max_position=8192, layer_specs=specs, norm_groups=groups,
        bos_token_id=0, eos_token_id=-1)


ARCHITECTURES.update({
    # CPU-runnable test config
    "tiny-derusun": _derusun_stack(
        "tiny-derusun", 96, 384, 4, delta_heads=4, delta_kv=2,
        delta_dim=16, delta_vdim=24, conv=3, rank=8, attn_heads=6,
        attn_kv=3, attn_dim=16, window=40, keep_first=2, softcap=10.0,
        lat_heads=4, lat_dim=16, lat_rot=8, lat_vdim=12, kv_rank=24,
        ff=160, limit=2.0, groups=3),
    # llama-3.2-1b-sized stack (same width, depth, ff and vocab)
    "derusun-1b": _derusun_stack(
        "derusun-1b", 2048, 128256, 16, delta_heads=32, delta_kv=16,
        delta_dim=64, delta_vdim=64, conv=4, rank=64, attn_heads=32,
        attn_kv=8, attn_dim=64, window=1024, keep_first=4, softcap=30.0,
        lat_heads=32, lat_dim=64, lat_rot=32, lat_vdim=64, kv_rank=256,
        ff=8192),
    # llama-3-8b-sized layers (width 4096, head dim 128, ff 14336)
    "derusun-8b": _derusun_stack(
        "derusun-8b", 4096, 128256, 32, delta_heads=32, delta_kv=16,
        delta_dim=128, delta_vdim=128, conv=4, rank=128, attn_heads=32,
        attn_kv=8, attn_dim=128, window=2048, keep_first=4, softcap=30.0,
        lat_heads=32, lat_dim=128, lat_rot=64, lat_vdim=128, kv_rank=512,
        ff=14336),
})


def _bipulorn_stack(
    name: str, width: int, vocab: int, n_layers: int, *, attn_heads: int,
    attn_kv: int, attn_dim: int, window: int, rot_dims: int,
    rot_factor: float, ssd_heads: int, ssd_vdim: int, ssd_state: int,
    ssd_groups: int, ssd_norm_groups: int, conv: int, gla_heads: int,
    gla_dim: int, gla_vdim: int, decay_rank: int, tau: float,
    lstm_heads: int, lstm_dim: int, lstm_vdim: int, gate_cap: float,
    experts: int, identity: int, top: int, expert_ff: int, shared_ff: int,
    route_scale: float = 1.0, softcap: float = 30.0,
) -> ModelConfig:
    """A Bipulorn stack in the repeating order pair (window attention +
    state-space), gated linear attention, pair, matrix LSTM; sequential
    sublayers with normalised, channel-scaled outputs, every layer with a
    routed feed-forward (identity outputs, score correction, gated shared
    expert)."""
    specs = []
    for i in range(n_layers):
        k = i % 4
        if k in (0, 2):
            left = MixerSpec(
                kind="attention", heads=attn_heads, kv_heads=attn_kv,
                dim=attn_dim, vdim=attn_dim, scale=attn_dim ** -0.5,
                window=window, rope=True, rot_dims=rot_dims,
                rot_base=10000.0, rot_factor=rot_factor, bias=True,
                out_bias=True, out_gate=True)
            right = MixerSpec(
                kind="ssd", heads=ssd_heads, dim=ssd_state, state=ssd_state,
                vdim=ssd_vdim, groups=ssd_groups,
                norm_groups=ssd_norm_groups, conv=conv, rope=False)
            mixer = MixerSpec(kind="pair", heads=attn_heads, dim=attn_dim,
                              rope=False, left=left, right=right)
        elif k == 1:
            mixer = MixerSpec(kind="gla", heads=gla_heads, dim=gla_dim,
                              vdim=gla_vdim, tau=tau, decay_rank=decay_rank,
                              rope=False)
        else:
            mixer = MixerSpec(kind="mlstm", heads=lstm_heads, dim=lstm_dim,
                              vdim=lstm_vdim, gate_cap=gate_cap, rope=False)
        mlp = MlpSpec(
            kind="moe", ff=expert_ff, act="silu", experts=experts, top=top,
            score="softmax", renormalize=True, shared_ff=shared_ff,
            correction=True, identity=identity, route_scale=route_scale,
            renorm_eps=1e-20)
        specs.append(LayerSpec(mixer=mixer, mlp=mlp, parallel=False,
                               post_norm=True, layer_scale=True))
    return ModelConfig(
        name=name, family="bipulorn", hidden_size=width,
        num_layers=n_layers, num_q_heads=attn_heads, num_kv_heads=attn_kv,
        head_dim=attn_dim, intermediate_size=max(expert_ff, shared_ff),
        vocab_size=vocab, max_position=8192, layer_specs=specs,
        logit_softcap=softcap, bos_token_id=0, eos_token_id=-1)


ARCHITECTURES.update({
    # CPU-runnable test config
    "tiny-bipulorn": _bipulorn_stack(
        "tiny-bipulorn", 96, 384, 4, attn_heads=6, attn_kv=3, attn_dim=16,
        window=40, rot_dims=8, rot_factor=2.0, ssd_heads=6, ssd_vdim=16,
        ssd_state=24, ssd_groups=3, ssd_norm_groups=2, conv=3, gla_heads=3,
        gla_dim=16, gla_vdim=32, decay_rank=8, tau=8.0, lstm_heads=3,
        lstm_dim=16, lstm_vdim=32, gate_cap=12.0, experts=5, identity=2,
        top=2, expert_ff=32, shared_ff=64, route_scale=1.5),
    # llama-3.2-1b-sized stack (same width, depth and vocab)
    "bipulorn-1b": _bipulorn_stack(
        "bipulorn-1b", 2048, 128256, 16, attn_heads=32, attn_kv=8,
        attn_dim=64, window=1024, rot_dims=64, rot_factor=1.0,
        ssd_heads=64, ssd_vdim=64, ssd_state=128, ssd_groups=1,
        ssd_norm_groups=1, conv=4, gla_heads=8, gla_dim=128, gla_vdim=256,
        decay_rank=16, tau=16.0, lstm_heads=16, lstm_dim=128,
        lstm_vdim=128, gate_cap=15.0, experts=8, identity=2, top=2,
        expert_ff=2048, shared_ff=2048),
    # llama-3-8b-sized layers (width 4096, head dim 128)
    "bipulorn-8b": _bipulorn_stack(
        "bipulorn-8b", 4096, 128256, 32, attn_heads=32, attn_kv=8,
        attn_dim=128, window=2048, rot_dims=128, rot_factor=1.0,
        ssd_heads=128, ssd_vdim=64, ssd_state=128, ssd_groups=1,
        ssd_norm_groups=1, conv=4, gla_heads=16, gla_dim=128, gla_vdim=256,
        decay_rank=16, tau=16.0, lstm_heads=32, lstm_dim=128,
        lstm_vdim=128, gate_cap=15.0, experts=8, identity=2, top=2,
        expert_ff=3584, shared_ff=3584),
})


def _dogidra_stack(
    name: str, width: int, vocab: int, n_layers: int, *, attn_heads: int,
    attn_kv: int, attn_dim: int, attn_vdim: int, window: int, pool: int,
    rot_dims: int, rot_scaling: Optional[tuple], gru: int, experts: int,
    top: int, expert_ff: int, shared_ff: int, taps: int, loop: tuple,
    softcap: float = 50.0, route_scale: float = 2.0,
    left_scale: float = 1.0, right_scale: float = 1.0,
    embedding_scale: float = 1.0,
) -> ModelConfig:
    """A Dogidra stack: every layer a pair of windowed attention with
    pooled far blocks and a minimal gated recurrent unit (weighted sum),
    then a routed feed-forward of ungated squared-relu experts with a
    shared expert; layer norms, input convolutions of `taps` taps, the
    span `loop` = (start, stop, times) repeated."""
    specs = []
    for _ in range(n_layers):
        left = MixerSpec(
            kind="attention", heads=attn_heads, kv_heads=attn_kv,
            dim=attn_dim, vdim=attn_vdim, scale=attn_dim ** -0.5,
            window=window, window_pool=pool, softcap=softcap, rope=True,
            rot_dims=rot_dims, rot_base=10000.0, rot_layout="half",
            rot_scaling=rot_scaling, qk_norm_all=True)
        right = MixerSpec(kind="mingru", heads=1, dim=1, vdim=gru,
                          rope=False)
        mixer = MixerSpec(
            kind="pair", heads=attn_heads, dim=attn_dim, rope=False,
            left=left, right=right, combine="weighted",
            left_scale=left_scale, right_scale=right_scale)
        mlp = MlpSpec(
            kind="moe", ff=expert_ff, act="relu2", gated=False,
            experts=experts, top=top, score="sigmoid", renormalize=False,
            shared_ff=shared_ff, shared_gate=False, correction=True,
            route_scale=route_scale)
        specs.append(LayerSpec(mixer=mixer, mlp=mlp, parallel=False,
                               norm="layer", input_conv=taps))
    return ModelConfig(
        name=name, family="dogidra", hidden_size=width,
        num_layers=n_layers, num_q_heads=attn_heads, num_kv_heads=attn_kv,
        head_dim=attn_dim, intermediate_size=max(expert_ff, shared_ff),
        vocab_size=vocab, max_position=8192, layer_specs=specs,
        embedding_scale=embedding_scale, loop=loop,
        tie_word_embeddings=True, bos_token_id=0, eos_token_id=-1)


ARCHITECTURES.update({
    # CPU-runnable test config
    "tiny-dogidra": _dogidra_stack(
        "tiny-dogidra", 96, 384, 4, attn_heads=6, attn_kv=3, attn_dim=16,
        attn_vdim=8, window=40, pool=8, rot_dims=8,
        rot_scaling=(2.0, 64, 8.0, 1.0), gru=128, experts=5, top=2,
        expert_ff=32, shared_ff=64, taps=3, loop=(1, 3, 2),
        embedding_scale=8.0),
    # llama-3.2-1b-sized stack (same width and vocab; 12 layers, the middle
    # four run twice: 16 layer runs)
    "dogidra-1b": _dogidra_stack(
        "dogidra-1b", 2048, 128256, 12, attn_heads=32, attn_kv=8,
        attn_dim=64, attn_vdim=64, window=1024, pool=64, rot_dims=64,
        rot_scaling=(8.0, 2048, 16.0, 1.0), gru=4096, experts=8, top=2,
        expert_ff=2048, shared_ff=2048, taps=4, loop=(4, 8, 2)),
    # llama-3-8b-sized layers (width 4096, head dim 128)
    "dogidra-8b": _dogidra_stack(
        "dogidra-8b", 4096, 128256, 24, attn_heads=32, attn_kv=8,
        attn_dim=128, attn_vdim=128, window=2048, pool=64, rot_dims=128,
        rot_scaling=(8.0, 2048, 16.0, 1.0), gru=8192, experts=8, top=2,
        expert_ff=3584, shared_ff=3584, taps=4, loop=(8, 16, 2)),
})


@dataclass
class CacheConfig:
    block_size: int = 16
    # Either an explicit block count (tests) or a fraction of free GPU memory.
    num_gpu_blocks: Optional[int] = None
    gpu_memory_utilization: float = 0.85
    enable_prefix_caching: bool = True
    # Host-DRAM KV offload pool size in GiB (0 disables). LMCache-equivalent
    # surface: reference LMCACHE_MAX_LOCAL_CPU_SIZE
    # (deployment-vllm-multi.yaml:336-343).
    cpu_offload_gb: float = 0.0
    # remote cacheserver data plane ("host:port"), shared across instances
    # (reference cacheserverSpec / LMCACHE_REMOTE_URL)
    remote_kv_url: Optional[str] = None
    remote_kv_serde: str = "cachegen"  # raw | cachegen | cachegen4
    # "bf16" (raw) or "int8" (CacheGen-style row-quantized serde, halves
    # host-pool bytes; reference LMCACHE remote serde surface)
    offload_dtype: str = "bf16"
    # KV cache storage dtype: "auto"/"bf16" or "fp8"/"fp8_e4m3" (OCP e4m3;
    # halves decode KV bandwidth; vLLM --kv-cache-dtype parity)
    kv_cache_dtype: str = "auto"


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 8192
    enable_chunked_prefill: bool = True
    # Cap on how many prompt tokens a single prefill chunk may carry.
    max_prefill_chunk: int = 8192
    # n-gram (prompt-lookup) speculative decoding: propose up to K draft
    # tokens per greedy decode by matching the sequence's trailing n-gram
    # against its own history; the drafts are verified in one multi-token
    # step through the prefill path. 0 = off.
    num_speculative_tokens: int = 0
    ngram_min: int = 2
    ngram_max: int = 4


@dataclass
class ParallelConfig:
    tensor_parallel_size: int = 1
    pipeline_parallel_size: int = 1
    # >1 splits each step's batch into M microbatches and issues them
    # back-to-back through the PP stages so stage k computes microbatch i
    # while stage k-1 computes i+1 (in-flight pipelining; see pipeline.py)
    pp_microbatches: int = 1
    rank: int = 0
    # disaggregated prefill role: None | "prefill" | "decode"
    kv_role: Optional[str] = None


@dataclass
class EngineConfig:
    model: str = "llama-3-8b"
    dtype: str = "bfloat16"
    max_model_len: int = 4096
    seed: int = 0
    weights_path: Optional[str] = None  # safetensors dir (optional)
    tokenizer: str = "synthetic"  # or a path to a tokenizer.json dir
    enforce_eager: bool = False  # True disables hipGraph decode capture
    # Mixed prefill+decode steps: True (default) runs one unified eager
    # batch so each layer's weights are read ONCE per step instead of
    # once for the decode graph replay and once for the prefill GEMMs —
    # measured +15-25% output tok/s AND lower TTFT at every load from 32
    # to 320 users on MI355X (graph replay remains for pure-decode
    # steps). False restores the split graph+eager mixed path.
    unified_mixed_steps: bool = True
    # graph-safe batched LoRA (BGMV slots); when False, adapters still run
    # through the eager grouped path
    # one-step-lagged sampling: the host schedules/launches step N+1 while
    # step N's sampled tokens are still in flight (decode inputs gather
    # from the previous step's device tensor). Greedy-exact; steps with
    # non-greedy sampling, penalties, logprobs or speculative chunks fall
    # back to the synchronous path transparently.
    async_scheduling: bool = False
    # weight quantization: None (bf16) or "fp8" (OCP e4m3 weights +
    # dynamic per-tensor activation quant through the fp8 MFMA pipe)
    quantization: Optional[str] = None
    # draft-model speculative decoding (engine/draft.py): architecture
    # name of the (smaller, same-vocab) proposer; None = n-gram drafts
    speculative_model: Optional[str] = None
    speculative_weights_path: Optional[str] = None
    enable_lora: bool = False
    max_loras: int = 4
    max_lora_rank: int = 16
    cache: CacheConfig = field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)
    parallel: ParallelConfig = field(default_factory=ParallelConfig)

    def model_config(self) -> ModelConfig:
        import os

        if os.path.isfile(os.path.join(self.model, "config.json")):
            # a checkpoint folder: its config.json names the architecture
            from production_stack_amd.engine.models.registry import (
                config_from_dir,
            )

            cfg = config_from_dir(self.model)
            if self.weights_path is None:
                self.weights_path = self.model
            if self.max_model_len > cfg.max_position:
                cfg = dataclasses.replace(
                    cfg, max_position=self.max_model_len)
            return cfg
        if self.model not in ARCHITECTURES:
            raise ValueError(
                f"unknown model architecture {self.model!r}; "
                f"known: {sorted(ARCHITECTURES)}"
            )
        cfg = ARCHITECTURES[self.model]
        if self.max_model_len > cfg.max_position:
            cfg = dataclasses.replace(cfg, max_position=self.max_model_len)
        return cfg
