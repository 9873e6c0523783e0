"""Model hyper-parameters, read from GGUF metadata, plus presets for the architectures the reference
advertises (reference `README.md:43-59`: Llama 2 7B/13B/70B, Mistral, Phi-2, Mixtral ...) and the
BASELINE.json configs (Llama-2-7B Q4_K_M, Mistral-7B, Llama-2-70B, Mixtral-8x7B, Phi-2).
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, field, replace
from typing import Any

ROPE_NORM = 0   # rotate adjacent pairs (x[2i], x[2i+1]) -- llama.cpp "normal" mode (llama GGUF)
ROPE_NEOX = 2   # rotate halves (x[i], x[i + n_rot/2]) -- phi2 / gpt-neox

# GGUF `general.architecture` values this engine runs, mapped to its internal arch. llama.cpp writes
# "llama" for Llama 2 / Code Llama / Vicuna / Mistral / Mixtral (MoE via expert_count).
SUPPORTED_ARCHS = {"llama": "llama", "phi2": "phi2", "gemma": "gemma"}


class UnsupportedArchitecture(ValueError):
    """A GGUF whose `general.architecture` this engine does not implement: loading must fail loudly
    rather than run the weights through the wrong graph (VERDICT r2 missing #3)."""


@dataclass
class ModelConfig:
    arch: str = "llama"            # "llama" (also Mistral / Mixtral / CodeLlama / Vicuna), "phi2", "gemma"
    n_vocab: int = 32000
    n_embd: int = 4096
    n_layer: int = 32
    n_head: int = 32
    n_head_kv: int = 32
    n_ff: int = 11008
    n_rot: int = 128
    rope_base: float = 10000.0
    rope_mode: int = ROPE_NORM
    norm_eps: float = 1e-5
    ctx_len: int = 4096
    n_expert: int = 0
    n_expert_used: int = 0
    sliding_window: int = 0
    n_embd_head: int = 0           # head dim when not n_embd / n_head (Gemma: attention.key_length = 256)
    bos_id: int = 1
    eos_id: int = 2
    name: str = ""
    extra: dict[str, Any] = field(default_factory=dict)

    @property
    def head_dim(self) -> int:
        return self.n_embd_head or self.n_embd // self.n_head

    @property
    def n_embd_q(self) -> int:
        return self.head_dim * self.n_head

    @property
    def gelu_glu(self) -> bool:
        """GeGLU FFN (gelu(gate) * up) instead of SwiGLU (Gemma)."""
        return self.arch == "gemma"

    @property
    def embed_scale(self) -> float:
        """Token embeddings are multiplied by sqrt(n_embd) (Gemma; llama.cpp build_gemma)."""
        return float(self.n_embd) ** 0.5 if self.arch == "gemma" else 1.0

    @property
    def n_embd_kv(self) -> int:
        return self.head_dim * self.n_head_kv

    @property
    def gqa(self) -> int:
        return self.n_head // self.n_head_kv

    @property
    def uses_layernorm(self) -> bool:
        return self.arch == "phi2"

    def to_dict(self) -> dict:
        return asdict(self)

    @classmethod
    def from_gguf_metadata(cls, md: dict[str, Any]) -> "ModelConfig":
        if "general.architecture" not in md:
            raise UnsupportedArchitecture("GGUF has no general.architecture")
        arch = str(md["general.architecture"])
        if arch not in SUPPORTED_ARCHS:
            raise UnsupportedArchitecture(
                f"unsupported model architecture {arch!r} (supported: {', '.join(sorted(SUPPORTED_ARCHS))})")
        p = arch + "."

        def g(k, default=None):
            return md.get(p + k, default)

        tokens = md.get("tokenizer.ggml.tokens")
        n_embd = int(g("embedding_length"))
        n_head = int(g("attention.head_count"))
        head = int(g("attention.key_length", n_embd // n_head))
        if int(g("attention.value_length", head)) != head:
            raise UnsupportedArchitecture("attention.value_length != attention.key_length")
        check_head_dim(head)
        cfg = cls(
            arch=SUPPORTED_ARCHS[arch],
            n_vocab=int(g("vocab_size", len(tokens) if tokens is not None else 32000)),
            n_embd=n_embd,
            n_layer=int(g("block_count")),
            n_head=n_head,
            n_head_kv=int(g("attention.head_count_kv", n_head)),
            n_ff=int(g("feed_forward_length")),
            n_rot=int(g("rope.dimension_count", head)),
            rope_base=float(g("rope.freq_base", 10000.0)),
            rope_mode=ROPE_NEOX if arch in ("phi2", "gemma") else ROPE_NORM,  # llama.cpp llama_rope_type
            norm_eps=float(g("attention.layer_norm_rms_epsilon", g("attention.layer_norm_epsilon", 1e-5))),
            ctx_len=int(g("context_length", 4096)),
            n_expert=int(g("expert_count", 0)),
            n_expert_used=int(g("expert_used_count", 0)),
            sliding_window=int(g("attention.sliding_window", 0) or 0),
            n_embd_head=head if head != n_embd // n_head else 0,
            bos_id=int(md.get("tokenizer.ggml.bos_token_id", 1)),
            eos_id=int(md.get("tokenizer.ggml.eos_token_id", 2)),
            name=str(md.get("general.name", "")),
        )
        return cfg

    def to_gguf_metadata(self) -> dict[str, Any]:
        a = self.arch if self.arch in ("phi2", "gemma") else "llama"
        p = a + "."
        md: dict[str, Any] = {
            "general.architecture": a,
            "general.name": self.name or a,
            p + "context_length": self.ctx_len,
            p + "embedding_length": self.n_embd,
            p + "block_count": self.n_layer,
            p + "feed_forward_length": self.n_ff,
            p + "rope.dimension_count": self.n_rot,
            p + "attention.head_count": self.n_head,
            p + "attention.head_count_kv": self.n_head_kv,
        }
        if self.n_embd_head or a == "gemma":
            md[p + "attention.key_length"] = self.head_dim
            md[p + "attention.value_length"] = self.head_dim
        if a == "phi2":
            md[p + "attention.layer_norm_epsilon"] = float(self.norm_eps)
        else:
            md[p + "attention.layer_norm_rms_epsilon"] = float(self.norm_eps)
            md[p + "rope.freq_base"] = float(self.rope_base)
        if self.n_expert:
            md[p + "expert_count"] = self.n_expert
            md[p + "expert_used_count"] = self.n_expert_used
        return md


# attention kernels (csrc/kernels/attention.hip) exist for these KV row widths; a head dim that is not
# one of them runs in the next one up (zero-padded cache rows, masked q / output): Orca Mini's 100 -> 112
ATTN_ROW_DIMS = (64, 80, 96, 112, 128, 256)


def cache_head_dim(head: int) -> int:
    """KV cache row width on the GPU for head dim `head` (the CPU backends keep `head`)."""
    for d in ATTN_ROW_DIMS:
        if head <= d:
            return d
    raise UnsupportedArchitecture(f"head dim {head} exceeds the largest attention kernel ({ATTN_ROW_DIMS[-1]})")


def check_head_dim(head: int) -> None:
    """Refuse at load what the GPU attention kernels cannot serve, instead of loading a model whose
    attention would silently not run (a head dim without a kernel used to no-op)."""
    if head <= 0 or head % 4 or cache_head_dim(head) - head >= 16:
        raise UnsupportedArchitecture(
            f"unsupported attention head dim {head} (supported: {', '.join(map(str, ATTN_ROW_DIMS))}, "
            "or a multiple of 4 up to 15 below one of them)")


PRESETS: dict[str, ModelConfig] = {
    # BASELINE headline: Llama-2-7B Q4_K_M
    "llama2-7b": ModelConfig(name="llama2-7b"),
    "llama2-13b": ModelConfig(name="llama2-13b", n_embd=5120, n_layer=40, n_head=40, n_head_kv=40,
                              n_ff=13824),
    "llama2-70b": ModelConfig(name="llama2-70b", n_embd=8192, n_layer=80, n_head=64, n_head_kv=8,
                              n_ff=28672),
    "mistral-7b": ModelConfig(name="mistral-7b", n_head_kv=8, n_ff=14336, ctx_len=32768,
                              rope_base=1000000.0),
    "mixtral-8x7b": ModelConfig(name="mixtral-8x7b", n_head_kv=8, n_ff=14336, ctx_len=32768,
                                rope_base=1000000.0, n_expert=8, n_expert_used=2),
    # Orca Mini 3B (reference README.md:55): OpenLLaMA-3B shapes, head dim 100; Q4_0 (its E = 3200 is not a
    # multiple of the 256-weight K-quant super-block)
    "orca-mini-3b": ModelConfig(name="orca-mini-3b", n_embd=3200, n_layer=26, n_head=32, n_head_kv=32,
                                n_ff=8640, n_rot=100, ctx_len=2048),
    "phi2": ModelConfig(name="phi2", arch="phi2", n_vocab=51200, n_embd=2560, n_layer=32, n_head=32,
                        n_head_kv=32, n_ff=10240, n_rot=32, rope_mode=ROPE_NEOX, norm_eps=1e-5,
                        ctx_len=2048, bos_id=50256, eos_id=50256),
    # Gemma (reference README.md:58-59): GeGLU, sqrt(E) embedding scale, head dim 256, MQA (2B),
    # NEOX RoPE, tied output. GGUF norm weights already carry Gemma's (1 + w) (llama.cpp converter)
    "gemma-2b": ModelConfig(name="gemma-2b", arch="gemma", n_vocab=256000, n_embd=2048, n_layer=18, n_head=8,
                            n_head_kv=1, n_ff=16384, n_rot=256, n_embd_head=256, rope_mode=ROPE_NEOX,
                            norm_eps=1e-6, ctx_len=8192, bos_id=2, eos_id=1),
    "gemma-7b": ModelConfig(name="gemma-7b", arch="gemma", n_vocab=256000, n_embd=3072, n_layer=28, n_head=16,
                            n_head_kv=16, n_ff=24576, n_rot=256, n_embd_head=256, rope_mode=ROPE_NEOX,
                            norm_eps=1e-6, ctx_len=8192, bos_id=2, eos_id=1),
    # small shapes of the same families for tests (K multiples of 256 so every quant type applies)
    "tiny-gemma": ModelConfig(name="tiny-gemma", arch="gemma", n_vocab=512, n_embd=256, n_layer=2, n_head=2,
                              n_head_kv=1, n_ff=512, n_rot=256, n_embd_head=256, rope_mode=ROPE_NEOX,
                              norm_eps=1e-6, ctx_len=256, bos_id=2, eos_id=1),
    "tiny-llama": ModelConfig(name="tiny-llama", n_vocab=512, n_embd=256, n_layer=2, n_head=4,
                              n_head_kv=2, n_ff=512, n_rot=64, ctx_len=256),
    # head dim 128 (the fused batch-1 attention half, attn8.hip): MHA and GQA 4
    "tiny-llama-d128": ModelConfig(name="tiny-llama-d128", n_vocab=512, n_embd=512, n_layer=3, n_head=4,
                                   n_head_kv=4, n_ff=768, n_rot=128, ctx_len=512),
    "tiny-llama-d128-gqa": ModelConfig(name="tiny-llama-d128-gqa", n_vocab=512, n_embd=512, n_layer=3, n_head=4,
                                       n_head_kv=1, n_ff=768, n_rot=128, ctx_len=512),
    # head dim 100 (Orca Mini), E not a multiple of 256: Q4_0 / Q8_0 files
    "tiny-orca": ModelConfig(name="tiny-orca", n_vocab=512, n_embd=800, n_layer=2, n_head=8, n_head_kv=8,
                             n_ff=2176, n_rot=100, ctx_len=256),
    "tiny-mixtral": ModelConfig(name="tiny-mixtral", n_vocab=512, n_embd=256, n_layer=2, n_head=4,
                                n_head_kv=2, n_ff=512, n_rot=64, ctx_len=256, n_expert=4,
                                n_expert_used=2),
    "tiny-phi2": ModelConfig(name="tiny-phi2", arch="phi2", n_vocab=512, n_embd=256, n_layer=2,
                             n_head=4, n_head_kv=4, n_ff=1024, n_rot=32, rope_mode=ROPE_NEOX,
                             ctx_len=256, bos_id=0, eos_id=0),
    # tensor-parallel test shapes: every row-parallel K spans >= 2 super-blocks per rank at TP=2
    "tiny-llama-tp": ModelConfig(name="tiny-llama-tp", n_vocab=512, n_embd=1024, n_layer=2, n_head=16,
                                 n_head_kv=4, n_ff=1024, n_rot=64, ctx_len=256),
    # n_ff = 3 super-blocks: TP=2 ranks hold an uneven 512 / 256 FFN split (as Llama-2-7B's 43 blocks)
    "tiny-llama-tp-odd": ModelConfig(name="tiny-llama-tp-odd", n_vocab=512, n_embd=1024, n_layer=2, n_head=16,
                                     n_head_kv=4, n_ff=768, n_rot=64, ctx_len=256),
    "tiny-phi2-tp": ModelConfig(name="tiny-phi2-tp", arch="phi2", n_vocab=512, n_embd=1024, n_layer=2,
                                n_head=16, n_head_kv=16, n_ff=2048, n_rot=32, rope_mode=ROPE_NEOX,
                                ctx_len=256, bos_id=0, eos_id=0),
    # TP = 8 (BASELINE config 4's degree, Llama-2-70B's 8:1 query / KV head ratio): one KV head, four query
    # heads, one FFN super-block and 64 vocab rows per rank
    "tiny-llama-tp8": ModelConfig(name="tiny-llama-tp8", n_vocab=512, n_embd=2048, n_layer=2, n_head=32,
                                  n_head_kv=8, n_ff=2048, n_rot=64, ctx_len=256),
    "tiny-mixtral-tp": ModelConfig(name="tiny-mixtral-tp", n_vocab=512, n_embd=1024, n_layer=2, n_head=16,
                                   n_head_kv=4, n_ff=1024, n_rot=64, ctx_len=256, n_expert=4,
                                   n_expert_used=2),
}


def preset(name: str, **overrides) -> ModelConfig:
    return replace(PRESETS[name], **overrides)


# ---------------------------------------------------------------------------------------------------
# Layer-list models: a model given as a folder with config.json + model.safetensors whose config lists
# heterogeneous layers (each with its own sequence mixer and feed-forward), optionally with a span of
# layers that runs several times over the same weights. `STACK_ARCHS` maps config.json's "architecture"
# to the reader that turns it into a StackConfig; the engine (engine/stack_runner.py) runs any StackConfig.

MIX_ATTENTION = 0   # softmax attention over a paged key/value cache
MIX_RETENTION = 1   # decayed linear attention with a per-sequence state matrix
MIX_LATENT = 2      # softmax attention whose keys and values come from one cached low-rank latent per token
MIX_MLSTM = 3       # matrix memory with exponential input / forget gates and a running stabiliser
MIX_MAMBA2 = 4      # selective state space layer (scalar decay per head) behind a short causal convolution
MIX_GLA = 5         # gated linear attention: a state matrix whose rows (key channels) decay by a per-token vector
STATE_MIXERS = (MIX_RETENTION, MIX_MLSTM, MIX_MAMBA2, MIX_GLA)   # mixers that own a per-sequence state slot

BLOCK_PARALLEL = 0  # x <- x + m (mixer(LN(x)) + ff(LN(x))): one norm, both sublayers read it
BLOCK_POSTNORM = 1  # x <- x + LN1(mixer(x)), then x <- x + LN2(ff(x)): the norm sits on the sublayer's output
BLOCK_SANDWICH = 2  # x <- x + s1 N1b(mixer(conv_in(N1(x)))), then x <- x + s2 N2b(ff(N2(x))): scalar-weight RMS norms
                    # before and after each sublayer, per-channel scales on the results, a short causal convolution
                    # added to the mixer's input
BLOCK_PRENORM = 3   # x <- x + mixer(N1(x)), then x <- x + ff(N2(x)): RMS norms with a weight vector on the sublayers' inputs

FF_MOE = 0          # routed experts (+ shared expert)
FF_DENSE = 1        # W_down act(W_up h), act = relu(z)^2
FF_GLU = 2          # W_down (act(W_gate h) * (W_up h)), act = the tanh form of gelu
ACT_GELU_TANH = 0   # activation of a gated dense feed-forward (FF_GLU)
ACT_RELU = 1
ROUTE_TOPK_SOFTMAX = 0   # top-k of (logits + bias), softmax over the chosen logits
ROUTE_SCORE_GROUPS = 1   # softmax over all outputs; choice by score + correction inside the best expert groups;
                         # weights = the chosen scores; trailing outputs may be identity experts
ROUTE_SIGMOID_GROUPS = 2  # sigmoid scores; a group ranks by the sum of its two largest scores; the chosen scores are
                          # divided by their sum and multiplied by a constant
GATE_NONE = 0
GATE_ELEMENT = 1            # the mixer's output is multiplied element by element with sigmoid(W_g h)
GATE_HEAD = 2               # one sigmoid gate per head


QK_NORM_NONE = 0
QK_NORM_WEIGHT_FIRST = 1    # RMS norm with a [dim] weight shared by the heads, before the rotation
QK_NORM_UNIT_LAST = 2       # division by the root mean square (no weight), after the rotation
SINK_NONE = 0
SINK_LEARNED = 1            # exp(sink_h), a learned number per head, joins the softmax denominator
SINK_ONE = 2                # a sink of score 0: the denominator holds one extra 1


def rotary_inv_freq(dims: int, base: float, scaling: tuple = ()) -> list:
    """Rotary frequencies f_i = base^(-2i / dims), i < dims / 2, in float64, with the scaling a config names."""
    import math
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f
    if scaling[0] == "linear":
        return [x / float(scaling[1]) for x in f]
    if scaling[0] != "bands":
        raise UnsupportedArchitecture(f"unknown rotary scaling {scaling[0]!r}")
    _, factor, low, high, original = scaling
    out = []
    for x in f:
        wave = 2.0 * math.pi / x
        if wave < original / high:
            out.append(x)
        elif wave > original / low:
            out.append(x / factor)
        else:
            t = (original / wave - low) / (high - low)
            out.append((1.0 - t) * x / factor + t * x)
    return out


@dataclass
class MixerSpec:
    kind: int = MIX_ATTENTION
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64               # per-head query / key size
    vdim: int = 64              # per-head value size
    # attention
    scale: float = 1.0          # score multiplier
    softcap: float = 0.0        # score <- cap * tanh(score / cap); 0 = none
    qtemp_coef: float = 0.0     # q *= 1 + coef * ln(floor((p + 1) / every) + 1); 0 = none
    qtemp_every: int = 1
    # retention
    decay: tuple = ()           # per-head state decay
    rot_dims: int = 0           # rotary dims per head (rotate-half pairing), 0 = none
    rot_base: float = 10000.0
    # latent attention: per head `dim` plain + `rot_dim` rotated query / key dims (adjacent-pair rotation of
    # the first rot_dims of the rotated part), keys / values expanded from a latent of kv_rank; a per-head
    # sink in the softmax denominator; sigmoid output gate
    rot_dim: int = 0
    kv_rank: int = 0
    # mlstm
    gate_cap: float = 0.0       # gate pre-activations pass cap * tanh(z / cap)
    # mamba2: heads x vdim channels, `state` rows per head, `groups` shared B / C groups
    state: int = 0
    groups: int = 1
    conv: int = 1               # taps of the causal convolution (the last one is the current token's)
    norm_groups: int = 1        # the gated output is RMS-normed in this many equal parts
    # attention options of the sandwich block's mixers
    bias: bool = False          # q, k, v (and with o_bias the output) projections carry biases
    o_bias: bool = False
    rot_scaling: tuple = ()     # () none; ("linear", factor); ("bands", factor, low, high, original): long waves
                                # divided by factor, short ones kept, a linear blend between
    qk_norm: int = QK_NORM_NONE
    sink: int = SINK_NONE
    talk: bool = False          # the heads' softmax weights are mixed by a [heads, heads] matrix before the values
    v_from_k: bool = False      # the values are the projected keys (before norm and rotation); no value projection
    # gated linear attention
    tau: float = 1.0            # decay = sigmoid(z)^(1 / tau)
    decay_rank: int = 0         # inner size of the low-rank map that gives z (read from the tensor's shape)
    # a second mixer that reads the same input; the layer's result is left_scale * this + right_scale * right
    right: "MixerSpec | None" = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    # attention options of the pre-norm block's mixers
    window: int = 0             # > 0: position i sees only j with 0 <= i - j < window
    maps: int = 1               # 2: differential attention, every head holds two query / key maps [map 1 | map 2] over the
                                # same values; o = a1 - lambda a2, unit RMS per head, times (1 - diff)
    diff: float = 0.0           # lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (learned vectors of size dim)
    gate: int = GATE_NONE       # sigmoid output gate from the mixer's input
    rot_pairs: bool = False     # the rotation pairs dims (2i, 2i + 1) instead of (i, i + rot_dims / 2)
    score_talk: bool = False    # the heads' SCORES, each times its own factor, are mixed by a [heads, heads] matrix
                                # before the softmax

    @property
    def n_q(self) -> int:
        return self.heads * self.dim * self.maps

    @property
    def n_k(self) -> int:
        return self.kv_heads * self.dim * self.maps

    @property
    def n_v(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def n_out(self) -> int:     # input width of the output projection
        return self.heads * self.vdim

    @property
    def n_out_all(self) -> int:  # with the second mixer's beside it
        return self.n_out + (self.right.n_out if self.right is not None else 0)

    @property
    def conv_channels(self) -> int:   # mamba2: x | B | C pass the convolution
        return self.heads * self.vdim + 2 * self.groups * self.state

    @property
    def cache_dim(self) -> int:       # latent attention: cached row = latent | shared rotated key part
        return self.kv_rank + self.rot_dim

    @property
    def state_floats(self) -> int:
        """float32 words of the per-sequence state of one run of this mixer."""
        if self.kind in (MIX_RETENTION, MIX_GLA):
            return self.heads * self.dim * self.vdim
        if self.kind == MIX_MLSTM:      # S [H][dim][vdim] | n [H][dim] | m [H]
            return self.heads * (self.dim * self.vdim + self.dim + 1)
        if self.kind == MIX_MAMBA2:     # S [H][state][vdim] | the convolution's last taps - 1 inputs
            return self.heads * self.state * self.vdim + (self.conv - 1) * self.conv_channels
        return 0


@dataclass
class MoESpec:
    experts: int = 0
    top: int = 0
    ff: int = 0
    shared_ff: int = 0          # 0 = no shared expert
    kind: int = FF_MOE          # FF_DENSE: only `ff` counts
    route: int = ROUTE_TOPK_SOFTMAX
    identity: int = 0           # trailing router outputs whose "expert" returns its input
    group_count: int = 1        # experts (identity ones included) form this many groups of neighbours
    group_keep: int = 1         # only experts of the best group_keep groups can be chosen
    shared_gate: bool = True    # the shared expert sits behind a scalar sigmoid gate
    act: int = ACT_GELU_TANH    # FF_GLU: the gate's activation
    route_scale: float = 1.0    # ROUTE_SIGMOID_GROUPS: factor on the normalised weights

    @property
    def n_router(self) -> int:
        return self.experts + self.identity


@dataclass
class LayerSpec:
    mixer: MixerSpec = field(default_factory=MixerSpec)
    mlp: MoESpec | None = None


@dataclass
class StackConfig:
    arch: str = "bizulix"
    n_vocab: int = 0
    n_embd: int = 0
    layers: list = field(default_factory=list)   # [LayerSpec]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0         # 0 = no repeated span
    norm_eps: float = 1e-5
    residual_mult: float = 1.0
    logit_softcap: float = 0.0
    block: int = BLOCK_PARALLEL
    embed_scale: float = 1.0
    logit_scale: float = 1.0    # logits = head x * logit_scale
    canon_taps: int = 1         # sandwich block: taps of the convolution added to the mixer's input (the last one is
                                # the current token's; with 1 nothing is carried between tokens)
    ctx_len: int = 1 << 20      # the design has no positional table: bounded by the cache pool only
    bos_id: int = 0
    eos_id: int = -1            # no tokenizer ships with these models: generation never stops on a token
    name: str = ""
    n_expert: int = 0           # (ModelConfig field the serving code reads; routing is per layer here)
    n_expert_used: int = 0

    @property
    def n_layer(self) -> int:
        return len(self.layers)

    def runs(self) -> list[tuple[int, int, bool]]:
        """(layer, pass, opens a pass) in execution order: the repeated span [loop_start, loop_stop) runs
        loop_times times in a row; every run has its own cache or state."""
        L = len(self.layers)
        if self.loop_times <= 0:
            return [(i, 0, False) for i in range(L)]
        a, b = self.loop_start, self.loop_stop
        out = [(i, 0, False) for i in range(a)]
        for p in range(self.loop_times):
            out += [(i, p, i == a) for i in range(a, b)]
        return out + [(i, 0, False) for i in range(b, L)]

    @property
    def has_state(self) -> bool:
        """Some layer carries a recurrent state: a cached prefix cannot be cut back to an earlier length."""
        return self.canon_taps > 1 or any(s.mixer.kind in STATE_MIXERS or s.mixer.right is not None for s in self.layers)

    def run_state_floats(self, li: int) -> int:
        """float32 words of the per-sequence state of one run of layer li: the mixer's (and its second mixer's) state
        matrix, then, in a sandwich block, the last canon_taps - 1 inputs of the input convolution."""
        m = self.layers[li].mixer
        n = m.state_floats + (m.right.state_floats if m.right is not None else 0)
        if self.block == BLOCK_SANDWICH:
            n += (self.canon_taps - 1) * self.n_embd
        return n

    def to_dict(self) -> dict:
        return asdict(self)

    # -- config.json of the Bizulix design
    @classmethod
    def from_bizulix(cls, c: dict) -> "StackConfig":
        layers = []
        for ent in c["layers"]:
            m = ent["mixer"]
            if ent["type"] == "attention":
                qt = m.get("q_temp") or {}
                mx = MixerSpec(kind=MIX_ATTENTION, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                               dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                               softcap=float(m.get("softcap") or 0.0), qtemp_coef=float(qt.get("coef", 0.0)),
                               qtemp_every=int(qt.get("every", 1)))
            elif ent["type"] == "retention":
                rot = m.get("rot") or {}
                mx = MixerSpec(kind=MIX_RETENTION, heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]),
                               vdim=int(m.get("vdim", m["dim"])), decay=tuple(float(d) for d in m["decay"]),
                               rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)))
                if len(mx.decay) != mx.heads:
                    raise UnsupportedArchitecture("retention: one decay per head expected")
                if mx.rot_dims % 2 or mx.rot_dims > mx.dim:
                    raise UnsupportedArchitecture("retention: rot.dims must be even and at most dim")
            else:
                raise UnsupportedArchitecture(f"unknown mixer type {ent['type']!r}")
            if mx.heads % mx.kv_heads:
                raise UnsupportedArchitecture("heads must be a multiple of kv_heads")
            mlp = None
            f = ent.get("mlp")
            if f:
                if f.get("kind", "moe") != "moe":
                    raise UnsupportedArchitecture(f"unknown feed-forward kind {f.get('kind')!r}")
                sh = f.get("shared") or {}
                mlp = MoESpec(experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                              ff=int(f["expert"]["ff"]), shared_ff=int(sh.get("ff", 0)))
                if not 0 < mlp.top <= mlp.experts:
                    raise UnsupportedArchitecture("router: top must be in 1..experts")
            layers.append(LayerSpec(mixer=mx, mlp=mlp))
        loop = c.get("loop") or {}
        cfg = cls(arch="bizulix", n_vocab=int(c["vocab"]), n_embd=int(c["width"]), layers=layers,
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 0)) if loop else 0, norm_eps=float(c["norm"]["eps"]),
                  residual_mult=float(c.get("residual_mult", 1.0)), logit_softcap=float(c.get("logit_softcap") or 0.0),
                  name=str(c.get("name", "")))
        if cfg.loop_times and not 0 <= cfg.loop_start < cfg.loop_stop <= len(layers):
            raise UnsupportedArchitecture("loop: need 0 <= start < stop <= number of layers")
        return cfg

    def to_bizulix(self) -> dict:
        """The config.json this configuration is read from (random-init fixtures, tests)."""
        out = []
        for s in self.layers:
            m = s.mixer
            if m.kind == MIX_ATTENTION:
                d = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale)
                if m.softcap:
                    d["softcap"] = m.softcap
                if m.qtemp_coef:
                    d["q_temp"] = dict(coef=m.qtemp_coef, every=m.qtemp_every)
                ent = dict(type="attention", mixer=d)
            else:
                d = dict(heads=m.heads, dim=m.dim, vdim=m.vdim, decay=list(m.decay))
                if m.rot_dims:
                    d["rot"] = dict(dims=m.rot_dims, base=m.rot_base)
                ent = dict(type="retention", mixer=d)
            f = s.mlp
            ent["mlp"] = None if f is None else dict(
                kind="moe", router=dict(experts=f.experts, top=f.top), expert=dict(ff=f.ff),
                **({"shared": dict(ff=f.shared_ff)} if f.shared_ff else {}))
            out.append(ent)
        c = dict(architecture="Bizulix", vocab=self.n_vocab, width=self.n_embd, layers=out,
                 norm=dict(eps=self.norm_eps), residual_mult=self.residual_mult)
        if self.logit_softcap:
            c["logit_softcap"] = self.logit_softcap
        if self.loop_times:
            c["loop"] = dict(start=self.loop_start, stop=self.loop_stop, times=self.loop_times)
        return c

    # -- config.json of the Norevik design
    @classmethod
    def from_norevik(cls, c: dict) -> "StackConfig":
        def bad(msg):
            raise UnsupportedArchitecture("Norevik: " + msg)

        layers = []
        for ent in c["layers"]:
            m, t = ent["mixer"], ent["type"]
            if t == "latent_attention":
                rot = m.get("rot") or {}
                mx = MixerSpec(kind=MIX_LATENT, heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]), vdim=int(m["vdim"]),
                               scale=float(m["scale"]), rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]),
                               rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot.get("base", 10000.0)))
                if mx.rot_dims % 2 or mx.rot_dims > mx.rot_dim:
                    bad("rot.dims must be even and at most rot_dim")
            elif t == "mlstm":
                mx = MixerSpec(kind=MIX_MLSTM, heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]),
                               vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]))
                if mx.gate_cap <= 0:
                    bad("gate_cap must be positive")
            elif t == "mamba2":
                mx = MixerSpec(kind=MIX_MAMBA2, heads=int(m["heads"]), kv_heads=int(m["groups"]), dim=int(m["state"]),
                               vdim=int(m["vdim"]), state=int(m["state"]), groups=int(m["groups"]), conv=int(m["conv"]),
                               norm_groups=int(m.get("norm_groups", 1)))
                if mx.groups <= 0 or mx.heads % mx.groups:
                    bad("heads must be a multiple of groups")
                if mx.norm_groups <= 0 or (mx.heads * mx.vdim) % mx.norm_groups:
                    bad("heads * vdim must be a multiple of norm_groups")
                if mx.conv < 1:
                    bad("conv must be at least 1")
            else:
                raise UnsupportedArchitecture(f"unknown mixer type {t!r}")
            if min(mx.heads, mx.dim, mx.vdim) <= 0:
                bad("mixer sizes must be positive")
            mlp = None
            f = ent.get("mlp")
            if f:
                kind = f.get("kind")
                if kind == "dense":
                    mlp = MoESpec(kind=FF_DENSE, ff=int(f["ff"]))
                elif kind == "moe":
                    r, sh = f["router"], f.get("shared") or {}
                    gr = r.get("groups") or {}
                    mlp = MoESpec(kind=FF_MOE, route=ROUTE_SCORE_GROUPS, experts=int(r["experts"]), top=int(r["top"]),
                                  ff=int(f["expert"]["ff"]), shared_ff=int(sh.get("ff", 0)), identity=int(r.get("identity", 0)),
                                  group_count=int(gr.get("count", 1)), group_keep=int(gr.get("keep", gr.get("count", 1))),
                                  shared_gate=False)
                    if not 0 < mlp.top <= mlp.n_router:
                        bad("router: top must be in 1..experts + identity")
                    if mlp.group_count < 1 or mlp.n_router % mlp.group_count or not 0 < mlp.group_keep <= mlp.group_count:
                        bad("router: groups must divide the router outputs, keep in 1..count")
                    if mlp.group_keep * (mlp.n_router // mlp.group_count) < mlp.top:
                        bad("router: the kept groups hold fewer experts than top")
                else:
                    raise UnsupportedArchitecture(f"unknown feed-forward kind {kind!r}")
            layers.append(LayerSpec(mixer=mx, mlp=mlp))
        return cls(arch="norevik", n_vocab=int(c["vocab"]), n_embd=int(c["width"]), layers=layers,
                   norm_eps=float(c["norm"]["eps"]), block=BLOCK_POSTNORM,
                   embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)), name=str(c.get("name", "")))

    def to_norevik(self) -> dict:
        """The config.json this configuration is read from (random-init fixtures, tests)."""
        out = []
        for s in self.layers:
            m = s.mixer
            if m.kind == MIX_LATENT:
                ent = dict(type="latent_attention", mixer=dict(
                    heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale,
                    rot=dict(dims=m.rot_dims, base=m.rot_base)))
            elif m.kind == MIX_MLSTM:
                ent = dict(type="mlstm", mixer=dict(heads=m.heads, dim=m.dim, vdim=m.vdim, gate_cap=m.gate_cap))
            elif m.kind == MIX_MAMBA2:
                ent = dict(type="mamba2", mixer=dict(heads=m.heads, vdim=m.vdim, state=m.state, groups=m.groups,
                                                      conv=m.conv, norm_groups=m.norm_groups))
            else:
                raise UnsupportedArchitecture("Norevik has no mixer of this kind")
            f = s.mlp
            if f is None:
                ent["mlp"] = None
            elif f.kind == FF_DENSE:
                ent["mlp"] = dict(kind="dense", ff=f.ff)
            else:
                ent["mlp"] = dict(kind="moe", expert=dict(ff=f.ff),
                                  router=dict(experts=f.experts, top=f.top, identity=f.identity,
                                              groups=dict(count=f.group_count, keep=f.group_keep)),
                                  **({"shared": dict(ff=f.shared_ff)} if f.shared_ff else {}))
            out.append(ent)
        return dict(architecture="Norevik", vocab=self.n_vocab, width=self.n_embd, layers=out,
                    norm=dict(eps=self.norm_eps), embedding=dict(scale=self.embed_scale))

    # -- config.json of the Suvunex design
    @classmethod
    def from_suvunex(cls, c: dict) -> "StackConfig":
        def bad(msg):
            raise UnsupportedArchitecture("Suvunex: " + msg)

        def attention(m: dict, **kw) -> MixerSpec:
            rot = m.get("rot") or {}
            sc = rot.get("scaling") or {}
            if not sc:
                scaling = ()
            elif "original" in sc:
                scaling = ("bands", float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
                if scaling[3] == scaling[2]:
                    bad("rot.scaling: high and low must differ")
            else:
                scaling = ("linear", float(sc["factor"]))
            mx = MixerSpec(kind=MIX_ATTENTION, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                           dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                           rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_scaling=scaling,
                           bias=True, **kw)
            if mx.rot_dims % 2 or mx.rot_dims > mx.dim:
                bad("rot.dims must be even and at most dim")
            if min(mx.heads, mx.kv_heads, mx.dim, mx.vdim) <= 0 or mx.heads % mx.kv_heads:
                bad("heads must be a positive multiple of kv_heads")
            return mx

        layers = []
        for ent in c["layers"]:
            m, t = ent["mixer"], ent["type"]
            if t == "parallel":
                mx = attention(m["left"], o_bias=True, qk_norm=QK_NORM_UNIT_LAST, sink=SINK_ONE)
                r = m["right"]
                mx.right = MixerSpec(kind=MIX_GLA, heads=int(r["heads"]), kv_heads=int(r["heads"]), dim=int(r["dim"]),
                                     vdim=int(r["vdim"]), tau=float(r["tau"]))
                if min(mx.right.heads, mx.right.dim, mx.right.vdim) <= 0 or mx.right.tau <= 0:
                    bad("right: sizes and tau must be positive")
                mx.left_scale, mx.right_scale = float(m["left_scale"]), float(m["right_scale"])
            elif t == "attention":
                mx = attention(m, qk_norm=QK_NORM_WEIGHT_FIRST, sink=SINK_LEARNED, talk=True, v_from_k=True)
                if mx.vdim != mx.dim:
                    bad("attention: the values are the keys, so vdim must equal dim")
            else:
                raise UnsupportedArchitecture(f"unknown mixer type {t!r}")
            mlp = None
            f = ent.get("mlp")
            if f:
                if f.get("kind") != "dense":
                    raise UnsupportedArchitecture(f"unknown feed-forward kind {f.get('kind')!r}")
                mlp = MoESpec(kind=FF_GLU, ff=int(f["ff"]))
                if mlp.ff <= 0:
                    bad("mlp.ff must be positive")
            layers.append(LayerSpec(mixer=mx, mlp=mlp))
        taps = int((c.get("canon") or {}).get("taps", 1))
        if taps < 1:
            bad("canon.taps must be at least 1")
        return cls(arch="suvunex", n_vocab=int(c["vocab"]), n_embd=int(c["width"]), layers=layers,
                   norm_eps=float(c["norm"]["eps"]), block=BLOCK_SANDWICH, canon_taps=taps,
                   embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(c.get("logit_scale", 1.0)), name=str(c.get("name", "")))

    def to_suvunex(self) -> dict:
        """The config.json this configuration is read from (random-init fixtures, tests)."""
        def attention(m: MixerSpec) -> dict:
            d = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale)
            if m.rot_dims:
                d["rot"] = dict(base=m.rot_base, dims=m.rot_dims)
                if m.rot_scaling and m.rot_scaling[0] == "linear":
                    d["rot"]["scaling"] = dict(factor=m.rot_scaling[1])
                elif m.rot_scaling:
                    _, fa, lo, hi, orig = m.rot_scaling
                    d["rot"]["scaling"] = dict(factor=fa, low=lo, high=hi, original=orig)
            return d

        out = []
        for s in self.layers:
            m = s.mixer
            if m.right is not None:
                r = m.right
                ent = dict(type="parallel", mixer=dict(left=attention(m), left_scale=m.left_scale, right_scale=m.right_scale,
                                                       right=dict(heads=r.heads, dim=r.dim, vdim=r.vdim, tau=r.tau)))
            elif m.kind == MIX_ATTENTION and m.talk:
                ent = dict(type="attention", mixer=attention(m))
            else:
                raise UnsupportedArchitecture("Suvunex has no mixer of this kind")
            ent["mlp"] = None if s.mlp is None else dict(kind="dense", ff=s.mlp.ff)
            out.append(ent)
        return dict(architecture="Suvunex", vocab=self.n_vocab, width=self.n_embd, layers=out, norm=dict(eps=self.norm_eps),
                    embedding=dict(scale=self.embed_scale), canon=dict(taps=self.canon_taps), logit_scale=self.logit_scale)

    # -- config.json of the Dekalorn design
    @classmethod
    def from_dekalorn(cls, c: dict) -> "StackConfig":
        def bad(msg):
            raise UnsupportedArchitecture("Dekalorn: " + msg)

        def rotary(m: dict, dim: int) -> dict:
            rot = m.get("rot") or {}
            sc = rot.get("scaling") or {}
            scaling = ()
            if sc:
                scaling = ("bands", float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
                if scaling[3] == scaling[2]:
                    bad("rot.scaling: high and low must differ")
            dims = int(rot.get("dims", dim if rot else 0))
            if dims % 2 or dims > dim:
                bad("rot.dims must be even and at most the rotated size")
            return dict(rot_dims=dims, rot_base=float(rot.get("base", 10000.0)), rot_scaling=scaling)

        def grouped(m: dict, **kw) -> MixerSpec:
            mx = MixerSpec(kind=MIX_ATTENTION, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                           dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                           window=int((m.get("mask") or {}).get("size", 0)), **kw)
            if min(mx.heads, mx.kv_heads, mx.dim, mx.vdim) <= 0 or mx.heads % mx.kv_heads or mx.window < 0:
                bad("heads must be a positive multiple of kv_heads")
            return mx

        layers = []
        for ent in c["layers"]:
            m, t = ent["mixer"], ent["type"]
            if t == "latent_attention":
                mx = MixerSpec(kind=MIX_LATENT, heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]), vdim=int(m["vdim"]),
                               scale=float(m["scale"]), rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]), gate=GATE_HEAD,
                               rot_pairs=True, **rotary(m, int(m["rot_dim"])))
                if min(mx.heads, mx.dim, mx.vdim, mx.kv_rank) <= 0 or mx.rot_dim < 0:
                    bad("latent attention sizes must be positive")
            elif t == "attention":
                mx = grouped(m, maps=2, diff=float(m["diff"]), gate=GATE_ELEMENT)
            elif t == "attention_2":
                mx = grouped(m, score_talk=True, rot_pairs=True, **rotary(m, int(m["dim"])))
            else:
                raise UnsupportedArchitecture(f"unknown mixer type {t!r}")
            mlp = None
            f = ent.get("mlp")
            if f:
                kind = f.get("kind")
                if kind == "dense":
                    mlp = MoESpec(kind=FF_GLU, ff=int(f["ff"]), act=ACT_RELU)
                    if mlp.ff <= 0:
                        bad("mlp.ff must be positive")
                elif kind == "moe":
                    r = f["router"]
                    gr = r.get("groups") or {}
                    mlp = MoESpec(kind=FF_MOE, route=ROUTE_SIGMOID_GROUPS, experts=int(r["experts"]), top=int(r["top"]),
                                  ff=int(f["expert"]["ff"]), group_count=int(gr.get("count", 1)),
                                  group_keep=int(gr.get("keep", gr.get("count", 1))), route_scale=float(r.get("scale", 1.0)),
                                  shared_gate=False)
                    if not 0 < mlp.top <= mlp.experts or mlp.ff <= 0:
                        bad("router: top must be in 1..experts")
                    if mlp.group_count < 1 or mlp.experts % mlp.group_count or not 0 < mlp.group_keep <= mlp.group_count:
                        bad("router: groups must divide the experts, keep in 1..count")
                    if mlp.group_keep * (mlp.experts // mlp.group_count) < mlp.top:
                        bad("router: the kept groups hold fewer experts than top")
                else:
                    raise UnsupportedArchitecture(f"unknown feed-forward kind {kind!r}")
            layers.append(LayerSpec(mixer=mx, mlp=mlp))
        loop = c.get("loop") or {}
        cfg = cls(arch="dekalorn", n_vocab=int(c["vocab"]), n_embd=int(c["width"]), layers=layers,
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 0)) if loop else 0, norm_eps=float(c["norm"]["eps"]), block=BLOCK_PRENORM,
                  name=str(c.get("name", "")))
        if cfg.loop_times and not 0 <= cfg.loop_start < cfg.loop_stop <= len(layers):
            bad("loop: need 0 <= start < stop <= number of layers")
        return cfg

    def to_dekalorn(self) -> dict:
        """The config.json this configuration is read from (random-init fixtures, tests)."""
        def rotary(m: MixerSpec) -> dict:
            d = dict(base=m.rot_base, dims=m.rot_dims)
            if m.rot_scaling:
                _, fa, lo, hi, orig = m.rot_scaling
                d["scaling"] = dict(factor=fa, low=lo, high=hi, original=orig)
            return d

        out = []
        for s in self.layers:
            m = s.mixer
            if m.kind == MIX_LATENT:
                ent = dict(type="latent_attention", mixer=dict(heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim,
                                                               kv_rank=m.kv_rank, scale=m.scale, rot=rotary(m)))
            elif m.kind == MIX_ATTENTION and m.maps == 2:
                ent = dict(type="attention", mixer=dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim,
                                                        scale=m.scale, diff=m.diff, mask=dict(size=m.window)))
            elif m.kind == MIX_ATTENTION and m.score_talk:
                ent = dict(type="attention_2", mixer=dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim,
                                                          scale=m.scale, mask=dict(size=m.window), rot=rotary(m)))
            else:
                raise UnsupportedArchitecture("Dekalorn has no mixer of this kind")
            f = s.mlp
            if f is None:
                ent["mlp"] = None
            elif f.kind == FF_GLU:
                ent["mlp"] = dict(kind="dense", ff=f.ff)
            else:
                ent["mlp"] = dict(kind="moe", expert=dict(ff=f.ff),
                                  router=dict(experts=f.experts, top=f.top, scale=f.route_scale,
                                              groups=dict(count=f.group_count, keep=f.group_keep)))
            out.append(ent)
        c = dict(architecture="Dekalorn", vocab=self.n_vocab, width=self.n_embd, layers=out, norm=dict(eps=self.norm_eps))
        if self.loop_times:
            c["loop"] = dict(start=self.loop_start, stop=self.loop_stop, times=self.loop_times)
        return c

    def to_config_json(self) -> dict:
        if self.arch == "dekalorn":
            return self.to_dekalorn()
        if self.arch == "suvunex":
            return self.to_suvunex()
        return self.to_norevik() if self.arch == "norevik" else self.to_bizulix()


STACK_ARCHS = {"Bizulix": StackConfig.from_bizulix, "Norevik": StackConfig.from_norevik, "Suvunex": StackConfig.from_suvunex,
               "Dekalorn": StackConfig.from_dekalorn}


def is_stack_model(path: str) -> bool:
    """A model folder (config.json + model.safetensors) rather than a GGUF file."""
    import os
    return os.path.isdir(path) and os.path.exists(os.path.join(path, "config.json"))


def load_stack_config(path: str) -> StackConfig:
    import json
    import os
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    arch = c.get("architecture")
    if arch not in STACK_ARCHS:
        raise UnsupportedArchitecture(
            f"unsupported model architecture {arch!r} (config.json models: {', '.join(sorted(STACK_ARCHS))})")
    return STACK_ARCHS[arch](c)
