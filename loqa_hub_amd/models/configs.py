"""Model configurations for the on-GPU STT -> intent -> TTS pipeline.

Dimensions are public model-card facts. Weights are always
seeded random-init (no network, no checkpoints); ``loqa_hub_amd.engine.weights``
can also map safetensors files when they exist locally.
"""
from __future__ import annotations

from dataclasses import dataclass, replace


@dataclass(frozen=True)
class LlamaConfig:
    name: str
    d_model: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    ffn_dim: int
    vocab_size: int
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    tie_embeddings: bool = False
    max_positions: int = 8192
    # Llama-3.1-style RoPE frequency scaling: (factor, low_freq_factor,
    # high_freq_factor, original_max_positions), or None
    rope_scaling: tuple | None = None

    @property
    def qkv_dim(self) -> int:
        return (self.n_heads + 2 * self.n_kv_heads) * self.head_dim

    def n_params(self) -> int:
        d, f = self.d_model, self.ffn_dim
        per = d * self.qkv_dim + self.n_heads * self.head_dim * d + 3 * d * f + 2 * d
        emb = self.vocab_size * d * (1 if self.tie_embeddings else 2)
        return self.n_layers * per + emb + d


LLAMA_CONFIGS = {
    "tinyllama": LlamaConfig("tinyllama-1.1b", 2048, 22, 32, 4, 64, 5632, 32000, rope_theta=10000.0),
    "llama3.2-1b": LlamaConfig("llama-3.2-1b", 2048, 16, 32, 8, 64, 8192, 128256, tie_embeddings=True,
                               rope_scaling=(32.0, 1.0, 4.0, 8192)),
    "llama3.2-3b": LlamaConfig("llama-3.2-3b", 3072, 28, 24, 8, 128, 8192, 128256, tie_embeddings=True,
                               rope_scaling=(32.0, 1.0, 4.0, 8192)),
    "llama3-8b": LlamaConfig("llama-3-8b", 4096, 32, 32, 8, 128, 14336, 128256),
    "llama3-70b": LlamaConfig("llama-3-70b", 8192, 80, 64, 8, 128, 28672, 128256),
    # small shapes for CPU tests / smoke
    "test-tiny": LlamaConfig("test-tiny", 256, 2, 4, 2, 64, 512, 4096, tie_embeddings=True,
                             max_positions=2048),
}


@dataclass(frozen=True)
class WhisperConfig:
    name: str
    n_mels: int
    d_model: int
    enc_layers: int
    dec_layers: int
    n_heads: int
    vocab_size: int
    n_audio_ctx: int = 1500
    n_text_ctx: int = 448

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_heads

    @property
    def ffn_dim(self) -> int:
        return 4 * self.d_model


WHISPER_CONFIGS = {
    "whisper-tiny": WhisperConfig("whisper-tiny", 80, 384, 4, 4, 6, 51865),
    "whisper-base": WhisperConfig("whisper-base", 80, 512, 6, 6, 8, 51865),
    "whisper-small": WhisperConfig("whisper-small", 80, 768, 12, 12, 12, 51865),
    "whisper-large-v3": WhisperConfig("whisper-large-v3", 128, 1280, 32, 32, 20, 51866),
    "test-whisper": WhisperConfig("test-whisper", 80, 128, 2, 2, 2, 4096, n_audio_ctx=1500),
}


@dataclass(frozen=True)
class VitsConfig:
    """VITS (text encoder + stochastic duration + flow + HiFi-GAN) at the public
    'vits-ljs' sizes; sample rate 22.05 kHz, hop 256."""
    name: str
    n_symbols: int = 178
    hidden: int = 192
    filter_channels: int = 768
    n_heads: int = 2
    enc_layers: int = 6
    kernel_size: int = 3
    flow_layers: int = 4
    wn_layers: int = 4
    inter_channels: int = 192
    upsample_rates: tuple = (8, 8, 2, 2)
    upsample_initial: int = 512
    resblock_kernels: tuple = (3, 7, 11)
    resblock_dilations: tuple = ((1, 3, 5), (1, 3, 5), (1, 3, 5))
    sample_rate: int = 22050
    window: int = 4
    # checkpoints (public VITS / MMS-TTS): the stochastic duration predictor
    # and the sampling constants of the published models
    sdp: bool = False
    sdp_filter: int = 192
    sdp_flows: int = 4
    sdp_bins: int = 10
    sdp_tail: float = 5.0
    sdp_kernel: int = 3
    noise_scale: float = 0.667
    noise_scale_duration: float = 0.8
    speaking_rate: float = 1.0
    upsample_kernels: tuple = ()          # () -> 2r for r > 2, else 4
    leaky_slope: float = 0.1
    # multi-speaker checkpoints (VCTK-style): a speaker embedding conditions
    # the duration predictor, every flow WaveNet layer and the vocoder input
    n_speakers: int = 1
    speaker_dim: int = 0


VITS_CONFIGS = {
    "vits-ljs": VitsConfig("vits-ljs"),
    "test-vits": VitsConfig("test-vits", hidden=64, filter_channels=128, enc_layers=2, flow_layers=2,
                            wn_layers=2, inter_channels=64, upsample_initial=256),
}


def llama_config(name: str, **over) -> LlamaConfig:
    c = LLAMA_CONFIGS[name]
    return replace(c, **over) if over else c


def whisper_config(name: str, **over) -> WhisperConfig:
    c = WHISPER_CONFIGS[name]
    return replace(c, **over) if over else c


def vits_config(name: str, **over) -> VitsConfig:
    c = VITS_CONFIGS[name]
    return replace(c, **over) if over else c


# --------------------------------------------------------------------------
# A checkpoint's own config.json (Hugging Face naming): any Llama-family or
# Whisper checkpoint, not only the named sizes above
def llama_config_from_hf(d: dict, name: str = "checkpoint") -> LlamaConfig:
    H = int(d["num_attention_heads"])
    D = int(d.get("head_dim") or int(d["hidden_size"]) // H)
    rs = d.get("rope_scaling") or None
    scaling = None
    if rs:
        kind = rs.get("rope_type", rs.get("type"))
        if kind != "llama3":
            raise ValueError(f"{name}: rope_scaling type {kind!r} is not supported")
        scaling = (float(rs["factor"]), float(rs.get("low_freq_factor", 1.0)),
                   float(rs.get("high_freq_factor", 4.0)),
                   int(rs.get("original_max_position_embeddings", 8192)))
    return LlamaConfig(name, int(d["hidden_size"]), int(d["num_hidden_layers"]), H,
                       int(d.get("num_key_value_heads", H)), D, int(d["intermediate_size"]),
                       int(d["vocab_size"]), rope_theta=float(d.get("rope_theta", 10000.0)),
                       norm_eps=float(d.get("rms_norm_eps", 1e-5)),
                       tie_embeddings=bool(d.get("tie_word_embeddings", False)),
                       max_positions=min(int(d.get("max_position_embeddings", 8192)), 8192),
                       rope_scaling=scaling)


def whisper_config_from_hf(d: dict, name: str = "checkpoint") -> WhisperConfig:
    c = WhisperConfig(name, int(d["num_mel_bins"]), int(d["d_model"]), int(d["encoder_layers"]),
                      int(d["decoder_layers"]), int(d["encoder_attention_heads"]),
                      int(d["vocab_size"]), n_audio_ctx=int(d.get("max_source_positions", 1500)),
                      n_text_ctx=int(d.get("max_target_positions", 448)))
    if int(d.get("encoder_ffn_dim", c.ffn_dim)) != c.ffn_dim:
        raise ValueError(f"{name}: encoder_ffn_dim {d['encoder_ffn_dim']} != 4 * d_model")
    return c


def vits_config_from_hf(d: dict, name: str = "checkpoint") -> VitsConfig:
    """A Hugging Face VITS / MMS-TTS config.json (``VitsConfig`` field names)."""
    return VitsConfig(
        name, n_symbols=d["vocab_size"], hidden=d["hidden_size"], filter_channels=d["ffn_dim"],
        n_heads=d["num_attention_heads"], enc_layers=d["num_hidden_layers"],
        kernel_size=d.get("ffn_kernel_size", 3), flow_layers=d.get("prior_encoder_num_flows", 4),
        wn_layers=d.get("prior_encoder_num_wavenet_layers", 4), inter_channels=d["flow_size"],
        upsample_rates=tuple(d["upsample_rates"]), upsample_initial=d["upsample_initial_channel"],
        resblock_kernels=tuple(d["resblock_kernel_sizes"]),
        resblock_dilations=tuple(tuple(x) for x in d["resblock_dilation_sizes"]),
        sample_rate=d.get("sampling_rate", 16000), window=d.get("window_size", 4),
        sdp=bool(d.get("use_stochastic_duration_prediction", True)),
        sdp_filter=d.get("duration_predictor_filter_channels", 256),
        sdp_flows=d.get("duration_predictor_num_flows", 4),
        sdp_bins=d.get("duration_predictor_flow_bins", 10),
        sdp_tail=float(d.get("duration_predictor_tail_bound", 5.0)),
        sdp_kernel=d.get("duration_predictor_kernel_size", 3),
        noise_scale=float(d.get("noise_scale", 0.667)),
        noise_scale_duration=float(d.get("noise_scale_duration", 0.8)),
        speaking_rate=float(d.get("speaking_rate", 1.0)),
        upsample_kernels=tuple(d.get("upsample_kernel_sizes", ())),
        leaky_slope=float(d.get("leaky_relu_slope", 0.1)),
        n_speakers=int(d.get("num_speakers", 1)),
        speaker_dim=int(d.get("speaker_embedding_size", 0)) if d.get("num_speakers", 1) > 1 else 0)


def checkpoint_config(path: str):
    """The config.json dict in (or beside) a checkpoint, or None."""
    import json
    import os
    if not path:
        return None
    d = path if os.path.isdir(path) else os.path.dirname(os.path.abspath(path))
    f = os.path.join(d, "config.json")
    if not os.path.isfile(f):
        return None
    with open(f, encoding="utf-8") as fh:
        return json.load(fh)


# --------------------------------------------------------------------------
# Pipizen: a hybrid decoder whose config.json lists its layers one by one.
# Every size and constant is taken from that file (or a tensor's shape).
@dataclass(frozen=True)
class RotaryConfig:
    dims: int                       # rotated entries (pairs 2i, 2i+1), <= rot_dim
    base: float
    yarn: tuple | None = None       # (factor, original, fast, slow)
    # the checkpoint pairs entry i with entry i + dims / 2 (rotate-half layout);
    # a loader may fold this into the interleaved layout by permuting rows
    half: bool = False


@dataclass(frozen=True)
class LatentAttnConfig:
    heads: int
    dim: int                        # unrotated query/key size per head
    rot_dim: int                    # rotated query/key size per head (key part shared)
    vdim: int
    kv_rank: int
    scale: float
    rot: RotaryConfig
    kv_from: int | None = None      # reuse that layer's latent cache
    q_rank: int = 0                 # > 0: queries go through an RMS-normed latent of this size
    gate: bool = False              # heads' outputs times sigmoid(W_g h), per entry


@dataclass(frozen=True)
class LightningConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                       # "dense" | "moe"
    ff: int = 0                     # dense width / expert width
    experts: int = 0
    identity: int = 0               # trailing router outputs that pass the input through
    top: int = 0
    groups: int = 1
    keep: int = 1
    shared_ff: int = 0              # 0: no shared expert
    # "swiglu": down(silu(gate x) * (up x)); "relu2": down(relu(up x)^2), no gate
    act: str = "swiglu"
    # "swiglu" / "geglu" (the tanh form of GELU on the gate) for dense layers
    # router: "softmax_all" scores every output and weighs by the plain score;
    # "softmax_top" takes the largest logits (+ bias) and weighs by the softmax
    # over the chosen ones only; "sigmoid" scores every output by the logistic
    # function of its logit and weighs by the plain score
    router: str = "softmax_all"
    # a group of experts ranks by the sum of its ``group_rank`` best scores
    group_rank: int = 1


@dataclass(frozen=True)
class HybridLayerConfig:
    kind: str                       # "latent_attention" | "lightning" | "attention"
    mixer: object
    mlp: FeedForwardConfig | None


@dataclass(frozen=True)
class PipizenConfig:
    name: str
    vocab_size: int
    d_model: int
    norm_eps: float
    layers: tuple

    @property
    def n_layers(self) -> int:
        return len(self.layers)


def pipizen_config_from_json(d: dict, name: str = "pipizen") -> PipizenConfig:
    layers = []
    for i, L in enumerate(d["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "latent_attention":
            r = m["rot"]
            sc = r.get("scaling")
            rot = RotaryConfig(int(r["dims"]), float(r["base"]),
                               (float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                float(sc["slow"])) if sc else None)
            src = m.get("kv_from")
            mixer = LatentAttnConfig(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]),
                                     int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]), rot,
                                     None if src is None else int(src))
            if mixer.kv_from is not None and not 0 <= mixer.kv_from < i:
                raise ValueError(f"layer {i}: kv_from {mixer.kv_from} is not an earlier layer")
        elif kind == "lightning":
            mixer = LightningConfig(int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                    tuple(float(v) for v in m["decay"]))
            if len(mixer.decay) != mixer.heads:
                raise ValueError(f"layer {i}: one decay per head expected")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = L.get("mlp")
        if not f:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForwardConfig("dense", int(f["ff"]))
        elif f["kind"] == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            mlp = FeedForwardConfig("moe", int(f["expert"]["ff"]), int(r["experts"]),
                                    int(r.get("identity", 0)), int(r["top"]),
                                    int(g.get("count", 1)), int(g.get("keep", g.get("count", 1))),
                                    int((f.get("shared") or {}).get("ff", 0)))
            if (mlp.experts + mlp.identity) % mlp.groups:
                raise ValueError(f"layer {i}: router outputs do not split into {mlp.groups} groups")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(HybridLayerConfig(kind, mixer, mlp))
    for i, L in enumerate(layers):
        if L.kind == "latent_attention" and L.mixer.kv_from is not None:
            s = layers[L.mixer.kv_from]
            if s.kind != "latent_attention" or s.mixer.kv_from is not None:
                raise ValueError(f"layer {i}: kv_from must name a latent layer with its own cache")
    return PipizenConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]),
                         tuple(layers))


# --------------------------------------------------------------------------
# Sodonex: a decoder whose mixer is chunked sigmoid attention (keys double as
# values, short convolutions on the projections, token shift, per-head output
# gate), with post-sublayer scalar-gain RMS norms and a mixture of relu^2
# experts. Every size and constant is taken from config.json or a tensor's shape.
@dataclass(frozen=True)
class ChunkAttnConfig:
    heads: int
    kv_heads: int
    dim: int                        # query / key size per head
    vdim: int                       # value size per head (the values are the keys: == dim)
    taps: int                       # short causal convolution on q and k
    chunk: int                      # a query sees earlier keys of its own chunk only
    scale: float
    rot: RotaryConfig               # rotate-half layout on the first rot.dims entries


@dataclass(frozen=True)
class SodonexConfig:
    name: str
    vocab_size: int
    d_model: int
    norm_eps: float
    residual_mult: float
    embed_scale: float
    layers: tuple

    @property
    def n_layers(self) -> int:
        return len(self.layers)


def sodonex_config_from_json(d: dict, name: str = "sodonex") -> SodonexConfig:
    layers = []
    for i, L in enumerate(d["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        r = m["rot"]
        mixer = ChunkAttnConfig(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]),
                                int(m.get("vdim", m["dim"])), int(m["conv"]),
                                int(m["mask"]["size"]), float(m["scale"]),
                                RotaryConfig(int(r["dims"]), float(r["base"])))
        if mixer.heads % mixer.kv_heads:
            raise ValueError(f"layer {i}: {mixer.heads} heads do not split over "
                             f"{mixer.kv_heads} key/value heads")
        if mixer.vdim != mixer.dim:
            raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
        if mixer.rot.dims % 2 or not 0 <= mixer.rot.dims <= mixer.dim:
            raise ValueError(f"layer {i}: rot.dims {mixer.rot.dims} does not fit a head of {mixer.dim}")
        if mixer.taps < 1 or mixer.chunk < 1:
            raise ValueError(f"layer {i}: conv taps and mask size must be positive")
        f = L.get("mlp")
        if not f:
            mlp = None
        elif f["kind"] == "moe":
            r = f["router"]
            mlp = FeedForwardConfig("moe", int(f["expert"]["ff"]), int(r["experts"]), 0,
                                    int(r["top"]), act="relu2", router="softmax_top")
            if not 0 < mlp.top <= mlp.experts:
                raise ValueError(f"layer {i}: top {mlp.top} of {mlp.experts} experts")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(HybridLayerConfig(kind, mixer, mlp))
    return SodonexConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]),
                         float(d["residual_mult"]), float(d["embedding"]["scale"]), tuple(layers))


# --------------------------------------------------------------------------
# Movinex: a pre-norm decoder (RMS norms with weights stored around zero, a
# learned per-coordinate scale on every sublayer output) whose config.json
# lists its layers; a stretch of layers may run several times in a row with the
# same weights. Mixers: softmax attention (full causal with a position-dependent
# query temperature, or sliding-window with kept first tokens, interleaved
# rotary, score soft-capping, keys doubling as values and an output gate) and
# Mamba-2 state-space layers. Feed-forwards: dense GeGLU or a sigmoid-routed
# mixture of SwiGLU experts. Every size and constant comes from config.json or
# a tensor's shape.
@dataclass(frozen=True)
class SoftmaxAttnConfig:
    heads: int
    kv_heads: int
    dim: int                        # query / key size per head
    vdim: int                       # value size per head
    scale: float
    bias: bool = False              # q / k / v projections carry biases
    values_from_keys: bool = False  # no value projection: v = k as projected
    gate: bool = False              # heads' outputs times sigmoid(W_g h), per entry
    rot: RotaryConfig | None = None     # interleaved pairs on the first rot.dims entries
    q_temp: tuple | None = None     # (coef, every): q *= 1 + coef ln(floor((p + 1) / every) + 1)
    softcap: float = 0.0            # score <- cap tanh(score / cap); 0: none
    window: int = 0                 # key j visible if p - j < window ...; 0: every earlier key
    keep_first: int = 0             # ... or j < keep_first
    # "head": q and k divided by their root mean square per head after rotation,
    # no weight; "whole": RMS norm over the whole q (and k) projection with a
    # weight vector of that size, before rotation
    qk_norm: str = "head"
    zero_sink: bool = False         # the softmax denominator holds one more term exp(0)


@dataclass(frozen=True)
class Mamba2Config:
    heads: int
    vdim: int                       # channels per head
    state: int                      # N
    groups: int                     # B / C groups shared by neighbouring heads
    taps: int                       # causal convolution on x | B | C
    norm_groups: int                # the gated output is RMS-normed in this many parts

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int                       # layers start .. stop - 1 ...
    times: int                      # ... run this many times in a row


@dataclass(frozen=True)
class MovinexConfig:
    name: str
    vocab_size: int
    d_model: int
    norm_eps: float
    logit_scale: float
    layers: tuple
    loop: LoopConfig | None = None

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list[tuple[int, bool]]:
        """The layers in execution order as (layer index, first of a pass of the
        repeated stretch); every run has a cache or state of its own."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        out = [(i, False) for i in range(lp.start)]
        for _ in range(lp.times):
            out += [(i, i == lp.start) for i in range(lp.start, lp.stop)]
        return out + [(i, False) for i in range(lp.stop, n)]


def movinex_config_from_json(d: dict, name: str = "movinex") -> MovinexConfig:
    layers = []
    for i, L in enumerate(d["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind in ("attention", "attention_2"):
            # the two kinds differ in what they have at all: the first one biases,
            # a value projection and the query temperature; the second one rotary
            # positions, the soft cap, the window with kept tokens and the gate
            second = kind == "attention_2"
            r = m.get("rot") if second else None
            qt = None if second else m.get("q_temp")
            mk = (m.get("mask") or {}) if second else {}
            mixer = SoftmaxAttnConfig(
                int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m["scale"]), bias=not second, values_from_keys=second, gate=second,
                rot=RotaryConfig(int(r["dims"]), float(r["base"])) if r else None,
                q_temp=(float(qt["coef"]), int(qt["every"])) if qt else None,
                softcap=float(m.get("softcap") or 0.0) if second else 0.0,
                window=int(mk.get("size") or 0), keep_first=int(mk.get("keep_first") or 0))
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: {mixer.heads} heads do not split over "
                                 f"{mixer.kv_heads} key/value heads")
            if mixer.values_from_keys and mixer.vdim != mixer.dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
            if mixer.rot and (mixer.rot.dims % 2 or not 0 <= mixer.rot.dims <= mixer.dim):
                raise ValueError(f"layer {i}: rot.dims {mixer.rot.dims} does not fit a head")
            if mixer.q_temp and mixer.q_temp[1] < 1:
                raise ValueError(f"layer {i}: q_temp.every must be positive")
        elif kind == "mamba2":
            mixer = Mamba2Config(int(m["heads"]), int(m["vdim"]), int(m["state"]),
                                 int(m.get("groups", 1)), int(m["conv"]),
                                 int(m.get("norm_groups", 1)))
            if mixer.heads % mixer.groups or mixer.inner % mixer.norm_groups or mixer.taps < 1:
                raise ValueError(f"layer {i}: heads, groups and norm_groups do not fit")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = L.get("mlp")
        if not f:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForwardConfig("dense", int(f["ff"]), act="geglu")
        elif f["kind"] == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            mlp = FeedForwardConfig("moe", int(f["expert"]["ff"]), int(r["experts"]), 0,
                                    int(r["top"]), int(g.get("count", 1)),
                                    int(g.get("keep", g.get("count", 1))), router="sigmoid",
                                    group_rank=2)
            if mlp.experts % mlp.groups or not 0 < mlp.keep <= mlp.groups:
                raise ValueError(f"layer {i}: {mlp.experts} experts do not split into "
                                 f"{mlp.groups} groups")
            if not 0 < mlp.top <= mlp.keep * (mlp.experts // mlp.groups):
                raise ValueError(f"layer {i}: top {mlp.top} exceeds the eligible experts")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(HybridLayerConfig(kind, mixer, mlp))
    lp = d.get("loop")
    loop = None
    if lp:
        loop = LoopConfig(int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 1:
            raise ValueError("loop: start, stop and times do not fit the layer list")
        if loop.start == loop.stop:
            loop = None
    return MovinexConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]),
                         float(d.get("logit_scale", 1.0)), tuple(layers), loop)


# --------------------------------------------------------------------------
# Vilulix: a decoder of parallel layers, x <- x + mixer(norm1(x)) + ff(norm2(x))
# with both RMS norms (weights stored around zero) reading the same x. A
# stretch of layers may run several times in a row with the same weights, the
# embedding output added to x before every pass but the first. Mixers: a
# stabilised matrix memory with exponential gates (mLSTM), latent attention
# with a query latent and an output gate, and a pair of mixers side by side -
# sliding-window softmax attention with a zero sink beside a gated delta rule
# with short convolutions. Dense SwiGLU feed-forwards; the logits are
# soft-capped. Every size and constant comes from config.json or a tensor's
# shape.
@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int                        # query / key size per head
    vdim: int
    gate_cap: float                 # gate pre-activations pass cap tanh(z / cap)


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int                      # value heads
    kv_heads: int                   # query / key heads shared by heads / kv_heads neighbours
    dim: int
    vdim: int
    taps: int                       # short causal convolution on q, k and v

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: SoftmaxAttnConfig
    right: DeltaRuleConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class VilulixConfig:
    name: str
    vocab_size: int
    d_model: int
    norm_eps: float
    logit_softcap: float            # 0: none
    layers: tuple
    loop: LoopConfig | None = None

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list[tuple[int, bool]]:
        """The layers in execution order as (layer index, first of a LATER pass
        of the repeated stretch: the embedding output is added before it);
        every run has a cache or state of its own."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        out = [(i, False) for i in range(lp.start)]
        for t in range(lp.times):
            out += [(i, t > 0 and i == lp.start) for i in range(lp.start, lp.stop)]
        return out + [(i, False) for i in range(lp.stop, n)]


def _rot_half(r: dict, size: int, where: str) -> RotaryConfig:
    rot = RotaryConfig(int(r["dims"]), float(r["base"]), half=True)
    if rot.dims % 2 or not 0 <= rot.dims <= size:
        raise ValueError(f"{where}: rot.dims {rot.dims} does not fit {size} entries")
    return rot


def vilulix_config_from_json(d: dict, name: str = "vilulix") -> VilulixConfig:
    layers = []
    for i, L in enumerate(d["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "mlstm":
            mixer = MatrixMemoryConfig(int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                       float(m["gate_cap"]))
            if mixer.gate_cap <= 0:
                raise ValueError(f"layer {i}: gate_cap must be positive")
        elif kind == "latent_attention":
            mixer = LatentAttnConfig(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]),
                                     int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]),
                                     _rot_half(m["rot"], int(m["rot_dim"]), f"layer {i}"),
                                     q_rank=int(m["q_rank"]), gate=True)
            if mixer.q_rank < 1 or mixer.kv_rank < 1:
                raise ValueError(f"layer {i}: latent sizes must be positive")
        elif kind == "parallel":
            a, r = m["left"], m["right"]
            left = SoftmaxAttnConfig(int(a["heads"]), int(a["kv_heads"]), int(a["dim"]),
                                     int(a["vdim"]), float(a["scale"]),
                                     rot=_rot_half(a["rot"], int(a["dim"]), f"layer {i}"),
                                     window=int(a["mask"]["size"]), qk_norm="whole", zero_sink=True)
            right = DeltaRuleConfig(int(r["heads"]), int(r["kv_heads"]), int(r["dim"]),
                                    int(r["vdim"]), int(r["conv"]))
            if left.heads % left.kv_heads or right.heads % right.kv_heads:
                raise ValueError(f"layer {i}: heads do not split over the key/value heads")
            if left.window < 1 or right.taps < 1:
                raise ValueError(f"layer {i}: mask size and conv taps must be positive")
            mixer = ParallelMixerConfig(left, right, float(m["left_scale"]),
                                        float(m["right_scale"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = L.get("mlp")
        if not f:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForwardConfig("dense", int(f["ff"]))
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(HybridLayerConfig(kind, mixer, mlp))
    lp = d.get("loop")
    loop = None
    if lp:
        loop = LoopConfig(int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 1:
            raise ValueError("loop: start, stop and times do not fit the layer list")
        if loop.start == loop.stop or loop.times == 1:
            loop = None
    return VilulixConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]),
                         float(d.get("logit_softcap") or 0.0), tuple(layers), loop)
