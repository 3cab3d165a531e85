"""Engine and model-architecture configuration.

The reference has a default-only consensus config; the native
engine adds EngineConfig — model preset/path, dtype, TP degree, KV block
size, hipGraph toggle — exposed through ``KLLMs(**kwargs)``.

Presets cover the BASELINE.json configs: Llama-3-8B (TP=1 headline),
Llama-3-70B (TP=8), Mixtral-8x7B (MoE), plus tiny CPU-testable variants.
"""

from __future__ import annotations

from typing import List, Literal, Optional, Union

from pydantic import BaseModel, Field


class ModelArchConfig(BaseModel):
    """Transformer architecture hyperparameters (Llama/Mixtral family)."""

    arch: Literal["llama", "mixtral"] = "llama"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: Optional[int] = None  # defaults to hidden_size // num_heads
    rope_theta: float = 500000.0
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    # Qwen2-family: bias on the fused QKV projection (o_proj stays bias-free)
    attention_qkv_bias: bool = False
    # HF rope_scaling dict (Llama-3.1 "llama3" banded NTK, "linear");
    # None = plain RoPE
    rope_scaling: Optional[dict] = None
    # MoE (mixtral only)
    num_experts: int = 0
    num_experts_per_tok: int = 2

    @property
    def head_dim_(self) -> int:
        return self.head_dim or (self.hidden_size // self.num_heads)


class RotarySpec(BaseModel):
    """Rotary position parameters of one attention mixer: the first ``dims``
    dimensions of each head rotate in pairs (``layout``) with frequency
    base^(-2i/dims); ``scaling`` is the banded frequency rescale
    (factor / low / high / original context), None = plain."""

    base: float = 10000.0
    dims: int = 0
    scaling: Optional[dict] = None
    # "pairs": entry 2i rotates with 2i+1; "half": entry i with i + dims/2
    layout: Literal["pairs", "half"] = "pairs"


class BlockAttnSpec(BaseModel):
    """Softmax attention whose causal mask is cut into aligned blocks of
    ``mask_size`` positions (0 = plain causal). ``values_from_keys``: no value
    projection, the values are the un-rotated keys."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int = 0
    rot: RotarySpec = Field(default_factory=RotarySpec)
    values_from_keys: bool = True
    qk_bias: bool = True
    head_gate: bool = True


class DecayLinearAttnSpec(BaseModel):
    """Linear attention with one constant decay per head:
    S <- decay_h S + k v^T, o = S^T q."""

    heads: int
    dim: int
    vdim: int
    decay: List[float]


class ParallelMixerSpec(BaseModel):
    left: BlockAttnSpec
    right: DecayLinearAttnSpec


class ChannelDeltaSpec(BaseModel):
    """Gated delta rule with a decay per head and key channel, short causal
    convolutions of ``conv`` taps on q/k/v."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # bottleneck widths of the two low-rank projections (decay, output gate);
    # a checkpoint fixes them by its tensor shapes
    decay_rank: int = 16
    gate_rank: int = 16


class GluSpec(BaseModel):
    """Clamped gated-linear-unit feed-forward: g = min(gate, limit),
    u = clamp(up, +-limit), y = g * sigmoid(alpha g) * (u + 1)."""

    kind: Literal["dense"] = "dense"
    ff: int
    limit: float
    alpha: float = 1.702


class MaskedAttnSpec(BaseModel):
    """GQA softmax attention without rotation whose causal mask is a sliding
    window of ``mask_size`` positions (0 = plain causal) that also keeps the
    first ``keep_first`` positions of the sequence; q and k pass an RMS norm
    per head (one weight of size ``dim`` shared by the heads). ``sink``: the
    softmax denominator holds one more term exp(0) that carries no value.
    The concatenated heads are gated elementwise by sigmoid(W_g h)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int = 0
    keep_first: int = 0
    sink: bool = True


class WkvSpec(BaseModel):
    """Time mixing with a decay per head and key channel that depends on the
    token: S <- diag(w_t) S + k v^T, read before the update with a bonus for
    the current token; inputs are mixed with the previous token's."""

    heads: int
    dim: int
    # bottleneck of the decay's low-rank projection; a checkpoint fixes it by
    # its tensor shapes
    decay_rank: int = 16


class MlstmSpec(BaseModel):
    """Matrix memory with exponential input gate, sigmoid forget gate (both
    soft-capped at ``gate_cap``) and a running maximum as stabiliser."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float


class SharedExpertSpec(BaseModel):
    """An expert that every token passes; its output is scaled by sigmoid of
    one more projection of the input (a scalar per token). ``limit`` is the
    clamp of a clamped-GLU expert (None: as the routed experts' form says)."""

    ff: int
    limit: Optional[float] = None


class RoutedExpertsSpec(BaseModel):
    """Mixture of silu-GLU experts behind a router. ``score`` turns the router
    logits into scores: softmax over all outputs, or sigmoid of each. The last
    ``identity`` router outputs are experts that return their input. The
    choice is made on score (+ correction, if the checkpoint has one) among
    the experts of the best ``group_keep`` of ``group_count`` groups of
    neighbours. The chosen scores weigh the experts, renormalised to sum 1 or
    as they are; the weight multiplies the expert's output or its input
    (``weight_on``). ``shared``: one more expert that runs for every token."""

    kind: Literal["moe"] = "moe"
    experts: int
    identity: int = 0
    top: int
    group_count: int = 1
    group_keep: int = 1
    ff: int
    score: Literal["softmax", "sigmoid"] = "softmax"
    renormalize: bool = True
    correction: bool = True
    weight_on: Literal["output", "input"] = "output"
    shared: Optional[SharedExpertSpec] = None
    # the experts' form: silu(gate) * up, or the clamped GLU
    # min(gate, limit) sigmoid(alpha min(gate, limit)) (clamp(up, +-limit) + 1)
    act: Literal["silu", "clamped"] = "silu"
    limit: float = 0.0
    alpha: float = 1.702


class BigramSpec(BaseModel):
    buckets: int
    mul_prev: int
    mul_cur: int


class LoopSpec(BaseModel):
    start: int
    stop: int
    times: int


class MedilixLayerSpec(BaseModel):
    type: Literal["attention", "wkv", "mlstm"]
    attention: Optional[MaskedAttnSpec] = None
    wkv: Optional[WkvSpec] = None
    mlstm: Optional[MlstmSpec] = None
    mlp: Optional[Union[GluSpec, RoutedExpertsSpec]] = None


class MedilixArchConfig(BaseModel):
    """A decoder with parallel layers x <- x + mixer(norm1 x) + ff(norm2 x),
    three mixer types (windowed attention with a sink, wkv, mlstm), dense or
    routed feed-forwards, a grouped RMS norm, a hashed bigram embedding added
    to the token embedding and an optional run of layers that repeats with
    shared weights. Every size comes from the checkpoint's config.json."""

    arch: Literal["medilix"] = "medilix"
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float = 1e-5
    norm_groups: int = 1
    embed_scale: float = 1.0
    bigram: Optional[BigramSpec] = None
    layers: List[MedilixLayerSpec]
    loop: Optional[LoopSpec] = None
    max_position_embeddings: int = 1 << 24
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_runs(self) -> List[tuple]:
        """(layer index, starts a pass of the loop) per layer run, in
        execution order: the looped range runs ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        looped = [(i, i == a) for i in range(a, b)] * times
        return [(i, False) for i in range(a)] + looped + [(i, False) for i in range(b, n)]

    @classmethod
    def from_checkpoint_config(cls, d: dict, shapes: Optional[dict] = None) -> "MedilixArchConfig":
        """Parse the family's config.json (keys: vocab, width, norm.eps,
        norm.groups, embedding.scale / .bigram, loop, layers[].type / .mixer /
        .mlp). ``shapes`` (tensor name -> shape, from the safetensors header)
        supplies what config.json leaves to the tensors: the decay rank."""
        shapes = shapes or {}
        layers = []
        for li, spec in enumerate(d["layers"]):
            m = spec["mixer"]
            mlp = spec.get("mlp")
            ff = None
            if mlp:
                if mlp.get("kind", "dense") == "dense":
                    ff = GluSpec(ff=mlp["ff"], limit=mlp["limit"])
                elif mlp["kind"] == "moe":
                    r = mlp["router"]
                    grp = r.get("groups") or {}
                    ff = RoutedExpertsSpec(experts=r["experts"], identity=r.get("identity", 0), top=r["top"],
                                           group_count=grp.get("count", 1), group_keep=grp.get("keep", 1),
                                           ff=mlp["expert"]["ff"])
                else:
                    raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            kind = spec["type"]
            if kind == "attention":
                mask = m.get("mask") or {}
                layers.append(MedilixLayerSpec(type=kind, mlp=ff, attention=MaskedAttnSpec(
                    heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=m["scale"],
                    mask_size=mask.get("size", 0), keep_first=mask.get("keep_first", 0))))
            elif kind == "wkv":
                layers.append(MedilixLayerSpec(type=kind, mlp=ff, wkv=WkvSpec(
                    heads=m["heads"], dim=m["dim"],
                    decay_rank=(shapes.get(f"l{li}.mix.w1") or [16])[0])))
            elif kind == "mlstm":
                layers.append(MedilixLayerSpec(type=kind, mlp=ff, mlstm=MlstmSpec(
                    heads=m["heads"], dim=m["dim"], vdim=m["vdim"], gate_cap=m["gate_cap"])))
            else:
                raise ValueError(f"unknown layer type {kind!r}")
        emb = d.get("embedding") or {}
        bg = emb.get("bigram")
        lp = d.get("loop")
        if lp and (lp["times"] < 1 or not 0 <= lp["start"] < lp["stop"] <= len(layers)):
            raise ValueError(f"loop {lp} does not fit {len(layers)} layers")
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], rms_norm_eps=d["norm"]["eps"],
                   norm_groups=d["norm"].get("groups", 1), embed_scale=emb.get("scale", 1.0),
                   bigram=BigramSpec(**bg) if bg else None, layers=layers,
                   loop=LoopSpec(**lp) if lp else None)


def _medilix_preset(vocab, width, depth, heads, kv_heads, dim, mask, keep, r_heads, r_dim, m_heads, m_dim,
                    m_vdim, ff, experts, top, expert_ff, pattern="awm", loop=None, groups=2,
                    identity=2) -> MedilixArchConfig:
    """Random-init presets of the family: ``pattern`` repeats over the depth
    ('a' attention + dense ff, 'w' wkv + routed experts, 'm' mlstm + dense ff)."""
    import math as _math

    layers = []
    for i in range(depth):
        c = pattern[i % len(pattern)]
        dense = GluSpec(ff=ff, limit=7.0)
        moe = RoutedExpertsSpec(experts=experts, identity=identity, top=top, group_count=2, group_keep=1,
                                ff=expert_ff)
        if c == "a":
            layers.append(MedilixLayerSpec(type="attention", mlp=dense, attention=MaskedAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=1.0 / _math.sqrt(dim),
                mask_size=mask, keep_first=keep)))
        elif c == "w":
            layers.append(MedilixLayerSpec(type="wkv", mlp=moe, wkv=WkvSpec(
                heads=r_heads, dim=r_dim, decay_rank=max(8, width // 64))))
        else:
            layers.append(MedilixLayerSpec(type="mlstm", mlp=dense, mlstm=MlstmSpec(
                heads=m_heads, dim=m_dim, vdim=m_vdim, gate_cap=15.0)))
    return MedilixArchConfig(vocab_size=vocab, hidden_size=width, norm_groups=groups, embed_scale=1.0,
                             bigram=BigramSpec(buckets=max(7, vocab // 2 - 1), mul_prev=131, mul_cur=5),
                             layers=layers, loop=LoopSpec(**loop) if loop else None)


class LatentAttnSpec(BaseModel):
    """Softmax attention whose keys and values are up-projections of one
    shared latent row per token. Per head the query has ``dim`` unrotated and
    ``rot_dim`` rotated entries; the token's down-projection gives the latent
    (``kv_rank`` entries, RMS-normed) and one rotated key part shared by all
    heads. Only those two are cached. Causal sliding window of ``mask_size``
    positions (0 = plain causal); per-head sigmoid output gate."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    mask_size: int = 0
    rot: RotarySpec = Field(default_factory=RotarySpec)
    head_gate: bool = True


class ActFFSpec(BaseModel):
    """Two-matrix feed-forward W_down act(W_up h); act = tanh-form gelu."""

    kind: Literal["dense"] = "dense"
    ff: int
    act: Literal["gelu_tanh"] = "gelu_tanh"


class MitunexLayerSpec(BaseModel):
    type: Literal["latent_attention"] = "latent_attention"
    attention: LatentAttnSpec
    mlp: Optional[Union[ActFFSpec, RoutedExpertsSpec]] = None
    # index of the layer whose weights this one uses (its own index = own weights)
    weights_of: int


class MitunexArchConfig(BaseModel):
    """A decoder of post-normed layers x <- x + norm(mixer(x)),
    x <- x + norm(ff(x)) over an fp32 residual. The embedding adds a learned
    position row and is RMS-normed. Every mixer is latent attention with a
    sliding window; feed-forwards are a gelu layer, routed experts with
    sigmoid scores and a shared expert, or absent. A layer may use another
    layer's weights with a cache of its own. The logits are scaled and
    soft-capped. Every size comes from the checkpoint's config.json."""

    arch: Literal["mitunex"] = "mitunex"
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float = 1e-6
    layers: List[MitunexLayerSpec]
    max_position_embeddings: int = 2048
    logit_scale: float = 1.0
    logit_softcap: float = 0.0          # 0 = none
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_checkpoint_config(cls, d: dict, shapes: Optional[dict] = None) -> "MitunexArchConfig":
        """Parse the family's config.json (keys: vocab, width, norm.eps,
        max_positions, logit_scale, logit_softcap, layers[].type / .mixer /
        .mlp / .weights_of)."""
        layers = []
        for li, spec in enumerate(d["layers"]):
            if spec["type"] != "latent_attention":
                raise ValueError(f"unknown layer type {spec['type']!r}")
            m = spec["mixer"]
            rot = m.get("rot") or {}
            mask = m.get("mask") or {}
            att = LatentAttnSpec(heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                                 kv_rank=m["kv_rank"], scale=m["scale"], mask_size=mask.get("size") or 0,
                                 rot=RotarySpec(base=rot.get("base", 10000.0), dims=rot.get("dims", m["rot_dim"])))
            if att.rot.dims != att.rot_dim:
                raise ValueError("the rotated part of a latent-attention head is rotated whole")
            mlp = spec.get("mlp")
            ff = None
            if mlp:
                kind = mlp.get("kind", "dense")
                if kind == "dense":
                    ff = ActFFSpec(ff=mlp["ff"])
                elif kind == "moe":
                    r = mlp["router"]
                    sh = mlp.get("shared")
                    ff = RoutedExpertsSpec(experts=r["experts"], top=r["top"], ff=mlp["expert"]["ff"],
                                           score="sigmoid", renormalize=False, correction=False,
                                           weight_on="input",
                                           shared=SharedExpertSpec(ff=sh["ff"]) if sh else None)
                else:
                    raise ValueError(f"unknown feed-forward kind {kind!r}")
            src = spec.get("weights_of", li)
            if src is None:
                src = li
            if not 0 <= src < len(d["layers"]) or d["layers"][src].get("weights_of", src) not in (src, None):
                raise ValueError(f"layer {li}: weights_of {src} does not name a layer with weights of its own")
            layers.append(MitunexLayerSpec(attention=att, mlp=ff, weights_of=src))
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], rms_norm_eps=d["norm"]["eps"], layers=layers,
                   max_position_embeddings=d.get("max_positions", 2048), logit_scale=d.get("logit_scale") or 1.0,
                   logit_softcap=d.get("logit_softcap") or 0.0)


def _mitunex_preset(vocab, width, depth, heads, dim, rot_dim, vdim, kv_rank, mask, ff, experts, top, expert_ff,
                    shared_ff, pattern="dm", share_from=None, max_pos=8192) -> MitunexArchConfig:
    """Random-init presets of the family: ``pattern`` repeats over the depth
    ('d' gelu feed-forward, 'm' routed experts + shared expert, 'n' none);
    layers from ``share_from`` on use the weights of layer share_from - 1."""
    import math as _math

    layers = []
    for i in range(depth):
        c = pattern[i % len(pattern)]
        att = LatentAttnSpec(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                             scale=1.0 / _math.sqrt(dim + rot_dim), mask_size=mask,
                             rot=RotarySpec(base=1e6, dims=rot_dim))
        mlp = None
        if c == "d":
            mlp = ActFFSpec(ff=ff)
        elif c == "m":
            mlp = RoutedExpertsSpec(experts=experts, top=top, ff=expert_ff, score="sigmoid", renormalize=False,
                                    correction=False, weight_on="input",
                                    shared=SharedExpertSpec(ff=shared_ff) if shared_ff else None)
        src = i
        if share_from is not None and i >= share_from:
            src = share_from - 1
            att, mlp = layers[src].attention, layers[src].mlp
        layers.append(MitunexLayerSpec(attention=att, mlp=mlp, weights_of=src))
    return MitunexArchConfig(vocab_size=vocab, hidden_size=width, layers=layers, max_position_embeddings=max_pos,
                             logit_scale=1.5, logit_softcap=30.0)


class PoolWindowAttnSpec(BaseModel):
    """GQA softmax attention over a sliding window of ``mask_size`` positions
    (0 = plain causal) plus, when ``pool`` > 0, one key and value per aligned
    block of ``pool`` positions that lies wholly before the window: the means
    of the block's cached keys and values. q and k pass an RMS norm over the
    whole projection (all heads at once, one weight per entry) before the
    rotation; scores are soft-capped at ``softcap`` (0 = none). ``kv_from``:
    the layer has no key/value projections and reads the cache of that
    earlier layer (own queries, mask and pooling)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    mask_size: int = 0
    pool: int = 0
    rot: RotarySpec = Field(default_factory=lambda: RotarySpec(layout="half"))
    kv_from: Optional[int] = None


class Mamba2Spec(BaseModel):
    """State-space mixer with a scalar decay per head and token:
    S <- exp(-exp(A_h) dt) S + dt B x^T, y = S^T C + D_h x; x, B, C pass a
    short causal convolution of ``conv`` taps with bias and silu; B and C are
    shared by the heads of a group; the output is gated by silu(z) and then
    RMS-normed in ``norm_groups`` equal parts."""

    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1


class PironexLayerSpec(BaseModel):
    type: Literal["attention", "mamba2", "latent_attention"]
    attention: Optional[PoolWindowAttnSpec] = None
    mamba2: Optional[Mamba2Spec] = None
    latent: Optional[LatentAttnSpec] = None
    mlp: Optional[RoutedExpertsSpec] = None


class PironexArchConfig(BaseModel):
    """A decoder whose sublayers are layer-normed before and after,
    x <- x + ln(sublayer(canon(ln(x)))), where canon adds a short causal
    convolution over time to the sublayer's input; after every layer the
    stream is replaced by a learned weighted sum of the embedding output and
    all layer results so far. Mixers: windowed attention with pooled blocks
    (optionally on another layer's cache), mamba2, latent attention;
    feed-forward: routed clamped-GLU experts with a gated shared expert, or
    none. The LM head is the embedding table. Every size comes from the
    checkpoint's config.json."""

    arch: Literal["pironex"] = "pironex"
    vocab_size: int
    hidden_size: int
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    canon_taps: int = 1
    layers: List[PironexLayerSpec]
    max_position_embeddings: int = 1 << 24
    tie_word_embeddings: bool = True

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_checkpoint_config(cls, d: dict, shapes: Optional[dict] = None) -> "PironexArchConfig":
        """Parse the family's config.json (keys: vocab, width, norm.eps,
        embedding.scale, canon.taps, layers[].type / .mixer / .mlp)."""
        layers = []
        for li, spec in enumerate(d["layers"]):
            m = spec["mixer"]
            kind = spec["type"]
            mlp = spec.get("mlp")
            ff = None
            if mlp:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
                r, sh = mlp["router"], mlp.get("shared")
                ff = RoutedExpertsSpec(experts=r["experts"], top=r["top"], ff=mlp["expert"]["ff"], score="softmax",
                                       renormalize=True, correction=False, act="clamped",
                                       limit=mlp["expert"]["limit"],
                                       shared=SharedExpertSpec(ff=sh["ff"], limit=sh["limit"]) if sh else None)
            mask = m.get("mask") or {}
            rot = m.get("rot") or {}
            if kind == "attention":
                src = m.get("kv_from")
                if src is not None:
                    other = d["layers"][src] if 0 <= src < li else None
                    if other is None or other["type"] != "attention" or other["mixer"].get("kv_from") is not None:
                        raise ValueError(f"layer {li}: kv_from {src} does not name an earlier attention layer "
                                         f"with keys and values of its own")
                layers.append(PironexLayerSpec(type=kind, mlp=ff, attention=PoolWindowAttnSpec(
                    heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=m["scale"],
                    softcap=m.get("softcap") or 0.0, mask_size=mask.get("size") or 0, pool=mask.get("pool") or 0,
                    rot=RotarySpec(base=rot.get("base", 10000.0), dims=rot.get("dims") or 0, layout="half"),
                    kv_from=src)))
            elif kind == "mamba2":
                layers.append(PironexLayerSpec(type=kind, mlp=ff, mamba2=Mamba2Spec(
                    heads=m["heads"], vdim=m["vdim"], state=m["state"], groups=m["groups"], conv=m["conv"],
                    norm_groups=m.get("norm_groups") or 1)))
            elif kind == "latent_attention":
                att = LatentAttnSpec(heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                                     kv_rank=m["kv_rank"], scale=m["scale"], mask_size=mask.get("size") or 0,
                                     rot=RotarySpec(base=rot.get("base", 10000.0),
                                                    dims=rot.get("dims") or m["rot_dim"]),
                                     head_gate=False)
                if att.rot.dims != att.rot_dim:
                    raise ValueError("the rotated part of a latent-attention head is rotated whole")
                layers.append(PironexLayerSpec(type=kind, mlp=ff, latent=att))
            else:
                raise ValueError(f"unknown layer type {kind!r}")
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], norm_eps=d["norm"]["eps"],
                   embed_scale=(d.get("embedding") or {}).get("scale", 1.0),
                   canon_taps=(d.get("canon") or {}).get("taps", 1), layers=layers)


def _pironex_preset(vocab, width, depth, heads, kv_heads, dim, mask, pool, m_heads, m_vdim, m_state, m_groups,
                    l_heads, l_dim, l_rot, l_vdim, l_rank, l_mask, experts, top, expert_ff, shared_ff,
                    pattern="mlamla", taps=3) -> PironexArchConfig:
    """Random-init presets of the family: ``pattern`` repeats over the depth
    ('m' mamba2, 'l' latent attention, 'a' attention; a later 'a' reads the
    first one's keys and values)."""
    import math as _math

    layers = []
    first_att = None
    for i in range(depth):
        c = pattern[i % len(pattern)]
        ff = RoutedExpertsSpec(experts=experts, top=top, ff=expert_ff, score="softmax", renormalize=True,
                               correction=False, act="clamped", limit=7.0,
                               shared=SharedExpertSpec(ff=shared_ff, limit=7.0) if shared_ff else None)
        if c == "a":
            layers.append(PironexLayerSpec(type="attention", mlp=ff, attention=PoolWindowAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=1.0 / _math.sqrt(dim), softcap=50.0,
                mask_size=mask, pool=pool, rot=RotarySpec(base=500000.0, dims=dim // 2, layout="half"),
                kv_from=first_att)))
            if first_att is None:
                first_att = i
        elif c == "m":
            layers.append(PironexLayerSpec(type="mamba2", mlp=ff, mamba2=Mamba2Spec(
                heads=m_heads, vdim=m_vdim, state=m_state, groups=m_groups, conv=4, norm_groups=m_groups)))
        else:
            layers.append(PironexLayerSpec(type="latent_attention", mlp=ff, latent=LatentAttnSpec(
                heads=l_heads, dim=l_dim, rot_dim=l_rot, vdim=l_vdim, kv_rank=l_rank,
                scale=1.0 / _math.sqrt(l_dim + l_rot), mask_size=l_mask,
                rot=RotarySpec(base=1e6, dims=l_rot), head_gate=False)))
    return PironexArchConfig(vocab_size=vocab, hidden_size=width, embed_scale=1.0, canon_taps=taps, layers=layers)


class HybridLayerSpec(BaseModel):
    type: Literal["parallel", "channel_delta"]
    parallel: Optional[ParallelMixerSpec] = None
    channel_delta: Optional[ChannelDeltaSpec] = None
    mlp: Optional[GluSpec] = None


class HybridArchConfig(BaseModel):
    """A decoder whose layers are listed one by one, each with its own
    sequence mixer (attention and/or recurrent) and optional feed-forward —
    the Zutalix family. Every size comes from the checkpoint's config.json."""

    arch: Literal["zutalix"] = "zutalix"
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float = 1e-6
    layers: List[HybridLayerSpec]
    # no rotary table: angles are computed from the position in the kernel
    max_position_embeddings: int = 1 << 24
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_checkpoint_config(cls, d: dict, shapes: Optional[dict] = None) -> "HybridArchConfig":
        """Parse the family's config.json (keys: vocab, width, norm.eps,
        layers[].type / .mixer / .mlp). ``shapes`` (tensor name -> shape, from
        the safetensors header) supplies the sizes config.json leaves to the
        tensors: the low-rank bottlenecks."""
        layers = []
        shapes = shapes or {}
        for li, spec in enumerate(d["layers"]):
            m = spec["mixer"]
            mlp = spec.get("mlp")
            glu = GluSpec(kind=mlp.get("kind", "dense"), ff=mlp["ff"], limit=mlp["limit"]) if mlp else None
            if spec["type"] == "parallel":
                le, ri = m["left"], m["right"]
                rot = le.get("rot") or {}
                left = BlockAttnSpec(
                    heads=le["heads"], kv_heads=le["kv_heads"], dim=le["dim"], vdim=le["vdim"],
                    scale=le["scale"], mask_size=(le.get("mask") or {}).get("size", 0),
                    rot=RotarySpec(base=rot.get("base", 10000.0), dims=rot.get("dims", 0),
                                   scaling=rot.get("scaling")),
                )
                right = DecayLinearAttnSpec(heads=ri["heads"], dim=ri["dim"], vdim=ri["vdim"],
                                            decay=list(ri["decay"]))
                layers.append(HybridLayerSpec(type="parallel", mlp=glu,
                                              parallel=ParallelMixerSpec(left=left, right=right)))
            elif spec["type"] == "channel_delta":
                layers.append(HybridLayerSpec(type="channel_delta", mlp=glu, channel_delta=ChannelDeltaSpec(
                    heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], conv=m["conv"],
                    decay_rank=(shapes.get(f"l{li}.mix.a1") or [16])[0],
                    gate_rank=(shapes.get(f"l{li}.mix.g1") or [16])[0])))
            else:
                raise ValueError(f"unknown layer type {spec['type']!r}")
        return cls(vocab_size=d["vocab"], hidden_size=d["width"],
                   rms_norm_eps=d["norm"]["eps"], layers=layers)


def _zutalix_preset(vocab, width, n_par, heads, kv_heads, dim, mask, lin_heads, lin_dim, lin_vdim,
                    d_heads, d_kv, d_dim, d_vdim, ff, pattern="ppd", rot_dims=None, conv=4,
                    scaling=None) -> HybridArchConfig:
    """Random-init presets of the family: ``pattern`` repeats over the depth
    ('p' = parallel layer with feed-forward, 'd' = delta layer without)."""
    import math as _math

    layers = []
    for i in range(n_par):
        if pattern[i % len(pattern)] == "p":
            left = BlockAttnSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                                 scale=1.0 / _math.sqrt(dim), mask_size=mask,
                                 rot=RotarySpec(base=500000.0, dims=rot_dims or dim, scaling=scaling))
            right = DecayLinearAttnSpec(
                heads=lin_heads, dim=lin_dim, vdim=lin_vdim,
                decay=[_math.exp(-1.0 / (2.0 ** (1 + 2 * h))) for h in range(lin_heads)])
            layers.append(HybridLayerSpec(type="parallel", parallel=ParallelMixerSpec(left=left, right=right),
                                          mlp=GluSpec(ff=ff, limit=7.0)))
        else:
            layers.append(HybridLayerSpec(type="channel_delta", channel_delta=ChannelDeltaSpec(
                heads=d_heads, kv_heads=d_kv, dim=d_dim, vdim=d_vdim, conv=conv,
                decay_rank=max(8, width // 32), gate_rank=max(8, width // 32))))
    return HybridArchConfig(vocab_size=vocab, hidden_size=width, layers=layers)


MODEL_PRESETS: dict = {
    # Llama-3-8B — the BASELINE headline config
    "llama-3-8b": ModelArchConfig(
        arch="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
        num_layers=32, num_heads=32, num_kv_heads=8, rope_theta=500000.0,
    ),
    # Llama-3.1: same dims, banded-NTK rope scaling to 128k context
    "llama-3.1-8b": ModelArchConfig(
        arch="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
        num_layers=32, num_heads=32, num_kv_heads=8, rope_theta=500000.0,
        max_position_embeddings=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    ),
    "llama-3-70b": ModelArchConfig(
        arch="llama", vocab_size=128256, hidden_size=8192, intermediate_size=28672,
        num_layers=80, num_heads=64, num_kv_heads=8, rope_theta=500000.0,
    ),
    "mixtral-8x7b": ModelArchConfig(
        arch="mixtral", vocab_size=32000, hidden_size=4096, intermediate_size=14336,
        num_layers=32, num_heads=32, num_kv_heads=8, rope_theta=1e6,
        num_experts=8, num_experts_per_tok=2, rms_norm_eps=1e-5,
    ),
    # Mid preset for GPU kernel/engine tests: real head_dim (128), small depth
    "mid-llama": ModelArchConfig(
        arch="llama", vocab_size=2048, hidden_size=512, intermediate_size=1024,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        max_position_embeddings=2048,
    ),
    "mid-qwen": ModelArchConfig(
        arch="llama", vocab_size=2048, hidden_size=512, intermediate_size=1024,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        max_position_embeddings=2048, attention_qkv_bias=True,
        tie_word_embeddings=True,
    ),
    "mid-mixtral": ModelArchConfig(
        arch="mixtral", vocab_size=2048, hidden_size=512, intermediate_size=1024,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        num_experts=4, num_experts_per_tok=2, max_position_embeddings=2048,
    ),
    # Tiny CPU-testable presets (same code paths, toy sizes)
    "tiny-llama": ModelArchConfig(
        arch="llama", vocab_size=512, hidden_size=64, intermediate_size=128,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        max_position_embeddings=512,
    ),
    # tiny variant with 4 KV heads so gloo TP=4 tests divide evenly
    "tiny-llama-kv4": ModelArchConfig(
        arch="llama", vocab_size=512, hidden_size=128, intermediate_size=256,
        num_layers=2, num_heads=8, num_kv_heads=4, rope_theta=10000.0,
        max_position_embeddings=512,
    ),
    "tiny-mixtral": ModelArchConfig(
        arch="mixtral", vocab_size=512, hidden_size=64, intermediate_size=128,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        num_experts=4, num_experts_per_tok=2, max_position_embeddings=512,
    ),
    # Qwen2 family: Llama compute graph + QKV bias (+ tied embeddings on
    # the small members); head_dim 128 so every HIP kernel applies as-is
    "qwen2-7b": ModelArchConfig(
        arch="llama", vocab_size=152064, hidden_size=3584, intermediate_size=18944,
        num_layers=28, num_heads=28, num_kv_heads=4, rope_theta=1e6,
        rms_norm_eps=1e-6, max_position_embeddings=32768, attention_qkv_bias=True,
    ),
    "tiny-qwen": ModelArchConfig(
        arch="llama", vocab_size=512, hidden_size=64, intermediate_size=128,
        num_layers=2, num_heads=4, num_kv_heads=2, rope_theta=10000.0,
        max_position_embeddings=512, attention_qkv_bias=True,
        tie_word_embeddings=True,
    ),
    # Zutalix family (listed-layer hybrid: block-local softmax attention +
    # decayed linear attention in parallel, gated-delta layers between)
    "tiny-zutalix": _zutalix_preset(
        vocab=512, width=64, n_par=3, heads=4, kv_heads=2, dim=16, mask=24,
        lin_heads=2, lin_dim=8, lin_vdim=16, d_heads=2, d_kv=1, d_dim=16, d_vdim=24, ff=96),
    "mid-zutalix": _zutalix_preset(
        vocab=2048, width=512, n_par=3, heads=4, kv_heads=2, dim=128, mask=256,
        lin_heads=4, lin_dim=64, lin_vdim=128, d_heads=4, d_kv=2, d_dim=64, d_vdim=128, ff=1024),
    # layer shapes of real models at reduced depth, and the dense Llama stack
    # of the same width / depth / heads / ff beside each (bench.py
    # --compare-families)
    "zutalix-8b-l6": _zutalix_preset(
        vocab=32000, width=4096, n_par=6, heads=32, kv_heads=8, dim=128, mask=2048,
        lin_heads=32, lin_dim=128, lin_vdim=128, d_heads=32, d_kv=16, d_dim=128, d_vdim=128, ff=14336),
    "llama-8b-l6": ModelArchConfig(
        arch="llama", vocab_size=32000, hidden_size=4096, intermediate_size=14336,
        num_layers=6, num_heads=32, num_kv_heads=8, rope_theta=500000.0),
    "zutalix-1b-l6": _zutalix_preset(
        vocab=32000, width=2048, n_par=6, heads=16, kv_heads=4, dim=128, mask=1024,
        lin_heads=16, lin_dim=64, lin_vdim=128, d_heads=16, d_kv=8, d_dim=64, d_vdim=128, ff=8192),
    "llama-1b-l6": ModelArchConfig(
        arch="llama", vocab_size=32000, hidden_size=2048, intermediate_size=8192,
        num_layers=6, num_heads=16, num_kv_heads=4, rope_theta=500000.0),
    # Medilix family (parallel layers; windowed attention with a sink, wkv and
    # mlstm mixers; dense and routed feed-forwards; looped layer range)
    "tiny-medilix": _medilix_preset(
        vocab=512, width=64, depth=4, heads=4, kv_heads=2, dim=16, mask=24, keep=3, r_heads=2, r_dim=16,
        m_heads=2, m_dim=8, m_vdim=16, ff=96, experts=4, top=2, expert_ff=48,
        loop={"start": 1, "stop": 3, "times": 2}),
    "mid-medilix": _medilix_preset(
        vocab=2048, width=512, depth=3, heads=4, kv_heads=2, dim=128, mask=256, keep=4, r_heads=8, r_dim=64,
        m_heads=4, m_dim=64, m_vdim=128, ff=1024, experts=8, top=2, expert_ff=256),
    # layer shapes of real models at reduced depth, beside llama-{1b,8b}-l6
    "medilix-8b-l6": _medilix_preset(
        vocab=32000, width=4096, depth=6, heads=32, kv_heads=8, dim=128, mask=2048, keep=4, r_heads=64,
        r_dim=64, m_heads=32, m_dim=64, m_vdim=128, ff=14336, experts=8, top=2, expert_ff=7168, identity=0),
    "medilix-1b-l6": _medilix_preset(
        vocab=32000, width=2048, depth=6, heads=16, kv_heads=4, dim=128, mask=1024, keep=4, r_heads=32,
        r_dim=64, m_heads=16, m_dim=64, m_vdim=128, ff=8192, experts=8, top=2, expert_ff=4096, identity=0),
    # Mitunex family (post-normed layers; latent attention with a sliding
    # window; gelu and routed feed-forwards; layers that share weights)
    "tiny-mitunex": _mitunex_preset(
        vocab=512, width=64, depth=4, heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=32, mask=24, ff=96,
        experts=6, top=2, expert_ff=48, shared_ff=40, share_from=3, max_pos=512),
    "mid-mitunex": _mitunex_preset(
        vocab=2048, width=512, depth=3, heads=8, dim=64, rot_dim=32, vdim=64, kv_rank=128, mask=256, ff=1024,
        experts=8, top=2, expert_ff=256, shared_ff=256, max_pos=2048),
    # layer shapes of real models at reduced depth, beside llama-/medilix-{1b,8b}-l6
    "mitunex-8b-l6": _mitunex_preset(
        vocab=32000, width=4096, depth=6, heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=512, mask=2048,
        ff=14336, experts=8, top=2, expert_ff=7168, shared_ff=2048),
    "mitunex-1b-l6": _mitunex_preset(
        vocab=32000, width=2048, depth=6, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512, mask=1024,
        ff=8192, experts=8, top=2, expert_ff=4096, shared_ff=1024),
    # Pironex family (layer-normed sublayers with a short input convolution,
    # depth-weighted stream; mamba2, latent attention and windowed attention
    # with pooled blocks; routed clamped-GLU experts)
    "tiny-pironex": _pironex_preset(
        vocab=512, width=64, depth=6, heads=4, kv_heads=2, dim=16, mask=24, pool=4, m_heads=4, m_vdim=16,
        m_state=8, m_groups=2, l_heads=4, l_dim=16, l_rot=8, l_vdim=24, l_rank=32, l_mask=24, experts=6, top=2,
        expert_ff=48, shared_ff=40),
    "mid-pironex": _pironex_preset(
        vocab=2048, width=512, depth=3, heads=4, kv_heads=2, dim=128, mask=256, pool=16, m_heads=8, m_vdim=64,
        m_state=64, m_groups=2, l_heads=8, l_dim=64, l_rot=32, l_vdim=64, l_rank=128, l_mask=256, experts=8,
        top=2, expert_ff=256, shared_ff=256, pattern="mla"),
    # layer shapes of real models at reduced depth, beside llama-/mitunex-{1b,8b}-l6
    "pironex-8b-l6": _pironex_preset(
        vocab=32000, width=4096, depth=6, heads=32, kv_heads=8, dim=128, mask=2048, pool=64, m_heads=64,
        m_vdim=64, m_state=128, m_groups=8, l_heads=32, l_dim=128, l_rot=64, l_vdim=128, l_rank=512, l_mask=2048,
        experts=8, top=2, expert_ff=7168, shared_ff=2048),
    "pironex-1b-l6": _pironex_preset(
        vocab=32000, width=2048, depth=6, heads=16, kv_heads=4, dim=128, mask=1024, pool=64, m_heads=32,
        m_vdim=64, m_state=128, m_groups=4, l_heads=16, l_dim=128, l_rot=64, l_vdim=128, l_rank=512, l_mask=1024,
        experts=8, top=2, expert_ff=4096, shared_ff=1024),
}


class EngineConfig(BaseModel):
    """Runtime configuration for the local engine."""

    model: str = "llama-3-8b"          # preset name or path to a weights dir
    weights_path: Optional[str] = None  # safetensors dir; None = random init
    dtype: Literal["bfloat16", "float32", "float16"] = "bfloat16"
    seed: int = 0

    # Parallelism: TP over RCCL/xGMI (one process per GPU)
    tp_size: int = 1

    # KV cache
    kv_block_size: int = 16
    # "bf16" (default, matches compute dtype) or "fp8_e4m3" (half the KV
    # traffic/footprint; OCP e4m3 with PER-ROW dequant scales — each
    # (token, head) row is stored as x/s with s = amax(|row|)/448 kept in a
    # parallel fp32 [NB, KVH, BS] tensor (~3% overhead), so outlier-heavy
    # real checkpoints don't saturate e4m3's +-448 range)
    kv_cache_dtype: Literal["bf16", "fp8_e4m3"] = "bf16"
    # Fraction of free HBM given to the KV cache after weights are resident
    kv_memory_fraction: float = 0.70
    max_kv_blocks: Optional[int] = None  # explicit cap (used on CPU/tests)

    max_seq_len: int = 8192
    max_batch_size: int = 256
    # recurrent-state slots (models with linear-attention / delta-rule /
    # convolution state keep one slot per live sequence); None = derived
    # from max_batch_size
    max_state_slots: Optional[int] = None

    # embeddings.create backend: "token_mean" mean-pools the model's token
    # embeddings (semantically meaningful once real weights are loaded);
    # "ngram" is a deterministic signed char-3-gram hashing embedder whose
    # cosine tracks STRING similarity with no weights at all; "auto" picks
    # ngram under random init and token_mean when a checkpoint is loaded
    embedding_mode: Literal["auto", "token_mean", "ngram"] = "auto"

    # Decode-step hipGraph capture
    use_hip_graphs: bool = True
    # constrained decoding: allow optional JSON whitespace between tokens
    # (default emits compact JSON — smaller DFA, fewer wasted tokens)
    constrained_whitespace: bool = False
    # cross-request prefix caching: full prompt blocks are published to a
    # digest-keyed cache; later prompts sharing the prefix skip re-prefilling
    # it (LRU + eviction under allocator pressure)
    enable_prefix_caching: bool = True
    prefix_cache_fraction: float = 0.5  # max fraction of KV blocks held
    # ignore hits shorter than this: a short cached head saves less prefill
    # than the tail's decode-mode forward costs over the packed kernel
    prefix_cache_min_tokens: int = 128

    # scheduler: prefill prompts longer than this in slices interleaved with
    # decode steps, so a long prompt doesn't stall running streams
    # (None = whole-prompt prefill at admission)
    prefill_chunk_tokens: Optional[int] = None
    hip_graph_batch_sizes: list[int] = Field(default_factory=lambda: [1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 160, 192, 224, 256])

    # Generation defaults
    default_max_new_tokens: int = 512
    # default: the checkpoint's generation_config.json eos_token_id (which
    # may be a LIST — Llama-3 stops on <|eot_id|> OR <|end_of_text|>),
    # else the tokenizer's
    eos_token_id: Optional[Union[int, List[int]]] = None

    # Device ("cuda" is ROCm/HIP under torch-rocm; "cpu" for tests)
    device: Optional[str] = None

    def effective_weights_dir(self) -> Optional[str]:
        """The directory to load safetensors from: explicit weights_path, or
        the model path itself when it is a directory holding safetensors
        (README contract: model = preset name OR path to a weights dir).
        None = deterministic random init."""
        import glob as _glob
        import os as _os

        if self.weights_path:
            return self.weights_path
        if _os.path.isdir(str(self.model)) and _glob.glob(_os.path.join(self.model, "*.safetensors")):
            return self.model
        return None

    def resolve_arch(self):
        if self.model in MODEL_PRESETS:
            return MODEL_PRESETS[self.model]
        # A path: read config.json (HF-style) next to the weights
        import json
        import os

        cfg_path = os.path.join(self.weights_path or self.model, "config.json")
        if not os.path.exists(cfg_path):
            # OpenAI-style model-not-found error instead of a raw ENOENT
            raise ValueError(
                f"model {self.model!r} is neither a preset "
                f"({', '.join(sorted(MODEL_PRESETS))}) nor a directory with a "
                f"config.json (model_not_found)"
            )
        with open(cfg_path) as f:
            hf = json.load(f)
        family = str(hf.get("architecture", "")).lower()
        if family in ("zutalix", "medilix", "mitunex", "pironex"):
            from .weights import safetensors_shapes

            reader = {"zutalix": HybridArchConfig, "medilix": MedilixArchConfig,
                      "mitunex": MitunexArchConfig, "pironex": PironexArchConfig}[family]
            return reader.from_checkpoint_config(hf, safetensors_shapes(os.path.dirname(cfg_path)))
        arch = "mixtral" if "mixtral" in hf.get("model_type", "").lower() or hf.get("num_local_experts") else "llama"
        return ModelArchConfig(
            arch=arch,
            vocab_size=hf["vocab_size"],
            hidden_size=hf["hidden_size"],
            intermediate_size=hf["intermediate_size"],
            num_layers=hf["num_hidden_layers"],
            num_heads=hf["num_attention_heads"],
            num_kv_heads=hf.get("num_key_value_heads", hf["num_attention_heads"]),
            rope_theta=hf.get("rope_theta", 10000.0),
            rms_norm_eps=hf.get("rms_norm_eps", 1e-5),
            max_position_embeddings=hf.get("max_position_embeddings", 8192),
            tie_word_embeddings=hf.get("tie_word_embeddings", False),
            num_experts=hf.get("num_local_experts", 0),
            num_experts_per_tok=hf.get("num_experts_per_tok", 2),
            # Qwen2 configs carry no attention_bias key but always use QKV
            # bias; Llama-style configs say so explicitly
            attention_qkv_bias=hf.get(
                "attention_bias", hf.get("model_type", "").lower() == "qwen2"),
            rope_scaling=hf.get("rope_scaling"),
        )
