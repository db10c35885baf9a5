"""Typed model configuration read from the architecture's own config.json keys.

The reference hands config.json to a library class and reads attributes where it needs
them (ullm/config.py:43, ullm/models/qwen3.py:139-157,207,224,268,
ullm/core/model_runner.py:31-73).  Here the keys are parsed once into a frozen
dataclass; every size and constant the model uses comes from this object.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, fields
from typing import Any, Mapping, Optional


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model configuration."""


_REQUIRED = object()


def _take(d: Mapping[str, Any], key: str, kind, default=_REQUIRED):
    if key not in d or d[key] is None:
        if default is _REQUIRED:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    try:
        if kind is bool:
            if not isinstance(v, (bool, int)):
                raise TypeError
            return bool(v)
        if kind is int:
            if isinstance(v, bool) or int(v) != v:
                raise TypeError
            return int(v)
        if kind is float:
            return float(v)
        if kind is str:
            if not isinstance(v, str):
                raise TypeError
            return v
    except (TypeError, ValueError):
        pass
    raise ConfigError(f"config.json: key '{key}' has value {v!r}, expected {kind.__name__}")


@dataclass(frozen=True)
class Qwen3Config:
    """Keys of a Qwen3 dense config.json.

    Defaults follow the reference: ``head_dim = hidden_size // num_attention_heads``
    (ullm/models/qwen3.py:78, ullm/core/model_runner.py:60-63), ``rope_theta = 1e6``
    (qwen3.py:144), ``attention_bias = False`` (qwen3.py:146); ``rms_norm_eps`` is read
    without a default (qwen3.py:145).  ``tie_word_embeddings`` and the sliding-window
    keys are not read by the reference (it always owns a separate lm_head,
    qwen3.py:267-270, and never masks by distance); they are read here so that a tied
    checkpoint binds and a windowed config chooses a windowed mixer layer by layer.
    """

    architectures: tuple
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    attention_bias: bool
    tie_word_embeddings: bool
    hidden_act: str
    use_sliding_window: bool
    sliding_window: int
    max_window_layers: int
    layer_types: tuple            # per layer "full_attention" / "sliding_attention", or () where config.json has no list
    torch_dtype: str
    eos_token_id: int             # the first stop id config.json names (-1: none)
    eos_token_ids: tuple          # all of them: config.json may hold a list
    initializer_range: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        archs = d.get("architectures")
        if not isinstance(archs, (list, tuple)) or not archs:
            raise ConfigError("config.json: required key 'architectures' is missing or empty")
        hidden = _take(d, "hidden_size", int)
        nq = _take(d, "num_attention_heads", int)
        nkv = _take(d, "num_key_value_heads", int, nq)
        if nq <= 0 or nkv <= 0 or nq % nkv != 0:
            raise ConfigError(
                f"config.json: num_attention_heads={nq} must be a positive multiple of "
                f"num_key_value_heads={nkv}")
        head_dim = _take(d, "head_dim", int, None)
        if head_dim is None:
            if hidden % nq != 0:
                raise ConfigError(
                    f"config.json: no 'head_dim' and hidden_size={hidden} is not a multiple "
                    f"of num_attention_heads={nq}")
            head_dim = hidden // nq
        use_window = _take(d, "use_sliding_window", bool, False)
        window = _take(d, "sliding_window", int, 0)
        layers = _take(d, "num_hidden_layers", int)
        max_window_layers = _take(d, "max_window_layers", int, layers)
        if use_window and window <= 0:
            raise ConfigError("config.json: use_sliding_window is true but 'sliding_window' "
                              "is missing or not positive")
        kinds = d.get("layer_types")
        if kinds is None:
            kinds = ()
        elif (not isinstance(kinds, (list, tuple)) or len(kinds) != layers
              or any(k not in ("full_attention", "sliding_attention") for k in kinds)):
            raise ConfigError(f"config.json: layer_types={kinds!r} must name 'full_attention' or 'sliding_attention' "
                              f"for each of the {layers} layers")
        elif "sliding_attention" in kinds and not use_window:
            raise ConfigError("config.json: layer_types names sliding_attention layers but use_sliding_window is "
                              "not true: which keys such a layer sees is not defined")
        act = _take(d, "hidden_act", str, "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act={act!r}; this architecture's "
                              "feed-forward is SwiGLU (silu)")
        dtype = d.get("dtype") or d.get("torch_dtype") or "bfloat16"
        if not isinstance(dtype, str):
            raise ConfigError(f"config.json: dtype={dtype!r} is not a string")
        eos = d.get("eos_token_id")
        eos_ids = tuple(eos) if isinstance(eos, (list, tuple)) else (() if eos is None else (eos,))
        for e in eos_ids:
            if isinstance(e, bool) or not isinstance(e, int) or e < 0:
                raise ConfigError(f"config.json: eos_token_id={eos!r} must be a token id or a list of token ids")
        # The reference builds its rotation angles from rope_theta alone (ullm/models/qwen3.py:97-102,
        # ullm/layers/rotary_embedding.py:52-75) and so does this engine: a config that asks for scaled
        # angles would run with wrong ones, so it is refused rather than served quietly.
        scaling = d.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, Mapping) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"config.json: rope_scaling={scaling!r} is not supported (only absent, null or "
                                  "type 'default': the rotation angles come from rope_theta alone)")
        cfg = cls(
            architectures=tuple(str(a) for a in archs),
            vocab_size=_take(d, "vocab_size", int),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=head_dim,
            intermediate_size=_take(d, "intermediate_size", int),
            max_position_embeddings=_take(d, "max_position_embeddings", int),
            rms_norm_eps=_take(d, "rms_norm_eps", float),
            rope_theta=_take(d, "rope_theta", float, 1000000.0),
            attention_bias=_take(d, "attention_bias", bool, False),
            tie_word_embeddings=_take(d, "tie_word_embeddings", bool, False),
            hidden_act=act,
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=max_window_layers,
            layer_types=tuple(kinds),
            torch_dtype=dtype,
            eos_token_id=int(eos_ids[0]) if eos_ids else -1,
            eos_token_ids=tuple(int(e) for e in eos_ids),
            initializer_range=_take(d, "initializer_range", float, 0.02),
        )
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "head_dim",
                     "intermediate_size", "max_position_embeddings"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"config.json: '{name}' must be positive, got {getattr(cfg, name)}")
        if cfg.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim={cfg.head_dim} must be even for rotary pairs")
        if cfg.rms_norm_eps < 0:
            raise ConfigError("config.json: 'rms_norm_eps' must not be negative")
        return cfg

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        d["eos_token_ids"] = list(self.eos_token_ids)
        if self.layer_types:
            d["layer_types"] = list(self.layer_types)
        else:
            del d["layer_types"]
        return d

    def window_of_layer(self, layer: int) -> int:
        """Keys a query of this layer may look back over, itself included; 0 = all.  A per-layer list in
        config.json decides where there is one, else the layers from ``max_window_layers`` on have the window."""
        if not self.use_sliding_window:
            return 0
        if self.layer_types:
            return self.sliding_window if self.layer_types[layer] == "sliding_attention" else 0
        return self.sliding_window if layer >= self.max_window_layers else 0


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json in the model folder")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def config_field_names(cls) -> list:
    return [f.name for f in fields(cls)]


@dataclass(frozen=True)
class PamopelLayer:
    """One layer of a Pamopel config.json: ``type`` names the mixer, ``mixer`` holds its sizes and constants as
    (key, value) pairs, ``mlp`` those of the feed-forward or None for a layer without one."""
    type: str
    mixer: tuple
    mlp: Optional[tuple]

    def mixer_dict(self) -> dict:
        return dict(self.mixer)

    def mlp_dict(self) -> Optional[dict]:
        return None if self.mlp is None else dict(self.mlp)


_PAMOPEL_MIXER_KEYS = {
    "attention": (("heads", int), ("kv_heads", int), ("dim", int), ("vdim", int), ("scale", float), ("bias_max", int)),
    "mamba2": (("heads", int), ("vdim", int), ("state", int), ("groups", int), ("conv", int), ("norm_groups", int)),
}


@dataclass(frozen=True)
class PamopelConfig:
    """Keys of a Pamopel config.json: a stack whose layers are listed one by one (attention with a learned
    bias by distance and a gate per head, possibly reading another layer's keys and values; or a Mamba-2
    mixer), layer norms on both sides of every sublayer, and an embedding that adds a hashed bigram row and
    a sinusoidal position row to the token's."""
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple                   # of PamopelLayer
    norm_eps: float
    residual_mult: float
    logit_scale: float
    embedding_scale: float
    bigram_buckets: int             # 0: no bigram table
    bigram_mul_prev: int
    bigram_mul_cur: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "PamopelConfig":
        emb = d.get("embedding") or {}
        if not isinstance(emb, Mapping):
            raise ConfigError("config.json: key 'embedding' must be an object")
        big = emb.get("bigram") or {}
        norm = d.get("norm") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(raw_layers):
            kind = _take(L, "type", str)
            if kind not in _PAMOPEL_MIXER_KEYS:
                raise ConfigError(f"config.json: layer {i} has type {kind!r}; known: {sorted(_PAMOPEL_MIXER_KEYS)}")
            m = L.get("mixer")
            if not isinstance(m, Mapping):
                raise ConfigError(f"config.json: layer {i} has no 'mixer' object")
            try:
                mixer = [(key, _take(m, key, typ)) for key, typ in _PAMOPEL_MIXER_KEYS[kind]]
                if kind == "attention" and m.get("kv_from") is not None:
                    src = _take(m, "kv_from", int)
                    if not 0 <= src < i or raw_layers[src].get("type") != "attention" \
                            or (raw_layers[src].get("mixer") or {}).get("kv_from") is not None:
                        raise ConfigError(f"'kv_from': {src} must name an earlier attention layer with keys of its own")
                    mixer.append(("kv_from", src))
                mlp = L.get("mlp")
                if mlp is not None:
                    if not isinstance(mlp, Mapping) or _take(mlp, "kind", str) != "dense":
                        raise ConfigError("'mlp' must be null or an object of kind 'dense'")
                    mlp = (("kind", "dense"), ("ff", _take(mlp, "ff", int)))
            except ConfigError as e:
                raise ConfigError(f"{e} (layer {i})") from None
            layers.append(PamopelLayer(kind, tuple(mixer), mlp))
        return cls(
            architecture=_take(d, "architecture", str, "Pamopel"),
            vocab_size=_take(d, "vocab", int), hidden_size=_take(d, "width", int), layers=tuple(layers),
            norm_eps=_take(norm, "eps", float), residual_mult=_take(d, "residual_mult", float, 1.0),
            logit_scale=_take(d, "logit_scale", float, 1.0), embedding_scale=_take(emb, "scale", float, 1.0),
            bigram_buckets=_take(big, "buckets", int, 0), bigram_mul_prev=_take(big, "mul_prev", int, 0),
            bigram_mul_cur=_take(big, "mul_cur", int, 0))

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)


@dataclass(frozen=True)
class ZiferaxAttention:
    """Sizes and constants of one Ziferax attention mixer."""
    heads: int
    kv_heads: int
    dim: int                        # per-head query / key size; the values are the keys, so also the value size
    scale: float
    window: int                     # keys a query sees, itself included; 0: all
    rot_dims: int                   # leading dims of each head that are rotated; 0: none
    rot_base: float


@dataclass(frozen=True)
class ZiferaxExperts:
    """Sizes and constants of one Ziferax routed feed-forward."""
    experts: int                    # experts with tensors
    identity: int                   # router outputs beyond them whose expert returns its input
    top: int
    ff: int
    limit: float
    shared_ff: int                  # 0: no shared expert
    shared_limit: float


@dataclass(frozen=True)
class ZiferaxLayer:
    type: str
    mixer: ZiferaxAttention
    mlp: Optional[ZiferaxExperts]
    weights_of: Optional[int]       # the layer whose tensors this one uses (with a cache of its own), or None


@dataclass(frozen=True)
class ZiferaxConfig:
    """Keys of a Ziferax config.json: a stack of parallel blocks (one RMS norm, attention and a routed
    feed-forward that both read it, a multiplier on their sum), listed layer by layer.  Attention has biases on
    q, k and the output, values that are the keys before rotation, rotation of adjacent pairs over the heads' first
    ``rot.dims`` dims, a sliding window and a sink per head.  A layer with ``weights_of`` uses another layer's
    tensors.  The head is the embedding table."""
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple                   # of ZiferaxLayer
    norm_eps: float
    residual_mult: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ZiferaxConfig":
        norm = d.get("norm") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(raw_layers):
            try:
                if not isinstance(L, Mapping):
                    raise ConfigError("a layer must be an object")
                kind = _take(L, "type", str)
                if kind != "attention":
                    raise ConfigError(f"type {kind!r}; known: ['attention']")
                m = L.get("mixer")
                if not isinstance(m, Mapping):
                    raise ConfigError("no 'mixer' object")
                mask, rot = m.get("mask") or {}, m.get("rot") or {}
                dim = _take(m, "dim", int)
                att = ZiferaxAttention(
                    heads=_take(m, "heads", int), kv_heads=_take(m, "kv_heads", int), dim=dim,
                    scale=_take(m, "scale", float), window=_take(mask, "size", int, 0),
                    rot_dims=_take(rot, "dims", int, 0), rot_base=_take(rot, "base", float, 10000.0))
                if _take(m, "vdim", int, dim) != dim:
                    raise ConfigError(f"'vdim' = {m['vdim']} differs from 'dim' = {dim}: the values are the keys")
                if att.heads < 1 or att.kv_heads < 1 or att.heads % att.kv_heads or dim < 1:
                    raise ConfigError(f"{att.heads} heads over {att.kv_heads} kv heads of size {dim}")
                if att.rot_dims < 0 or att.rot_dims % 2 or att.rot_dims > dim or att.window < 0:
                    raise ConfigError(f"rot.dims = {att.rot_dims} must be even and at most dim = {dim}; mask.size >= 0")
                mlp = L.get("mlp")
                if mlp is not None:
                    if not isinstance(mlp, Mapping) or _take(mlp, "kind", str) != "moe":
                        raise ConfigError("'mlp' must be null or an object of kind 'moe'")
                    router, expert = mlp.get("router") or {}, mlp.get("expert") or {}
                    shared = mlp.get("shared") or {}
                    mlp = ZiferaxExperts(
                        experts=_take(router, "experts", int), identity=_take(router, "identity", int, 0),
                        top=_take(router, "top", int), ff=_take(expert, "ff", int), limit=_take(expert, "limit", float),
                        shared_ff=_take(shared, "ff", int, 0),
                        shared_limit=_take(shared, "limit", float, _take(expert, "limit", float)))
                    if mlp.experts < 0 or mlp.identity < 0 or not 1 <= mlp.top <= mlp.experts + mlp.identity:
                        raise ConfigError(f"top = {mlp.top} of {mlp.experts} experts and {mlp.identity} identity experts")
                    if (mlp.experts and mlp.ff < 1) or mlp.shared_ff < 0 or not mlp.limit > 0 or not mlp.shared_limit > 0:
                        raise ConfigError("expert sizes and limits must be positive")
                src = L.get("weights_of")
                if src is not None:
                    src = _take(L, "weights_of", int)
                    seen = {i}
                    while True:                                   # a layer may name one that names another: followed to the tensors
                        if not 0 <= src < len(raw_layers) or src in seen or not isinstance(raw_layers[src], Mapping):
                            raise ConfigError(f"'weights_of': {src} must lead to another layer with tensors of its own")
                        if raw_layers[src].get("weights_of") is None:
                            break
                        seen.add(src)
                        src = _take(raw_layers[src], "weights_of", int)
            except ConfigError as e:
                raise ConfigError(f"{e} (layer {i})") from None
            layers.append(ZiferaxLayer(kind, att, mlp, src))
        for i, L in enumerate(layers):
            if L.weights_of is not None:
                o = layers[L.weights_of]
                if (o.mixer, o.mlp) != (L.mixer, L.mlp):
                    raise ConfigError(f"config.json: layer {i} uses the tensors of layer {L.weights_of} but their "
                                      f"entries differ")
        cfg = cls(architecture=_take(d, "architecture", str, "Ziferax"), vocab_size=_take(d, "vocab", int),
                  hidden_size=_take(d, "width", int), layers=tuple(layers), norm_eps=_take(norm, "eps", float),
                  residual_mult=_take(d, "residual_mult", float, 1.0))
        if cfg.vocab_size < 1 or cfg.hidden_size < 1 or cfg.norm_eps < 0:
            raise ConfigError("config.json: 'vocab' and 'width' must be positive and 'norm.eps' not negative")
        return cfg

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)


@dataclass(frozen=True)
class RotaryScaling:
    """Frequencies stretched by wavelength: pairs that turn fewer than ``slow`` times over ``original`` positions
    have their frequency divided by ``factor``, pairs that turn more than ``fast`` times keep it, those between
    are blended linearly by their index; cosines and sines are multiplied by 0.1 ln(factor) + 1."""
    factor: float
    original: int
    fast: float
    slow: float


@dataclass(frozen=True)
class DovisunAttention:
    """Grouped-query attention without positions; queries and keys have unit root mean square per head and the
    softmax's denominator holds one more term exp(0)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float


@dataclass(frozen=True)
class DovisunLatentAttention:
    """Attention whose queries and keys/values go through latents; ``rot_dim`` rotated dims shared by all heads."""
    heads: int
    dim: int                        # unrotated query / key dims per head
    rot_dim: int                    # rotated dims per head (the keys' are one vector for all heads)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_scaling: Optional[RotaryScaling]


@dataclass(frozen=True)
class DovisunDense:
    ff: int


@dataclass(frozen=True)
class DovisunExperts:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class DovisunLayer:
    type: str                       # "attention" | "latent_attention"
    mixer: object                   # DovisunAttention | DovisunLatentAttention
    mlp: object                     # DovisunDense | DovisunExperts | None


@dataclass(frozen=True)
class DovisunConfig:
    """Keys of a Dovisun config.json: parallel blocks (one RMS norm, a mixer and a feed-forward that both read it)
    listed layer by layer, a run of layers that is passed several times on the same tensors with the embedding
    mixed into the stream ahead of every pass (``loop``), a scale on the embedding and a soft cap on the logits."""
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple                   # of DovisunLayer
    norm_eps: float
    embedding_scale: float
    logit_softcap: float            # 0: none
    loop_start: int
    loop_stop: int                  # layers loop_start .. loop_stop - 1 run loop_times times in a row; equal: no loop
    loop_times: int
    has_loop: bool = False          # config.json has a 'loop' object (and so the checkpoint the mixing matrix)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "DovisunConfig":
        norm, emb = d.get("norm") or {}, d.get("embedding") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(raw_layers):
            try:
                if not isinstance(L, Mapping):
                    raise ConfigError("a layer must be an object")
                kind, m = _take(L, "type", str), L.get("mixer")
                if not isinstance(m, Mapping):
                    raise ConfigError("no 'mixer' object")
                if kind == "attention":
                    dim = _take(m, "dim", int)
                    mixer = DovisunAttention(heads=_take(m, "heads", int), kv_heads=_take(m, "kv_heads", int), dim=dim,
                                             vdim=_take(m, "vdim", int, dim), scale=_take(m, "scale", float))
                    if mixer.heads < 1 or mixer.kv_heads < 1 or mixer.heads % mixer.kv_heads or dim < 1 or mixer.vdim < 1:
                        raise ConfigError(f"{mixer.heads} heads over {mixer.kv_heads} kv heads of sizes {dim} and {mixer.vdim}")
                elif kind == "latent_attention":
                    rot = m.get("rot") or {}
                    rot_dim = _take(m, "rot_dim", int)
                    sc = rot.get("scaling")
                    scaling = None
                    if sc is not None:
                        if not isinstance(sc, Mapping):
                            raise ConfigError("'rot.scaling' must be an object")
                        scaling = RotaryScaling(factor=_take(sc, "factor", float), original=_take(sc, "original", int),
                                                fast=_take(sc, "fast", float), slow=_take(sc, "slow", float))
                        if scaling.factor <= 0 or scaling.original < 1 or scaling.fast <= 0 or scaling.slow <= 0:
                            raise ConfigError("'rot.scaling': factor, original, fast and slow must be positive")
                    dim = _take(m, "dim", int)
                    mixer = DovisunLatentAttention(
                        heads=_take(m, "heads", int), dim=dim, rot_dim=rot_dim, vdim=_take(m, "vdim", int, dim),
                        q_rank=_take(m, "q_rank", int), kv_rank=_take(m, "kv_rank", int), scale=_take(m, "scale", float),
                        rot_base=_take(rot, "base", float, 10000.0), rot_scaling=scaling)
                    if _take(rot, "dims", int, rot_dim) != rot_dim:
                        raise ConfigError(f"'rot.dims' = {rot['dims']} differs from 'rot_dim' = {rot_dim}: the rotated part is rotated whole")
                    if mixer.heads < 1 or dim < 1 or rot_dim < 0 or rot_dim % 2 or mixer.vdim < 1 \
                            or mixer.q_rank < 1 or mixer.kv_rank < 1:
                        raise ConfigError("latent attention sizes must be positive and 'rot_dim' even")
                else:
                    raise ConfigError(f"type {kind!r}; known: ['attention', 'latent_attention']")
                mlp = L.get("mlp")
                if mlp is not None:
                    if not isinstance(mlp, Mapping):
                        raise ConfigError("'mlp' must be null or an object")
                    mlp_kind = _take(mlp, "kind", str)
                    if mlp_kind == "dense":
                        mlp = DovisunDense(ff=_take(mlp, "ff", int))
                        if mlp.ff < 1:
                            raise ConfigError("'mlp.ff' must be positive")
                    elif mlp_kind == "moe":
                        router, expert = mlp.get("router") or {}, mlp.get("expert") or {}
                        mlp = DovisunExperts(experts=_take(router, "experts", int), top=_take(router, "top", int),
                                             ff=_take(expert, "ff", int))
                        if mlp.ff < 1 or not 1 <= mlp.top <= mlp.experts:
                            raise ConfigError(f"top = {mlp.top} of {mlp.experts} experts of size {mlp.ff}")
                    else:
                        raise ConfigError(f"'mlp.kind' = {mlp_kind!r}; known: ['dense', 'moe']")
            except ConfigError as e:
                raise ConfigError(f"{e} (layer {i})") from None
            layers.append(DovisunLayer(kind, mixer, mlp))
        loop = d.get("loop") or {}
        if not isinstance(loop, Mapping):
            raise ConfigError("config.json: key 'loop' must be an object")
        start, stop = _take(loop, "start", int, 0), _take(loop, "stop", int, 0)
        cfg = cls(architecture=_take(d, "architecture", str, "Dovisun"), vocab_size=_take(d, "vocab", int),
                  hidden_size=_take(d, "width", int), layers=tuple(layers), norm_eps=_take(norm, "eps", float),
                  embedding_scale=_take(emb, "scale", float, 1.0), logit_softcap=_take(d, "logit_softcap", float, 0.0),
                  loop_start=start, loop_stop=stop, loop_times=_take(loop, "times", int, 1),
                  has_loop=d.get("loop") is not None)
        if cfg.vocab_size < 1 or cfg.hidden_size < 1 or cfg.norm_eps < 0 or cfg.logit_softcap < 0:
            raise ConfigError("config.json: 'vocab' and 'width' must be positive, 'norm.eps' and 'logit_softcap' not negative")
        if not 0 <= start <= stop <= len(layers) or cfg.loop_times < 1:
            raise ConfigError(f"config.json: 'loop' = layers {start} .. {stop} - 1, {cfg.loop_times} times, of {len(layers)} layers")
        return cfg

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def loops(self) -> bool:
        """Whether a run of layers is passed at all (and so the embedding mixed in ahead of each pass)."""
        return self.loop_stop > self.loop_start


# ----------------------------------------------------------------------------------------- Kumudra

@dataclass(frozen=True)
class Llama3RotaryScaling:
    """Frequencies stretched by wavelength: pairs whose wavelength exceeds original/low turn ``factor`` times slower,
    those below original/high are kept, those between are blended linearly in original/wavelength."""
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class KumudraAttention:
    """The softmax half of a parallel mixer: grouped-query attention with biases, a partial rotation, a window."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int                     # keys a query sees, itself included; 0: all
    rot_dims: int                   # 0: no rotation
    rot_base: float
    rot_scaling: Optional[Llama3RotaryScaling]


@dataclass(frozen=True)
class KumudraTimeMix:
    """The recurrent half of a parallel mixer: token-shifted projections, a decay per key channel, a bonus."""
    heads: int
    dim: int
    rank: int                       # inner size of the decay's two-layer product where no checkpoint decides it


@dataclass(frozen=True)
class KumudraParallel:
    left: KumudraAttention
    right: KumudraTimeMix
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class KumudraGLA:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int


@dataclass(frozen=True)
class KumudraLightning:
    heads: int
    dim: int
    vdim: int
    decay: tuple                    # one per head


@dataclass(frozen=True)
class KumudraDense:
    ff: int


@dataclass(frozen=True)
class KumudraExperts:
    experts: int
    top: int
    ff: int
    scale: float


@dataclass(frozen=True)
class KumudraLayer:
    type: str                       # "parallel" | "gla" | "lightning"
    mixer: object
    mlp: object                     # KumudraDense | KumudraExperts | None


KUMUDRA_DEFAULT_RANK = 16           # what random weights are drawn with; a checkpoint's tensors have the rank they have


@dataclass(frozen=True)
class KumudraConfig:
    """Keys of a Kumudra config.json: layers listed one by one (a mixer of three kinds, a dense or routed feed-forward
    or none), several copies of the residual stream that every sublayer reads a mix of and writes back into
    (``streams``), a run of layers passed several times on the same tensors (``loop``), a multiplier on what joins the
    stream, a scale on the embedding; layer norms without a bias; the head is the embedding table."""
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple                   # of KumudraLayer
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    streams: int
    loop_start: int
    loop_stop: int
    loop_times: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KumudraConfig":
        norm, emb = d.get("norm") or {}, d.get("embedding") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(raw_layers):
            try:
                if not isinstance(L, Mapping):
                    raise ConfigError("a layer must be an object")
                kind, m = _take(L, "type", str), L.get("mixer")
                if not isinstance(m, Mapping):
                    raise ConfigError("no 'mixer' object")
                if kind == "parallel":
                    mixer = KumudraParallel(left=_kumudra_attention(m.get("left")), right=_kumudra_time_mix(m.get("right")),
                                            left_scale=_take(m, "left_scale", float, 1.0),
                                            right_scale=_take(m, "right_scale", float, 1.0))
                elif kind == "gla":
                    dim = _take(m, "dim", int)
                    mixer = KumudraGLA(heads=_take(m, "heads", int), dim=dim, vdim=_take(m, "vdim", int, dim),
                                       tau=_take(m, "tau", float, 1.0), rank=_take(m, "rank", int, KUMUDRA_DEFAULT_RANK))
                    if mixer.heads < 1 or dim < 1 or mixer.vdim < 1 or mixer.tau <= 0 or mixer.rank < 1:
                        raise ConfigError("gated linear attention: sizes and 'tau' must be positive")
                elif kind == "lightning":
                    dim, decay = _take(m, "dim", int), m.get("decay")
                    heads = _take(m, "heads", int)
                    if not isinstance(decay, (list, tuple)) or len(decay) != heads:
                        raise ConfigError(f"'decay' must list one number for each of the {heads} heads")
                    mixer = KumudraLightning(heads=heads, dim=dim, vdim=_take(m, "vdim", int, dim),
                                             decay=tuple(float(v) for v in decay))
                    if heads < 1 or dim < 1 or mixer.vdim < 1:
                        raise ConfigError("lightning attention: sizes must be positive")
                else:
                    raise ConfigError(f"type {kind!r}; known: ['gla', 'lightning', 'parallel']")
                mlp = L.get("mlp")
                if mlp is not None:
                    if not isinstance(mlp, Mapping):
                        raise ConfigError("'mlp' must be null or an object")
                    mlp_kind = _take(mlp, "kind", str)
                    if mlp_kind == "dense":
                        mlp = KumudraDense(ff=_take(mlp, "ff", int))
                        if mlp.ff < 1:
                            raise ConfigError("'mlp.ff' must be positive")
                    elif mlp_kind == "moe":
                        router, expert = mlp.get("router") or {}, mlp.get("expert") or {}
                        mlp = KumudraExperts(experts=_take(router, "experts", int), top=_take(router, "top", int),
                                             ff=_take(expert, "ff", int), scale=_take(router, "scale", float, 1.0))
                        if mlp.ff < 1 or not 1 <= mlp.top <= mlp.experts:
                            raise ConfigError(f"top = {mlp.top} of {mlp.experts} experts of size {mlp.ff}")
                    else:
                        raise ConfigError(f"'mlp.kind' = {mlp_kind!r}; known: ['dense', 'moe']")
            except ConfigError as e:
                raise ConfigError(f"{e} (layer {i})") from None
            layers.append(KumudraLayer(kind, mixer, mlp))
        loop = d.get("loop") or {}
        if not isinstance(loop, Mapping):
            raise ConfigError("config.json: key 'loop' must be an object")
        start, stop = _take(loop, "start", int, 0), _take(loop, "stop", int, 0)
        cfg = cls(architecture=_take(d, "architecture", str, "Kumudra"), vocab_size=_take(d, "vocab", int),
                  hidden_size=_take(d, "width", int), layers=tuple(layers), norm_eps=_take(norm, "eps", float),
                  embedding_scale=_take(emb, "scale", float, 1.0), residual_mult=_take(d, "residual_mult", float, 1.0),
                  streams=_take(d, "streams", int, 1), loop_start=start, loop_stop=stop,
                  loop_times=_take(loop, "times", int, 1))
        if cfg.vocab_size < 1 or cfg.hidden_size < 1 or cfg.norm_eps < 0 or cfg.streams < 1:
            raise ConfigError("config.json: 'vocab', 'width' and 'streams' must be positive, 'norm.eps' not negative")
        if not 0 <= start <= stop <= len(layers) or cfg.loop_times < 1:
            raise ConfigError(f"config.json: 'loop' = layers {start} .. {stop} - 1, {cfg.loop_times} times, of {len(layers)} layers")
        return cfg

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def run_order(self) -> list:
        """Layer indices in the order they run."""
        n, a, b = len(self.layers), self.loop_start, self.loop_stop
        if b <= a:
            return list(range(n))
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))


def _kumudra_attention(m) -> KumudraAttention:
    if not isinstance(m, Mapping):
        raise ConfigError("a parallel mixer needs a 'left' object")
    dim = _take(m, "dim", int)
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    sc = rot.get("scaling")
    scaling = None
    if sc is not None:
        if not isinstance(sc, Mapping):
            raise ConfigError("'rot.scaling' must be an object")
        scaling = Llama3RotaryScaling(factor=_take(sc, "factor", float), low=_take(sc, "low", float),
                                      high=_take(sc, "high", float), original=_take(sc, "original", float))
        if scaling.factor <= 0 or scaling.original <= 0 or scaling.low <= 0 or scaling.high <= 0:
            raise ConfigError("'rot.scaling': factor, low, high and original must be positive")
    a = KumudraAttention(heads=_take(m, "heads", int), kv_heads=_take(m, "kv_heads", int), dim=dim,
                         vdim=_take(m, "vdim", int, dim), scale=_take(m, "scale", float, dim ** -0.5),
                         window=_take(mask, "size", int, 0), rot_dims=_take(rot, "dims", int, 0),
                         rot_base=_take(rot, "base", float, 10000.0), rot_scaling=scaling)
    if a.heads < 1 or a.kv_heads < 1 or a.heads % a.kv_heads or dim < 1 or a.vdim < 1 or a.window < 0:
        raise ConfigError(f"{a.heads} heads over {a.kv_heads} kv heads of sizes {dim} and {a.vdim}, window {a.window}")
    if a.rot_dims < 0 or a.rot_dims % 2 or a.rot_dims > dim:
        raise ConfigError(f"'rot.dims' = {a.rot_dims} must be even and at most 'dim' = {dim}")
    return a


def _kumudra_time_mix(m) -> KumudraTimeMix:
    if not isinstance(m, Mapping):
        raise ConfigError("a parallel mixer needs a 'right' object")
    r = KumudraTimeMix(heads=_take(m, "heads", int), dim=_take(m, "dim", int),
                       rank=_take(m, "rank", int, KUMUDRA_DEFAULT_RANK))
    if r.heads < 1 or r.dim < 1 or r.rank < 1:
        raise ConfigError("time mixing: 'heads', 'dim' and 'rank' must be positive")
    return r
