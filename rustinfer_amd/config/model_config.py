"""Typed model configuration read from a model folder's ``config.json``.

Every size and constant of the model comes from here; no part of the engine
carries a size of its own.  Keys, defaults and meanings follow the reference's
``HfConfig`` / ``build_load_config`` (crates/infer-worker/src/bin/worker_main.rs:55-181,
:389-449) with the differences listed in ``LlamaConfig``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json (or launch file) that cannot be used."""


def _require(d: Dict[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d[key], key, typ, where)


def _typed(value, key: str, typ, where: str):
    if typ is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{where}: '{key}' must be an integer, got {value!r}")
        return int(value)
    if typ is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{where}: '{key}' must be a number, got {value!r}")
        return float(value)
    if typ is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"{where}: '{key}' must be true or false, got {value!r}")
        return value
    if typ is str:
        if not isinstance(value, str):
            raise ConfigError(f"{where}: '{key}' must be a string, got {value!r}")
        return value
    raise TypeError(typ)


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json.  Only ``rope_type == "llama3"`` rescales
    (crates/infer-worker/src/bin/worker_main.rs:393-404); the reference silently
    ignores other types, this engine refuses them."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> Optional["RopeScaling"]:
        rope_type = d.get("rope_type", d.get("type"))
        if rope_type is None:
            raise ConfigError(f"{where}: rope_scaling has no 'rope_type'")
        if rope_type == "default":
            return None
        if rope_type != "llama3":
            raise ConfigError(
                f"{where}: rope_scaling.rope_type {rope_type!r} is not supported "
                f"(supported: 'default', 'llama3')")
        w = where + ".rope_scaling"
        rs = RopeScaling(
            rope_type="llama3",
            factor=_require(d, "factor", float, w),
            low_freq_factor=_require(d, "low_freq_factor", float, w),
            high_freq_factor=_require(d, "high_freq_factor", float, w),
            original_max_position_embeddings=_require(
                d, "original_max_position_embeddings", int, w),
        )
        if rs.factor <= 0:
            raise ConfigError(f"{w}: factor must be > 0")
        if rs.high_freq_factor <= rs.low_freq_factor:
            raise ConfigError(f"{w}: high_freq_factor must exceed low_freq_factor")
        if rs.low_freq_factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError(f"{w}: low_freq_factor and original_max_position_embeddings must be > 0")
        return rs


class ModelConfig:
    """Base of every architecture's typed configuration.

    A subclass is a dataclass with ``from_dict`` (parse + validate config.json)
    and ``to_dict`` (what the random-weights mode writes back as config.json).
    """

    architecture: str = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


DEFAULT_EOS_IDS = (128001, 128008, 128009)  # worker_main.rs:327-373 fallback
MAX_HEAD_DIM = 256      # the attention kernel that takes any head size keeps one head's features in a block of this many lanes


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    """Dense Llama-3 decoder (``LlamaForCausalLM``).

    Differences from the reference's reader: ``tie_word_embeddings`` is read (the
    reference decides by the presence of ``lm_head.weight``,
    crates/infer-worker/src/models/decoder.rs:245-262) and cross-checked by the
    loader; ``hidden_act`` must be ``silu`` and ``attention_bias``/``mlp_bias``
    must be false if present, because this architecture's parts have neither.
    """

    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    vocab_size: int = 0
    max_position_embeddings: int = 4096     # worker_main.rs:173-175
    rms_norm_eps: float = 1e-5              # worker_main.rs:176-178
    rope_theta: float = 10000.0             # worker_main.rs:179-181
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    eos_token_ids: tuple = DEFAULT_EOS_IDS
    architecture: str = "LlamaForCausalLM"

    # derived sizes (reference: ModelDims, crates/infer-worker/src/domain/model.rs:12-54)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def qkv_dim(self) -> int:
        return self.q_dim + 2 * self.kv_dim

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "LlamaConfig":
        d = dict(d)
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        if heads <= 0:
            raise ConfigError(f"{where}: num_attention_heads must be > 0")
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size {hidden} is not divisible by "
                    f"num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads          # worker_main.rs:390-392
        head_dim = _typed(head_dim, "head_dim", int, where)
        rs = d.get("rope_scaling")
        if rs is not None and not isinstance(rs, dict):
            raise ConfigError(f"{where}: rope_scaling must be an object")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids = DEFAULT_EOS_IDS
        elif isinstance(eos, list):
            eos_ids = tuple(_typed(e, "eos_token_id", int, where) for e in eos)
        else:
            eos_ids = (_typed(eos, "eos_token_id", int, where),)
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"{where}: hidden_act {act!r} is not supported (only 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"{where}: {key}=true is not supported by this architecture")
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=_require(d, "intermediate_size", int, where),
            num_hidden_layers=_require(d, "num_hidden_layers", int, where),
            num_attention_heads=heads,
            num_key_value_heads=_require(d, "num_key_value_heads", int, where),
            head_dim=head_dim,
            vocab_size=_require(d, "vocab_size", int, where),
            max_position_embeddings=_typed(d.get("max_position_embeddings", 4096),
                                           "max_position_embeddings", int, where),
            rms_norm_eps=_typed(d.get("rms_norm_eps", 1e-5), "rms_norm_eps", float, where),
            rope_theta=_typed(d.get("rope_theta", 10000.0), "rope_theta", float, where),
            rope_scaling=RopeScaling.from_dict(rs, where) if rs is not None else None,
            tie_word_embeddings=_typed(d.get("tie_word_embeddings", False),
                                       "tie_word_embeddings", bool, where),
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        for key in ("hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim",
                    "vocab_size", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{where}: {key} must be > 0, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for rotary pairs")
        if self.head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: head_dim {self.head_dim} exceeds {MAX_HEAD_DIM}, the largest head "
                              f"the attention kernels take")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"{where}: rms_norm_eps must be > 0")
        if not (self.rope_theta > 0):
            raise ConfigError(f"{where}: rope_theta must be > 0")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "eos_token_id": list(self.eos_token_ids),
        }
        if self.rope_scaling is not None:
            d["rope_scaling"] = asdict(self.rope_scaling)
        return d


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    # generation_config.json's eos ids win over config.json's (worker_main.rs:327-373)
    gen = os.path.join(model_dir, "generation_config.json")
    if os.path.isfile(gen):
        try:
            with open(gen, "r", encoding="utf-8") as f:
                g = json.load(f)
            if isinstance(g, dict) and g.get("eos_token_id") is not None:
                d["eos_token_id"] = g["eos_token_id"]
        except (OSError, json.JSONDecodeError):
            pass
    return d


# ---------------------------------------------------------------------------
# Tedelix: a decoder whose layers are listed one by one in config.json
# ---------------------------------------------------------------------------
def _obj(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: '{key}' must be an object")
    return v


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Mixer ``attention``: grouped softmax attention in a sliding window, rotary angles on the
    first ``rot_dims`` features of queries and keys, values turned by their position."""
    heads: int
    kv_heads: int
    dim: int                  # size of a query / key head
    vdim: int                 # size of a value head
    window: int               # a query sees itself and the window - 1 positions before it
    rot_base: float
    rot_dims: int
    scale: float
    kind: str = "attention"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "WindowAttentionSpec":
        rot, mask = _obj(m, "rot", where), _obj(m, "mask", where)
        s = WindowAttentionSpec(
            heads=_require(m, "heads", int, where), kv_heads=_require(m, "kv_heads", int, where),
            dim=_require(m, "dim", int, where), vdim=_require(m, "vdim", int, where),
            window=_require(mask, "size", int, where + ".mask"),
            rot_base=_require(rot, "base", float, where + ".rot"), rot_dims=_require(rot, "dims", int, where + ".rot"),
            scale=_require(m, "scale", float, where))
        if min(s.heads, s.kv_heads, s.dim, s.vdim, s.window) <= 0 or s.heads % s.kv_heads:
            raise ConfigError(f"{where}: heads, kv_heads, dim, vdim and mask.size must be > 0 and heads a multiple of kv_heads")
        if s.rot_dims <= 0 or s.rot_dims % 2 or s.rot_dims > s.dim or s.vdim % 2 or not s.rot_base > 0:
            raise ConfigError(f"{where}: rot.dims must be even and within dim, vdim even, rot.base > 0")
        if s.dim > MAX_HEAD_DIM or s.vdim > MAX_HEAD_DIM or s.heads // s.kv_heads > 32:
            raise ConfigError(f"{where}: heads of more than {MAX_HEAD_DIM} features or more than 32 query heads a "
                              f"key/value head are beyond the attention kernels")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "mask": {"size": self.window}, "rot": {"base": self.rot_base, "dims": self.rot_dims},
                "scale": self.scale}


@dataclass(frozen=True)
class LightningSpec:
    """Mixer ``lightning``: linear attention with one fixed decay for each head."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    kind: str = "lightning"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "LightningSpec":
        decay = m.get("decay")
        if not isinstance(decay, list):
            raise ConfigError(f"{where}: 'decay' must be a list with one number for each head")
        s = LightningSpec(heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where),
                          vdim=_require(m, "vdim", int, where),
                          decay=tuple(_typed(x, "decay", float, where) for x in decay))
        if min(s.heads, s.dim, s.vdim) <= 0 or len(s.decay) != s.heads:
            raise ConfigError(f"{where}: heads, dim, vdim must be > 0 and 'decay' hold {s.heads} numbers")
        if s.dim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: dim {s.dim} exceeds {MAX_HEAD_DIM}, the most key rows the state kernel takes")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class GeneralDeltaSpec:
    """Mixer ``general_delta``: a generalized delta rule with a decay and a removal rate for each
    key channel; keys, values and readers all of size ``dim``."""
    heads: int
    dim: int
    # rows of the first of the two matrices behind the decay: config.json does not give it, the
    # checkpoint's tensor does (``TedelixConfig.complete_from_checkpoint``); None: not known yet
    decay_rank: Optional[int] = None
    kind: str = "general_delta"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "GeneralDeltaSpec":
        s = GeneralDeltaSpec(heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where))
        if s.heads <= 0 or s.dim <= 0 or s.dim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: heads must be > 0 and dim in [1, {MAX_HEAD_DIM}]")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim}


TEDELIX_MIXERS = {"attention": WindowAttentionSpec, "lightning": LightningSpec, "general_delta": GeneralDeltaSpec}


@dataclass(frozen=True)
class TedelixLayer:
    mixer: Any                       # one of the specs above
    ff: Optional[int] = None         # width of the dense feed-forward, None: the layer has none

    @property
    def type(self) -> str:
        return self.mixer.kind


@dataclass(frozen=True)
class TedelixConfig(ModelConfig):
    """``{"architecture": "Tedelix", "vocab", "width", "norm": {"eps"}, "logit_scale",
    "logit_softcap", "layers": [{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}]}``.
    Every layer is parallel (one norm; mixer and feed-forward read its output); the head shares
    the embedding table; the model has no end-of-sequence token of its own."""

    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    layers: tuple = ()
    eos_token_ids: tuple = ()
    architecture: str = "Tedelix"

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "TedelixConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(layers_in):
            w = f"{where}.layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{w}: must be an object")
            kind = _require(entry, "type", str, w)
            if kind not in TEDELIX_MIXERS:
                raise ConfigError(f"{w}: unknown mixer type {kind!r} (known: {', '.join(sorted(TEDELIX_MIXERS))})")
            mixer = TEDELIX_MIXERS[kind].from_dict(_obj(entry, "mixer", w), w + ".mixer")
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{w}: 'mlp' must be null or an object of kind 'dense'")
                ff = _require(mlp, "ff", int, w + ".mlp")
                if ff <= 0:
                    raise ConfigError(f"{w}.mlp: ff must be > 0")
            layers.append(TedelixLayer(mixer, ff))
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where) for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab_size=_require(d, "vocab", int, where), hidden_size=_require(d, "width", int, where),
                  norm_eps=_require(_obj(d, "norm", where), "eps", float, where + ".norm"),
                  logit_scale=_typed(d.get("logit_scale", 1.0), "logit_scale", float, where),
                  logit_softcap=_typed(d.get("logit_softcap", 0.0), "logit_softcap", float, where),
                  layers=tuple(layers), eos_token_ids=eos_ids)
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or not cfg.norm_eps > 0 or cfg.logit_softcap < 0:
            raise ConfigError(f"{where}: vocab and width must be > 0, norm.eps > 0, logit_softcap >= 0")
        return cfg

    def complete_from_checkpoint(self, shapes: Dict[str, Any]) -> "TedelixConfig":
        """The sizes that only a tensor's shape gives (``shapes``: checkpoint name -> shape): the
        rank of each delta-rule layer's decay input, the rows of ``l<i>.mix.w1``."""
        layers = []
        for i, layer in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.w1")
            if isinstance(layer.mixer, GeneralDeltaSpec) and shape is not None and len(shape) == 2:
                layer = TedelixLayer(GeneralDeltaSpec(layer.mixer.heads, layer.mixer.dim, int(shape[0])), layer.ff)
            layers.append(layer)
        return TedelixConfig(**{**self.__dict__, "layers": tuple(layers)})

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
            "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap,
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


# ---------------------------------------------------------------------------
# Belorax: layers listed one by one; the norm sits on each sub-layer's output
# ---------------------------------------------------------------------------
@dataclass(frozen=True)
class YarnScaling:
    """Rotary frequencies stretched band by band: pairs that turn more than ``fast`` times over
    ``original`` positions keep their frequency, pairs that turn fewer than ``slow`` times have it
    divided by ``factor``, a linear ramp over the pair index between; cos and sin are multiplied by
    ``0.1 ln(factor) + 1``."""
    factor: float
    original: int
    fast: float
    slow: float

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> "YarnScaling":
        s = YarnScaling(factor=_require(d, "factor", float, where), original=_require(d, "original", int, where),
                        fast=_require(d, "fast", float, where), slow=_require(d, "slow", float, where))
        if not (s.factor > 0 and s.original > 0 and s.fast > 0 and s.slow > 0):
            raise ConfigError(f"{where}: factor, original, fast and slow must be > 0")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


def _rot_of(m: Dict[str, Any], where: str):
    """(base, dims, scaling) of a mixer's 'rot' object."""
    rot = _obj(m, "rot", where)
    base, dims = _require(rot, "base", float, where + ".rot"), _require(rot, "dims", int, where + ".rot")
    sc = rot.get("scaling")
    if sc is not None and not isinstance(sc, dict):
        raise ConfigError(f"{where}.rot: 'scaling' must be an object or null")
    if not base > 0 or dims <= 0 or dims % 2:
        raise ConfigError(f"{where}.rot: base must be > 0 and dims even and > 0")
    return base, dims, (YarnScaling.from_dict(sc, where + ".rot.scaling") if sc is not None else None)


def _rot_dict(base, dims, scaling=None) -> Dict[str, Any]:
    d = {"base": base, "dims": dims}
    if scaling is not None:
        d["scaling"] = scaling.to_dict()
    return d


@dataclass(frozen=True)
class NormedAttentionSpec:
    """Mixer ``attention``: grouped softmax attention over all earlier positions, queries and keys
    normed head by head, no rotation, a query temperature that grows with the position's logarithm;
    ``kv_from``: the layer whose keys and values this one reads instead of making its own."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float = 0.0
    temp_every: int = 0           # 0: no temperature
    kv_from: Optional[int] = None
    kind: str = "attention"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "NormedAttentionSpec":
        temp = m.get("q_temp")
        if temp is not None and not isinstance(temp, dict):
            raise ConfigError(f"{where}: 'q_temp' must be an object or null")
        kv_from = m.get("kv_from")
        s = NormedAttentionSpec(
            heads=_require(m, "heads", int, where), kv_heads=_require(m, "kv_heads", int, where),
            dim=_require(m, "dim", int, where), vdim=_require(m, "vdim", int, where),
            scale=_require(m, "scale", float, where),
            temp_coef=_require(temp, "coef", float, where + ".q_temp") if temp is not None else 0.0,
            temp_every=_require(temp, "every", int, where + ".q_temp") if temp is not None else 0,
            kv_from=_typed(kv_from, "kv_from", int, where) if kv_from is not None else None)
        if min(s.heads, s.kv_heads, s.dim, s.vdim) <= 0 or s.heads % s.kv_heads:
            raise ConfigError(f"{where}: heads, kv_heads, dim and vdim must be > 0 and heads a multiple of kv_heads")
        if temp is not None and s.temp_every <= 0:
            raise ConfigError(f"{where}.q_temp: every must be > 0")
        if s.dim > MAX_HEAD_DIM or s.vdim > MAX_HEAD_DIM or s.heads // s.kv_heads > 32:
            raise ConfigError(f"{where}: heads of more than {MAX_HEAD_DIM} features or more than 32 query heads a "
                              f"key/value head are beyond the attention kernels")
        return s

    def to_dict(self) -> Dict[str, Any]:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.temp_every > 0:
            d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Mixer ``latent_attention``: keys and values of all heads come from one latent vector of
    ``kv_rank`` features a token, plus one rotated key part of ``rot_dim`` features shared by the heads."""
    heads: int
    dim: int                 # unrotated query/key features a head
    rot_dim: int             # rotated query/key features a head
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[YarnScaling] = None
    kind: str = "latent_attention"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "LatentAttentionSpec":
        base, dims, scaling = _rot_of(m, where)
        s = LatentAttentionSpec(
            heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where),
            rot_dim=_require(m, "rot_dim", int, where), vdim=_require(m, "vdim", int, where),
            kv_rank=_require(m, "kv_rank", int, where), scale=_require(m, "scale", float, where),
            rot_base=base, rot_dims=dims, rot_scaling=scaling)
        if min(s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank) <= 0:
            raise ConfigError(f"{where}: heads, dim, rot_dim, vdim and kv_rank must be > 0")
        if s.rot_dims > s.rot_dim:
            raise ConfigError(f"{where}: rot.dims {s.rot_dims} exceeds rot_dim {s.rot_dim}")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": _rot_dict(self.rot_base, self.rot_dims, self.rot_scaling)}


@dataclass(frozen=True)
class RetentionSpec:
    """Mixer ``retention``: linear attention with one fixed decay a head, rotated queries and keys."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[YarnScaling] = None
    kind: str = "retention"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "RetentionSpec":
        decay = m.get("decay")
        if not isinstance(decay, list):
            raise ConfigError(f"{where}: 'decay' must be a list with one number for each head")
        base, dims, scaling = _rot_of(m, where)
        s = RetentionSpec(heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where),
                          vdim=_require(m, "vdim", int, where),
                          decay=tuple(_typed(x, "decay", float, where) for x in decay), rot_base=base, rot_dims=dims,
                          rot_scaling=scaling)
        if min(s.heads, s.dim, s.vdim) <= 0 or len(s.decay) != s.heads:
            raise ConfigError(f"{where}: heads, dim, vdim must be > 0 and 'decay' hold {s.heads} numbers")
        if s.dim > MAX_HEAD_DIM or s.rot_dims > s.dim:
            raise ConfigError(f"{where}: dim {s.dim} exceeds {MAX_HEAD_DIM}, the most key rows the state kernel takes, "
                              f"or rot.dims {s.rot_dims} exceeds dim")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay),
                "rot": _rot_dict(self.rot_base, self.rot_dims, self.rot_scaling)}


BELORAX_MIXERS = {"attention": NormedAttentionSpec, "latent_attention": LatentAttentionSpec, "retention": RetentionSpec}


@dataclass(frozen=True)
class FeedForwardSpec:
    """``dense``: one gated feed-forward of width ``ff``.  ``moe``: ``experts`` of them of width ``ff``
    each, of which a token uses ``top``."""
    kind: str
    ff: int
    experts: int = 0
    top: int = 0

    @staticmethod
    def from_dict(mlp: Dict[str, Any], where: str) -> "FeedForwardSpec":
        kind = _require(mlp, "kind", str, where)
        if kind == "dense":
            s = FeedForwardSpec("dense", _require(mlp, "ff", int, where))
        elif kind == "moe":
            router = _obj(mlp, "router", where)
            s = FeedForwardSpec("moe", _require(_obj(mlp, "expert", where), "ff", int, where + ".expert"),
                                _require(router, "experts", int, where + ".router"), _require(router, "top", int, where + ".router"))
            if not (0 < s.top <= s.experts):
                raise ConfigError(f"{where}.router: need 0 < top <= experts")
        else:
            raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: dense, moe)")
        if s.ff <= 0:
            raise ConfigError(f"{where}: ff must be > 0")
        return s

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class BeloraxLayer:
    mixer: Any                                # one of the specs above
    mlp: Optional[FeedForwardSpec] = None     # None: the layer has no feed-forward

    @property
    def type(self) -> str:
        return self.mixer.kind


@dataclass(frozen=True)
class BeloraxConfig(ModelConfig):
    """``{"architecture": "Belorax", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"},
    "residual_mult", "layers": [{"type", "mixer": {...}, "mlp": {...} | null}]}``.  Each sub-layer
    reads the residual stream itself and its output is normed before it is added, times
    ``residual_mult``; the head has a matrix of its own; no end-of-sequence token of its own."""

    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    residual_mult: float = 1.0
    layers: tuple = ()
    eos_token_ids: tuple = ()
    architecture: str = "Belorax"

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "BeloraxConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(layers_in):
            w = f"{where}.layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{w}: must be an object")
            kind = _require(entry, "type", str, w)
            if kind not in BELORAX_MIXERS:
                raise ConfigError(f"{w}: unknown mixer type {kind!r} (known: {', '.join(sorted(BELORAX_MIXERS))})")
            mixer = BELORAX_MIXERS[kind].from_dict(_obj(entry, "mixer", w), w + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None and not isinstance(mlp, dict):
                raise ConfigError(f"{w}: 'mlp' must be null or an object")
            layers.append(BeloraxLayer(mixer, FeedForwardSpec.from_dict(mlp, w + ".mlp") if mlp is not None else None))
        for i, layer in enumerate(layers):
            j = getattr(layer.mixer, "kv_from", None)
            if j is None:
                continue
            w = f"{where}.layers[{i}].mixer"
            if not (0 <= j < i) or not isinstance(layers[j].mixer, NormedAttentionSpec) or layers[j].mixer.kv_from is not None:
                raise ConfigError(f"{w}: kv_from must name an earlier attention layer that has keys and values of its own")
            a, b = layer.mixer, layers[j].mixer
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise ConfigError(f"{w}: kv_heads, dim and vdim must equal those of layer {j}, whose keys and values it reads")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where) for e in (eos if isinstance(eos, list) else [eos]))
        emb = d.get("embedding")
        if emb is not None and not isinstance(emb, dict):
            raise ConfigError(f"{where}: 'embedding' must be an object")
        cfg = cls(vocab_size=_require(d, "vocab", int, where), hidden_size=_require(d, "width", int, where),
                  norm_eps=_require(_obj(d, "norm", where), "eps", float, where + ".norm"),
                  embedding_scale=_typed(emb.get("scale", 1.0), "scale", float, where + ".embedding") if emb else 1.0,
                  residual_mult=_typed(d.get("residual_mult", 1.0), "residual_mult", float, where),
                  layers=tuple(layers), eos_token_ids=eos_ids)
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or not cfg.norm_eps > 0:
            raise ConfigError(f"{where}: vocab and width must be > 0, norm.eps > 0")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
            "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
            "residual_mult": self.residual_mult,
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


# ---------------------------------------------------------------------------
# Pilavik: a norm before and after every sub-layer, a gate on each sub-layer's result, a stretch
# of layers that runs several times
# ---------------------------------------------------------------------------
@dataclass(frozen=True)
class GatedDeltaSpec:
    """Mixer ``delta``: the gated delta rule on ``heads`` value heads of ``vdim`` that share ``kv_heads``
    query/key heads of ``dim``; q, k, v pass a causal convolution of ``conv`` taps."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    kind: str = "delta"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "GatedDeltaSpec":
        s = GatedDeltaSpec(heads=_require(m, "heads", int, where), kv_heads=_require(m, "kv_heads", int, where),
                           dim=_require(m, "dim", int, where), vdim=_require(m, "vdim", int, where),
                           conv=_require(m, "conv", int, where))
        if min(s.heads, s.kv_heads, s.dim, s.vdim, s.conv) <= 0 or s.heads % s.kv_heads:
            raise ConfigError(f"{where}: heads, kv_heads, dim, vdim and conv must be > 0 and heads a multiple of kv_heads")
        if s.dim > MAX_HEAD_DIM or s.conv > 8:
            raise ConfigError(f"{where}: dim {s.dim} exceeds {MAX_HEAD_DIM}, the most key rows the state kernel takes, "
                              f"or conv {s.conv} exceeds the 8 taps the convolution kernel takes")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class SinkLatentAttentionSpec:
    """Mixer ``latent_attention`` of this design: keys and values from one latent a token (see
    ``LatentAttentionSpec``), an unstretched interleaved rotation, a sliding window of ``window`` positions
    (None: all) and a learned sink a head in the softmax's denominator."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int] = None
    kind: str = "latent_attention"

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "SinkLatentAttentionSpec":
        base, dims, scaling = _rot_of(m, where)
        if scaling is not None:
            raise ConfigError(f"{where}.rot: this design's rotation is not stretched")
        mask = m.get("mask")
        if mask is not None and not isinstance(mask, dict):
            raise ConfigError(f"{where}: 'mask' must be an object or null")
        window = _require(mask, "size", int, where + ".mask") if mask is not None else None
        s = SinkLatentAttentionSpec(
            heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where),
            rot_dim=_require(m, "rot_dim", int, where), vdim=_require(m, "vdim", int, where),
            kv_rank=_require(m, "kv_rank", int, where), scale=_require(m, "scale", float, where),
            rot_base=base, rot_dims=dims, window=window)
        if min(s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank) <= 0 or (window is not None and window <= 0):
            raise ConfigError(f"{where}: heads, dim, rot_dim, vdim, kv_rank and mask.size must be > 0")
        if s.rot_dims > s.rot_dim:
            raise ConfigError(f"{where}: rot.dims {s.rot_dims} exceeds rot_dim {s.rot_dim}")
        return s

    def to_dict(self) -> Dict[str, Any]:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale, "rot": _rot_dict(self.rot_base, self.rot_dims)}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


PILAVIK_MIXERS = {"delta": GatedDeltaSpec, "latent_attention": SinkLatentAttentionSpec}


@dataclass(frozen=True)
class PilavikFeedForwardSpec:
    """``dense``: one feed-forward of width ``ff`` (biases, an activation that norms powers).  ``moe``:
    ``experts`` gated feed-forwards of width ``ff`` of which a token uses ``top``, weights times
    ``router_scale``, and a shared one of width ``shared_ff`` (0: none) for every token."""
    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    shared_ff: int = 0

    @staticmethod
    def from_dict(mlp: Dict[str, Any], where: str) -> "PilavikFeedForwardSpec":
        kind = _require(mlp, "kind", str, where)
        if kind == "dense":
            s = PilavikFeedForwardSpec("dense", _require(mlp, "ff", int, where))
        elif kind == "moe":
            router = _obj(mlp, "router", where)
            shared = mlp.get("shared")
            if shared is not None and not isinstance(shared, dict):
                raise ConfigError(f"{where}: 'shared' must be an object or null")
            s = PilavikFeedForwardSpec(
                "moe", _require(_obj(mlp, "expert", where), "ff", int, where + ".expert"),
                _require(router, "experts", int, where + ".router"), _require(router, "top", int, where + ".router"),
                _typed(router.get("scale", 1.0), "scale", float, where + ".router"),
                _require(shared, "ff", int, where + ".shared") if shared is not None else 0)
            if not (0 < s.top <= s.experts) or s.experts > 512 or s.shared_ff < 0:
                raise ConfigError(f"{where}: need 0 < top <= experts <= 512 and shared.ff >= 0")
        else:
            raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: dense, moe)")
        if s.ff <= 0:
            raise ConfigError(f"{where}: ff must be > 0")
        return s

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        d = {"kind": "moe", "expert": {"ff": self.ff},
             "router": {"experts": self.experts, "top": self.top, "scale": self.router_scale}}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class PilavikLayer:
    mixer: Any                                       # one of the specs above
    mlp: Optional[PilavikFeedForwardSpec] = None     # None: the layer has no feed-forward

    @property
    def type(self) -> str:
        return self.mixer.kind


@dataclass(frozen=True)
class PilavikConfig(ModelConfig):
    """``{"architecture": "Pilavik", "vocab", "width", "norm": {"eps"}, "layers": [{"type", "mixer": {...},
    "mlp": {...} | null}], "loop": {"start", "stop", "times"} | absent}``.  Layers ``start .. stop - 1`` run
    ``times`` times in a row with the same weights, each pass on a cache or state of its own; the head has
    a matrix of its own; no end-of-sequence token of its own."""

    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    layers: tuple = ()
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    has_loop: bool = False       # config.json has a 'loop' (the checkpoint then has the passes' vectors)
    eos_token_ids: tuple = ()
    architecture: str = "Pilavik"

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "PilavikConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(layers_in):
            w = f"{where}.layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{w}: must be an object")
            kind = _require(entry, "type", str, w)
            if kind not in PILAVIK_MIXERS:
                raise ConfigError(f"{w}: unknown mixer type {kind!r} (known: {', '.join(sorted(PILAVIK_MIXERS))})")
            mixer = PILAVIK_MIXERS[kind].from_dict(_obj(entry, "mixer", w), w + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None and not isinstance(mlp, dict):
                raise ConfigError(f"{w}: 'mlp' must be null or an object")
            layers.append(PilavikLayer(mixer, PilavikFeedForwardSpec.from_dict(mlp, w + ".mlp") if mlp is not None else None))
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError(f"{where}: 'loop' must be an object or null")
            w = where + ".loop"
            start, stop, times = _require(loop, "start", int, w), _require(loop, "stop", int, w), _require(loop, "times", int, w)
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"{w}: need 0 <= start <= stop <= {len(layers)} layers and times >= 1")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where) for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab_size=_require(d, "vocab", int, where), hidden_size=_require(d, "width", int, where),
                  norm_eps=_require(_obj(d, "norm", where), "eps", float, where + ".norm"),
                  layers=tuple(layers), loop_start=start, loop_stop=stop, loop_times=times, has_loop=loop is not None,
                  eos_token_ids=eos_ids)
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or not cfg.norm_eps > 0:
            raise ConfigError(f"{where}: vocab and width must be > 0, norm.eps > 0")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
            "norm": {"eps": self.norm_eps},
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers]}
        if self.has_loop:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


# ---------------------------------------------------------------------------
# Debuzen: pre-norm layers with a norm in groups and a token shift in front of the mixer; mixers that are
# two sub-mixers side by side (attention and a recurrence) or gated linear attention; a stretch of
# layers that runs several times behind a product over the stream and the embedded rows
# ---------------------------------------------------------------------------
DEFAULT_LOW_RANK = 16     # rows of the first of two matrices that make a decay's or a gate's input, where no checkpoint says


def _mask_of(m: Dict[str, Any], where: str):
    """(size, keep_first) of a mixer's 'mask' object."""
    mask = _obj(m, "mask", where)
    size = _require(mask, "size", int, where + ".mask")
    keep = _typed(mask.get("keep_first", 0), "keep_first", int, where + ".mask")
    if size <= 0 or keep < 0:
        raise ConfigError(f"{where}.mask: size must be > 0 and keep_first >= 0")
    return size, keep


@dataclass(frozen=True)
class MaskedAttentionSpec:
    """The attention half of a mixer of two: grouped heads (keys of ``dim``, values of ``vdim``), a rotation
    over the first ``rot_dims`` features, a sliding window of ``window`` positions behind which the first
    ``keep_first`` positions of a sequence stay in sight."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int
    rot_base: float
    rot_dims: int

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "MaskedAttentionSpec":
        base, dims, scaling = _rot_of(m, where)
        if scaling is not None:
            raise ConfigError(f"{where}.rot: this design's rotation is not stretched")
        size, keep = _mask_of(m, where)
        s = MaskedAttentionSpec(heads=_require(m, "heads", int, where), kv_heads=_require(m, "kv_heads", int, where),
                                dim=_require(m, "dim", int, where), vdim=_require(m, "vdim", int, where),
                                scale=_require(m, "scale", float, where), window=size, keep_first=keep,
                                rot_base=base, rot_dims=dims)
        if min(s.heads, s.kv_heads, s.dim, s.vdim) <= 0 or s.heads % s.kv_heads:
            raise ConfigError(f"{where}: heads, kv_heads, dim and vdim must be > 0 and heads a multiple of kv_heads")
        if s.rot_dims > s.dim or max(s.dim, s.vdim) > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: rot.dims {s.rot_dims} exceeds dim {s.dim}, or a head exceeds {MAX_HEAD_DIM} features")
        return s

    def to_dict(self) -> Dict[str, Any]:
        mask = {"size": self.window}
        if self.keep_first:
            mask["keep_first"] = self.keep_first
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "mask": mask, "rot": _rot_dict(self.rot_base, self.rot_dims)}


@dataclass(frozen=True)
class ChannelDeltaSpec:
    """The gated delta rule with a decay for every key channel; the decay's and the gate's inputs come through
    two matrices each, whose inner sizes (``decay_rank``, ``gate_rank``) the checkpoint's shapes give."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int = DEFAULT_LOW_RANK
    gate_rank: int = DEFAULT_LOW_RANK

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "ChannelDeltaSpec":
        s = ChannelDeltaSpec(heads=_require(m, "heads", int, where), kv_heads=_require(m, "kv_heads", int, where),
                             dim=_require(m, "dim", int, where), vdim=_require(m, "vdim", int, where),
                             conv=_require(m, "conv", int, where),
                             decay_rank=_typed(m.get("decay_rank", DEFAULT_LOW_RANK), "decay_rank", int, where),
                             gate_rank=_typed(m.get("gate_rank", DEFAULT_LOW_RANK), "gate_rank", int, where))
        if min(s.heads, s.kv_heads, s.dim, s.vdim, s.conv, s.decay_rank, s.gate_rank) <= 0 or s.heads % s.kv_heads:
            raise ConfigError(f"{where}: every size must be > 0 and heads a multiple of kv_heads")
        if s.dim > MAX_HEAD_DIM or s.conv > 8:
            raise ConfigError(f"{where}: dim {s.dim} exceeds {MAX_HEAD_DIM} or conv {s.conv} exceeds 8 taps")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class StateSpaceSpec:
    """A state-space mixer in its recurrent form: ``heads`` heads of ``vdim`` over a state of ``state`` rows,
    inputs shared by ``groups`` groups of heads, a convolution of ``conv`` taps, an output norm in
    ``norm_groups`` parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @staticmethod
    def from_dict(m: Dict[str, Any], where: str) -> "StateSpaceSpec":
        s = StateSpaceSpec(heads=_require(m, "heads", int, where), vdim=_require(m, "vdim", int, where),
                           state=_require(m, "state", int, where), groups=_require(m, "groups", int, where),
                           conv=_require(m, "conv", int, where), norm_groups=_require(m, "norm_groups", int, where))
        if min(s.heads, s.vdim, s.state, s.groups, s.conv, s.norm_groups) <= 0 or s.heads % s.groups \
                or (s.heads * s.vdim) % s.norm_groups:
            raise ConfigError(f"{where}: every size must be > 0, heads a multiple of groups, heads * vdim of norm_groups")
        if s.state > MAX_HEAD_DIM or s.conv > 8:
            raise ConfigError(f"{where}: state {s.state} exceeds {MAX_HEAD_DIM} or conv {s.conv} exceeds 8 taps")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class TwoMixerSpec:
    """Mixers ``parallel`` (attention with sigmoid weights and kept first positions beside the channel-gated
    delta rule) and ``parallel_2`` (softmax attention with a sink beside a state-space mixer): both halves read
    the same rows, and the result is ``left_scale * left + right_scale * right``.  A mask's ``keep_first`` is
    honoured in either (absent: none)."""
    kind: str
    left: MaskedAttentionSpec
    right: Any
    left_scale: float
    right_scale: float

    @staticmethod
    def from_dict(kind: str, m: Dict[str, Any], where: str) -> "TwoMixerSpec":
        right_cls = ChannelDeltaSpec if kind == "parallel" else StateSpaceSpec
        s = TwoMixerSpec(kind, MaskedAttentionSpec.from_dict(_obj(m, "left", where), where + ".left"),
                         right_cls.from_dict(_obj(m, "right", where), where + ".right"),
                         _require(m, "left_scale", float, where), _require(m, "right_scale", float, where))
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class GatedLinearSpec:
    """Mixer ``gla``: gated linear attention, a decay ``sigmoid(.)^(1 / tau)`` for every key channel whose input
    comes through two matrices (inner size ``decay_rank``, from the checkpoint's shapes)."""
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = DEFAULT_LOW_RANK
    kind: str = "gla"

    @staticmethod
    def from_dict(kind: str, m: Dict[str, Any], where: str) -> "GatedLinearSpec":
        s = GatedLinearSpec(heads=_require(m, "heads", int, where), dim=_require(m, "dim", int, where),
                            vdim=_require(m, "vdim", int, where), tau=_require(m, "tau", float, where),
                            decay_rank=_typed(m.get("decay_rank", DEFAULT_LOW_RANK), "decay_rank", int, where))
        if min(s.heads, s.dim, s.vdim, s.decay_rank) <= 0 or not s.tau > 0 or s.dim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: heads, dim, vdim and tau must be > 0 and dim at most {MAX_HEAD_DIM}")
        return s

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


DEBUZEN_MIXERS = {"parallel": TwoMixerSpec, "parallel_2": TwoMixerSpec, "gla": GatedLinearSpec}


@dataclass(frozen=True)
class DebuzenLayer:
    mixer: Any                    # TwoMixerSpec or GatedLinearSpec
    ff: Optional[int] = None      # width of the gated feed-forward; None: the layer has none

    @property
    def type(self) -> str:
        return self.mixer.kind


@dataclass(frozen=True)
class DebuzenConfig(ModelConfig):
    """``{"architecture": "Debuzen", "vocab", "width", "norm": {"eps", "groups"}, "logit_softcap", "layers":
    [{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}], "loop": {"start", "stop", "times"} |
    absent}``.  Every norm works in ``norm.groups`` equal parts of a row.  Layers ``start .. stop - 1`` run
    ``times`` times in a row with the same weights, each pass on a cache and state of its own, behind a
    product of the stream and the embedded rows; the head has a matrix of its own."""

    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    norm_groups: int = 1
    logit_softcap: float = 0.0
    layers: tuple = ()
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    has_loop: bool = False
    eos_token_ids: tuple = ()
    architecture: str = "Debuzen"

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "DebuzenConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(layers_in):
            w = f"{where}.layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{w}: must be an object")
            kind = _require(entry, "type", str, w)
            if kind not in DEBUZEN_MIXERS:
                raise ConfigError(f"{w}: unknown mixer type {kind!r} (known: {', '.join(sorted(DEBUZEN_MIXERS))})")
            mixer = DEBUZEN_MIXERS[kind].from_dict(kind, _obj(entry, "mixer", w), w + ".mixer")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(f"{w}: 'mlp' must be null or an object")
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{w}.mlp: unknown feed-forward kind {mlp.get('kind')!r} (known: dense)")
                ff = _require(mlp, "ff", int, w + ".mlp")
                if ff <= 0:
                    raise ConfigError(f"{w}.mlp: ff must be > 0")
            layers.append(DebuzenLayer(mixer, ff))
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError(f"{where}: 'loop' must be an object or null")
            w = where + ".loop"
            start, stop, times = _require(loop, "start", int, w), _require(loop, "stop", int, w), _require(loop, "times", int, w)
            if not (0 <= start < stop <= len(layers)) or times < 1:
                raise ConfigError(f"{w}: need 0 <= start < stop <= {len(layers)} layers and times >= 1")
        norm = _obj(d, "norm", where)
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where) for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab_size=_require(d, "vocab", int, where), hidden_size=_require(d, "width", int, where),
                  norm_eps=_require(norm, "eps", float, where + ".norm"),
                  norm_groups=_typed(norm.get("groups", 1), "groups", int, where + ".norm"),
                  logit_softcap=_typed(d.get("logit_softcap", 0.0) or 0.0, "logit_softcap", float, where),
                  layers=tuple(layers), loop_start=start, loop_stop=stop, loop_times=times, has_loop=loop is not None,
                  eos_token_ids=eos_ids)
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or not cfg.norm_eps > 0 or cfg.logit_softcap < 0:
            raise ConfigError(f"{where}: vocab and width must be > 0, norm.eps > 0, logit_softcap >= 0")
        if cfg.norm_groups <= 0 or cfg.hidden_size % cfg.norm_groups:
            raise ConfigError(f"{where}.norm: width {cfg.hidden_size} does not split into {cfg.norm_groups} equal parts")
        return cfg

    def complete_from_checkpoint(self, shapes: Dict[str, Any]) -> "DebuzenConfig":
        """The sizes that only a tensor's shape gives (``shapes``: checkpoint name -> shape): the inner sizes
        of the pairs of matrices that make decays and gates (rows of ``a1`` and ``g1``)."""
        from dataclasses import replace

        def rows(name, default):
            shape = shapes.get(name)
            return int(shape[0]) if shape is not None and len(shape) == 2 else default

        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, GatedLinearSpec):
                m = replace(m, decay_rank=rows(f"l{i}.mix.a1", m.decay_rank))
            elif isinstance(m.right, ChannelDeltaSpec):
                m = replace(m, right=replace(m.right, decay_rank=rows(f"l{i}.mix.right.a1", m.right.decay_rank),
                                             gate_rank=rows(f"l{i}.mix.right.g1", m.right.gate_rank)))
            layers.append(DebuzenLayer(m, layer.ff))
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
            "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "logit_softcap": self.logit_softcap,
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in self.layers]}
        if self.has_loop:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
