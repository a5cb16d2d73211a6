"""Typed configuration of the Mifutar architecture, read from config.json.

A Mifutar model is a list of layers, each with its own mixer (``"attention"`` or ``"mamba2"``) and an
optional feed-forward, around ``streams`` copies of the residual stream (hyper-connections).  Every size is
per layer: two layers of one model may differ in everything but the model width.

config.json keys: ``architecture``, ``vocab``, ``width``, ``streams``, ``logit_scale``, ``norm.eps`` and
``layers`` (a list of ``{"type", "mixer": {...}, "mlp": {...} or null}``); optional ``max_positions``.
Tensor names: ``embed``, ``head``, ``final.norm`` and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.hc1.*``, ``l<i>.hc2.*``.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

#: the design has no position limit of its own (sinusoidal positions, windows and recurrent state); this bounds
#: what a request may hold unless config.json says ``max_positions``
DEFAULT_MAX_POSITIONS = 1 << 20
#: base of the sinusoidal position vector (fixed by the design)
SINUSOID_BASE = 10000.0
#: slope of the sigmoid in the feed-forward's gate, and what is added to the clamped up branch (fixed by the design)
GATE_SIGMOID_SLOPE = 1.702
UP_OFFSET = 1.0


def _num(d: Dict[str, Any], key: str, where: str, kind=int, positive: bool = True):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where}: missing field '{key}'")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}: field '{key}' must be a number, got {v!r}")
    if kind is int:
        if int(v) != v:
            raise ConfigError(f"config.json: {where}: field '{key}' must be an integer, got {v!r}")
        v = int(v)
    else:
        v = float(v)
    if positive and not v > 0:
        raise ConfigError(f"config.json: {where}: field '{key}' must be positive, got {v!r}")
    return v


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    window: Optional[int]
    #: rows of the distance table.  The checkpoint's tensor says it; a configuration names it (``bias_buckets``)
    #: only where no checkpoint is there to say it: for random weights
    buckets: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        mask = d.get("mask")
        window = None
        if mask is not None:
            if not isinstance(mask, dict):
                raise ConfigError(f"config.json: {where}: 'mask' must be an object")
            if mask.get("size") is not None:
                window = _num(mask, "size", where + ".mask")
        m = cls(_num(d, "heads", where), _num(d, "kv_heads", where), _num(d, "dim", where),
                _num(d, "vdim", where) if d.get("vdim") is not None else _num(d, "dim", where),
                _num(d, "scale", where, float), _num(d, "bias_max", where), window,
                _num(d, "bias_buckets", where) if d.get("bias_buckets") is not None else None)
        if m.heads % m.kv_heads != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
        if m.vdim != m.dim:
            raise ConfigError(f"config.json: {where}: the values are the keys, so vdim ({m.vdim}) must equal dim ({m.dim})")
        return m

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "bias_max": self.bias_max}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.buckets is not None:
            d["bias_buckets"] = self.buckets
        return d


@dataclass(frozen=True)
class Mamba2Mixer:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, d, where):
        m = cls(*(_num(d, k, where) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")))
        if m.heads % m.groups != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of groups ({m.groups})")
        if (m.heads * m.vdim) % m.norm_groups != 0:
            raise ConfigError(f"config.json: {where}: heads * vdim ({m.heads * m.vdim}) must be a multiple of norm_groups ({m.norm_groups})")
        return m

    def to_dict(self):
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class DenseMlp:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("kind", "dense")
        if kind != "dense":
            raise ConfigError(f"config.json: {where}: feed-forward kind {kind!r} is not supported (only 'dense')")
        return cls(_num(d, "ff", where), _num(d, "limit", where, float))

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclass(frozen=True)
class MifutarLayer:
    type: str
    mixer: Any
    mlp: Optional[DenseMlp]


_MIXERS = {"attention": AttentionMixer, "mamba2": Mamba2Mixer}


@dataclass
class MifutarConfig:
    vocab: int
    width: int
    layers: List[MifutarLayer]
    streams: Optional[int] = None      # None: one residual stream with the plain sum, no connection tensors
    logit_scale: float = 1.0
    norm_eps: float = 1e-6
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_id: List[int] = field(default_factory=list)
    architecture: str = "Mifutar"

    # (names the engine's reports and sizing read from any configuration)
    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MifutarConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, ld in enumerate(layers_in):
            where = f"layers[{i}]"
            if not isinstance(ld, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = ld.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}: mixer type {kind!r} unknown (known: {', '.join(sorted(_MIXERS))})")
            if not isinstance(ld.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}: 'mixer' must be an object")
            mixer = _MIXERS[kind].from_dict(ld["mixer"], where + ".mixer")
            mlp = None
            if ld.get("mlp") is not None:
                if not isinstance(ld["mlp"], dict):
                    raise ConfigError(f"config.json: {where}: 'mlp' must be an object or null")
                mlp = DenseMlp.from_dict(ld["mlp"], where + ".mlp")
            layers.append(MifutarLayer(kind, mixer, mlp))
        norm = d.get("norm") or {}
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, list) else [int(eos)])
        return cls(
            vocab=_num(d, "vocab", "top level"),
            width=_num(d, "width", "top level"),
            layers=layers,
            streams=_num(d, "streams", "top level") if d.get("streams") is not None else None,
            logit_scale=_num(d, "logit_scale", "top level", float, positive=False) if d.get("logit_scale") is not None else 1.0,
            norm_eps=_num(norm, "eps", "norm", float) if norm.get("eps") is not None else 1e-6,
            max_positions=_num(d, "max_positions", "top level") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
            eos_token_id=eos_list,
            architecture=str(d.get("architecture", "Mifutar")),
        )

    @classmethod
    def from_json(cls, text: str) -> "MifutarConfig":
        try:
            d = json.loads(text)
        except json.JSONDecodeError as e:
            raise ConfigError(f"config.json: malformed JSON: {e}") from e
        if not isinstance(d, dict):
            raise ConfigError("config.json: top level must be an object")
        return cls.from_dict(d)

    def to_dict(self) -> Dict[str, Any]:
        d = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "logit_scale": self.logit_scale,
            "norm": {"eps": self.norm_eps},
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers],
        }
        if self.streams is not None:
            d["streams"] = self.streams
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    def to_json(self) -> str:
        return json.dumps(self.to_dict(), indent=1)

    # ---- derived ---------------------------------------------------------
    def num_parameters(self) -> int:
        from ..parts.inventory import expected_weights
        total = 0
        for info in expected_weights(self.build_spec()).values():
            n = 1
            for s in info.shape:
                n *= int(s) if s is not None else 0      # (a size only the checkpoint says: not counted)
            total += n
        return total

    def kv_bytes_per_token(self, elem_bytes: int = 2) -> int:
        return sum(2 * l.mixer.kv_heads * l.mixer.dim * elem_bytes for l in self.layers if l.type == "attention")

    def state_bytes_per_request(self) -> int:
        total = 0
        for l in self.layers:
            if l.type == "mamba2":
                m = l.mixer
                total += 4 * (m.heads * m.state * m.vdim + (m.conv - 1) * (m.heads * m.vdim + 2 * m.groups * m.state))
        return total

    def describe(self) -> Dict[str, Any]:
        """What ``tempura inspect`` prints of this architecture."""
        def layer(l):
            m = l.mixer
            if l.type == "attention":
                mix = (f"attention {m.heads} heads ({m.kv_heads} key/value) of {m.dim}, window {m.window or 'none'}, "
                       f"distance bias up to {m.bias_max}")
            else:
                mix = (f"mamba2 {m.heads} heads of {m.vdim}, state {m.state}, {m.groups} groups, {m.conv} taps, "
                       f"norm in {m.norm_groups} parts")
            return mix + (f"; feed-forward {l.mlp.ff}, limit {l.mlp.limit:g}" if l.mlp is not None else "; no feed-forward")
        return {"hidden_size": self.width, "vocab_size": self.vocab, "streams": self.streams or 1,
                "logit_scale": self.logit_scale, "norm_eps": self.norm_eps, "max_positions": self.max_positions,
                "layers": [layer(l) for l in self.layers],
                "kv_bytes_per_token_bf16": self.kv_bytes_per_token(2), "state_bytes_per_request": self.state_bytes_per_request()}

    def build_spec(self) -> ModelSpec:
        layers = []
        s = self.streams or 1
        for i, l in enumerate(self.layers):
            p = f"l{i}"
            m = l.mixer
            if l.type == "attention":
                mixer = PartSpec(
                    "attention",
                    params={"num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "scale": m.scale,
                            "window": m.window, "position": PartSpec("none"), "values": "keys", "bias": True,
                            "distance_bias": {"kind": "log_buckets", "max_distance": m.bias_max, "buckets": m.buckets}},
                    weights={"q": f"{p}.mix.q", "k": f"{p}.mix.k", "o": f"{p}.mix.o", "q_bias": f"{p}.mix.q.b",
                             "k_bias": f"{p}.mix.k.b", "distance_bias": f"{p}.mix.rel"})
            else:
                mixer = PartSpec(
                    "mamba2",
                    params={"num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state, "groups": m.groups,
                            "conv_taps": m.conv, "norm_groups": m.norm_groups, "norm_eps": self.norm_eps},
                    weights={"in": f"{p}.mix.in", "conv": f"{p}.mix.conv", "conv_bias": f"{p}.mix.conv.b",
                             "dt_bias": f"{p}.mix.dt_bias", "a_log": f"{p}.mix.A_log", "d": f"{p}.mix.D",
                             "norm": f"{p}.mix.norm", "out": f"{p}.mix.o"})
            norm = lambda name: PartSpec("rmsnorm", {"eps": self.norm_eps, "weight_offset": 1.0}, {"weight": name})
            hyper = lambda q: PartSpec("hyper_connection", {"streams": s},
                                       {"in": f"{p}.hc{q}.in", "out": f"{p}.hc{q}.out", "mix": f"{p}.hc{q}.mix"})
            parts = {"mixer_norm": norm(f"{p}.norm1"), "mixer": mixer}
            if self.streams is not None:
                parts["mixer_link"] = hyper(1)
            if l.mlp is not None:
                parts["ffn_norm"] = norm(f"{p}.norm2")
                parts["ffn"] = PartSpec(
                    "gated",
                    params={"intermediate_size": l.mlp.ff, "sigmoid_slope": GATE_SIGMOID_SLOPE, "limit": l.mlp.limit,
                            "up_offset": UP_OFFSET},
                    weights={"gate": f"{p}.mlp.gate", "up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
                if self.streams is not None:
                    parts["ffn_link"] = hyper(2)
            layers.append(LayerSpec("hyper", parts))
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.width,
            vocab_size=self.vocab,
            max_positions=self.max_positions,
            layers=layers,
            order=[LayerCall(i) for i in range(len(layers))],
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps, "weight_offset": 1.0}, {"weight": "final.norm"}),
            embedding=PartSpec("embedding", {"position": "sinusoid", "position_base": SINUSOID_BASE}, {"weight": "embed"}),
            lm_head=PartSpec("lm_head", {"tied": False, "scale": self.logit_scale}, {"weight": "head"}),
            eos_token_ids=list(self.eos_token_id),
            streams=s,
        )
