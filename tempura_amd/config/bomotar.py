"""Typed configuration of the Bomotar architecture, read from config.json.

A Bomotar model is a list of layers around one float32 residual stream.  Every layer has a norm before and a norm
behind each sublayer (what enters the stream is multiplied by ``residual_mult``), a ``parallel`` mixer (a softmax
attention with short convolutions, rotated positions with YaRN scaling and an output gate, beside a gated delta-rule
recurrence; the two are added with ``left_scale`` and ``right_scale``) and a feed-forward that is dense (GELU, tanh
form), a mixture of experts (SiLU-gated experts, a softmax router with a correction and groups) or absent.  A
layer with ``weights_of: j`` runs layer j's tensors with a cache and state of its own.  The embedding adds a row
of a hashed bigram table.  Every size is per layer.

config.json keys: ``architecture``, ``vocab``, ``width``, ``residual_mult``, ``norm.eps``,
``embedding.bigram.{buckets, mul_prev, mul_cur}`` and ``layers`` (a list of ``{"type": "parallel", "mixer": {"left":
{...}, "right": {...}, "left_scale", "right_scale"}, "mlp": {...} or null, "weights_of": j (optional)}``); optional
``max_positions``.  Tensor names: ``embed``, ``bigram``, ``head``, ``final.norm`` and per layer i ``l<i>.norm1``,
``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .mifutar import _num
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

#: the design has no position limit of its own; this bounds what a request may hold unless config.json says ``max_positions``
DEFAULT_MAX_POSITIONS = 1 << 20
#: what is added under the root when q and k of the recurrence are made unit vectors (fixed by the design)
UNIT_EPS = 1e-6
#: the magnitude of cosine and sine under YaRN scaling is YARN_MAG_SLOPE * ln(factor) + 1 (fixed by the design)
YARN_MAG_SLOPE = 0.1


def _obj(d, key, where, optional=False):
    v = d.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}: '{key}' must be an object")
    return v


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    #: YaRN scaling (factor, original, fast, slow) or None
    factor: Optional[float] = None
    original: Optional[float] = None
    fast: Optional[float] = None
    slow: Optional[float] = None

    @classmethod
    def from_dict(cls, d, where, dim):
        r = cls(_num(d, "dims", where), _num(d, "base", where, float))
        if r.dims % 2 != 0 or r.dims > dim:
            raise ConfigError(f"config.json: {where}: dims ({r.dims}) must be even and at most the head size ({dim})")
        sc = _obj(d, "scaling", where, optional=True)
        if sc is not None:
            w = where + ".scaling"
            r = cls(r.dims, r.base, _num(sc, "factor", w, float), _num(sc, "original", w, float), _num(sc, "fast", w, float),
                    _num(sc, "slow", w, float))
        return r

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.factor is not None:
            d["scaling"] = {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}
        return d

    def part(self, dim) -> PartSpec:
        params = {"head_dim": dim, "rotary_dim": self.dims, "theta": self.base}
        if self.factor is not None:
            params["scaling"] = {"type": "yarn", "factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}
            params["attn_factor"] = YARN_MAG_SLOPE * math.log(self.factor) + 1.0
        return PartSpec("rope", params)


@dataclass(frozen=True)
class LeftMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int
    rot: Optional[Rotation]

    @classmethod
    def from_dict(cls, d, where):
        dim = _num(d, "dim", where)
        rot = _obj(d, "rot", where, optional=True)
        m = cls(_num(d, "heads", where), _num(d, "kv_heads", where), dim,
                _num(d, "vdim", where) if d.get("vdim") is not None else dim, _num(d, "scale", where, float), _num(d, "conv", where),
                None if rot is None else Rotation.from_dict(rot, where + ".rot", dim))
        if m.heads % m.kv_heads != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
        return m

    def to_dict(self):
        d = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class RightMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    #: ranks of the decay's and the gate's low-rank projections: the checkpoint's tensors say them; a configuration
    #: names them (``decay_rank``, ``gate_rank``) only where no checkpoint is there to say it, for random weights
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        m = cls(_num(d, "heads", where), _num(d, "kv_heads", where), _num(d, "dim", where), _num(d, "vdim", where), _num(d, "conv", where),
                _num(d, "decay_rank", where) if d.get("decay_rank") is not None else None,
                _num(d, "gate_rank", where) if d.get("gate_rank") is not None else None)
        if m.heads % m.kv_heads != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
        return m

    def to_dict(self):
        d = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            d["gate_rank"] = self.gate_rank
        return d


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: LeftMixer
    right: RightMixer
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d, where):
        return cls(LeftMixer.from_dict(_obj(d, "left", where), where + ".left"), RightMixer.from_dict(_obj(d, "right", where), where + ".right"),
                   _num(d, "left_scale", where, float, positive=False), _num(d, "right_scale", where, float, positive=False))

    def to_dict(self):
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(), "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseMlp:
    ff: int

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class MoeMlp:
    ff: int
    experts: int
    top: int
    group_count: Optional[int] = None
    group_keep: Optional[int] = None

    def to_dict(self):
        router = {"experts": self.experts, "top": self.top}
        if self.group_count is not None:
            router["groups"] = {"count": self.group_count, "keep": self.group_keep}
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": router}


def _mlp_from_dict(d, where):
    kind = d.get("kind", "dense")
    if kind == "dense":
        return DenseMlp(_num(d, "ff", where))
    if kind == "moe":
        r = _obj(d, "router", where)
        g = _obj(r, "groups", where + ".router", optional=True)
        m = MoeMlp(_num(_obj(d, "expert", where), "ff", where + ".expert"), _num(r, "experts", where + ".router"), _num(r, "top", where + ".router"),
                   None if g is None else _num(g, "count", where + ".router.groups"), None if g is None else _num(g, "keep", where + ".router.groups"))
        if m.top > m.experts:
            raise ConfigError(f"config.json: {where}.router: top ({m.top}) exceeds experts ({m.experts})")
        if m.group_count is not None and (m.experts % m.group_count != 0 or m.group_keep > m.group_count
                                          or m.group_keep * (m.experts // m.group_count) < m.top):
            raise ConfigError(f"config.json: {where}.router.groups: count must divide experts, keep at most count, and the kept groups hold at least top experts")
        return m
    raise ConfigError(f"config.json: {where}: feed-forward kind {kind!r} unknown (known: dense, moe)")


@dataclass(frozen=True)
class BomotarLayer:
    type: str
    mixer: ParallelMixerConfig
    mlp: Any                            # DenseMlp, MoeMlp or None
    weights_of: Optional[int] = None    # the layer whose tensors this one runs (None: its own)


@dataclass
class BomotarConfig:
    vocab: int
    width: int
    layers: List[BomotarLayer]
    bigram_buckets: int
    bigram_mul_prev: int
    bigram_mul_cur: int
    residual_mult: float = 1.0
    norm_eps: float = 1e-6
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_id: List[int] = field(default_factory=list)
    architecture: str = "Bomotar"

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
    def from_dict(cls, d: Dict[str, Any]) -> "BomotarConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, ld in enumerate(layers_in):
            where = f"layers[{i}]"
            if not isinstance(ld, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            if ld.get("type") != "parallel":
                raise ConfigError(f"config.json: {where}: mixer type {ld.get('type')!r} unknown (known: parallel)")
            mixer = ParallelMixerConfig.from_dict(_obj(ld, "mixer", where), where + ".mixer")
            mlp = None
            if ld.get("mlp") is not None:
                mlp = _mlp_from_dict(_obj(ld, "mlp", where), where + ".mlp")
            src = ld.get("weights_of")
            if src is not None:
                src = _num(ld, "weights_of", where, positive=False)
                if not 0 <= src < len(layers_in) or not isinstance(layers_in[src], dict) or layers_in[src].get("weights_of") is not None:
                    raise ConfigError(f"config.json: {where}: weights_of must name a layer that has tensors of its own")
            layers.append(BomotarLayer("parallel", mixer, mlp, src))
        for i, l in enumerate(layers):
            if l.weights_of is not None and (layers[l.weights_of].mixer != l.mixer or layers[l.weights_of].mlp != l.mlp):
                raise ConfigError(f"config.json: layers[{i}]: a layer that runs layer {l.weights_of}'s tensors has that layer's sizes")
        norm = d.get("norm") or {}
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        bg = _obj(_obj(d, "embedding", "top level"), "bigram", "embedding")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, list) else [int(eos)])
        return cls(
            vocab=_num(d, "vocab", "top level"),
            width=_num(d, "width", "top level"),
            layers=layers,
            bigram_buckets=_num(bg, "buckets", "embedding.bigram"),
            bigram_mul_prev=_num(bg, "mul_prev", "embedding.bigram", positive=False),
            bigram_mul_cur=_num(bg, "mul_cur", "embedding.bigram", positive=False),
            residual_mult=_num(d, "residual_mult", "top level", float, positive=False) if d.get("residual_mult") is not None else 1.0,
            norm_eps=_num(norm, "eps", "norm", float) if norm.get("eps") is not None else 1e-6,
            max_positions=_num(d, "max_positions", "top level") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
            eos_token_id=eos_list,
            architecture=str(d.get("architecture", "Bomotar")),
        )

    @classmethod
    def from_json(cls, text: str) -> "BomotarConfig":
        try:
            d = json.loads(text)
        except json.JSONDecodeError as e:
            raise ConfigError(f"config.json: malformed JSON: {e}") from e
        if not isinstance(d, dict):
            raise ConfigError("config.json: top level must be an object")
        return cls.from_dict(d)

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            e = {"mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict(), "type": l.type}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        d = {
            "architecture": self.architecture,
            "embedding": {"bigram": {"buckets": self.bigram_buckets, "mul_cur": self.bigram_mul_cur, "mul_prev": self.bigram_mul_prev}},
            "layers": layers,
            "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult,
            "vocab": self.vocab,
            "width": self.width,
        }
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
        return sum(l.mixer.left.kv_heads * (l.mixer.left.dim + l.mixer.left.vdim) * elem_bytes for l in self.layers)

    def state_bytes_per_request(self) -> int:
        total = 4      # the embedding's previous token
        for l in self.layers:
            a, r = l.mixer.left, l.mixer.right
            total += 4 * (a.conv - 1) * (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim))
            total += 4 * ((r.conv - 1) * (2 * r.kv_heads * r.dim + r.heads * r.vdim) + r.heads * r.dim * r.vdim)
        return total

    def describe(self) -> Dict[str, Any]:
        """What ``tempura inspect`` prints of this architecture."""
        def layer(i, l):
            a, r = l.mixer.left, l.mixer.right
            mix = (f"{l.mixer.left_scale:g} x attention {a.heads} heads ({a.kv_heads} key/value) of {a.dim}, values of {a.vdim}, "
                   f"{a.conv} taps, " + ("no rotation" if a.rot is None else f"{a.rot.dims} rotated") +
                   f" + {l.mixer.right_scale:g} x delta rule {r.heads} heads ({r.kv_heads} key) of {r.dim}, values of {r.vdim}, {r.conv} taps")
            if l.mlp is None:
                ff = "no feed-forward"
            elif isinstance(l.mlp, DenseMlp):
                ff = f"feed-forward {l.mlp.ff}"
            else:
                ff = f"{l.mlp.experts} experts of {l.mlp.ff}, {l.mlp.top} a token" + \
                    (f", {l.mlp.group_keep} of {l.mlp.group_count} groups" if l.mlp.group_count is not None else "")
            return mix + "; " + ff + (f"; tensors of layer {l.weights_of}" if l.weights_of is not None else "")
        return {"hidden_size": self.width, "vocab_size": self.vocab, "residual_mult": self.residual_mult, "norm_eps": self.norm_eps,
                "max_positions": self.max_positions, "bigram_buckets": self.bigram_buckets,
                "layers": [layer(i, l) for i, l in enumerate(self.layers)],
                "kv_bytes_per_token_bf16": self.kv_bytes_per_token(2), "state_bytes_per_request": self.state_bytes_per_request()}

    def build_spec(self) -> ModelSpec:
        # one LayerSpec per layer that has tensors of its own; the run order names it once for itself and once for
        # every layer that runs its tensors (each run-order entry has a cache slot and a state row of its own)
        index, layers = {}, []
        for i, l in enumerate(self.layers):
            if l.weights_of is not None:
                continue
            index[i] = len(layers)
            p = f"l{i}"
            a, r = l.mixer.left, l.mixer.right
            left = PartSpec(
                "conv_attention",
                params={"num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "value_dim": a.vdim, "scale": a.scale,
                        "conv_taps": a.conv, "gate": True, "window": None,
                        "position": PartSpec("none") if a.rot is None else a.rot.part(a.dim)},
                weights={"q": f"{p}.mix.left.q", "k": f"{p}.mix.left.k", "v": f"{p}.mix.left.v", "q_conv": f"{p}.mix.left.q.conv",
                         "k_conv": f"{p}.mix.left.k.conv", "v_conv": f"{p}.mix.left.v.conv", "gate": f"{p}.mix.left.g", "o": f"{p}.mix.left.o"})
            right = PartSpec(
                "gated_delta",
                params={"num_heads": r.heads, "num_kv_heads": r.kv_heads, "head_dim": r.dim, "value_dim": r.vdim, "conv_taps": r.conv,
                        "norm_eps": self.norm_eps, "unit_eps": UNIT_EPS, "q_scale": r.dim ** -0.5, "decay_rank": r.decay_rank,
                        "gate_rank": r.gate_rank},
                weights={"q": f"{p}.mix.right.q", "k": f"{p}.mix.right.k", "v": f"{p}.mix.right.v", "q_conv": f"{p}.mix.right.q.conv",
                         "k_conv": f"{p}.mix.right.k.conv", "v_conv": f"{p}.mix.right.v.conv", "beta": f"{p}.mix.right.b",
                         "a_log": f"{p}.mix.right.A_log", "dt_bias": f"{p}.mix.right.dt_bias", "a1": f"{p}.mix.right.a1",
                         "a2": f"{p}.mix.right.a2", "g1": f"{p}.mix.right.g1", "g2": f"{p}.mix.right.g2", "norm": f"{p}.mix.right.norm",
                         "o": f"{p}.mix.right.o"})
            mixer = PartSpec("parallel", params={"branches": [left, right], "scales": [l.mixer.left_scale, l.mixer.right_scale]})
            pre = lambda name: PartSpec("rmsnorm", {"eps": self.norm_eps}, {"weight": name})
            post = lambda name: PartSpec("rmsnorm", {"eps": self.norm_eps, "scale": self.residual_mult}, {"weight": name})
            parts = {"mixer_norm": pre(f"{p}.norm1"), "mixer": mixer, "mixer_post_norm": post(f"{p}.norm1b")}
            if l.mlp is not None:
                parts["ffn_norm"] = pre(f"{p}.norm2")
                parts["ffn_post_norm"] = post(f"{p}.norm2b")
                if isinstance(l.mlp, DenseMlp):
                    parts["ffn"] = PartSpec("mlp", params={"intermediate_size": l.mlp.ff, "activation": "gelu_tanh"},
                                            weights={"up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
                else:
                    groups = None if l.mlp.group_count is None else {"count": l.mlp.group_count, "keep": l.mlp.group_keep}
                    parts["ffn"] = PartSpec("moe", params={"experts": l.mlp.experts, "top": l.mlp.top, "groups": groups,
                                                           "intermediate_size": l.mlp.ff},
                                            weights={"router": f"{p}.mlp.router", "correction": f"{p}.mlp.correction",
                                                     "gate": p + ".mlp.e{}.gate", "up": p + ".mlp.e{}.up", "down": p + ".mlp.e{}.down"})
            layers.append(LayerSpec("sandwich", parts))
        order = [LayerCall(index[l.weights_of if l.weights_of is not None else i]) for i, l in enumerate(self.layers)]
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.width,
            vocab_size=self.vocab,
            max_positions=self.max_positions,
            layers=layers,
            order=order,
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps}, {"weight": "final.norm"}),
            embedding=PartSpec("embedding", {"bigram": {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev,
                                                        "mul_cur": self.bigram_mul_cur}}, {"weight": "embed", "bigram": "bigram"}),
            lm_head=PartSpec("lm_head", {"tied": False}, {"weight": "head"}),
            eos_token_ids=list(self.eos_token_id),
        )
