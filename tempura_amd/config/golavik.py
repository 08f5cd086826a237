"""Typed configuration of the Golavik architecture, read from config.json.

A Golavik model is a list of layers around one float32 residual stream.  A layer has ONE norm (an RMS norm in
``norm.groups`` equal parts) whose output both sublayers read, each through a short causal convolution over time of
its own that is added to what it convolves (``canon.taps`` taps); the mixer's and the feed-forward's outputs enter the
stream together.  The mixer is one of ``channel_delta`` (a gated delta-rule recurrence with a decay per head and key
channel), ``general_delta`` (a generalized delta rule: decay per channel, a removal along the unit key, an additive
write) and ``latent_attention`` (softmax attention over a sliding window whose keys and values are expanded from one
compressed vector per token, with one rotated key part shared by the heads, YaRN frequency scaling and an output
gate).  The feed-forward is a mixture of SiLU-gated experts with a sigmoid router (groups of neighbouring experts are
ranked by the sum of their two best scores; weights are the chosen scores over their sum, times a constant) or
absent.  ``loop`` runs a range of layers several times in a row with the same tensors, every pass with a cache and
state of its own and a learned vector added to the stream before its first layer.  The output head is the embedding
table.

config.json keys: ``architecture``, ``vocab``, ``width``, ``norm.{eps, groups}``, ``canon.taps``, ``loop.{start, stop,
times}`` (optional) and ``layers`` (a list of ``{"type", "mixer": {...}, "mlp": {...} or null}``); optional
``max_positions``.  Tensor names: ``embed``, ``loop.step``, ``final.norm`` and per layer i ``l<i>.norm1``,
``l<i>.canon1``, ``l<i>.canon2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .bomotar import DEFAULT_MAX_POSITIONS, UNIT_EPS, Rotation, _obj
from .llama import ConfigError
from .mifutar import _num
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

#: the generalized delta rule's decay is exp(-DECAY_RATE * sigmoid(.)) (fixed by the design)
DECAY_RATE = math.exp(-0.5)
#: what is added to the sum of the chosen experts' scores before the division (fixed by the design)
ROUTE_SUM_EPS = 1e-20
#: a group of experts is ranked by the sum of this many of its best scores (fixed by the design)
GROUP_BEST = 2


def _opt(d, key, where):
    return _num(d, key, where) if d.get(key) is not None else None


@dataclass(frozen=True)
class ChannelDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    #: ranks of the decay's and the gate's low-rank projections: the checkpoint's tensors say them; a configuration
    #: names them only where no checkpoint is there to say it, for random weights
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        m = cls(_num(d, "heads", where), _num(d, "kv_heads", where), _num(d, "dim", where), _num(d, "vdim", where),
                _num(d, "conv", where), _opt(d, "decay_rank", where), _opt(d, "gate_rank", where))
        if m.heads % m.kv_heads != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
        return m

    def to_dict(self):
        d = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        for k in ("decay_rank", "gate_rank"):
            if getattr(self, k) is not None:
                d[k] = getattr(self, k)
        return d

    def part(self, p, eps) -> PartSpec:
        return PartSpec(
            "gated_delta",
            params={"num_heads": self.heads, "num_kv_heads": self.kv_heads, "head_dim": self.dim, "value_dim": self.vdim,
                    "conv_taps": self.conv, "norm_eps": eps, "unit_eps": UNIT_EPS, "q_scale": self.dim ** -0.5,
                    "decay_rank": self.decay_rank, "gate_rank": self.gate_rank},
            weights={"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "q_conv": f"{p}.q.conv", "k_conv": f"{p}.k.conv",
                     "v_conv": f"{p}.v.conv", "beta": f"{p}.b", "a_log": f"{p}.A_log", "dt_bias": f"{p}.dt_bias",
                     "a1": f"{p}.a1", "a2": f"{p}.a2", "g1": f"{p}.g1", "g2": f"{p}.g2", "norm": f"{p}.norm", "o": f"{p}.o"})

    def state_floats(self):
        return (self.conv - 1) * (2 * self.kv_heads * self.dim + self.heads * self.vdim) + self.heads * self.dim * self.vdim

    def text(self):
        return f"channel delta rule, {self.heads} heads ({self.kv_heads} key) of {self.dim}, values of {self.vdim}, {self.conv} taps"


@dataclass(frozen=True)
class GeneralDelta:
    heads: int
    dim: int
    #: rank of the decay's low-rank projection (the checkpoint's own; named only for random weights)
    decay_rank: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        return cls(_num(d, "heads", where), _num(d, "dim", where), _opt(d, "decay_rank", where))

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        return d

    def part(self, p, eps) -> PartSpec:
        return PartSpec(
            "general_delta",
            params={"num_heads": self.heads, "head_dim": self.dim, "norm_eps": eps, "unit_eps": UNIT_EPS,
                    "decay_rate": DECAY_RATE, "decay_rank": self.decay_rank},
            weights={"r": f"{p}.r", "k": f"{p}.k", "v": f"{p}.v", "gate": f"{p}.g", "a": f"{p}.a", "a_bias": f"{p}.a.b",
                     "w1": f"{p}.w1", "w2": f"{p}.w2", "w0": f"{p}.w0", "norm": f"{p}.norm", "o": f"{p}.o"})

    def state_floats(self):
        return self.heads * self.dim * self.dim

    def text(self):
        return f"general delta rule, {self.heads} heads of {self.dim}"


@dataclass(frozen=True)
class LatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: Rotation
    window: Optional[int]

    @classmethod
    def from_dict(cls, d, where):
        rot_dim = _num(d, "rot_dim", where)
        rot = Rotation.from_dict(_obj(d, "rot", where), where + ".rot", rot_dim)
        if rot.dims != rot_dim:
            raise ConfigError(f"config.json: {where}: rot.dims ({rot.dims}) must equal rot_dim ({rot_dim})")
        mask = _obj(d, "mask", where, optional=True)
        return cls(_num(d, "heads", where), _num(d, "dim", where), rot_dim, _num(d, "vdim", where), _num(d, "kv_rank", where),
                   _num(d, "scale", where, float), rot, None if mask is None else _num(mask, "size", where + ".mask"))

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": self.rot.to_dict(), "rot_dim": self.rot_dim,
             "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d

    def part(self, p, eps) -> PartSpec:
        return PartSpec(
            "latent_attention",
            params={"num_heads": self.heads, "head_dim": self.dim, "rotary_dim": self.rot_dim, "value_dim": self.vdim,
                    "latent_dim": self.kv_rank, "scale": self.scale, "window": self.window, "norm_eps": eps, "gate": True,
                    "position": self.rot.part(self.rot_dim)},
            weights={"q": f"{p}.q", "down": f"{p}.dkv", "latent_norm": f"{p}.dkv.norm", "up_k": f"{p}.uk", "up_v": f"{p}.uv",
                     "gate": f"{p}.g", "o": f"{p}.o"})

    def state_floats(self):
        return 0

    def text(self):
        return (f"latent attention, {self.heads} heads of {self.dim} + {self.rot_dim} rotated, values of {self.vdim}, latent of "
                f"{self.kv_rank}" + (f", window {self.window}" if self.window is not None else ""))


_MIXERS = {"channel_delta": ChannelDelta, "general_delta": GeneralDelta, "latent_attention": LatentAttention}


@dataclass(frozen=True)
class ExpertsMlp:
    ff: int
    experts: int
    top: int
    scale: float = 1.0
    group_count: Optional[int] = None
    group_keep: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("kind", "moe")
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: feed-forward kind {kind!r} unknown (known: moe)")
        r = _obj(d, "router", where)
        g = _obj(r, "groups", where + ".router", optional=True)
        m = cls(_num(_obj(d, "expert", where), "ff", where + ".expert"), _num(r, "experts", where + ".router"),
                _num(r, "top", where + ".router"),
                _num(r, "scale", where + ".router", float, positive=False) if r.get("scale") is not None else 1.0,
                None if g is None else _num(g, "count", where + ".router.groups"),
                None if g is None else _num(g, "keep", where + ".router.groups"))
        if m.top > m.experts:
            raise ConfigError(f"config.json: {where}.router: top ({m.top}) exceeds experts ({m.experts})")
        if m.group_count is not None and (m.experts % m.group_count != 0 or m.group_keep > m.group_count
                                          or m.group_keep * (m.experts // m.group_count) < m.top):
            raise ConfigError(f"config.json: {where}.router.groups: count must divide experts, keep at most count, and the kept groups hold at least top experts")
        return m

    def to_dict(self):
        router = {"experts": self.experts, "scale": self.scale, "top": self.top}
        if self.group_count is not None:
            router["groups"] = {"count": self.group_count, "keep": self.group_keep}
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": router}

    def part(self, p) -> PartSpec:
        groups = None if self.group_count is None else {"count": self.group_count, "keep": self.group_keep}
        return PartSpec("moe", params={"experts": self.experts, "top": self.top, "groups": groups, "intermediate_size": self.ff,
                                       "score": "sigmoid", "group_best": GROUP_BEST, "normalize": True, "sum_eps": ROUTE_SUM_EPS,
                                       "scale": self.scale},
                        weights={"router": f"{p}.router", "gate": p + ".e{}.gate", "up": p + ".e{}.up", "down": p + ".e{}.down"})


@dataclass(frozen=True)
class GolavikLayer:
    type: str
    mixer: Any                       # ChannelDelta, GeneralDelta or LatentAttention
    mlp: Optional[ExpertsMlp]


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass
class GolavikConfig:
    vocab: int
    width: int
    layers: List[GolavikLayer]
    canon_taps: int
    norm_eps: float = 1e-6
    norm_groups: int = 1
    loop: Optional[Loop] = None
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_id: List[int] = field(default_factory=list)
    architecture: str = "Golavik"

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
    def from_dict(cls, d: Dict[str, Any]) -> "GolavikConfig":
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
            mixer = _MIXERS[kind].from_dict(_obj(ld, "mixer", where), where + ".mixer")
            mlp = ExpertsMlp.from_dict(_obj(ld, "mlp", where), where + ".mlp") if ld.get("mlp") is not None else None
            layers.append(GolavikLayer(kind, mixer, mlp))
        norm = _obj(d, "norm", "top level", optional=True) or {}
        width = _num(d, "width", "top level")
        groups = _num(norm, "groups", "norm") if norm.get("groups") is not None else 1
        if width % groups != 0:
            raise ConfigError(f"config.json: norm.groups ({groups}) must divide width ({width})")
        loop = None
        lp = _obj(d, "loop", "top level", optional=True)
        if lp is not None:
            loop = Loop(_num(lp, "start", "loop", positive=False), _num(lp, "stop", "loop", positive=False), _num(lp, "times", "loop"))
            if not 0 <= loop.start <= loop.stop <= len(layers):
                raise ConfigError(f"config.json: loop: start ({loop.start}) and stop ({loop.stop}) must lie in order within the {len(layers)} layers")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, list) else [int(eos)])
        return cls(
            vocab=_num(d, "vocab", "top level"),
            width=width,
            layers=layers,
            canon_taps=_num(_obj(d, "canon", "top level"), "taps", "canon"),
            norm_eps=_num(norm, "eps", "norm", float) if norm.get("eps") is not None else 1e-6,
            norm_groups=groups,
            loop=loop,
            max_positions=_num(d, "max_positions", "top level") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
            eos_token_id=eos_list,
            architecture=str(d.get("architecture", "Golavik")),
        )

    @classmethod
    def from_json(cls, text: str) -> "GolavikConfig":
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
            "canon": {"taps": self.canon_taps},
            "layers": [{"mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict(), "type": l.type} for l in self.layers],
            "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
            "vocab": self.vocab,
            "width": self.width,
        }
        if self.loop is not None:
            d["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    def to_json(self) -> str:
        return json.dumps(self.to_dict(), indent=1)

    # ---- derived ---------------------------------------------------------
    def run_order(self):
        """[(layer, pass number or None)] in the order the layers run; a looped layer appears once a pass."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lp = self.loop
        order = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t) for i in range(lp.start, lp.stop)]
        return order + [(i, None) for i in range(lp.stop, n)]

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
        return sum(self.layers[i].mixer.heads * (self.layers[i].mixer.dim + self.layers[i].mixer.rot_dim + self.layers[i].mixer.vdim) * elem_bytes
                   for i, _ in self.run_order() if isinstance(self.layers[i].mixer, LatentAttention))

    def state_bytes_per_request(self) -> int:
        return sum(4 * ((self.canon_taps - 1) * self.width + self.layers[i].mixer.state_floats()) for i, _ in self.run_order())

    def describe(self) -> Dict[str, Any]:
        """What ``tempura inspect`` prints of this architecture."""
        def layer(l):
            if l.mlp is None:
                ff = "no feed-forward"
            else:
                ff = f"{l.mlp.experts} experts of {l.mlp.ff}, {l.mlp.top} a token, weights times {l.mlp.scale:g}" + \
                    (f", {l.mlp.group_keep} of {l.mlp.group_count} groups" if l.mlp.group_count is not None else "")
            return l.mixer.text() + "; " + ff
        info = {"hidden_size": self.width, "vocab_size": self.vocab, "norm_eps": self.norm_eps, "norm_groups": self.norm_groups,
                "input_convolution_taps": self.canon_taps, "max_positions": self.max_positions,
                "layers": [layer(l) for l in self.layers],
                "kv_bytes_per_token_bf16": self.kv_bytes_per_token(2), "state_bytes_per_request": self.state_bytes_per_request()}
        if self.loop is not None:
            info["loop"] = f"layers {self.loop.start} to {self.loop.stop - 1}, {self.loop.times} times"
        return info

    def build_spec(self) -> ModelSpec:
        norm = lambda name: PartSpec("rmsnorm", {"eps": self.norm_eps, "groups": self.norm_groups}, {"weight": name})
        layers = []
        for i, l in enumerate(self.layers):
            p = f"l{i}"
            taps = [f"{p}.canon1"] + ([f"{p}.canon2"] if l.mlp is not None else [])
            # (a layer without a feed-forward has no use for the second convolution; a checkpoint may hold it all the same)
            names = {"taps": taps} if l.mlp is not None else {"taps": taps, "unused": [f"{p}.canon2"]}
            parts = {"norm": norm(f"{p}.norm1"), "mixer": l.mixer.part(f"{p}.mix", self.norm_eps),
                     "inputs": PartSpec("residual_conv", {"taps": self.canon_taps}, names)}
            if l.mlp is not None:
                parts["ffn"] = l.mlp.part(f"{p}.mlp")
            layers.append(LayerSpec("shared_norm", parts))
        # every entry of the run order has a cache slot and a state row of its own; the first layer of a pass of the
        # loop adds that pass's row of the step table to the stream before it runs
        order = []
        for i, t in self.run_order():
            before = None
            if t is not None and i == self.loop.start:
                before = PartSpec("add_row", {"row": t, "rows": self.loop.times}, {"table": "loop.step"})
            order.append(LayerCall(i, None, before))
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.width,
            vocab_size=self.vocab,
            max_positions=self.max_positions,
            layers=layers,
            order=order,
            final_norm=norm("final.norm"),
            embedding=PartSpec("embedding", {}, {"weight": "embed"}),
            lm_head=PartSpec("lm_head", {"tied": True}, {"weight": "head"}),
            eos_token_ids=list(self.eos_token_id),
        )
