"""Typed configuration of the Zemarax architecture, read from config.json.

A Zemarax model is a list of layers around one float32 residual stream.  Every layer has a norm before and a norm
behind each sublayer (RMS norms whose weights are stored around zero), one of three mixers and a feed-forward or none:

* ``attention``: grouped-query softmax attention without positions, a norm per head on q and k, values of their own
  size, a ``scale`` given as it is, a sliding window under which the first tokens stay visible, a sink per head;
* ``mlstm``: a matrix-memory recurrence with capped exponential gates and a running maximum;
* ``latent_attention``: causal softmax attention whose keys and values are maps of one cached latent a token, queries
  through a latent of their own, a sink per head; with ``kv_from: j`` the layer reads layer j's latents.

Feed-forwards: ``dense`` (SiLU-gated) or ``moe`` (ungated experts with the exact GELU, a router with a bias whose
weights are a softmax over the chosen logits, optionally a shared expert behind a sigmoid gate of one number a token).
The embedding multiplies the token's row by ``embedding.scale`` and adds a row of a hashed bigram table and a learned
row per position; the logits are multiplied by ``logit_scale``.

config.json keys: ``architecture``, ``vocab``, ``width``, ``max_positions``, ``logit_scale``, ``norm.eps``,
``embedding.{scale, bigram.{buckets, mul_prev, mul_cur}}`` and ``layers`` (a list of ``{"type", "mixer": {...},
"mlp": {...} or null}``).  Tensor names: ``embed``, ``bigram``, ``pos``, ``head``, ``final.norm`` and per layer i
``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .bomotar import DEFAULT_MAX_POSITIONS, _obj
from .llama import ConfigError
from .mifutar import _num
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

#: the activation of a routed or shared expert (fixed by the design; the dense feed-forward is SiLU-gated)
EXPERT_ACTIVATION = "gelu_erf"
#: the weight of every norm of a layer and of the model's last norm is stored as its deviation from one
NORM_WEIGHT_OFFSET = 1.0
MIXERS = ("attention", "mlstm", "latent_attention")


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None
    keep_first: int = 0

    @classmethod
    def from_dict(cls, d, where):
        mask = _obj(d, "mask", where, optional=True)
        dim = _num(d, "dim", where)
        m = cls(_num(d, "heads", where), _num(d, "kv_heads", where), dim, _num(d, "vdim", where) if d.get("vdim") is not None else dim,
                _num(d, "scale", where, float),
                None if mask is None else _num(mask, "size", where + ".mask"),
                0 if mask is None or mask.get("keep_first") is None else _num(mask, "keep_first", where + ".mask", positive=False))
        if m.heads % m.kv_heads != 0:
            raise ConfigError(f"config.json: {where}: heads ({m.heads}) must be a multiple of kv_heads ({m.kv_heads})")
        return m

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            d["mask"] = {"keep_first": self.keep_first, "size": self.window}
        return d


@dataclass(frozen=True)
class MlstmMixer:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d, where):
        return cls(_num(d, "heads", where), _num(d, "dim", where), _num(d, "vdim", where), _num(d, "gate_cap", where, float))

    def to_dict(self):
        return {"dim": self.dim, "gate_cap": self.gate_cap, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    q_rank: Optional[int]      # (None: the query latent's size is the tensors' own)
    scale: float
    kv_from: Optional[int] = None

    @classmethod
    def from_dict(cls, d, where):
        dim = _num(d, "dim", where)
        return cls(_num(d, "heads", where), dim, _num(d, "vdim", where) if d.get("vdim") is not None else dim, _num(d, "kv_rank", where),
                   _num(d, "q_rank", where) if d.get("q_rank") is not None else None,
                   _num(d, "scale", where, float), None if d.get("kv_from") is None else _num(d, "kv_from", where, positive=False))

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "scale": self.scale, "vdim": self.vdim}
        if self.q_rank is not None:
            d["q_rank"] = self.q_rank
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


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
    shared_ff: Optional[int] = None

    def to_dict(self):
        d = {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


def _mlp_from_dict(d, where):
    kind = d.get("kind", "dense")
    if kind == "dense":
        return DenseMlp(_num(d, "ff", where))
    if kind == "moe":
        r = _obj(d, "router", where)
        sh = _obj(d, "shared", where, optional=True)
        m = MoeMlp(_num(_obj(d, "expert", where), "ff", where + ".expert"), _num(r, "experts", where + ".router"), _num(r, "top", where + ".router"),
                   None if sh is None else _num(sh, "ff", where + ".shared"))
        if m.top > m.experts:
            raise ConfigError(f"config.json: {where}.router: top ({m.top}) exceeds experts ({m.experts})")
        return m
    raise ConfigError(f"config.json: {where}: feed-forward kind {kind!r} unknown (known: dense, moe)")


@dataclass(frozen=True)
class ZemaraxLayer:
    type: str
    mixer: Any      # AttentionMixer, MlstmMixer or LatentMixer
    mlp: Any        # DenseMlp, MoeMlp or None


@dataclass
class ZemaraxConfig:
    vocab: int
    width: int
    layers: List[ZemaraxLayer]
    max_positions: Optional[int]      # rows of the position table (None: the tensor's own first dimension)
    bigram_buckets: int
    bigram_mul_prev: int
    bigram_mul_cur: int
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    norm_eps: float = 1e-6
    eos_token_id: List[int] = field(default_factory=list)
    architecture: str = "Zemarax"

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
        return self.max_positions if self.max_positions is not None else DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZemaraxConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, ld in enumerate(layers_in):
            where = f"layers[{i}]"
            if not isinstance(ld, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = ld.get("type")
            md = _obj(ld, "mixer", where)
            if kind == "attention":
                mixer = AttentionMixer.from_dict(md, where + ".mixer")
            elif kind == "mlstm":
                mixer = MlstmMixer.from_dict(md, where + ".mixer")
            elif kind == "latent_attention":
                mixer = LatentMixer.from_dict(md, where + ".mixer")
            else:
                raise ConfigError(f"config.json: {where}: mixer type {kind!r} unknown (known: {', '.join(MIXERS)})")
            mlp = None if ld.get("mlp") is None else _mlp_from_dict(_obj(ld, "mlp", where), where + ".mlp")
            layers.append(ZemaraxLayer(kind, mixer, mlp))
        for i, l in enumerate(layers):
            if l.type == "latent_attention" and l.mixer.kv_from is not None:
                j = l.mixer.kv_from
                src = layers[j] if 0 <= j < i else None
                if src is None or src.type != "latent_attention" or src.mixer.kv_from is not None or src.mixer.kv_rank != l.mixer.kv_rank:
                    raise ConfigError(f"config.json: layers[{i}].mixer: kv_from must name an earlier latent_attention layer with a latent "
                                      "of its own and of this layer's kv_rank")
        norm = d.get("norm") or {}
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        emb = _obj(d, "embedding", "top level")
        bg = _obj(emb, "bigram", "embedding")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, list) else [int(eos)])
        return cls(
            vocab=_num(d, "vocab", "top level"),
            width=_num(d, "width", "top level"),
            layers=layers,
            max_positions=_num(d, "max_positions", "top level") if d.get("max_positions") is not None else None,
            bigram_buckets=_num(bg, "buckets", "embedding.bigram"),
            bigram_mul_prev=_num(bg, "mul_prev", "embedding.bigram", positive=False),
            bigram_mul_cur=_num(bg, "mul_cur", "embedding.bigram", positive=False),
            embedding_scale=_num(emb, "scale", "embedding", float, positive=False) if emb.get("scale") is not None else 1.0,
            logit_scale=_num(d, "logit_scale", "top level", float, positive=False) if d.get("logit_scale") is not None else 1.0,
            norm_eps=_num(norm, "eps", "norm", float) if norm.get("eps") is not None else 1e-6,
            eos_token_id=eos_list,
            architecture=str(d.get("architecture", "Zemarax")),
        )

    @classmethod
    def from_json(cls, text: str) -> "ZemaraxConfig":
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
            "embedding": {"bigram": {"buckets": self.bigram_buckets, "mul_cur": self.bigram_mul_cur, "mul_prev": self.bigram_mul_prev},
                          "scale": self.embedding_scale},
            "layers": [{"mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict(), "type": l.type} for l in self.layers],
            "logit_scale": self.logit_scale,
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab,
            "width": self.width,
        }
        if self.max_positions is not None:
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
                n *= int(s) if s is not None else 0
            total += n
        return total

    def kv_bytes_per_token(self, elem_bytes: int = 2) -> int:
        total = 0
        for l in self.layers:
            if l.type == "attention":
                total += l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) * elem_bytes
            elif l.type == "latent_attention" and l.mixer.kv_from is None:
                total += 2 * l.mixer.kv_rank * elem_bytes      # (the latent as key and, transposed, as value)
        return total

    def state_bytes_per_request(self) -> int:
        total = 4      # the embedding's previous token
        for l in self.layers:
            if l.type == "mlstm":
                total += 4 * l.mixer.heads * (l.mixer.vdim + 1) * (l.mixer.dim + 1)
        return total

    def describe(self) -> Dict[str, Any]:
        """What ``tempura inspect`` prints of this architecture."""
        def layer(l):
            m = l.mixer
            if l.type == "attention":
                mix = (f"attention {m.heads} heads ({m.kv_heads} key/value) of {m.dim}, values of {m.vdim}, " +
                       ("no window" if m.window is None else f"window {m.window} keeping the first {m.keep_first}") + ", sink")
            elif l.type == "mlstm":
                mix = f"mlstm {m.heads} heads of {m.dim} x {m.vdim}, gates capped at {m.gate_cap:g}"
            else:
                mix = (f"latent attention {m.heads} heads of {m.dim}, values of {m.vdim}, latent {m.kv_rank}, query latent {m.q_rank}, sink" +
                       (f", latents of layer {m.kv_from}" if m.kv_from is not None else ""))
            if l.mlp is None:
                ff = "no feed-forward"
            elif isinstance(l.mlp, DenseMlp):
                ff = f"feed-forward {l.mlp.ff}"
            else:
                ff = f"{l.mlp.experts} experts of {l.mlp.ff}, {l.mlp.top} a token" + \
                    (f", shared expert of {l.mlp.shared_ff}" if l.mlp.shared_ff is not None else "")
            return mix + "; " + ff
        return {"hidden_size": self.width, "vocab_size": self.vocab, "norm_eps": self.norm_eps, "max_positions": self.max_position_embeddings,
                "embedding_scale": self.embedding_scale, "logit_scale": self.logit_scale, "bigram_buckets": self.bigram_buckets,
                "layers": [layer(l) for l in self.layers],
                "kv_bytes_per_token_bf16": self.kv_bytes_per_token(2), "state_bytes_per_request": self.state_bytes_per_request()}

    def build_spec(self) -> ModelSpec:
        layers, order = [], []
        norm = lambda name: PartSpec("rmsnorm", {"eps": self.norm_eps, "weight_offset": NORM_WEIGHT_OFFSET}, {"weight": name})
        for i, l in enumerate(self.layers):
            p, m = f"l{i}", l.mixer
            cache = None
            if l.type == "attention":
                mixer = PartSpec(
                    "attention",
                    params={"num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim, "scale": m.scale,
                            "window": m.window, "keep_first": m.keep_first if m.window is not None else 0, "sink": True,
                            "qk_norm": {"eps": self.norm_eps}, "position": PartSpec("none")},
                    weights={"q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "o": f"{p}.mix.o", "q_norm": f"{p}.mix.q.norm",
                             "k_norm": f"{p}.mix.k.norm", "sink": f"{p}.mix.sink"})
            elif l.type == "mlstm":
                mixer = PartSpec(
                    "mlstm",
                    params={"num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim, "gate_cap": m.gate_cap, "norm_eps": self.norm_eps,
                            "q_scale": m.dim ** -0.5},
                    weights={"q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "gate": f"{p}.mix.g", "o": f"{p}.mix.o",
                             "norm": f"{p}.mix.norm", "i": f"{p}.mix.i", "i_bias": f"{p}.mix.i.b", "f": f"{p}.mix.f", "f_bias": f"{p}.mix.f.b"})
            else:
                own = m.kv_from is None
                weights = {"dq": f"{p}.mix.dq", "dq_norm": f"{p}.mix.dq.norm", "uq": f"{p}.mix.uq", "uk": f"{p}.mix.uk", "uv": f"{p}.mix.uv",
                           "o": f"{p}.mix.o", "sink": f"{p}.mix.sink"}
                if own:
                    weights.update({"dkv": f"{p}.mix.dkv", "dkv_norm": f"{p}.mix.dkv.norm"})
                mixer = PartSpec(
                    "latent_cache_attention",
                    params={"num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim, "latent_dim": m.kv_rank, "query_rank": m.q_rank,
                            "scale": m.scale, "norm_eps": self.norm_eps, "sink": True, "own_latent": own},
                    weights=weights)
                # a layer with latents of its own names its cache slot after itself; one that borrows names the lender's
                cache = i if own else m.kv_from
            parts = {"mixer_norm": norm(f"{p}.norm1"), "mixer": mixer, "mixer_post_norm": norm(f"{p}.norm1b")}
            if l.mlp is not None:
                parts["ffn_norm"] = norm(f"{p}.norm2")
                parts["ffn_post_norm"] = norm(f"{p}.norm2b")
                if isinstance(l.mlp, DenseMlp):
                    parts["ffn"] = PartSpec("gated", params={"intermediate_size": l.mlp.ff},
                                            weights={"gate": f"{p}.mlp.gate", "up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
                else:
                    params = {"experts": l.mlp.experts, "top": l.mlp.top, "intermediate_size": l.mlp.ff, "expert": "plain",
                              "activation": EXPERT_ACTIVATION, "normalize": True, "sum_eps": 0.0}
                    weights = {"router": f"{p}.mlp.router", "router_bias": f"{p}.mlp.router.b", "up": p + ".mlp.e{}.up",
                               "down": p + ".mlp.e{}.down"}
                    if l.mlp.shared_ff is not None:
                        params["shared"] = {"intermediate_size": l.mlp.shared_ff, "activation": EXPERT_ACTIVATION}
                        weights.update({"shared_up": f"{p}.mlp.shared.up", "shared_down": f"{p}.mlp.shared.down",
                                        "shared_gate": f"{p}.mlp.shared.sg"})
                    parts["ffn"] = PartSpec("moe", params=params, weights=weights)
            layers.append(LayerSpec("sandwich", parts))
            order.append(LayerCall(i, cache))
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.width,
            vocab_size=self.vocab,
            max_positions=self.max_position_embeddings,
            layers=layers,
            order=order,
            final_norm=norm("final.norm"),
            embedding=PartSpec("embedding", {"scale": self.embedding_scale, "position": "learned", "max_positions": self.max_positions,
                                             "bigram": {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev,
                                                        "mul_cur": self.bigram_mul_cur}},
                               {"weight": "embed", "bigram": "bigram", "position": "pos"}),
            lm_head=PartSpec("lm_head", {"tied": False, "scale": self.logit_scale}, {"weight": "head"}),
            eos_token_ids=list(self.eos_token_id),
        )
