"""Dirozen: a decoder whose layers are listed one by one in config.json.

config.json holds ``architecture`` (a string), ``vocab``, ``width``, ``norm.eps`` and ``layers``: for each layer its
``type`` (the mixer), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``: ``kind`` and ``ff``,
or null for a layer without one).  Every size and constant is taken from there; the tensors are named
``embed``, ``l<i>.norm1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``final.norm`` and ``head``.

A layer: n = norm1(x); x <- x + (mixer(n) + ff(n)), with norm1 an RMSNorm whose weight is stored as its distance
from one.  The mixer ``attention``: grouped query heads over key/value heads that are one tensor (the values are the
keys as projected, before their norm), q and k divided by their root mean square per head without weights, a query
temperature 1 + coef * ln(floor((position + 1) / every) + 1), scores scaled by ``scale``, all earlier positions
visible, no rotation, and a sigmoid gate per head on the output (``g``).  The feed-forward ``dense``:
down(silu(gate(n)) * up(n)).  All of that is said to the engine as parameters of its parts (``model_spec``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, JsonReader, ModelConfig, require_positive
from ..models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

ARCHITECTURE = "Dirozen"
MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense",)


@dataclass
class DirozenLayer:
    """One entry of ``layers``, checked."""

    type: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float
    temp_every: int
    ff: Optional[int]        # None: no feed-forward

    def to_dict(self) -> Dict[str, Any]:
        return {
            "type": self.type,
            "mixer": {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                      "q_temp": {"coef": self.temp_coef, "every": self.temp_every}, "scale": self.scale,
                      "vdim": self.vdim},
            "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"},
        }


@dataclass
class DirozenConfig(ModelConfig):
    vocab_size: int
    width: int
    norm_eps: float
    layers: List[DirozenLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    # An option of the engine, not a key of config.json (the design has no rotation or table that ends somewhere):
    # the most positions a request may reach.
    max_positions: int = 1 << 20
    architecture: str = ARCHITECTURE

    engine_options = {
        "max_positions": {"type": int, "help": "the most positions a request may reach (the design sets no limit)"}}

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Dict[str, Any], origin: str = "<dict>", generation: Optional[Dict[str, Any]] = None,
                  generation_origin: str = "<dict>") -> "DirozenConfig":
        r = JsonReader(data, origin)
        norm = r.raw("norm")
        if not isinstance(norm, dict):
            raise ConfigError(f"'{origin}': key 'norm' must be an object with 'eps'")
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"'{origin}': key 'layers' must be a list with at least one layer")
        layers = [cls._read_layer(entry, f"{origin}: layers[{i}]") for i, entry in enumerate(listed)]
        cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"),
                  norm_eps=JsonReader(norm, f"{origin}: norm").number("eps"), layers=layers,
                  eos_token_ids=r.int_or_int_list("eos_token_id"))
        cfg.read_generation_defaults(generation, generation_origin)
        cfg.validate(origin)
        return cfg

    @staticmethod
    def _read_layer(entry: Any, origin: str) -> DirozenLayer:
        if not isinstance(entry, dict):
            raise ConfigError(f"'{origin}' must be an object")
        r = JsonReader(entry, origin)
        kind = r.string("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"'{origin}': there is no mixer '{kind}' (known: {', '.join(MIXER_TYPES)})")
        mixer = r.raw("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"'{origin}': key 'mixer' must be an object")
        m = JsonReader(mixer, f"{origin}.mixer")
        temp = m.raw("q_temp")
        if not isinstance(temp, dict):
            raise ConfigError(f"'{origin}.mixer': key 'q_temp' must be an object with 'coef' and 'every'")
        t = JsonReader(temp, f"{origin}.mixer.q_temp")
        ff = None
        mlp = r.raw("mlp")
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise ConfigError(f"'{origin}': key 'mlp' must be an object or null")
            f = JsonReader(mlp, f"{origin}.mlp")
            if f.string("kind") not in MLP_KINDS:
                raise ConfigError(f"'{origin}.mlp': there is no feed-forward '{f.string('kind')}' "
                                  f"(known: {', '.join(MLP_KINDS)})")
            ff = f.integer("ff")
        return DirozenLayer(type=kind, heads=m.integer("heads"), kv_heads=m.integer("kv_heads"), dim=m.integer("dim"),
                            vdim=m.integer("vdim", m.integer("dim")), scale=m.number("scale"), temp_coef=t.number("coef"),
                            temp_every=t.integer("every"), ff=ff)

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        require_positive(origin, vocab=self.vocab_size, width=self.width, max_positions=self.max_positions)
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"'{origin}': norm.eps ({self.norm_eps}) must not be negative")
        if not self.layers:
            raise ConfigError(f"'{origin}': a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"{origin}: layers[{i}]"
            require_positive(where, heads=layer.heads, kv_heads=layer.kv_heads, dim=layer.dim, vdim=layer.vdim,
                             every=layer.temp_every)
            if layer.ff is not None:
                require_positive(where, ff=layer.ff)
            if layer.heads % layer.kv_heads:
                raise ConfigError(f"'{where}': {layer.heads} query heads cannot be shared out evenly over "
                                  f"{layer.kv_heads} key/value heads")
            if layer.vdim != layer.dim:
                raise ConfigError(f"'{where}': the values are the keys as projected, so vdim ({layer.vdim}) must equal "
                                  f"dim ({layer.dim})")
            if layer.dim % 2:
                raise ConfigError(f"'{where}': dim ({layer.dim}) must be even (the kernels take a head in pairs)")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": [layer.to_dict() for layer in self.layers],
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab_size,
            "width": self.width,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------ the model
    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "weight_offset": 1.0, "tensor": ""})
        layers = []
        for i, layer in enumerate(self.layers):
            mixer = PartSpec("attention", {
                "hidden_size": self.width,
                "num_heads": layer.heads,
                "num_kv_heads": layer.kv_heads,
                "head_dim": layer.dim,
                "values": "keys",
                "qk_norm": True,
                "qk_norm_weights": False,
                "qk_norm_eps": self.norm_eps,
                "query_temperature": {"coef": layer.temp_coef, "every": layer.temp_every},
                "scale": layer.scale,
                "window": None,
                "position": None,
                "output_gate": True,
                "names": {"q": "q", "k": "k", "o": "o", "gate": "g"},
                "prefix": "mix",
            })
            ffn = None
            if layer.ff is not None:
                ffn = PartSpec("gated_mlp", {
                    "hidden_size": self.width,
                    "intermediate_size": layer.ff,
                    "activation": "silu",
                    "names": {"gate": "gate", "up": "up", "down": "down"},
                    "prefix": "mlp",
                })
            layers.append(LayerSpec(prefix=f"l{i}", mixer=mixer, ffn=ffn, norms={"norm": norm},
                                    block=PartSpec("parallel", {"norm": "norm1"})))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.width,
            max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "embed"}),
            layers=layers,
            order=[RunSpec(layer=i) for i in range(len(layers))],
            final_norm=norm,
            final_norm_prefix="final.norm",
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "head",
                                      "tied": False}),
            positions={},
        )
        spec.validate()
        return spec
