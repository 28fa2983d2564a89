"""Kesovik: a decoder whose layers are listed one by one in config.json, with the norm after the sum.

config.json holds ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``postln_alpha``,
``logit_softcap`` and ``layers``: for each layer its ``type`` (the mixer), the mixer's sizes and constants (``mixer``)
and its feed-forward (``mlp``, or null for none).  Every size and constant is taken from there.  Tensors:
``embed``, ``l<i>.norm1`` / ``norm2`` / ``ls1`` / ``ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.

The model: x = embed[token] * embedding.scale; per layer x <- norm1(alpha x + ls1 * mixer(x)), then
x <- norm2(alpha x + ls2 * ff(x)) (RMSNorms with plain weights; the sublayers read x itself); logits =
head(final.norm(x)), then cap * tanh(logits / cap).

Mixers.  ``lightning``: linear attention with a constant decay per head and a float32 state per request (``heads``,
``dim``, ``vdim``, ``decay``).  ``parallel``: two mixers side by side on the same input, ``left_scale * left +
right_scale * right``; left is softmax attention with grouped key/value heads (``heads``, ``kv_heads``, ``dim``,
``vdim``), biases on q, k and v, one norm over the whole q projection and one over the whole k projection, a rotation
on the first ``rot.dims`` channels of every head in adjacent pairs (``rot.base``), ``scale`` on the scores and a sliding
window of ``mask.size`` tokens; right is lightning attention.

Feed-forwards.  ``dense``: down(relu(up x)^2).  ``moe``: ``router.experts`` gated experts of width ``expert.ff`` plus
``router.identity`` identity experts, ``router.top`` of them a token, chosen by softmax score plus a stored correction,
weighted by their scores divided by their sum; and a shared gated expert (``shared.ff``) for every token.

All of that is said to the engine as parameters of registered parts (``model_spec``); there is no model class.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, JsonReader, ModelConfig, require_positive
from ..models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

ARCHITECTURE = "Kesovik"
MIXER_TYPES = ("lightning", "parallel")
MLP_KINDS = ("dense", "moe")


def _object(value: Any, where: str, what: str) -> Dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"'{where}': key '{what}' must be an object")
    return value


@dataclass
class LightningSizes:
    heads: int
    dim: int
    vdim: int
    decay: List[float]

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "LightningSizes":
        r = JsonReader(data, where)
        decay = r.raw("decay")
        if not isinstance(decay, list) or not all(isinstance(v, (int, float)) and not isinstance(v, bool) for v in decay):
            raise ConfigError(f"'{where}': key 'decay' must be a list of numbers, one a head")
        dim = r.integer("dim")
        return cls(heads=r.integer("heads"), dim=dim, vdim=r.integer("vdim", dim), decay=[float(v) for v in decay])

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, dim=self.dim, vdim=self.vdim)
        if len(self.decay) != self.heads:
            raise ConfigError(f"'{where}': {len(self.decay)} decays for {self.heads} heads")
        if not all(0.0 <= v <= 1.0 for v in self.decay):
            raise ConfigError(f"'{where}': a decay must lie between 0 and 1")
        if self.dim > 256:
            raise ConfigError(f"'{where}': the state's kernel takes at most 256 key channels a head, dim is {self.dim}")

    def to_dict(self) -> Dict[str, Any]:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]       # None: config.json names no mask, every earlier token is visible
    rot_base: float
    rot_dims: int               # 0: config.json names no rotation

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "WindowAttentionSizes":
        r = JsonReader(data, where)
        dim = r.integer("dim")
        window, base, dims = None, 1.0, 0
        if r.raw("mask") is not None:
            window = JsonReader(_object(r.raw("mask"), where, "mask"), f"{where}.mask").integer("size")
        if r.raw("rot") is not None:
            rot = JsonReader(_object(r.raw("rot"), where, "rot"), f"{where}.rot")
            base, dims = rot.number("base"), rot.integer("dims")
        return cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads", r.integer("heads")), dim=dim,
                   vdim=r.integer("vdim", dim), scale=r.number("scale"), window=window, rot_base=base, rot_dims=dims)

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim)
        if self.window is not None:
            require_positive(where, window=self.window)
        if self.heads % self.kv_heads:
            raise ConfigError(f"'{where}': {self.heads} query heads cannot be shared out evenly over {self.kv_heads} "
                              "key/value heads")
        if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"'{where}': rot.dims ({self.rot_dims}) must be even and at most dim ({self.dim})")
        if self.rot_dims and not self.rot_base > 0:
            raise ConfigError(f"'{where}': rot.base must be positive")

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return out


@dataclass
class KesovikMLP:
    kind: str
    ff: int = 0                 # dense: the inner width; moe: an expert's
    experts: int = 0
    identity: int = 0
    top: int = 0
    shared_ff: Optional[int] = None

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "KesovikMLP":
        r = JsonReader(data, where)
        kind = r.string("kind")
        if kind not in MLP_KINDS:
            raise ConfigError(f"'{where}': there is no feed-forward '{kind}' (known: {', '.join(MLP_KINDS)})")
        if kind == "dense":
            return cls(kind=kind, ff=r.integer("ff"))
        router = JsonReader(_object(r.raw("router"), where, "router"), f"{where}.router")
        expert = JsonReader(_object(r.raw("expert"), where, "expert"), f"{where}.expert")
        shared = r.raw("shared")
        shared_ff = None
        if shared is not None:
            shared_ff = JsonReader(_object(shared, where, "shared"), f"{where}.shared").integer("ff")
        return cls(kind=kind, ff=expert.integer("ff"), experts=router.integer("experts"),
                   identity=router.integer("identity", 0), top=router.integer("top"), shared_ff=shared_ff)

    def check(self, where: str) -> None:
        require_positive(where, ff=self.ff)
        if self.kind == "moe":
            require_positive(where, experts=self.experts, top=self.top)
            if self.identity < 0 or self.top > self.experts + self.identity:
                raise ConfigError(f"'{where}': {self.top} of {self.experts} + {self.identity} experts cannot be chosen")
            if self.shared_ff is not None:
                require_positive(where, shared_ff=self.shared_ff)

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        out: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe",
                               "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass
class KesovikLayer:
    type: str
    lightning: Optional[LightningSizes] = None      # type "lightning": the mixer; "parallel": its right branch
    left: Optional[WindowAttentionSizes] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    mlp: Optional[KesovikMLP] = None

    def to_dict(self) -> Dict[str, Any]:
        if self.type == "lightning":
            mixer = self.lightning.to_dict()
        else:
            mixer = {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.lightning.to_dict(),
                     "right_scale": self.right_scale}
        return {"mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass
class KesovikConfig(ModelConfig):
    vocab_size: int
    width: int
    norm_eps: float
    embedding_scale: float = 1.0
    postln_alpha: float = 1.0
    logit_softcap: float = 0.0      # 0: none
    layers: List[KesovikLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    # An option of the engine, not a key of config.json: the most positions a request may reach.
    max_positions: int = 1 << 20
    architecture: str = ARCHITECTURE

    engine_options = {
        "max_positions": {"type": int, "help": "the most positions a request may reach (the design sets no limit)"}}

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Dict[str, Any], origin: str = "<dict>", generation: Optional[Dict[str, Any]] = None,
                  generation_origin: str = "<dict>") -> "KesovikConfig":
        r = JsonReader(data, origin)
        norm = JsonReader(_object(r.raw("norm"), origin, "norm"), f"{origin}: norm")
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"'{origin}': key 'layers' must be a list with at least one layer")
        scale = 1.0
        if r.raw("embedding") is not None:
            scale = JsonReader(_object(r.raw("embedding"), origin, "embedding"), f"{origin}: embedding").number("scale", 1.0)
        cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"), norm_eps=norm.number("eps"),
                  embedding_scale=scale, postln_alpha=r.number("postln_alpha", 1.0),
                  logit_softcap=r.number("logit_softcap", 0.0),
                  layers=[cls._read_layer(entry, f"{origin}: layers[{i}]") for i, entry in enumerate(listed)],
                  eos_token_ids=r.int_or_int_list("eos_token_id"))
        cfg.read_generation_defaults(generation, generation_origin)
        cfg.validate(origin)
        return cfg

    @staticmethod
    def _read_layer(entry: Any, origin: str) -> KesovikLayer:
        if not isinstance(entry, dict):
            raise ConfigError(f"'{origin}' must be an object")
        r = JsonReader(entry, origin)
        kind = r.string("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"'{origin}': there is no mixer '{kind}' (known: {', '.join(MIXER_TYPES)})")
        mixer = _object(r.raw("mixer"), origin, "mixer")
        layer = KesovikLayer(type=kind)
        if kind == "lightning":
            layer.lightning = LightningSizes.read(mixer, f"{origin}.mixer")
        else:
            m = JsonReader(mixer, f"{origin}.mixer")
            layer.left = WindowAttentionSizes.read(_object(m.raw("left"), f"{origin}.mixer", "left"), f"{origin}.mixer.left")
            layer.lightning = LightningSizes.read(_object(m.raw("right"), f"{origin}.mixer", "right"), f"{origin}.mixer.right")
            layer.left_scale = m.number("left_scale", 1.0)
            layer.right_scale = m.number("right_scale", 1.0)
        mlp = r.raw("mlp")
        if mlp is not None:
            layer.mlp = KesovikMLP.read(_object(mlp, origin, "mlp"), f"{origin}.mlp")
        return layer

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        require_positive(origin, vocab=self.vocab_size, width=self.width, max_positions=self.max_positions)
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"'{origin}': norm.eps ({self.norm_eps}) must not be negative")
        if self.logit_softcap < 0.0:
            raise ConfigError(f"'{origin}': logit_softcap ({self.logit_softcap}) must not be negative")
        if not self.layers:
            raise ConfigError(f"'{origin}': a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"{origin}: layers[{i}]"
            layer.lightning.check(f"{where}.mixer" + (".right" if layer.type == "parallel" else ""))
            if layer.left is not None:
                layer.left.check(f"{where}.mixer.left")
            if layer.mlp is not None:
                layer.mlp.check(f"{where}.mlp")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architecture": self.architecture,
            "embedding": {"scale": self.embedding_scale},
            "layers": [layer.to_dict() for layer in self.layers],
            "logit_softcap": self.logit_softcap,
            "norm": {"eps": self.norm_eps},
            "postln_alpha": self.postln_alpha,
            "vocab": self.vocab_size,
            "width": self.width,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------ the model
    def _lightning_params(self, sizes: LightningSizes, prefix: str) -> Dict[str, Any]:
        return {"hidden_size": self.width, "num_heads": sizes.heads, "head_dim": sizes.dim, "value_dim": sizes.vdim,
                "decay": list(sizes.decay), "norm_eps": self.norm_eps, "activation": "silu", "prefix": prefix}

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "tensor": ""})
        layers = []
        positions: Dict[str, PartSpec] = {}
        for i, layer in enumerate(self.layers):
            if layer.type == "lightning":
                mixer = PartSpec("lightning", self._lightning_params(layer.lightning, "mix"))
            else:
                left = layer.left
                rope = None
                if left.rot_dims:
                    rope = f"rope:{left.rot_base!r}:{left.rot_dims}:{left.dim}"
                    positions.setdefault(rope, PartSpec("rope", {"theta": left.rot_base, "rotary_dim": left.rot_dims,
                                                                 "head_dim": left.dim, "pairing": "interleaved"}))
                attention = {"hidden_size": self.width, "num_heads": left.heads, "num_kv_heads": left.kv_heads,
                             "head_dim": left.dim, "value_dim": left.vdim, "bias": True, "qk_norm": "projection",
                             "qk_norm_eps": self.norm_eps, "scale": left.scale, "window": left.window,
                             "position": rope, "prefix": "left"}
                mixer = PartSpec("side_by_side", {
                    "hidden_size": self.width, "prefix": "mix",
                    "branches": [
                        {"kind": "attention_rows", "params": attention, "scale": layer.left_scale},
                        {"kind": "lightning", "params": self._lightning_params(layer.lightning, "right"),
                         "scale": layer.right_scale}]})
            ffn = None
            if layer.mlp is not None and layer.mlp.kind == "dense":
                ffn = PartSpec("mlp", {"hidden_size": self.width, "intermediate_size": layer.mlp.ff,
                                       "activation": "relu2", "prefix": "mlp"})
            elif layer.mlp is not None:
                m = layer.mlp
                ffn = PartSpec("routed_experts", {"hidden_size": self.width, "expert_size": m.ff, "num_experts": m.experts,
                                                  "num_identity": m.identity, "top": m.top, "correction": True,
                                                  "shared_size": m.shared_ff, "prefix": "mlp"})
            layers.append(LayerSpec(prefix=f"l{i}", mixer=mixer, ffn=ffn, norms={"mixer_norm": norm, "ffn_norm": norm},
                                    block=PartSpec("postnorm", {"alpha": self.postln_alpha, "mixer_norm": "norm1",
                                                                "ffn_norm": "norm2", "mixer_scale": "ls1",
                                                                "ffn_scale": "ls2"})))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.width,
            max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "embed",
                                             "scale": self.embedding_scale}),
            layers=layers,
            order=[RunSpec(layer=i) for i in range(len(layers))],
            final_norm=norm,
            final_norm_prefix="final.norm",
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "head",
                                      "tied": False, "softcap": self.logit_softcap}),
            positions=positions,
        )
        spec.validate()
        return spec
