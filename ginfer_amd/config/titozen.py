"""Typed configuration of the Titozen decoder, read from its own config.json keys.

config.json names the architecture under `architecture` and gives: `vocab`, `width`, `norm.eps`, `canon.taps` (the taps
of the short convolution in front of every mixer) and `layers`, a list whose entries name the mixer (`type`: "hgrn2" or
"latent_attention"), the mixer's sizes (`mixer`) and the feed-forward (`mlp`: {kind: "dense", ff, limit}, or null for a
layer without one).  Layers may differ from one another in kind and in every size.

What the design fixes (no key of config.json): the position vectors' base 10000, the feed-forward's sigmoid factor
1.702 and its shift of the linear branch by 1, the sink and the output gate of the latent attention, the norms on the
sublayers' outputs with one gain each.  There is no limit on positions and no end-of-sequence token in config.json.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .registry import register_architecture, ConfigError
from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec

POSITION_BASE = 10000.0
FEED_FORWARD_SIGMOID_FACTOR = 1.702
FEED_FORWARD_LINEAR_SHIFT = 1.0
# positions are counted in 32-bit floats inside the position vectors: whole numbers are exact up to 2^24
MAX_POSITIONS = 1 << 24

# how the checkpoints spell the parts' tensor prefixes: layer i is "l<i>", and inside it
LAYER_TENSOR_NAMES = dict(mixer="mix", feed_forward="mlp", mixer_norm="norm1", feed_forward_norm="norm2",
                          input_conv="canon1")
MODEL_TENSOR_NAMES = dict(embedding="embed", final_norm="final.norm", head="head")

_MIXER_KEYS = {"hgrn2": ("heads", "dim", "vdim"),
               "latent_attention": ("heads", "dim", "vdim", "q_rank", "kv_rank", "scale")}


def _int(d, key, where, minimum=1):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError("config.json: %s %r must be an integer >= %d, got %r" % (where, key, minimum, v))
    return v


def _number(d, key, where):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError("config.json: %s %r must be a number, got %r" % (where, key, v))
    return float(v)


@dataclass
class TitozenLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@register_architecture("Titozen", "titozen")
@dataclass
class TitozenConfig:
    vocab: int
    width: int
    eps: float
    taps: int
    layers: List[TitozenLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)

    architecture = "Titozen"

    @classmethod
    def from_dict(cls, d):
        missing = [k for k in ("vocab", "width", "norm", "canon", "layers") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): %s" % ", ".join(missing))
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, l in enumerate(d["layers"]):
            where = "layer %d" % i
            kind = l.get("type")
            if kind not in _MIXER_KEYS:
                raise ConfigError("config.json: %s has the unknown mixer type %r (known: %s)"
                                  % (where, kind, ", ".join(sorted(_MIXER_KEYS))))
            m = l.get("mixer") or {}
            lacking = [k for k in _MIXER_KEYS[kind] if k not in m]
            if lacking:
                raise ConfigError("config.json: %s (%s) lacks the mixer key(s): %s" % (where, kind, ", ".join(lacking)))
            mixer = {k: _int(m, k, where + " mixer") for k in ("heads", "dim", "vdim")}
            if kind == "latent_attention":
                mixer.update(q_rank=_int(m, "q_rank", where + " mixer"), kv_rank=_int(m, "kv_rank", where + " mixer"),
                             scale=_number(m, "scale", where + " mixer"))
                mask = m.get("mask")             # no mask (or null): every earlier position is seen
                mixer["mask"] = None if mask is None else dict(size=_int(mask, "size", where + " mixer mask"))
            mlp = l.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError("config.json: %s has the unknown feed-forward kind %r (known: dense)"
                                      % (where, mlp.get("kind")))
                mlp = dict(kind="dense", ff=_int(mlp, "ff", where + " mlp"), limit=_number(mlp, "limit", where + " mlp"))
                if not mlp["limit"] > 0:
                    raise ConfigError("config.json: %s mlp 'limit' must be positive" % where)
            layers.append(TitozenLayer(kind, mixer, mlp))
        eps = _number(d["norm"], "eps", "norm")
        if not eps > 0:
            raise ConfigError("config.json: norm 'eps' must be positive")
        vocab = _int(d, "vocab", "")
        eos = d.get("eos_token_id")
        eos = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        return cls(vocab=vocab, width=_int(d, "width", ""), eps=eps, taps=_int(d["canon"], "taps", "canon"), layers=layers,
                   eos_token_ids=eos)

    def to_dict(self):
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 canon=dict(taps=self.taps),
                 layers=[dict(type=l.type, mixer=dict(l.mixer), mlp=None if l.mlp is None else dict(l.mlp))
                         for l in self.layers])
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    def model_spec(self):
        W = self.width
        norm = PartSpec("scalar_rmsnorm", dict(size=W, eps=self.eps))
        conv = PartSpec("short_causal", dict(width=W, taps=self.taps))
        layers = []
        for i, l in enumerate(self.layers):
            m = l.mixer
            if l.type == "hgrn2":
                mixer = PartSpec("hgrn2", dict(hidden_size=W, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                                               eps=self.eps))
            else:
                mixer = PartSpec("latent_attention", dict(
                    hidden_size=W, num_heads=m["heads"], head_dim=m["dim"], value_dim=m["vdim"], q_rank=m["q_rank"],
                    kv_rank=m["kv_rank"], scale=m["scale"], window=None if m["mask"] is None else m["mask"]["size"],
                    eps=self.eps, sink=True, gated=True))
            parts = dict(mixer=mixer, mixer_norm=norm, input_conv=conv)
            if l.mlp is not None:
                parts["feed_forward"] = PartSpec("clamped_glu", dict(
                    hidden_size=W, intermediate_size=l.mlp["ff"], limit=l.mlp["limit"],
                    alpha=FEED_FORWARD_SIGMOID_FACTOR, shift=FEED_FORWARD_LINEAR_SHIFT))
                parts["feed_forward_norm"] = norm
            layers.append(LayerSpec(prefix="l%d" % i, parts=parts, arrangement="outnorm", names=dict(LAYER_TENSOR_NAMES)))
        spec = ModelSpec(
            hidden_size=W, vocab_size=self.vocab, layers=layers,
            schedule=[ScheduleEntry(i) for i in range(len(layers))],
            embedding=PartSpec("sinusoidal_normed", dict(vocab_size=self.vocab, hidden_size=W, eps=self.eps,
                                                         base=POSITION_BASE)),
            final_norm=norm,
            head=PartSpec("lm_head", dict(vocab_size=self.vocab, hidden_size=W, tied=False, weight_name="")),
            max_positions=MAX_POSITIONS, eos_token_ids=list(self.eos_token_ids), names=dict(MODEL_TENSOR_NAMES))
        spec.validate()
        return spec
