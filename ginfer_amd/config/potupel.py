"""Typed configuration of the Potupel decoder, read from its own config.json keys.

config.json names the architecture under `architecture` and gives: `vocab`, `width`, `norm.eps`, optionally `loop`
({start, stop, times}: the layers start .. stop - 1 run `times` times in a row with the same weights, each pass with
a cache of its own) and `layers`, a list whose entries name the mixer (`type`: "attention"), the mixer's sizes
(`mixer`: heads, kv_heads, dim, vdim, scale, optionally conv = the taps of the short convolution behind the
projections, and rot = {base, dims, optionally scaling = {factor, low, high, original}}) and the feed-forward (`mlp`:
{kind: "dense", ff}, {kind: "moe", router: {experts, top}, expert: {ff}, optionally shared: {ff}}, or null for a layer
without one).  Layers may differ from one another in every size.

What the design fixes (no key of config.json): gains of norms are stored around zero (g = 1 + stored); the softmax's
sink has the score 0; the head is the embedding table; the re-entry of the loop reads [x; x0] and adds one vector per
pass; the dense feed-forward squares a relu, the experts gate with silu.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .registry import register_architecture, ConfigError
from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec

NORM_GAIN_OFFSET = 1.0
SINK_SCORE = 0.0
# positions are counted in 32-bit floats where angles are made: whole numbers are exact far beyond this; the rotation's
# tables are as long as the longest sequence the engine is set up for, never longer than this
MAX_POSITIONS = 1 << 20

# how the checkpoints spell things: layer i is "l<i>"; the output norms' tensors and the layer scales stand in the layer
# itself (l<i>.norm1b, l<i>.ls1), so their role is spelt "" and the part is told the tensors' names
LAYER_TENSOR_NAMES = dict(mixer="mix", feed_forward="mlp", mixer_norm="norm1", feed_forward_norm="norm2",
                          mixer_out_norm="", feed_forward_out_norm="")
MODEL_TENSOR_NAMES = dict(embedding="embed", final_norm="final.norm", head="head", reentry="loop")


def _int(d, key, where, minimum=1):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError("config.json: %s %r must be an integer >= %d, got %r" % (where, key, minimum, v))
    return v


def _number(d, key, where, positive=False):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError("config.json: %s %r must be a %snumber, got %r" % (where, key, "positive " if positive else "", v))
    return float(v)


@dataclass
class PotupelLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


def _read_mixer(m, where):
    if not isinstance(m, dict):
        raise ConfigError("config.json: %s has no mixer sizes" % where)
    out = {k: _int(m, k, where + " mixer") for k in ("heads", "kv_heads", "dim", "vdim")}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError("config.json: %s: heads %d is not a multiple of kv_heads %d" % (where, out["heads"], out["kv_heads"]))
    out["scale"] = _number(m, "scale", where + " mixer")
    out["conv"] = None if m.get("conv") is None else _int(m, "conv", where + " mixer")
    rot = m.get("rot")
    if rot is not None:
        r = dict(base=_number(rot, "base", where + " rot", positive=True), dims=_int(rot, "dims", where + " rot", minimum=2))
        if r["dims"] % 2 or r["dims"] > out["dim"]:
            raise ConfigError("config.json: %s rot 'dims' must be even and at most dim %d, got %d" % (where, out["dim"], r["dims"]))
        sc = rot.get("scaling")
        r["scaling"] = None if sc is None else {k: _number(sc, k, where + " rot scaling", positive=True)
                                                for k in ("factor", "low", "high", "original")}
        if r["scaling"] is not None and not r["scaling"]["high"] > r["scaling"]["low"]:
            raise ConfigError("config.json: %s rot scaling needs high > low" % where)
        rot = r
    out["rot"] = rot
    return out


def _read_mlp(mlp, where):
    if mlp is None:
        return None
    kind = mlp.get("kind") if isinstance(mlp, dict) else None
    if kind == "dense":
        return dict(kind="dense", ff=_int(mlp, "ff", where + " mlp"))
    if kind == "moe":
        out = dict(kind="moe", router=dict(experts=_int(mlp.get("router"), "experts", where + " mlp router"),
                                           top=_int(mlp.get("router"), "top", where + " mlp router")),
                   expert=dict(ff=_int(mlp.get("expert"), "ff", where + " mlp expert")))
        if out["router"]["top"] > out["router"]["experts"]:
            raise ConfigError("config.json: %s mlp router: top %d of %d experts" % (where, out["router"]["top"], out["router"]["experts"]))
        shared = mlp.get("shared")
        out["shared"] = None if shared is None else dict(ff=_int(shared, "ff", where + " mlp shared"))
        return out
    raise ConfigError("config.json: %s has the unknown feed-forward kind %r (known: dense, moe)" % (where, kind))


@register_architecture("Potupel", "potupel")
@dataclass
class PotupelConfig:
    vocab: int
    width: int
    eps: float
    layers: List[PotupelLayer] = field(default_factory=list)
    loop: Optional[Dict[str, int]] = None
    eos_token_ids: List[int] = field(default_factory=list)

    architecture = "Potupel"

    @classmethod
    def from_dict(cls, d):
        missing = [k for k in ("vocab", "width", "norm", "layers") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): %s" % ", ".join(missing))
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, l in enumerate(d["layers"]):
            where = "layer %d" % i
            if not isinstance(l, dict) or l.get("type") != "attention":
                raise ConfigError("config.json: %s has the unknown mixer type %r (known: attention)"
                                  % (where, l.get("type") if isinstance(l, dict) else l))
            layers.append(PotupelLayer("attention", _read_mixer(l.get("mixer"), where), _read_mlp(l.get("mlp"), where)))
        loop = d.get("loop")
        if loop is not None:
            loop = dict(start=_int(loop, "start", "loop", minimum=0), stop=_int(loop, "stop", "loop", minimum=0),
                        times=_int(loop, "times", "loop", minimum=0))
            if not loop["start"] <= loop["stop"] <= len(layers):
                raise ConfigError("config.json: loop needs 0 <= start <= stop <= %d layers, got %d .. %d"
                                  % (len(layers), loop["start"], loop["stop"]))
        eos = d.get("eos_token_id")
        eos = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        return cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), eps=_number(d["norm"], "eps", "norm", positive=True),
                   layers=layers, loop=loop, eos_token_ids=eos)

    def to_dict(self):
        def mixer(m):
            out = {k: m[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale")}
            if m["conv"] is not None:
                out["conv"] = m["conv"]
            if m["rot"] is not None:
                out["rot"] = dict(base=m["rot"]["base"], dims=m["rot"]["dims"])
                if m["rot"]["scaling"] is not None:
                    out["rot"]["scaling"] = dict(m["rot"]["scaling"])
            return out

        def mlp(f):
            if f is None or f["kind"] == "dense":
                return None if f is None else dict(f)
            out = dict(kind="moe", router=dict(f["router"]), expert=dict(f["expert"]))
            if f["shared"] is not None:
                out["shared"] = dict(f["shared"])
            return out
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 layers=[dict(type=l.type, mixer=mixer(l.mixer), mlp=mlp(l.mlp)) for l in self.layers])
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    def schedule(self):
        """The runs in order; a run that a pass of the loop starts before carries the pass's number.  Returns (entries,
        passes that start behind the last run)."""
        n = len(self.layers)
        if self.loop is None:
            return [ScheduleEntry(i) for i in range(n)], ()
        entries, pending = [], []

        def run(i):
            entries.append(ScheduleEntry(i, enter=tuple(pending)))
            del pending[:]
        for i in range(self.loop["start"]):
            run(i)
        for t in range(self.loop["times"]):
            pending.append(t)
            for i in range(self.loop["start"], self.loop["stop"]):
                run(i)
        for i in range(self.loop["stop"], n):
            run(i)
        return entries, tuple(pending)

    def model_spec(self):
        W = self.width
        offset = NORM_GAIN_OFFSET

        def norm(name=""):
            return PartSpec("rmsnorm", dict(size=W, eps=self.eps, gain_offset=offset, weight_name=name))

        def out_norm(gain, scale):
            return PartSpec("scaled_output_rmsnorm", dict(size=W, eps=self.eps, gain_offset=offset, gain_name=gain, scale_name=scale))
        layers = []
        for i, l in enumerate(self.layers):
            m = l.mixer
            position = None
            if m["rot"] is not None:
                position = PartSpec("rope_neox", dict(theta=m["rot"]["base"], rotary_dim=m["rot"]["dims"], max_positions=MAX_POSITIONS,
                                                      scaling=m["rot"]["scaling"], wide_frequencies=True))
            mixer = PartSpec("conv_attention", dict(
                hidden_size=W, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
                scale=m["scale"], taps=m["conv"], position=position, sink=SINK_SCORE, window=None))
            parts = dict(mixer=mixer, mixer_norm=norm(), mixer_out_norm=out_norm("norm1b", "ls1"))
            if l.mlp is not None:
                if l.mlp["kind"] == "dense":
                    parts["feed_forward"] = PartSpec("squared_relu", dict(hidden_size=W, intermediate_size=l.mlp["ff"]))
                else:
                    parts["feed_forward"] = PartSpec("routed_glu", dict(
                        hidden_size=W, num_experts=l.mlp["router"]["experts"], top_k=l.mlp["router"]["top"],
                        expert_size=l.mlp["expert"]["ff"],
                        shared_size=None if l.mlp["shared"] is None else l.mlp["shared"]["ff"], router_bias=True))
                parts["feed_forward_norm"] = norm()
                parts["feed_forward_out_norm"] = out_norm("norm2b", "ls2")
            layers.append(LayerSpec(prefix="l%d" % i, parts=parts, arrangement="sandwich", names=dict(LAYER_TENSOR_NAMES)))
        schedule, tail = self.schedule()
        spec = ModelSpec(
            hidden_size=W, vocab_size=self.vocab, layers=layers, schedule=schedule,
            embedding=PartSpec("embedding", dict(vocab_size=self.vocab, hidden_size=W, weight_name="")),
            final_norm=norm(),
            head=PartSpec("lm_head", dict(vocab_size=self.vocab, hidden_size=W, tied=True)),
            max_positions=MAX_POSITIONS, eos_token_ids=list(self.eos_token_ids), names=dict(MODEL_TENSOR_NAMES),
            reentry=None if self.loop is None else PartSpec("concat_projection", dict(hidden_size=W, passes=self.loop["times"])),
            tail_enter=tail)
        spec.validate()
        return spec
