"""The Zugutar decoder's configuration: config.json to a ModelSpec.

config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, `logit_scale`, a
list `layers` and, optionally, `loop`.  Every layer has a `type` (which mixer), the mixer's sizes
(`mixer`) and its feed-forward (`mlp`, or null for none):

* "attention": grouped-query attention without rotation (`heads`, `kv_heads`, `dim`, `vdim`, `scale`);
  the query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1) (`q_temp`: `coef`,
  `every`); an ordinary softmax over the earlier positions; a sigmoid gate on every element of the heads;
* "parallel": two mixers side by side on the same input, each output RMS-normed over the width with a
  gain (`left.out`, `right.out`), and half their sum taken.  `left`: attention whose queries and keys are
  normed per head with a gain shared by the heads, the first `rot.dims` places of a head rotated in
  half-apart pairs (`rot.base`), a sink of score 0 in the softmax (one more in its denominator) and a gate a
  head.  `right`: a selective state-space mixer (`heads`, `vdim`, `state`, `groups`, `conv`, `norm_groups`);
* `mlp` {"kind": "moe"}: `router.experts` gated units of `expert.ff`, of which a token takes the
  `router.top` with the largest sigmoid scores, each fed the token's row times its score (not
  renormalised); `shared` (`ff`): one more unit for every token, times the sigmoid of a logit of its own.

A layer is h = norm1(x); x += mixer(h) + mlp(h) with an RMS norm whose gain is stored around zero (1 + w).
`loop` = {start, stop, times}: layers start .. stop - 1 run `times` times in a row with the same tensors,
each pass with caches and states of its own; before every pass but the first the embedding's output is
added to the stream.  Layer i's tensors start with `l<i>.`; beside them there are `embed` (also the head:
logits = embed norm(x) logit_scale) and `final.norm`.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, get_number, get_whole

# the design leaves positions unbounded; the engine sizes its block tables by this unless told otherwise
UNBOUNDED_POSITIONS = 1 << 20


def _object(cfg: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = cfg.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json {where}{key} = {v!r} is not an object")
    return v


class ZugutarConfig(ModelConfig):
    architecture = "Zugutar"
    model_type = "zugutar"

    def __init__(self, cfg: Dict[str, Any]):
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        self.cfg = copy.deepcopy(cfg)
        self.width = get_whole(cfg, "width")
        self.vocab = get_whole(cfg, "vocab")
        self.eps = get_number(_object(cfg, "norm", ""), "eps")
        self.logit_scale = get_number(cfg, "logit_scale", 1.0)
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers is not a list of layers")
        self.layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json layers[{i}] is not an object")
            self.layers.append({"mixer": self._mixer(entry.get("type"), _object(entry, "mixer", where), where + "mixer."),
                                "mlp": self._mlp(entry.get("mlp"), where)})
        loop = _object(cfg, "loop", "", optional=True)
        self.loop = None
        if loop is not None:
            start, stop = get_whole(loop, "start", minimum=0), get_whole(loop, "stop", minimum=0)
            times = get_whole(loop, "times", minimum=0)
            if not start <= stop <= len(layers):
                raise ConfigError(f"config.json loop: layers {start} .. {stop} - 1 of {len(layers)}")
            self.loop = (start, stop, times)

    # ------------------------------------------------------------------ the parts of a layer
    def _heads(self, mixer: Dict[str, Any]) -> Dict[str, Any]:
        return {"hidden_size": self.width, "heads": get_whole(mixer, "heads"), "kv_heads": get_whole(mixer, "kv_heads"),
                "dim": get_whole(mixer, "dim"), "vdim": get_whole(mixer, "vdim"), "scale": get_number(mixer, "scale"),
                "eps": self.eps, "maps": 1, "values": "projected", "mask": {"kind": "causal"}}

    def _mixer(self, kind, mixer: Dict[str, Any], where: str) -> PartSpec:
        if kind == "attention":
            temp = _object(mixer, "q_temp", where, optional=True)
            q_temp = None
            if temp is not None and get_number(temp, "coef", 0.0, positive=False) != 0.0:
                q_temp = {"coef": get_number(temp, "coef", positive=False), "every": get_whole(temp, "every")}
            return PartSpec("masked_attention", {**self._heads(mixer), "gate": "elements", "q_temp": q_temp, "position": None})
        if kind == "parallel":
            left, right = _object(mixer, "left", where), _object(mixer, "right", where)
            rot = _object(left, "rot", where + "left.", optional=True)
            position = None
            if rot is not None and get_whole(rot, "dims", minimum=0) > 0:
                position = PartSpec("rope", {"head_dim": get_whole(left, "dim"), "rotary_dim": get_whole(rot, "dims", minimum=2),
                                             "theta": get_number(rot, "base"), "pairing": "halves"})
            attention = PartSpec("masked_attention", {
                **self._heads(left), "qk_norm": True, "sink": 0.0, "gate": "heads", "position": position,
                "names": {"scope": "mix.left."}})
            state_space = PartSpec("selective_state_space", {
                "hidden_size": self.width, "heads": get_whole(right, "heads"), "vdim": get_whole(right, "vdim"),
                "state": get_whole(right, "state"), "groups": get_whole(right, "groups"), "conv": get_whole(right, "conv"),
                "norm_groups": get_whole(right, "norm_groups", 1), "eps": self.eps, "names": {"scope": "mix.right."}})
            return PartSpec("paired_mixers", {"hidden_size": self.width, "eps": self.eps, "mult": 0.5, "left": attention,
                                              "right": state_space})
        raise ConfigError(f"config.json {where[:-6]}type = {kind!r} is not a mixer of this design (attention, parallel)")

    def _mlp(self, mlp, where: str) -> Optional[PartSpec]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json {where}mlp = {mlp!r} is not an object")
        if mlp.get("kind") != "moe":
            raise ConfigError(f"config.json {where}mlp.kind = {mlp.get('kind')!r} is not a feed-forward of this design (moe)")
        expert, router = _object(mlp, "expert", where + "mlp."), _object(mlp, "router", where + "mlp.")
        shared = _object(mlp, "shared", where + "mlp.", optional=True)
        return PartSpec("routed_experts", {
            "hidden_size": self.width, "experts": get_whole(router, "experts"), "top": get_whole(router, "top"),
            "ff": get_whole(expert, "ff"), "limit": None, "alpha": 1.0, "shift": 0.0, "weight_on": "input",
            "router": {"scores": "sigmoid", "normalize": False},
            "shared": None if shared is None else {"ff": get_whole(shared, "ff"), "unit": "gated", "gate": "sg"}})

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "ZugutarConfig":
        return cls(cfg)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.cfg)

    # ------------------------------------------------------------------ the model as data
    def run_order(self) -> List[tuple]:
        """(layer, whether a pass of the loop other than the first begins with it) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        order = [(i, False) for i in range(start)]
        for k in range(times):
            order += [(i, k > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "offset": 1.0})
        layers = [LayerSpec(block="parallel", mixer=layer["mixer"], feed_forward=layer["mlp"], norm=norm, prefix=f"l{i}.")
                  for i, layer in enumerate(self.layers)]
        # every run has a cache and a state of its own: a layer of the loop keeps one per pass
        order = [Run(layer=i, cache=at, enter=0 if again else None) for at, (i, again) in enumerate(self.run_order())]
        entries = (PartSpec("embedding_add", {"factor": 1.0}),) if any(again for _, again in self.run_order()) else ()
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "embed"}),
            layers=layers, order=order,
            final_norm=PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "tensor": "final.norm", "offset": 1.0}),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "head", "tied_to": "embed",
                                      "tied": True, "scale": self.logit_scale}),
            max_positions=UNBOUNDED_POSITIONS, entries=entries)
