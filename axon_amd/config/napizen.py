"""The Napizen decoder's configuration: config.json to a ModelSpec.

config.json names the design in `architecture` and gives `vocab`, `width`, `embedding.scale`,
`norm.eps`, `postln_alpha`, `logit_softcap` and a list `layers`.  Every layer has a `type` (which
mixer: "latent_attention", causal attention over a shared latent with a sink in its softmax and a gate
a head), the mixer's sizes (`mixer`: `heads`, `dim`, `rot_dim`, `vdim`, `kv_rank`, `scale`, and `rot`:
`base`, `dims`, optionally `scaling`: `factor`, `original`, `fast`, `slow`) and its feed-forward (`mlp`:
`kind` "dense" with `ff`; `kind` "moe" with `expert.ff` and `router`: `experts`, `top`, `scale`,
`groups`: `count`, `keep`; or null for none).  Layer i's tensors start with `l<i>.`; beside them there are
`embed`, `final.norm` and `head`.

A layer is x <- ln1(alpha x + mixer(x)); x <- ln2(alpha x + mlp(x)) with layer norms (a gain, no bias)
behind the sums and alpha = `postln_alpha`; the embedding row is multiplied by `embedding.scale`; the
logits are bent, cap tanh(z / cap) with cap = `logit_softcap`.  Queries and the shared key part rotate in
neighbouring pairs (2i, 2i + 1); with `scaling` the pairs' frequencies are ramped by pair index and cos
and sin are scaled (the position encoding's "ramp").  Feed-forwards are gated units, silu(gate) up; the
router's scores are sigmoids, the choice goes by score + `correction` within the best groups, the
weights are the chosen scores over their sum, times `router.scale`.
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


class NapizenConfig(ModelConfig):
    architecture = "Napizen"
    model_type = "napizen"

    def __init__(self, cfg: Dict[str, Any]):
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        self.cfg = copy.deepcopy(cfg)
        self.width = get_whole(cfg, "width")
        self.vocab = get_whole(cfg, "vocab")
        self.embedding_scale = get_number(_object(cfg, "embedding", "", optional=True) or {}, "scale", 1.0)
        self.eps = get_number(_object(cfg, "norm", ""), "eps")
        self.alpha = get_number(cfg, "postln_alpha", 1.0)
        self.softcap = get_number(cfg, "logit_softcap", 0.0, positive=False)
        if self.softcap < 0:
            raise ConfigError(f"config.json logit_softcap = {self.softcap} must not be below 0")
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers is not a list of layers")
        self.layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json layers[{i}] is not an object")
            kind = entry.get("type")
            if kind != "latent_attention":
                raise ConfigError(f"config.json {where}type = {kind!r} is not a mixer of this design (latent_attention)")
            self.layers.append({"mixer": self._mixer(_object(entry, "mixer", where), where + "mixer."),
                                "mlp": self._mlp(entry.get("mlp"), where)})

    def _mixer(self, mixer: Dict[str, Any], where: str) -> PartSpec:
        rot_dim = get_whole(mixer, "rot_dim", minimum=0)
        position = None
        if rot_dim:
            rot = _object(mixer, "rot", where)
            params = {"head_dim": rot_dim, "rotary_dim": get_whole(rot, "dims", minimum=2), "theta": get_number(rot, "base"),
                      "pairing": "neighbours"}
            scaling = _object(rot, "scaling", where + "rot.", optional=True)
            if scaling is not None:
                params["scaling"] = {"kind": "ramp", "factor": get_number(scaling, "factor"),
                                     "original": get_number(scaling, "original"), "fast": get_number(scaling, "fast"),
                                     "slow": get_number(scaling, "slow")}
            position = PartSpec("rope", params)
        return PartSpec("latent_attention", {
            "hidden_size": self.width, "heads": get_whole(mixer, "heads"), "dim": get_whole(mixer, "dim"), "rot_dim": rot_dim,
            "vdim": get_whole(mixer, "vdim"), "kv_rank": get_whole(mixer, "kv_rank"), "q_rank": 0,
            "scale": get_number(mixer, "scale"), "window": 0, "eps": self.eps, "gate": "heads", "sink": True,
            "position": position})

    def _mlp(self, mlp, where: str) -> Optional[PartSpec]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json {where}mlp = {mlp!r} is not an object")
        kind = mlp.get("kind")
        names = {"gate": "gate", "up": "up", "down": "down", "suffix": ""}
        if kind == "dense":
            return PartSpec("swiglu_mlp", {"hidden_size": self.width, "intermediate_size": get_whole(mlp, "ff"), "names": names})
        if kind == "moe":
            expert, router = _object(mlp, "expert", where + "mlp."), _object(mlp, "router", where + "mlp.")
            groups = _object(router, "groups", where + "mlp.router.", optional=True) or {}
            return PartSpec("routed_experts", {
                "hidden_size": self.width, "experts": get_whole(router, "experts"), "top": get_whole(router, "top"),
                "ff": get_whole(expert, "ff"), "limit": None, "alpha": 1.0, "shift": 0.0,
                "router": {"scores": "sigmoid", "correction": True, "groups": get_whole(groups, "count", 1),
                           "keep": get_whole(groups, "keep", 1), "scale": get_number(router, "scale", 1.0)}})
        raise ConfigError(f"config.json {where}mlp.kind = {kind!r} is not a feed-forward of this design (dense, moe)")

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "NapizenConfig":
        return cls(cfg)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.cfg)

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("layernorm", {"size": self.width, "eps": self.eps, "stream_alpha": self.alpha})
        layers = [LayerSpec(block="postnorm", mixer=layer["mixer"], feed_forward=layer["mlp"], norm=norm, prefix=f"l{i}.")
                  for i, layer in enumerate(self.layers)]
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "embed",
                                                   "scale": self.embedding_scale}),
            layers=layers, order=[Run(layer=i, cache=i) for i in range(len(layers))],
            final_norm=PartSpec("layernorm", {"size": self.width, "eps": self.eps, "tensor": "final.norm"}),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "head", "tied_to": "embed",
                                      "tied": False, "softcap": self.softcap}),
            max_positions=UNBOUNDED_POSITIONS)
