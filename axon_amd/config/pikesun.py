"""The Pikesun decoder's configuration: config.json to a ModelSpec.

config.json names the design in `architecture` and gives `vocab`, `width`, `embedding.scale`,
`norm.eps`, `residual_mult` and a list `layers`.  Every layer has a `type` (which mixer: "rglru",
a gated linear recurrence behind a short convolution, or "latent_attention", windowed attention
over a shared latent), the mixer's sizes (`mixer`) and its feed-forward (`mlp`: dense, a mixture
of experts with an optional shared expert, or null for none).  A layer with `weights_of: j` has
no tensors of its own: it runs layer j's with a cache or state of its own.  Layer i's tensors
start with `l<i>.`; beside them there are `embed`, `final.norm` and `head`.

A layer is x += m norm1(mixer(x)); x += m norm2(mlp(x)) with RMS norms on the sublayers' outputs
and m = `residual_mult`; the embedding row is multiplied by `embedding.scale`.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, get_number, get_whole

# the design leaves positions unbounded; the engine sizes its block tables by this unless told otherwise
UNBOUNDED_POSITIONS = 1 << 20
GATE_DECAY = 8.0            # log a = -8 r softplus(lam)
EXPERT_ALPHA = 1.702        # g sigmoid(1.702 g)


def _object(cfg: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = cfg.get(key)
    if v is None and optional:
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"config.json {where}{key} = {v!r} is not an object")
    return v


class PikesunConfig(ModelConfig):
    architecture = "Pikesun"
    model_type = "pikesun"

    def __init__(self, cfg: Dict[str, Any]):
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        self.cfg = copy.deepcopy(cfg)
        self.width = get_whole(cfg, "width")
        self.vocab = get_whole(cfg, "vocab")
        self.embedding_scale = get_number(_object(cfg, "embedding", "", optional=True) or {}, "scale", 1.0)
        self.eps = get_number(_object(cfg, "norm", ""), "eps")
        self.residual_mult = get_number(cfg, "residual_mult", 1.0)
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers is not a list of layers")
        self.layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json layers[{i}] is not an object")
            kind = entry.get("type")
            mixer = _object(entry, "mixer", where)
            if kind == "rglru":
                spec = PartSpec("gated_recurrence", {
                    "hidden_size": self.width, "width": get_whole(mixer, "width"), "blocks": get_whole(mixer, "blocks"),
                    "conv": get_whole(mixer, "conv"), "decay": GATE_DECAY})
            elif kind == "latent_attention":
                rot_dim = get_whole(mixer, "rot_dim", minimum=0)
                rot = _object(mixer, "rot", where + "mixer.", optional=rot_dim == 0)
                mask = _object(mixer, "mask", where + "mixer.", optional=True)
                position = None
                if rot_dim:
                    position = PartSpec("rope", {"head_dim": rot_dim, "rotary_dim": get_whole(rot, "dims", minimum=2),
                                                 "theta": get_number(rot, "base")})
                spec = PartSpec("latent_attention", {
                    "hidden_size": self.width, "heads": get_whole(mixer, "heads"), "dim": get_whole(mixer, "dim"),
                    "rot_dim": rot_dim, "vdim": get_whole(mixer, "vdim"), "kv_rank": get_whole(mixer, "kv_rank"),
                    "q_rank": get_whole(mixer, "q_rank"), "scale": get_number(mixer, "scale"),
                    "window": get_whole(mask, "size") if mask is not None else 0, "eps": self.eps, "gated": True,
                    "position": position})
            else:
                raise ConfigError(f"config.json {where}type = {kind!r} is not a mixer of this design (rglru, latent_attention)")
            owner = entry.get("weights_of")
            if owner is not None:
                owner = get_whole(entry, "weights_of", minimum=0)
                if owner >= len(layers) or owner == i or not isinstance(layers[owner], dict) or "weights_of" in layers[owner] \
                        or layers[owner].get("type") != kind:
                    raise ConfigError(f"config.json {where}weights_of = {owner} does not name a layer of type {kind} "
                                      "with tensors of its own")
            self.layers.append({"mixer": spec, "mlp": self._mlp(entry.get("mlp"), where), "owner": owner})

    def _mlp(self, mlp, where: str) -> Optional[PartSpec]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json {where}mlp = {mlp!r} is not an object")
        kind = mlp.get("kind")
        if kind == "dense":
            return PartSpec("dense_mlp", {"hidden_size": self.width, "ff": get_whole(mlp, "ff"), "activation": "gelu_tanh"})
        if kind == "moe":
            expert, router = _object(mlp, "expert", where + "mlp."), _object(mlp, "router", where + "mlp.")
            shared = _object(mlp, "shared", where + "mlp.", optional=True)
            return PartSpec("routed_experts", {
                "hidden_size": self.width, "experts": get_whole(router, "experts"), "top": get_whole(router, "top"),
                "ff": get_whole(expert, "ff"), "limit": get_number(expert, "limit"), "alpha": EXPERT_ALPHA,
                "shared": None if shared is None else {"ff": get_whole(shared, "ff"), "limit": get_number(shared, "limit")}})
        raise ConfigError(f"config.json {where}mlp.kind = {kind!r} is not a feed-forward of this design (dense, moe)")

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "PikesunConfig":
        return cls(cfg)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.cfg)

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "residual_mult": self.residual_mult})
        layers, index_of, order = [], {}, []
        for i, layer in enumerate(self.layers):
            if layer["owner"] is None:
                index_of[i] = len(layers)
                layers.append(LayerSpec(block="sublayer_norm", mixer=layer["mixer"], feed_forward=layer["mlp"], norm=norm,
                                        prefix=f"l{i}."))
        for i, layer in enumerate(self.layers):
            # a layer that runs another's tensors has a cache or state of its own
            order.append(Run(layer=index_of[i if layer["owner"] is None else layer["owner"]], cache=i))
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "embed",
                                                   "scale": self.embedding_scale}),
            layers=layers, order=order,
            final_norm=PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "tensor": "final.norm"}),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "head", "tied_to": "embed",
                                      "tied": False}),
            max_positions=UNBOUNDED_POSITIONS)
