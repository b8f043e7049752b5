"""The Figalorn decoder's configuration: config.json to a ModelSpec.

config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, a list
`layers` and, optionally, `loop`.  Every layer has a `type` (which mixer), the mixer's sizes
(`mixer`) and its feed-forward (`mlp`: {"kind": "dense", "ff": n}, or null for none):

* "attention": differential attention (two score maps a head over one set of values, combined
  with a factor made of four vectors and `diff`, normed), biases on q, k and v, rotation of the
  leading `rot.dims` of each map in neighbouring pairs with the frequencies stretched by
  wavelength (`rot.scaling`: factor, low, high, original), chunks of `mask.size` positions, a
  sigmoid gate on the heads;
* "attention_2": the values are the keys as projected, queries and keys normed per head with a
  gain, rotation in half-apart pairs with the frequencies ramped by pair index (`rot.scaling`:
  factor, original, fast, slow; cos and sin scaled), scores bent by `softcap`, a sliding window
  of `mask.size`.

A layer is x += mixer(norm1 x); x += mlp(norm2 x) with RMS norms whose gains are stored around
zero (1 + w), the feed-forward is down(gelu(up h)) with the exact GELU.  `loop` = {start, stop,
times}: layers start .. stop - 1 run `times` times in a row with the same tensors, each pass with
caches of its own and each beginning with x <- W_in [x ; x0] (`loop.in`, x0 the embedding's
output).  Layer i's tensors start with `l<i>.`; beside them there are `embed`, `final.norm`, `head`.
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


class FigalornConfig(ModelConfig):
    architecture = "Figalorn"
    model_type = "figalorn"

    def __init__(self, cfg: Dict[str, Any]):
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        self.cfg = copy.deepcopy(cfg)
        self.width = get_whole(cfg, "width")
        self.vocab = get_whole(cfg, "vocab")
        self.eps = get_number(_object(cfg, "norm", ""), "eps")
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers is not a list of layers")
        self.layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json layers[{i}] is not an object")
            self.layers.append({"mixer": self._mixer(entry.get("type"), _object(entry, "mixer", where), where),
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
    def _rotation(self, mixer, where: str, pairing: str, scaling_kind: str, keys) -> Optional[PartSpec]:
        rot = _object(mixer, "rot", where + "mixer.", optional=True)
        if rot is None or get_whole(rot, "dims", minimum=0) == 0:
            return None
        scaling = _object(rot, "scaling", where + "mixer.rot.", optional=True)
        params = {"head_dim": get_whole(mixer, "dim"), "rotary_dim": get_whole(rot, "dims", minimum=2),
                  "theta": get_number(rot, "base"), "pairing": pairing}
        if scaling is not None:
            params["scaling"] = {"kind": scaling_kind, **{k: get_number(scaling, k) for k in keys}}
        return PartSpec("rope", params)

    def _mixer(self, kind, mixer, where: str) -> PartSpec:
        if kind not in ("attention", "attention_2"):
            raise ConfigError(f"config.json {where}type = {kind!r} is not a mixer of this design (attention, attention_2)")
        mask = _object(mixer, "mask", where + "mixer.", optional=True)
        common = {"hidden_size": self.width, "heads": get_whole(mixer, "heads"), "kv_heads": get_whole(mixer, "kv_heads"),
                  "dim": get_whole(mixer, "dim"), "vdim": get_whole(mixer, "vdim"), "scale": get_number(mixer, "scale"),
                  "eps": self.eps}
        if kind == "attention":
            return PartSpec("masked_attention", {
                **common, "maps": 2, "diff": get_number(mixer, "diff", positive=False), "values": "projected", "bias": True,
                "gate": True, "mask": {"kind": "chunk", "size": get_whole(mask, "size")} if mask is not None else None,
                "position": self._rotation(mixer, where, "neighbours", "stretch", ("factor", "low", "high", "original"))})
        softcap = get_number(mixer, "softcap", 0.0)
        return PartSpec("masked_attention", {
            **common, "maps": 1, "values": "keys", "qk_norm": True, "softcap": softcap,
            "mask": {"kind": "window", "size": get_whole(mask, "size")} if mask is not None else None,
            "position": self._rotation(mixer, where, "halves", "ramp", ("factor", "original", "fast", "slow"))})

    def _mlp(self, mlp, where: str) -> Optional[PartSpec]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json {where}mlp = {mlp!r} is not an object")
        if mlp.get("kind") != "dense":
            raise ConfigError(f"config.json {where}mlp.kind = {mlp.get('kind')!r} is not a feed-forward of this design (dense)")
        return PartSpec("dense_mlp", {"hidden_size": self.width, "ff": get_whole(mlp, "ff"), "activation": "gelu_erf"})

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "FigalornConfig":
        return cls(cfg)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.cfg)

    # ------------------------------------------------------------------ the model as data
    def run_order(self) -> List[tuple]:
        """(layer, begins a pass of the loop) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        order = [(i, False) for i in range(start)]
        for _ in range(times):
            order += [(i, i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "offset": 1.0})
        layers = [LayerSpec(block="prenorm_short_names", mixer=layer["mixer"], feed_forward=layer["mlp"], norm=norm,
                            prefix=f"l{i}.") for i, layer in enumerate(self.layers)]
        # every run has a cache of its own: a layer of the loop keeps one per pass
        order = [Run(layer=i, cache=at, enter=0 if begins else None) for at, (i, begins) in enumerate(self.run_order())]
        entries = (PartSpec("embedding_mix", {"hidden_size": self.width, "tensor": "loop.in"}),) if self.loop is not None else ()
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "embed"}),
            layers=layers, order=order,
            final_norm=PartSpec("rmsnorm", {"size": self.width, "eps": self.eps, "tensor": "final.norm", "offset": 1.0}),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tensor": "head", "tied_to": "embed",
                                      "tied": False}),
            max_positions=UNBOUNDED_POSITIONS, entries=entries)
