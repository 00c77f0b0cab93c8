"""config.json of a Luvapel checkpoint.  Every size and every constant that may differ between checkpoints is read here;
what the design fixes (activation functions, the 1e-6 of the unit vectors, the exp(-1/2) of the decay, layouts of the
rotation) lives in the kernels.  Unknown mixer types / feed-forward kinds and inconsistent sizes are refused at load."""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

MIXERS = ("parallel", "general_delta")


def _need(d: Dict[str, Any], keys, what: str):
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"Luvapel {what}: missing {missing}")


@dataclass
class LayerConfig:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None
    weights_of: Optional[int] = None       # the layer whose tensors this one uses (own cache / state)

    def __post_init__(self):
        if self.type not in MIXERS:
            raise ValueError(f"Luvapel layer type {self.type!r}: one of {MIXERS}")
        m = self.mixer
        if self.type == "general_delta":
            _need(m, ("heads", "dim"), "general_delta mixer")
        else:
            _need(m, ("left", "right"), "parallel mixer")
            a, r = m["left"], m["right"]
            _need(a, ("heads", "kv_heads", "dim", "scale"), "parallel.left")
            a.setdefault("vdim", a["dim"])
            a.setdefault("rot", {"dims": 0, "base": 10000.0})          # an entry without them: no rotation / no window
            a.setdefault("mask", {"size": None})
            _need(r, ("heads", "kv_heads", "dim", "vdim", "conv"), "parallel.right")
            if int(a["heads"]) % int(a["kv_heads"]) or int(r["heads"]) % int(r["kv_heads"]):
                raise ValueError("parallel mixer: heads must be a multiple of kv_heads")
            if int(a["vdim"]) != int(a["dim"]):
                raise ValueError("parallel.left: the values are the projected keys, so vdim must equal dim")
            dims = int(a["rot"]["dims"])
            if dims % 2 or not 0 <= dims <= int(a["dim"]):
                raise ValueError(f"parallel.left: rot.dims {dims} for head dim {a['dim']}")
            if (a["mask"]["size"] is not None and int(a["mask"]["size"]) < 1) or int(r["conv"]) < 1:
                raise ValueError("parallel mixer: mask.size and conv are at least 1")
        if self.mlp is not None:
            if self.mlp.get("kind", "dense") != "dense":
                raise ValueError(f"Luvapel feed-forward kind {self.mlp.get('kind')!r}: 'dense'")
            _need(self.mlp, ("ff",), "feed-forward")


def _shape_sizes(lc: LayerConfig):
    """the sizes of an entry that decide tensor shapes (a borrowing layer must agree on them with its source; window,
    rotation, score scale are read from the layer's own entry)"""
    m = lc.mixer
    if lc.type == "general_delta":
        sizes = [int(m["heads"]), int(m["dim"])]
    else:
        a, r = m["left"], m["right"]
        sizes = [int(a[k]) for k in ("heads", "kv_heads", "dim")] + [int(r[k]) for k in ("heads", "kv_heads", "dim", "vdim", "conv")]
    return sizes + [int(lc.mlp["ff"]) if lc.mlp is not None else 0]


@dataclass
class ModelConfig:
    vocab: int = 0
    width: int = 0
    layers: List[LayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    model_type: str = "luvapel"
    eos_token_id: Any = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        layers = []
        for L in d["layers"]:
            src = L.get("weights_of")
            layers.append(LayerConfig(type=L["type"], mixer=copy.deepcopy(L["mixer"]), mlp=(dict(L["mlp"]) if L.get("mlp") else None),
                                      weights_of=None if src is None else int(src)))
        for i, lc in enumerate(layers):
            # the source may stand before or after the layer; a source that itself borrows is followed to the owner
            j, seen = lc.weights_of, {i}
            while j is not None:
                if not 0 <= j < len(layers) or j in seen:
                    raise ValueError(f"layer {i}: weights_of must lead to a layer that has tensors of its own")
                seen.add(j)
                if layers[j].weights_of is None:
                    break
                j = layers[j].weights_of
            if j is not None:
                o = layers[j]
                if o.type != lc.type or _shape_sizes(o) != _shape_sizes(lc):
                    raise ValueError(f"layer {i}: its sizes differ from layer {j}, whose weights it uses")
                lc.weights_of = j
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), eos_token_id=d.get("eos_token_id"))

    # names other parts of the package read from a text config
    @property
    def vocab_size(self):
        return self.vocab

    @property
    def hidden_size(self):
        return self.width

    @property
    def num_hidden_layers(self):
        return len(self.layers)
