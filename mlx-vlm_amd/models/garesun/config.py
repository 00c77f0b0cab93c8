"""config.json of a Garesun checkpoint.  Every size and every constant that may differ between checkpoints is read here;
what the design fixes (activation functions, the 1e-6 of the gated denominator, layouts of the rotations) lives in the
kernels.  Unknown mixer types / feed-forward kinds are refused at load, not at the first step."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

MIXERS = ("retention", "mlstm", "latent_attention")


@dataclass
class LayerConfig:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None

    def __post_init__(self):
        if self.type not in MIXERS:
            raise ValueError(f"Garesun layer type {self.type!r}: one of {MIXERS}")
        m = self.mixer
        need = {"retention": ("heads", "dim", "vdim", "decay", "rot"), "mlstm": ("heads", "dim", "vdim", "gate_cap"),
                "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot")}[self.type]
        missing = [k for k in need if k not in m]
        if missing:
            raise ValueError(f"Garesun {self.type} mixer: missing {missing}")
        if self.type == "retention" and len(m["decay"]) != m["heads"]:
            raise ValueError("retention: one decay per head")
        if self.mlp is not None:
            if self.mlp.get("kind", "moe") != "moe":
                raise ValueError(f"Garesun feed-forward kind {self.mlp.get('kind')!r}: 'moe'")
            r = self.mlp["router"]
            if not 0 < int(r["top"]) <= int(r["experts"]):
                raise ValueError("moe: 0 < top <= experts")

    # ---- feed-forward sizes (0 when absent)
    @property
    def experts(self) -> int:
        return int(self.mlp["router"]["experts"]) if self.mlp else 0

    @property
    def top(self) -> int:
        return int(self.mlp["router"]["top"]) if self.mlp else 0

    @property
    def expert_ff(self) -> int:
        return int(self.mlp["expert"]["ff"]) if self.mlp else 0

    @property
    def shared_ff(self) -> int:
        sh = (self.mlp or {}).get("shared")
        return int(sh["ff"]) if sh else 0


@dataclass
class ModelConfig:
    vocab: int = 0
    width: int = 0
    layers: List[LayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    side_dim: int = 0                      # per-layer token input width (0: none)
    model_type: str = "garesun"
    eos_token_id: Any = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        layers = [LayerConfig(type=L["type"], mixer=dict(L["mixer"]), mlp=(dict(L["mlp"]) if L.get("mlp") else None))
                  for L in d["layers"]]
        for i, L in enumerate(layers):
            src = L.mixer.get("kv_from")
            if L.type == "latent_attention" and src is not None:
                if not (0 <= int(src) < i) or layers[int(src)].type != "latent_attention" or layers[int(src)].mixer.get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier latent_attention layer that writes its own cache")
                s = layers[int(src)].mixer
                if (s["kv_rank"], s["rot_dim"], s["rot"]) != (L.mixer["kv_rank"], L.mixer["rot_dim"], L.mixer["rot"]):
                    raise ValueError(f"layer {i}: kv_from layer {src} has another kv_rank / rot_dim / rotation")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                   side_dim=int((d.get("token_side") or {}).get("dim", 0) or 0), eos_token_id=d.get("eos_token_id"))

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
