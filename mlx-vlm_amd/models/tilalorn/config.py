"""config.json of a Tilalorn checkpoint.  Every size and every constant that may differ between checkpoints is read here;
what the design fixes (activation functions, the rotate-half layout of the rotation, norm weights kept as offsets from one) lives
in the model code and the kernels.  Unknown mixer types / feed-forward kinds and inconsistent sizes are refused at load."""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

MIXERS = ("attention", "latent_attention")


def _need(d: Dict[str, Any], keys, what: str):
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"Tilalorn {what}: missing {missing}")


@dataclass
class LayerConfig:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None

    def __post_init__(self):
        if self.type not in MIXERS:
            raise ValueError(f"Tilalorn layer type {self.type!r}: one of {MIXERS}")
        m = self.mixer
        if self.type == "attention":
            _need(m, ("heads", "kv_heads", "dim", "scale"), "attention mixer")
            m.setdefault("vdim", m["dim"])
            if int(m["heads"]) % int(m["kv_heads"]) or int(m["kv_heads"]) < 1:
                raise ValueError("attention: heads must be a multiple of kv_heads")
            qt = m.get("q_temp")
            if qt is not None:
                _need(qt, ("coef", "every"), "attention q_temp")
                if int(qt["every"]) < 1:
                    raise ValueError("attention: q_temp.every is at least 1")
            if m.get("softcap") is not None and not float(m["softcap"]) > 0:
                raise ValueError("attention: softcap must be positive")
        else:
            _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"), "latent_attention mixer")
            Dr = int(m["rot_dim"])
            if Dr:
                _need(m, ("rot",), "latent_attention mixer")
                _need(m["rot"], ("base",), "latent_attention rot")
                if int(m["rot"].get("dims", Dr)) != Dr or Dr % 2:
                    raise ValueError(f"latent_attention: the rotated part is rot_dim wide and even (rot.dims {m['rot'].get('dims')}, rot_dim {Dr})")
        win = (m.get("mask") or {}).get("size")
        if win is not None and int(win) < 1:
            raise ValueError("mask.size is at least 1")
        if self.mlp is not None:
            kind = self.mlp.get("kind", "dense")
            if kind == "dense":
                _need(self.mlp, ("ff",), "dense feed-forward")
            elif kind == "moe":
                _need(self.mlp, ("expert", "router"), "mixture of experts")
                r = self.mlp["router"]
                _need(r, ("experts", "top"), "router")
                E, top = int(r["experts"]), int(r["top"])
                g = r.get("groups") or {}
                count, keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
                if not 0 < top <= E or count < 1 or E % count or not 0 < keep <= count or top > keep * (E // count):
                    raise ValueError("moe: 0 < top <= experts, experts a multiple of groups.count, 0 < groups.keep <= groups.count, "
                                     "top no more than the kept groups hold")
            else:
                raise ValueError(f"Tilalorn feed-forward kind {kind!r}: 'dense' or 'moe'")

    # ---- what the entry says, with the defaults of what it may leave out
    @property
    def window(self) -> int:
        """0: every earlier token is seen"""
        win = (self.mixer.get("mask") or {}).get("size")
        return int(win) if win is not None else 0

    @property
    def kv_from(self) -> Optional[int]:
        src = self.mixer.get("kv_from")
        return None if src is None else int(src)

    @property
    def moe(self) -> bool:
        return self.mlp is not None and self.mlp.get("kind", "dense") == "moe"

    @property
    def ff(self) -> int:
        if self.mlp is None:
            return 0
        return int(self.mlp["expert"]["ff"]) if self.moe else int(self.mlp["ff"])

    @property
    def router(self):
        """(experts, top, groups, kept groups, weight scale)"""
        r = self.mlp["router"]
        g = r.get("groups") or {}
        count = int(g.get("count", 1))
        return int(r["experts"]), int(r["top"]), count, int(g.get("keep", count)), float(r.get("scale", 1.0))


def _cache_sizes(lc: LayerConfig):
    m = lc.mixer
    if lc.type == "attention":
        return [int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])]
    return [int(m["kv_rank"]), int(m["rot_dim"]), float((m.get("rot") or {}).get("base", 0.0))]


@dataclass
class ModelConfig:
    vocab: int = 0
    width: int = 0
    layers: List[LayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    model_type: str = "tilalorn"
    eos_token_id: Any = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        _need(d, ("vocab", "width", "layers", "norm"), "config")
        raw = [copy.deepcopy(L["mixer"]) for L in d["layers"]]
        for i, m in enumerate(raw):
            # a layer that reads another layer's cache may leave the cache's sizes to that layer's entry
            j = m.get("kv_from")
            if j is not None and isinstance(j, int) and 0 <= j < len(raw) and j != i:
                for k in ("kv_heads", "vdim", "kv_rank", "rot_dim", "rot"):
                    if k not in m and k in raw[j]:
                        m[k] = copy.deepcopy(raw[j][k])
        layers = [LayerConfig(type=L["type"], mixer=m, mlp=(copy.deepcopy(L["mlp"]) if L.get("mlp") else None))
                  for L, m in zip(d["layers"], raw)]
        for i, lc in enumerate(layers):
            j = lc.kv_from
            if j is None:
                continue
            # the source's cache must hold this step's tokens when the layer runs: an earlier layer.  A source that itself
            # reads another layer's cache is followed to the layer that writes it
            while 0 <= j < i and layers[j].type == lc.type and layers[j].kv_from is not None:
                j = layers[j].kv_from
            if not 0 <= j < i or layers[j].type != lc.type:
                raise ValueError(f"layer {i}: kv_from must name an earlier {lc.type} layer")
            lc.mixer["kv_from"] = j
            if _cache_sizes(layers[j]) != _cache_sizes(lc):
                raise ValueError(f"layer {i}: layer {j}, whose cache it reads, has other cache sizes")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float(d["norm"]["eps"]),
                   residual_mult=float(d.get("residual_mult", 1.0)), eos_token_id=d.get("eos_token_id"))

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
