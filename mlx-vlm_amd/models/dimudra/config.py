"""config.json of a Dimudra checkpoint.  Every size and every constant that may differ between checkpoints is read here; what the
design fixes (activation functions, the rotate-half layout, two best members ranking a group of experts, the sink's score of 0)
lives in the model code and the kernels.  Unknown mixer types / feed-forward kinds and inconsistent sizes are refused at load."""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

MIXERS = ("parallel", "hgrn2", "attention")


def _need(d: Dict[str, Any], keys, what: str):
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"Dimudra {what}: missing {missing}")


def _check_attention(m: Dict[str, Any], what: str):
    _need(m, ("heads", "kv_heads", "dim", "scale"), what)
    m.setdefault("vdim", m["dim"])
    if int(m["kv_heads"]) < 1 or int(m["heads"]) % int(m["kv_heads"]):
        raise ValueError(f"{what}: heads must be a multiple of kv_heads")
    win = (m.get("mask") or {}).get("size")
    if win is not None and int(win) < 1:
        raise ValueError(f"{what}: mask.size is at least 1")
    rot = m.get("rot")
    if rot:
        _need(rot, ("base", "dims"), what + " rot")
        if int(rot["dims"]) % 2 or not 0 <= int(rot["dims"]) <= int(m["dim"]):
            raise ValueError(f"{what}: rot.dims is even and at most dim")


@dataclass
class LayerConfig:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None

    def __post_init__(self):
        if self.type not in MIXERS:
            raise ValueError(f"Dimudra layer type {self.type!r}: one of {MIXERS}")
        m = self.mixer
        if self.type == "parallel":
            _need(m, ("left", "right", "left_scale", "right_scale"), "parallel mixer")
            _check_attention(m["left"], "parallel mixer, left")
            _need(m["right"], ("inner", "state", "dt_rank", "conv"), "parallel mixer, right")
            r = m["right"]
            if min(int(r["inner"]), int(r["state"]), int(r["dt_rank"]), int(r["conv"])) < 1:
                raise ValueError("parallel mixer, right: inner, state, dt_rank and conv are at least 1")
        elif self.type == "hgrn2":
            _need(m, ("heads", "dim", "vdim"), "hgrn2 mixer")
        else:
            _check_attention(m, "attention mixer")
        if self.mlp is not None:
            kind = self.mlp.get("kind", "moe")
            if kind != "moe":
                raise ValueError(f"Dimudra feed-forward kind {kind!r}: 'moe'")
            _need(self.mlp, ("expert", "router"), "mixture of experts")
            _need(self.mlp["expert"], ("ff",), "expert")
            _need(self.mlp["router"], ("experts", "top"), "router")
            E, top, count, keep = self.router
            if not 0 < top <= E or count < 1 or E % count or not 0 < keep <= count or top > keep * (E // count):
                raise ValueError("moe: 0 < top <= experts, experts a multiple of groups.count, 0 < groups.keep <= groups.count, "
                                 "top no more than the kept groups hold")
            if self.mlp.get("shared"):
                _need(self.mlp["shared"], ("ff",), "shared expert")

    @property
    def router(self) -> Tuple[int, int, int, int]:
        """(experts, top, groups, kept groups)"""
        r = self.mlp["router"]
        g = r.get("groups") or {}
        count = int(g.get("count", 1))
        return int(r["experts"]), int(r["top"]), count, int(g.get("keep", count))

    @property
    def ff(self) -> int:
        return int(self.mlp["expert"]["ff"]) if self.mlp is not None else 0

    @property
    def shared_ff(self) -> int:
        return int(self.mlp["shared"]["ff"]) if self.mlp is not None and self.mlp.get("shared") else 0


def attention_constants(m: Dict[str, Any]):
    """(heads, kv_heads, dim, vdim, scale, window (0: none), rot dims, rot base) of an attention entry"""
    win = (m.get("mask") or {}).get("size")
    rot = m.get("rot") or {}
    return (int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), int(win) if win is not None else 0,
            int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))


@dataclass
class ModelConfig:
    vocab: int = 0
    width: int = 0
    layers: List[LayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    canon_taps: int = 0                    # 0: the mixers read the normed stream as it is
    loop: Tuple[int, int, int] = (0, 0, 1)      # layers start .. stop - 1 run `times` times in a row
    model_type: str = "dimudra"
    eos_token_id: Any = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        _need(d, ("vocab", "width", "layers", "norm"), "config")
        layers = [LayerConfig(type=L["type"], mixer=copy.deepcopy(L["mixer"]), mlp=(copy.deepcopy(L["mlp"]) if L.get("mlp") else None))
                  for L in d["layers"]]
        lp = d.get("loop") or {}
        a, b, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
        if lp and not (0 <= a <= b <= len(layers) and times >= 1):
            raise ValueError("loop: 0 <= start <= stop <= number of layers, times at least 1")
        taps = int((d.get("canon") or {}).get("taps", 0))
        if taps < 0 or taps > 16:
            raise ValueError("canon.taps: 1 to 16")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), canon_taps=taps, loop=(a, b, times),
                   eos_token_id=d.get("eos_token_id"))

    def runs(self) -> List[Tuple[int, bool]]:
        """The order in which layers run: [(layer, the embedding output is added to the stream before it)].  Every run has a
        cache / state of its own; the runs of one layer share its tensors."""
        a, b, times = self.loop
        n = len(self.layers)
        if b <= a or times <= 1:
            return [(i, False) for i in range(n)]
        out = [(i, False) for i in range(a)]
        for rep in range(times):
            out += [(i, rep > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

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
