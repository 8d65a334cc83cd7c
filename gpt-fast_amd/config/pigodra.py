"""Typed configuration of the Pigodra decoder: a stack whose layers are listed one by one in
``config.json``, each with a mixer of its own kind and sizes and an optional feed-forward.

    {"architecture": "Pigodra", "vocab": V, "width": D, "norm": {"eps": e},
     "embedding": {"scale": s},
     "layers": [{"type": "mlstm", "mixer": {"heads", "dim", "vdim", "gate_cap"}, "mlp": null},
                {"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "diff",
                           "mask": {"size", "keep_first"},
                           "rot": {"dims", "base", "scaling": {"factor"}}},
                 "mlp": {"kind": "dense", "ff": F}}, ...]}

Every size and constant is read from there; nothing is assumed equal between layers.
"""
from dataclasses import dataclass
from typing import Optional, Tuple


class ConfigError(ValueError):
    pass


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"Pigodra config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class MatrixMemoryMixer:
    heads: int
    dim: int
    vdim: int
    gate_cap: Optional[float]

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}
        if self.gate_cap is not None:
            d["gate_cap"] = self.gate_cap
        return d


@dataclass(frozen=True)
class DifferentialMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: Optional[float]
    diff: float
    window: Optional[int]
    keep_first: int
    rot_dims: int
    rot_base: float
    rot_factor: Optional[float]

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
             "diff": self.diff}
        if self.scale is not None:
            d["scale"] = self.scale
        if self.window is not None or self.keep_first:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        rot = {"dims": self.rot_dims, "base": self.rot_base}
        if self.rot_factor is not None:
            rot["scaling"] = {"factor": self.rot_factor}
        d["rot"] = rot
        return d


@dataclass(frozen=True)
class DenseMlp:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class PigodraLayer:
    type: str                 # "mlstm" | "attention"
    mixer: object
    mlp: Optional[DenseMlp]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_layer(i: int, d: dict) -> PigodraLayer:
    where = f"layers[{i}]"
    kind = _need(d, "type", where)
    m = _need(d, "mixer", where)
    if kind == "mlstm":
        cap = m.get("gate_cap")
        mixer = MatrixMemoryMixer(heads=int(_need(m, "heads", where)), dim=int(_need(m, "dim", where)),
                                  vdim=int(_need(m, "vdim", where)),
                                  gate_cap=None if cap is None else float(cap))
    elif kind == "attention":
        mask = m.get("mask") or {}
        rot = m.get("rot") or {}
        scaling = rot.get("scaling") or {}
        heads = int(_need(m, "heads", where))
        mixer = DifferentialMixer(
            heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(_need(m, "dim", where)),
            vdim=int(_need(m, "vdim", where)),
            scale=None if m.get("scale") is None else float(m["scale"]),
            diff=float(_need(m, "diff", where)),
            window=None if mask.get("size") is None else int(mask["size"]),
            keep_first=int(mask.get("keep_first") or 0),
            rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base", 10000.0)),
            rot_factor=None if scaling.get("factor") is None else float(scaling["factor"]))
        if mixer.heads % mixer.kv_heads:
            raise ConfigError(f"Pigodra config.json: {where}: {mixer.heads} heads do not divide "
                              f"into {mixer.kv_heads} kv_heads")
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
            raise ConfigError(f"Pigodra config.json: {where}: rot.dims {mixer.rot_dims} must be "
                              f"even and at most dim {mixer.dim}")
    else:
        raise ConfigError(f"Pigodra config.json: {where} has type '{kind}': mlstm or attention")
    mlp = d.get("mlp")
    if mlp is not None:
        if mlp.get("kind", "dense") != "dense":
            raise ConfigError(f"Pigodra config.json: {where}.mlp.kind '{mlp.get('kind')}': dense")
        mlp = DenseMlp(ff=int(_need(mlp, "ff", where + ".mlp")))
    return PigodraLayer(kind, mixer, mlp)


@dataclass(frozen=True)
class PigodraConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: Tuple[PigodraLayer, ...]
    max_positions: int = 1 << 20

    @staticmethod
    def from_dict(d: dict) -> "PigodraConfig":
        layers = _need(d, "layers", "the top level")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("Pigodra config.json: 'layers' must be a list of at least one layer")
        return PigodraConfig(
            vocab=int(_need(d, "vocab", "the top level")),
            width=int(_need(d, "width", "the top level")),
            norm_eps=float(_need(_need(d, "norm", "the top level"), "eps", "norm")),
            embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
            layers=tuple(_read_layer(i, l) for i, l in enumerate(layers)),
            max_positions=int(d.get("max_positions", 1 << 20)))

    def to_dict(self) -> dict:
        return {"architecture": "Pigodra", "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "layers": [l.to_dict() for l in self.layers]}

    # ------------------------------------------------------------------ named shapes
    @staticmethod
    def from_name(name: str) -> "PigodraConfig":
        """Shapes for measurements (random weights): ``pigodra-<width>``; heads of 128, three
        matrix-memory layers to one attention layer, a feed-forward in every layer."""
        key = name.lower()
        if key not in PRESETS:
            raise KeyError(f"no Pigodra preset '{name}'; known: {sorted(PRESETS)}")
        return PRESETS[key]()


def _stack(width: int, n_layers: int, ff: int, kv_heads: int, vocab: int = 32000,
           window: int = 1024) -> PigodraConfig:
    heads = width // 128
    layers = []
    for i in range(n_layers):
        if i % 4 == 3:
            layers.append(PigodraLayer("attention", DifferentialMixer(
                heads=heads // 2, kv_heads=max(1, kv_heads // 2), dim=128, vdim=256, scale=None,
                diff=0.2, window=window, keep_first=8, rot_dims=64, rot_base=500000.0,
                rot_factor=4.0), DenseMlp(ff)))
        else:
            layers.append(PigodraLayer("mlstm", MatrixMemoryMixer(
                heads=heads, dim=128, vdim=128, gate_cap=15.0), DenseMlp(ff)))
    return PigodraConfig(vocab=vocab, width=width, norm_eps=1e-6, embedding_scale=1.0,
                         layers=tuple(layers))


PRESETS = {
    # the widths, inner sizes, head sizes and vocabularies of the library's llama-3.1-8b and
    # llama-3.1-70b presets: the same rows of q, k, v and output per layer
    "pigodra-4096": lambda: _stack(4096, 32, 14336, 8, vocab=128256),
    "pigodra-8192": lambda: _stack(8192, 80, 28672, 8, vocab=128256),
}
