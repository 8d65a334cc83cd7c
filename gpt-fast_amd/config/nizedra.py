"""Typed configuration of the Nizedra decoder: a stack whose layers are listed one by one in
``config.json``, each with one of three mixers and an optional dense feed-forward, and a
stretch of layers that may run several times in a row with the same weights.

    {"architecture": "Nizedra", "vocab": V, "width": D, "norm": {"eps": e},
     "loop": {"start": a, "stop": b, "times": n},
     "layers": [{"type": "lightning", "mixer": {"heads", "dim", "vdim", "decay": [per head]}, "mlp": ...},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale",
                           "mask": {"size"}, "rot": {"dims", "base"}}, "mlp": ...},
                {"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "bias_max"},
                 "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Every size and constant is read from there; nothing is assumed equal between layers.  Sizes
that only a tensor's shape gives (the rows of an attention layer's distance table) are read
from the checkpoint by the loader, which accepts any number of them.
"""
from dataclasses import dataclass
from typing import Optional, Tuple


class ConfigError(ValueError):
    pass


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"Nizedra config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class LightningMixer:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: Optional[int]
    rot_dims: int
    rot_base: float

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
             "q_rank": self.q_rank, "kv_rank": self.kv_rank, "scale": self.scale,
             "rot": {"dims": self.rot_dims, "base": self.rot_base}}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class MixedHeadsMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]
    bias_max: float
    bias_rows: int            # rows of the distance table (the checkpoint's to say; see the loader)

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
             "scale": self.scale, "bias_max": self.bias_max, "bias_rows": self.bias_rows}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        return d


@dataclass(frozen=True)
class DenseMlp:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class NizedraLayer:
    type: str                 # "lightning" | "latent_attention" | "attention"
    mixer: object
    mlp: Optional[DenseMlp]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int

    def to_dict(self) -> dict:
        return {"start": self.start, "stop": self.stop, "times": self.times}


DEFAULT_BIAS_ROWS = 32


def _read_layer(i: int, d: dict) -> NizedraLayer:
    where = f"layers[{i}]"
    kind = _need(d, "type", where)
    m = _need(d, "mixer", where)
    if kind == "lightning":
        heads = int(_need(m, "heads", where))
        decay = _need(m, "decay", where)
        if not isinstance(decay, (list, tuple)):
            decay = [decay] * heads
        if len(decay) != heads:
            raise ConfigError(f"Nizedra config.json: {where}: {len(decay)} decays for {heads} heads")
        mixer = LightningMixer(heads=heads, dim=int(_need(m, "dim", where)),
                               vdim=int(_need(m, "vdim", where)),
                               decay=tuple(float(x) for x in decay))
    elif kind == "latent_attention":
        mask = m.get("mask") or {}
        rot = m.get("rot") or {}
        rot_dim = int(m.get("rot_dim") or 0)
        mixer = LatentMixer(
            heads=int(_need(m, "heads", where)), dim=int(_need(m, "dim", where)), rot_dim=rot_dim,
            vdim=int(_need(m, "vdim", where)), q_rank=int(_need(m, "q_rank", where)),
            kv_rank=int(_need(m, "kv_rank", where)), scale=float(_need(m, "scale", where)),
            window=None if mask.get("size") is None else int(mask["size"]),
            rot_dims=int(rot.get("dims", rot_dim) or 0), rot_base=float(rot.get("base", 10000.0)))
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
            raise ConfigError(f"Nizedra config.json: {where}: rot.dims {mixer.rot_dims} must be "
                              f"even and at most rot_dim {mixer.rot_dim}")
    elif kind == "attention":
        heads = int(_need(m, "heads", where))
        cap = m.get("softcap")
        mixer = MixedHeadsMixer(
            heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(_need(m, "dim", where)),
            vdim=int(_need(m, "vdim", where)), scale=float(_need(m, "scale", where)),
            softcap=None if not cap else float(cap), bias_max=float(_need(m, "bias_max", where)),
            bias_rows=int(m.get("bias_rows", DEFAULT_BIAS_ROWS)))
        if mixer.heads % mixer.kv_heads:
            raise ConfigError(f"Nizedra config.json: {where}: {mixer.heads} heads do not divide "
                              f"into {mixer.kv_heads} kv_heads")
    else:
        raise ConfigError(f"Nizedra config.json: {where} has type '{kind}': lightning, "
                          f"latent_attention or attention")
    mlp = d.get("mlp")
    if mlp is not None:
        if mlp.get("kind", "dense") != "dense":
            raise ConfigError(f"Nizedra config.json: {where}.mlp.kind '{mlp.get('kind')}': dense")
        mlp = DenseMlp(ff=int(_need(mlp, "ff", where + ".mlp")))
    return NizedraLayer(kind, mixer, mlp)


@dataclass(frozen=True)
class NizedraConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[NizedraLayer, ...]
    loop: Optional[Loop] = None
    max_positions: int = 1 << 20

    @staticmethod
    def from_dict(d: dict) -> "NizedraConfig":
        layers = _need(d, "layers", "the top level")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("Nizedra config.json: 'layers' must be a list of at least one layer")
        loop = d.get("loop")
        if loop is not None:
            loop = Loop(int(_need(loop, "start", "loop")), int(_need(loop, "stop", "loop")),
                        int(_need(loop, "times", "loop")))
            if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 0:
                raise ConfigError(f"Nizedra config.json: loop {loop.to_dict()} does not fit "
                                  f"{len(layers)} layers")
        return NizedraConfig(
            vocab=int(_need(d, "vocab", "the top level")),
            width=int(_need(d, "width", "the top level")),
            norm_eps=float(_need(_need(d, "norm", "the top level"), "eps", "norm")),
            layers=tuple(_read_layer(i, l) for i, l in enumerate(layers)),
            loop=loop, max_positions=int(d.get("max_positions", 1 << 20)))

    def to_dict(self) -> dict:
        d = {"architecture": "Nizedra", "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.norm_eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        return d

    def with_table_rows(self, rows_of_layer: dict) -> "NizedraConfig":
        """The same configuration with the rows of the distance tables that a checkpoint
        holds (layer index -> rows)."""
        import dataclasses
        layers = list(self.layers)
        for i, rows in rows_of_layer.items():
            if isinstance(layers[i].mixer, MixedHeadsMixer):
                layers[i] = dataclasses.replace(
                    layers[i], mixer=dataclasses.replace(layers[i].mixer, bias_rows=int(rows)))
        return dataclasses.replace(self, layers=tuple(layers))

    # ------------------------------------------------------------------ named shapes
    @staticmethod
    def from_name(name: str) -> "NizedraConfig":
        """Shapes for measurements (random weights): ``nizedra-<width>``."""
        key = name.lower()
        if key not in PRESETS:
            raise KeyError(f"no Nizedra preset '{name}'; known: {sorted(PRESETS)}")
        return PRESETS[key]()


def _stack(width: int, n_layers: int, ff: int, kv_heads: int, vocab: int,
           window: int = 1024) -> NizedraConfig:
    """Heads of 128; of every four layers two lightning layers, one latent attention (latent
    of 512, rotated part of 64) and one attention with mixed heads; a feed-forward in every
    layer; no loop."""
    heads = width // 128
    layers = []
    for i in range(n_layers):
        if i % 4 == 1:
            mixer = LatentMixer(heads=heads, dim=128, rot_dim=64, vdim=128, q_rank=width * 3 // 8,
                                kv_rank=512, scale=(128 + 64) ** -0.5, window=window, rot_dims=64,
                                rot_base=500000.0)
            kind = "latent_attention"
        elif i % 4 == 3:
            mixer = MixedHeadsMixer(heads=heads, kv_heads=kv_heads, dim=128, vdim=128,
                                    scale=128 ** -0.5 * 8.0, softcap=30.0, bias_max=4096.0,
                                    bias_rows=32)
            kind = "attention"
        else:
            decay = tuple(1.0 - 2.0 ** (-5.0 - 3.0 * h / max(heads - 1, 1)) for h in range(heads))
            mixer = LightningMixer(heads=heads, dim=128, vdim=128, decay=decay)
            kind = "lightning"
        layers.append(NizedraLayer(kind, mixer, DenseMlp(ff)))
    return NizedraConfig(vocab=vocab, width=width, norm_eps=1e-6, layers=tuple(layers))


PRESETS = {
    # the widths, head sizes and vocabularies of the library's llama-3.1-8b and llama-3.1-70b
    # presets; the dense feed-forward has two matrices where the gated one has three, so its
    # inner size is half again as large for the same weights per layer
    "nizedra-4096": lambda: _stack(4096, 32, 21504, 8, vocab=128256),
    "nizedra-8192": lambda: _stack(8192, 80, 43008, 8, vocab=128256),
}
