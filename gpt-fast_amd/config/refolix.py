"""Typed configuration of the Refolix decoder: a stack whose layers are listed one by one in
``config.json``; the norm of a layer stands after each sum; a layer's mixer is either two
mixers side by side (windowed attention with normed, partly rotated heads, and the gated delta
rule) or retention (a matrix state per head with a fixed decay), its feed-forward a mixture of
gated experts with a shared expert.

    {"architecture": "Refolix", "vocab": V, "width": D, "norm": {"eps": e}, "postln_alpha": a,
     "embedding": {"scale": c}, "logit_scale": s, "logit_softcap": cap,
     "layers": [{"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap",
                                    "mask": {"size"},
                                    "rot": {"dims", "base", "scaling": {"factor", "original",
                                                                        "fast", "slow"}}},
                           "right": {"heads", "kv_heads", "dim", "vdim", "conv"}},
                 "mlp": {"kind": "moe", "expert": {"ff"}, "shared": {"ff"} | null,
                         "router": {"experts", "top", "groups": {"count", "keep"}}} | null},
                {"type": "retention",
                 "mixer": {"heads", "dim", "vdim", "decay": [...], "rot": {"dims", "base"}},
                 "mlp": ...}, ...]}

Every size and constant is read from there; nothing is assumed equal between layers.
"""
from dataclasses import dataclass
from typing import Optional, Tuple


class ConfigError(ValueError):
    pass


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"Refolix config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class Rotation:
    """Rotary positions on the first ``dims`` elements of a head; ``scaling`` None or
    (factor, original, fast, slow)."""
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None

    @staticmethod
    def read(d, where: str) -> Optional["Rotation"]:
        if not d or not int(d.get("dims", 0)):
            return None
        sc = d.get("scaling")
        scaling = None
        if sc:
            scaling = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow"))
        r = Rotation(int(d["dims"]), float(_need(d, "base", where)), scaling)
        if r.dims % 2 or r.dims < 0:
            raise ConfigError(f"Refolix config.json: {where}.dims {r.dims} must be even")
        return r

    def to_dict(self) -> dict:
        d = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return d


@dataclass(frozen=True)
class WindowAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]
    window: Optional[int]
    rot: Optional[Rotation]

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
             "scale": self.scale}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class DeltaRule:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "conv": self.conv}


@dataclass(frozen=True)
class ParallelPair:
    left: WindowAttention
    right: DeltaRule

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class Retention:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation]

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class MoeMlp:
    experts: int
    top: int
    groups: int
    keep: int
    ff: int
    shared_ff: int            # 0: no shared expert

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top,
                           "groups": {"count": self.groups, "keep": self.keep}},
                "shared": {"ff": self.shared_ff} if self.shared_ff else None}


@dataclass(frozen=True)
class RefolixLayer:
    type: str                 # "parallel" | "retention"
    mixer: object
    mlp: Optional[MoeMlp]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_mlp(mlp, where: str) -> Optional[MoeMlp]:
    if mlp is None:
        return None
    if mlp.get("kind", "moe") != "moe":
        raise ConfigError(f"Refolix config.json: {where}.kind '{mlp.get('kind')}': moe")
    router = _need(mlp, "router", where)
    experts = int(_need(router, "experts", where + ".router"))
    top = int(_need(router, "top", where + ".router"))
    groups = router.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1)))
    shared = mlp.get("shared") or {}
    out = MoeMlp(experts=experts, top=top, groups=count, keep=keep,
                 ff=int(_need(_need(mlp, "expert", where), "ff", where + ".expert")),
                 shared_ff=int(shared.get("ff", 0) or 0))
    if count < 1 or experts % count or not 1 <= keep <= count:
        raise ConfigError(f"Refolix config.json: {where}: {experts} experts do not form "
                          f"{count} equal groups of which {keep} are kept")
    if not 1 <= top <= keep * (experts // count):
        raise ConfigError(f"Refolix config.json: {where}: top {top} of the "
                          f"{keep * (experts // count)} experts that can be chosen")
    return out


def _optional_float(d: dict, key: str) -> Optional[float]:
    v = d.get(key)
    return None if v is None else float(v)


def _read_layer(i: int, d: dict) -> RefolixLayer:
    where = f"layers[{i}]"
    kind = _need(d, "type", where)
    m = _need(d, "mixer", where)
    if kind == "parallel":
        l, r = _need(m, "left", where + ".mixer"), _need(m, "right", where + ".mixer")
        heads = int(_need(l, "heads", where + ".left"))
        dim = int(_need(l, "dim", where + ".left"))
        mask = l.get("mask") or {}
        left = WindowAttention(
            heads=heads, kv_heads=int(l.get("kv_heads", heads)), dim=dim, vdim=int(l.get("vdim", dim)),
            scale=float(_need(l, "scale", where + ".left")), softcap=_optional_float(l, "softcap"),
            window=None if mask.get("size") is None else int(mask["size"]),
            rot=Rotation.read(l.get("rot"), where + ".left.rot"))
        rheads = int(_need(r, "heads", where + ".right"))
        rdim = int(_need(r, "dim", where + ".right"))
        right = DeltaRule(heads=rheads, kv_heads=int(r.get("kv_heads", rheads)), dim=rdim,
                          vdim=int(r.get("vdim", rdim)), conv=int(_need(r, "conv", where + ".right")))
        for name, part in (("left", left), ("right", right)):
            if part.kv_heads < 1 or part.heads % part.kv_heads:
                raise ConfigError(f"Refolix config.json: {where}.{name}: {part.heads} heads do not "
                                  f"divide into {part.kv_heads} kv_heads")
        if left.rot is not None and left.rot.dims > left.dim:
            raise ConfigError(f"Refolix config.json: {where}.left: {left.rot.dims} rotated elements in "
                              f"heads of {left.dim}")
        if left.window is not None and left.window < 1:
            raise ConfigError(f"Refolix config.json: {where}.left.mask.size must be at least 1")
        if right.conv < 1:
            raise ConfigError(f"Refolix config.json: {where}.right.conv must be at least 1")
        mixer = ParallelPair(left, right)
    elif kind == "retention":
        heads = int(_need(m, "heads", where))
        dim = int(_need(m, "dim", where))
        decay = tuple(float(a) for a in _need(m, "decay", where))
        mixer = Retention(heads=heads, dim=dim, vdim=int(m.get("vdim", dim)), decay=decay,
                          rot=Rotation.read(m.get("rot"), where + ".rot"))
        if len(decay) != heads:
            raise ConfigError(f"Refolix config.json: {where}: {len(decay)} decays for {heads} heads")
        if mixer.rot is not None and mixer.rot.dims > dim:
            raise ConfigError(f"Refolix config.json: {where}: {mixer.rot.dims} rotated elements in "
                              f"heads of {dim}")
    else:
        raise ConfigError(f"Refolix config.json: {where} has type '{kind}': parallel or retention")
    return RefolixLayer(kind, mixer, _read_mlp(d.get("mlp"), where + ".mlp"))


@dataclass(frozen=True)
class RefolixConfig:
    vocab: int
    width: int
    norm_eps: float
    alpha: float                       # the stream's factor in every sum that is normed
    embedding_scale: float
    logit_scale: Optional[float]
    logit_softcap: Optional[float]
    layers: Tuple[RefolixLayer, ...]
    max_positions: int = 1 << 20       # the design has no table of positions: a bound for requests

    @staticmethod
    def from_dict(d: dict) -> "RefolixConfig":
        layers = _need(d, "layers", "the top level")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("Refolix config.json: 'layers' must be a list of at least one layer")
        return RefolixConfig(
            vocab=int(_need(d, "vocab", "the top level")),
            width=int(_need(d, "width", "the top level")),
            norm_eps=float(_need(_need(d, "norm", "the top level"), "eps", "norm")),
            alpha=float(d.get("postln_alpha", 1.0)),
            embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
            logit_scale=_optional_float(d, "logit_scale"),
            logit_softcap=_optional_float(d, "logit_softcap"),
            layers=tuple(_read_layer(i, l) for i, l in enumerate(layers)),
            max_positions=int(d.get("max_positions", 1 << 20)))

    def to_dict(self) -> dict:
        d = {"architecture": "Refolix", "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.norm_eps}, "postln_alpha": self.alpha,
             "embedding": {"scale": self.embedding_scale},
             "layers": [l.to_dict() for l in self.layers]}
        if self.logit_scale is not None:
            d["logit_scale"] = self.logit_scale
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d

    # ------------------------------------------------------------------ named shapes
    @staticmethod
    def from_name(name: str) -> "RefolixConfig":
        """Shapes for measurements (random weights): ``refolix-<width>``."""
        key = name.lower()
        if key not in PRESETS:
            raise KeyError(f"no Refolix preset '{name}'; known: {sorted(PRESETS)}")
        return PRESETS[key]()


def _stack(width: int, n_layers: int, ff: int, experts: int, top: int, shared_ff: int,
           kv_heads: int, vocab: int) -> RefolixConfig:
    """Heads of 128; three retention layers, then one pair of windowed attention (4,096 keys)
    and the delta rule, and so on; a mixture of experts in every layer."""
    heads = width // 128
    layers = []
    for i in range(n_layers):
        if i % 4 == 3:
            left = WindowAttention(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5,
                                   softcap=50.0, window=4096,
                                   rot=Rotation(64, 500000.0, (8.0, 8192.0, 32.0, 1.0)))
            right = DeltaRule(heads=heads // 2, kv_heads=heads // 4, dim=128, vdim=128, conv=4)
            mixer, kind = ParallelPair(left, right), "parallel"
        else:
            step = 5.0 / max(heads - 1, 1)
            decay = tuple(1.0 - 2.0 ** (-5.0 - step * h) for h in range(heads))
            mixer = Retention(heads=heads, dim=128, vdim=128, decay=decay, rot=Rotation(128, 1000000.0))
            kind = "retention"
        layers.append(RefolixLayer(kind, mixer, MoeMlp(experts=experts, top=top, groups=4, keep=2,
                                                       ff=ff, shared_ff=shared_ff)))
    return RefolixConfig(vocab=vocab, width=width, norm_eps=1e-6, alpha=2.0, embedding_scale=1.0,
                         logit_scale=None, logit_softcap=30.0, layers=tuple(layers))


PRESETS = {
    # the widths, head sizes and vocabulary of the library's other presets; per token four
    # routed gated experts and the shared one together are as large as those presets' feed-forwards
    "refolix-4096": lambda: _stack(4096, 32, 2048, 32, 4, 6144, 8, vocab=128256),
    "refolix-8192": lambda: _stack(8192, 80, 4096, 32, 4, 12288, 8, vocab=128256),
}
