"""Typed configuration of the Vusenex decoder: a stack whose layers are listed one by one in
``config.json``, each with one of two attention mixers and an optional mixture-of-experts
feed-forward; the embedded rows get a hashed token-pair embedding and a learned position
vector.

    {"architecture": "Vusenex", "vocab": V, "width": D, "max_positions": P, "norm": {"eps": e},
     "embedding": {"bigram": {"buckets": B, "mul_prev": a, "mul_cur": b}},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale",
                           "q_temp": {"coef", "every"}}, "mlp": ...},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "vdim", "kv_rank", "scale"},
                 "mlp": {"kind": "moe", "expert": {"ff"}, "shared": {"ff"} | null,
                         "router": {"experts", "top", "groups": {"count", "keep"}}} | null}, ...]}

Every size and constant is read from there; nothing is assumed equal between layers.
"""
from dataclasses import dataclass
from typing import Optional, Tuple


class ConfigError(ValueError):
    pass


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"Vusenex config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class SinkMixer:
    """Attention whose values are its keys, with a bias by the logarithm of the distance and a
    sink in the softmax."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: Optional[float]
    q_temp_every: int

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
             "scale": self.scale}
        if self.q_temp_coef is not None:
            d["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return d


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale}


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
class VusenexLayer:
    type: str                 # "attention" | "latent_attention"
    mixer: object
    mlp: Optional[MoeMlp]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_mlp(mlp, where: str) -> Optional[MoeMlp]:
    if mlp is None:
        return None
    if mlp.get("kind", "moe") != "moe":
        raise ConfigError(f"Vusenex config.json: {where}.kind '{mlp.get('kind')}': moe")
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
        raise ConfigError(f"Vusenex config.json: {where}: {experts} experts do not form "
                          f"{count} equal groups of which {keep} are kept")
    if not 1 <= top <= keep * (experts // count):
        raise ConfigError(f"Vusenex config.json: {where}: top {top} of the "
                          f"{keep * (experts // count)} experts that can be chosen")
    return out


def _read_layer(i: int, d: dict) -> VusenexLayer:
    where = f"layers[{i}]"
    kind = _need(d, "type", where)
    m = _need(d, "mixer", where)
    if kind == "attention":
        heads = int(_need(m, "heads", where))
        temp = m.get("q_temp") or {}
        mixer = SinkMixer(
            heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(_need(m, "dim", where)),
            vdim=int(m.get("vdim", m["dim"])), scale=float(_need(m, "scale", where)),
            q_temp_coef=None if "coef" not in temp else float(temp["coef"]),
            q_temp_every=int(temp.get("every", 1)))
        if mixer.heads % mixer.kv_heads:
            raise ConfigError(f"Vusenex config.json: {where}: {mixer.heads} heads do not divide "
                              f"into {mixer.kv_heads} kv_heads")
        if mixer.vdim != mixer.dim:
            raise ConfigError(f"Vusenex config.json: {where}: the values are the keys, so vdim "
                              f"{mixer.vdim} must equal dim {mixer.dim}")
        if mixer.q_temp_every < 1:
            raise ConfigError(f"Vusenex config.json: {where}: q_temp.every must be at least 1")
    elif kind == "latent_attention":
        mixer = LatentMixer(heads=int(_need(m, "heads", where)), dim=int(_need(m, "dim", where)),
                            vdim=int(_need(m, "vdim", where)),
                            kv_rank=int(_need(m, "kv_rank", where)),
                            scale=float(_need(m, "scale", where)))
    else:
        raise ConfigError(f"Vusenex config.json: {where} has type '{kind}': attention or "
                          f"latent_attention")
    return VusenexLayer(kind, mixer, _read_mlp(d.get("mlp"), where + ".mlp"))


@dataclass(frozen=True)
class VusenexConfig:
    vocab: int
    width: int
    norm_eps: float
    max_positions: int
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: Tuple[VusenexLayer, ...]

    @staticmethod
    def from_dict(d: dict) -> "VusenexConfig":
        layers = _need(d, "layers", "the top level")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("Vusenex config.json: 'layers' must be a list of at least one layer")
        pair = _need(_need(d, "embedding", "the top level"), "bigram", "embedding")
        c = VusenexConfig(
            vocab=int(_need(d, "vocab", "the top level")),
            width=int(_need(d, "width", "the top level")),
            norm_eps=float(_need(_need(d, "norm", "the top level"), "eps", "norm")),
            max_positions=int(d.get("max_positions", 0) or 0),     # 0: the table's rows say
            buckets=int(_need(pair, "buckets", "embedding.bigram")),
            mul_prev=int(_need(pair, "mul_prev", "embedding.bigram")),
            mul_cur=int(_need(pair, "mul_cur", "embedding.bigram")),
            layers=tuple(_read_layer(i, l) for i, l in enumerate(layers)))
        if c.buckets < 1 or c.mul_prev < 0 or c.mul_cur < 0:
            raise ConfigError("Vusenex config.json: embedding.bigram needs buckets >= 1 and "
                              "multipliers >= 0")
        return c

    def to_dict(self) -> dict:
        return {"architecture": "Vusenex", "vocab": self.vocab, "width": self.width,
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
                "embedding": {"bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev,
                                         "mul_cur": self.mul_cur}},
                "layers": [l.to_dict() for l in self.layers]}

    # ------------------------------------------------------------------ named shapes
    @staticmethod
    def from_name(name: str) -> "VusenexConfig":
        """Shapes for measurements (random weights): ``vusenex-<width>``."""
        key = name.lower()
        if key not in PRESETS:
            raise KeyError(f"no Vusenex preset '{name}'; known: {sorted(PRESETS)}")
        return PRESETS[key]()


def _stack(width: int, n_layers: int, ff: int, experts: int, top: int, shared_ff: int,
           kv_heads: int, vocab: int) -> VusenexConfig:
    """Heads of 128; latent attention (latent of 512) and attention with a sink in turn; a
    mixture of experts in every layer."""
    heads = width // 128
    layers = []
    for i in range(n_layers):
        if i % 2 == 0:
            mixer = LatentMixer(heads=heads, dim=128, vdim=128, kv_rank=512, scale=128 ** -0.5)
            kind = "latent_attention"
        else:
            mixer = SinkMixer(heads=heads, kv_heads=kv_heads, dim=128, vdim=128,
                              scale=128 ** -0.5 * 8.0, q_temp_coef=0.1, q_temp_every=1024)
            kind = "attention"
        layers.append(VusenexLayer(kind, mixer, MoeMlp(experts=experts, top=top, groups=4, keep=2,
                                                       ff=ff, shared_ff=shared_ff)))
    return VusenexConfig(vocab=vocab, width=width, norm_eps=1e-6, max_positions=131072,
                         buckets=262139, mul_prev=1000003, mul_cur=31, layers=tuple(layers))


PRESETS = {
    # the widths, head sizes and vocabulary of the library's Llama and Nizedra presets; per token
    # four routed experts and the shared one together are as large as those presets' feed-forwards
    "vusenex-4096": lambda: _stack(4096, 32, 3584, 32, 4, 7168, 8, vocab=128256),
    "vusenex-8192": lambda: _stack(8192, 80, 7168, 32, 4, 14336, 8, vocab=128256),
}
