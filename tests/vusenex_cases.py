"""Small Vusenex configurations for the tests; they differ from each other in every size and
option.  Weights are drawn by the library's random-weights mode and may be patched before
they are written."""
import json
import os

import torch


def _moe(experts, top, count, keep, ff, shared):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}},
            "shared": {"ff": shared} if shared else None}


def _attention(heads, kv, dim, scale, temp=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _latent(heads, dim, vdim, rank, scale, mlp=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}, "mlp": mlp}


def _model(width, vocab, eps, positions, pair, layers):
    return {"architecture": "Vusenex", "vocab": vocab, "width": width, "max_positions": positions,
            "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": pair[0], "mul_prev": pair[1], "mul_cur": pair[2]}},
            "layers": layers}


CASES = {
    # attention first; three kv heads for six heads; head sizes in multiples of 8; a temperature
    # that changes every 16 positions; three groups of which two are kept; a layer without a
    # feed-forward; a latent wider than a head
    "A": _model(96, 300, 1e-5, 640, (211, 31, 5), [
        _attention(6, 3, 16, 0.3, temp=(0.4, 16), mlp=_moe(6, 2, 3, 2, 40, 56)),
        _latent(3, 16, 24, 40, 0.25, mlp=_moe(4, 1, 2, 1, 24, 32)),
        _attention(2, 1, 24, 0.2, temp=(1.5, 5)),
        _latent(2, 24, 8, 16, 0.2, mlp=_moe(8, 3, 4, 2, 16, 0)),
    ]),
    # sizes that are multiples of 4 only; one head; a kv head per head; no temperature; one
    # group (every expert can be chosen); no shared expert; every expert chosen (top = experts)
    "B": _model(104, 211, 1e-6, 700, (97, 3, 11), [
        _latent(1, 20, 12, 28, 0.3, mlp=_moe(5, 2, 1, 1, 36, 0)),
        _attention(3, 3, 20, 0.22, mlp=_moe(3, 3, 1, 1, 28, 44)),
        _attention(1, 1, 12, 0.5, temp=(0.25, 64), mlp=_moe(4, 2, 4, 2, 20, 12)),
    ]),
    # values wider than 128 in the latent layer; a latent beyond 128; one kv head for all heads;
    # groups of one expert each; buckets fewer than the vocabulary
    "C": _model(64, 97, 1e-5, 600, (13, 7, 2), [
        _latent(4, 8, 144, 136, 0.35, mlp=_moe(6, 2, 6, 3, 24, 16)),
        _attention(8, 1, 8, 0.4, temp=(0.7, 1), mlp=_moe(2, 1, 2, 2, 48, 8)),
        _latent(2, 32, 16, 8, 0.18),
    ]),
    # a width and sizes that are multiples of two only: no kernel's fast form applies
    "O": _model(100, 131, 1e-5, 520, (50, 2, 3), [
        _attention(2, 1, 10, 0.3, temp=(0.5, 7), mlp=_moe(4, 2, 2, 1, 18, 10)),
        _latent(2, 10, 6, 14, 0.3, mlp=_moe(3, 1, 1, 1, 22, 6)),
    ]),
    # latent attention only; an odd number of experts of which all are chosen; multipliers of
    # one and more buckets than the vocabulary; one head whose latent has the head's size
    "L": _model(72, 150, 1e-6, 560, (301, 1, 1), [
        _latent(3, 12, 20, 24, 0.3, mlp=_moe(7, 7, 1, 1, 10, 14)),
        _latent(1, 40, 40, 40, 0.2, mlp=_moe(2, 2, 1, 1, 8, 0)),
    ]),
    # attention only, a kv head per head; a temperature that never changes within a test's
    # sequences; all groups kept; a first layer without a feed-forward
    "T": _model(48, 90, 1e-5, 530, (89, 11, 13), [
        _attention(4, 4, 8, 0.35, temp=(0.9, 1000)),
        _attention(2, 2, 24, 0.15, temp=(0.3, 2), mlp=_moe(9, 4, 3, 3, 12, 20)),
    ]),
}


def random_case(seed):
    """A configuration drawn from sizes that kernels treat differently (head sizes of 32 to 128,
    latents up to 320, several kv head ratios, experts in one to four groups), two to six
    layers in any order, now and then one without a feed-forward."""
    import random
    rng = random.Random(seed)
    width = rng.choice([128, 192, 256, 320, 384, 512])
    vocab = rng.choice([263, 500, 1000, 2048])
    layers = []
    for _ in range(rng.randint(2, 6)):
        experts = rng.choice([4, 6, 8, 12, 16])
        count = rng.choice([g for g in (1, 2, 3, 4) if experts % g == 0])
        keep = rng.randint(1, count)
        top = rng.randint(1, min(4, keep * (experts // count)))
        mlp = _moe(experts, top, count, keep, rng.choice([32, 48, 64, 96, 128, 160]), rng.choice([0, 64, 96, 128, 256]))
        if rng.random() < 0.15:
            mlp = None
        heads = rng.choice([2, 4, 6, 8])
        dim = rng.choice([32, 48, 64, 96, 128])
        if rng.random() < 0.5:
            kv = rng.choice([g for g in (1, 2, 3, 4, 8) if heads % g == 0])
            temp = None if rng.random() < 0.2 else (rng.choice([0.25, 0.5, 1.0]), rng.choice([16, 32, 64, 100, 128]))
            layers.append(_attention(heads, kv, dim, rng.choice([0.0625, 0.09375, 0.125, 0.2]), temp=temp, mlp=mlp))
        else:
            layers.append(_latent(heads, dim, rng.choice([32, 48, 64, 96, 128]), rng.choice([64, 96, 128, 192, 256, 320]),
                                  rng.choice([0.0884, 0.125, 0.177]), mlp=mlp))
    pair = (rng.choice([509, 2039, 4093]), rng.choice([31, 8191]), rng.choice([17, 131]))
    return _model(width, vocab, rng.choice([1e-5, 1e-6]), 1024, pair, layers)


def write_model(folder, config, seed, dtype="bfloat16", std=0.08, patch=None):
    """A model folder of ``config`` with seeded random weights; ``patch(tensors)`` may change
    them before they are written.  The router's rows are made large enough for clear choices,
    the gates' biases and the distance bias's numbers are given both small and large values."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.random_init import random_checkpoint
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    arch = gfa.config.registry.architecture_of(config)
    cfg = arch.read_config(config)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    tensors = random_checkpoint(arch.bindings(cfg), seed, dtype, std=std, norm_std=0.2)
    g = torch.Generator().manual_seed(seed + 1)
    for name in sorted(tensors):
        t = tensors[name]
        if name.endswith("mlp.router"):
            tensors[name] = (torch.randn(t.shape, generator=g) * 0.6).to(t.dtype)
        elif name.endswith(".r1"):
            tensors[name] = (torch.rand(t.shape, generator=g) * 1.5 + 0.1).to(t.dtype)
        elif name.endswith(".r2"):
            tensors[name] = (torch.rand(t.shape, generator=g) * 0.5 + 0.02).to(t.dtype)
        elif name in ("pos", "bigram"):
            tensors[name] = (torch.randn(t.shape, generator=g) * std).to(t.dtype)
    if patch is not None:
        patch(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def make_folder(tmp, name, seed=0, dtype="bfloat16", patch=None, tag=""):
    folder = os.path.join(str(tmp), f"vusenex_{name}_{dtype}_{seed}{tag}")
    if not os.path.isdir(folder):
        write_model(folder, CASES[name], seed, dtype, patch=patch)
    return folder
