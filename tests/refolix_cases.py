"""Small Refolix configurations for the tests; they differ from each other in every size and
option.  Weights are drawn by the library's random-weights mode and may be patched before
they are written."""
import json
import os

import torch


def _moe(experts, top, count, keep, ff, shared):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}},
            "shared": {"ff": shared} if shared else None}


def _rot(dims, base, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _left(heads, kv, dim, vdim, scale, window=None, softcap=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if softcap is not None:
        m["softcap"] = softcap
    if rot is not None:
        m["rot"] = rot
    return m


def _right(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _parallel(left, right, mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def _retention(heads, dim, vdim, decay, rot=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot is not None:
        m["rot"] = rot
    return {"type": "retention", "mixer": m, "mlp": mlp}


def _model(width, vocab, eps, alpha, embed_scale, logit_scale, logit_cap, layers):
    d = {"architecture": "Refolix", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "postln_alpha": alpha, "embedding": {"scale": embed_scale}, "layers": layers}
    if logit_scale is not None:
        d["logit_scale"] = logit_scale
    if logit_cap is not None:
        d["logit_softcap"] = logit_cap
    return d


CASES = {
    # the pair first; three kv heads for six heads and two key heads for four; values of
    # another size than the keys; a window of 40 keys; a third of each head rotated, with a
    # rescaled ladder whose ramp lies inside it; three groups of which two are kept; a
    # retention layer without a feed-forward whose heads are half rotated; no shared expert in
    # the last layer
    "A": _model(96, 300, 1e-5, 2.0, 1.5, 0.5, 20.0, [
        _parallel(_left(6, 3, 24, 16, 0.3, window=40, softcap=15.0, rot=_rot(8, 10000.0, (4.0, 64, 16.0, 2.0))),
                  _right(4, 2, 16, 8, 3), mlp=_moe(6, 2, 3, 2, 40, 56)),
        _retention(3, 16, 24, (0.9, 0.97, 0.995), rot=_rot(16, 50000.0), mlp=_moe(4, 1, 2, 1, 24, 32)),
        _retention(2, 24, 8, (0.8, 0.99), rot=_rot(12, 300.0)),
        _parallel(_left(2, 1, 16, 40, 0.2, window=70, softcap=50.0, rot=_rot(16, 1000.0)),
                  _right(2, 2, 8, 24, 4), mlp=_moe(8, 3, 4, 2, 16, 0)),
    ]),
    # sizes that are multiples of 4 only; a kv head per head; no window, no cap, no rotation in
    # the attention, none in one retention layer; one tap (no convolution); one group (every
    # expert can be chosen); every expert chosen; no factors on the embedding or the logits
    "B": _model(104, 211, 1e-6, 1.0, 1.0, None, None, [
        _retention(1, 20, 12, (0.96,), mlp=_moe(5, 2, 1, 1, 36, 0)),
        _parallel(_left(3, 3, 20, 12, 0.22), _right(3, 3, 12, 20, 1), mlp=_moe(3, 3, 1, 1, 28, 44)),
        _retention(4, 12, 28, (0.5, 0.9, 0.99, 0.999), rot=_rot(12, 10000.0), mlp=_moe(4, 2, 4, 2, 20, 12)),
    ]),
    # one kv head for all heads; a window of one key (a token sees itself only) and one of
    # exactly a page; groups of one expert each; five taps; one delta head; values wider than
    # 128 in retention; a ladder that is rescaled throughout (the ramp ends before it)
    "C": _model(64, 97, 1e-5, 3.0, 0.25, 2.0, 5.0, [
        _parallel(_left(8, 1, 8, 16, 0.4, window=1, softcap=4.0, rot=_rot(8, 100.0, (2.0, 16, 1000.0, 500.0))),
                  _right(1, 1, 32, 16, 5), mlp=_moe(6, 2, 6, 3, 24, 16)),
        _retention(2, 8, 144, (0.93, 0.999), rot=_rot(8, 20.0), mlp=_moe(2, 1, 2, 2, 48, 8)),
        _parallel(_left(4, 2, 32, 8, 0.18, window=64, rot=_rot(2, 7.0)), _right(6, 2, 8, 8, 2)),
    ]),
    # a width and sizes that are multiples of two only: no kernel's fast form applies
    "O": _model(100, 131, 1e-5, 1.5, 0.7, 0.3, 12.0, [
        _parallel(_left(2, 1, 10, 6, 0.3, window=33, softcap=9.0, rot=_rot(6, 50.0, (3.0, 40, 8.0, 1.0))),
                  _right(2, 1, 10, 6, 3), mlp=_moe(4, 2, 2, 1, 18, 10)),
        _retention(2, 10, 6, (0.9, 0.98), rot=_rot(10, 90.0), mlp=_moe(3, 1, 1, 1, 22, 6)),
    ]),
}


def random_case(seed):
    """A configuration drawn from sizes that kernels treat differently (head sizes of 32 to 128,
    several kv head ratios, windows around a page, two to five taps, experts in one to four
    groups), two to five layers in any order, now and then one without a feed-forward."""
    import random
    rng = random.Random(seed)
    width = rng.choice([128, 192, 256, 320, 384])
    vocab = rng.choice([263, 500, 1000])
    layers = []
    for _ in range(rng.randint(2, 5)):
        experts = rng.choice([4, 6, 8, 12, 16])
        count = rng.choice([g for g in (1, 2, 3, 4) if experts % g == 0])
        keep = rng.randint(1, count)
        top = rng.randint(1, min(4, keep * (experts // count)))
        mlp = _moe(experts, top, count, keep, rng.choice([32, 48, 64, 96]), rng.choice([0, 64, 96, 128]))
        if rng.random() < 0.15:
            mlp = None
        heads = rng.choice([2, 4, 6, 8])
        dim = rng.choice([32, 48, 64, 96, 128])
        if rng.random() < 0.5:
            kv = rng.choice([g for g in (1, 2, 3, 4, 8) if heads % g == 0])
            dims = rng.choice([d for d in (8, 16, 32, 64) if d <= dim])
            scaling = None if rng.random() < 0.4 else (rng.choice([2.0, 4.0, 8.0]), rng.choice([64, 256, 1024]),
                                                       rng.choice([16.0, 32.0]), rng.choice([1.0, 2.0]))
            left = _left(heads, kv, dim, rng.choice([32, 48, 64, 96]), rng.choice([0.0625, 0.125, 0.2]),
                         window=rng.choice([None, 17, 63, 64, 65, 100, 200]),
                         softcap=rng.choice([None, 10.0, 30.0]), rot=_rot(dims, rng.choice([1e4, 5e5]), scaling))
            rheads = rng.choice([2, 4, 6])
            right = _right(rheads, rng.choice([g for g in (1, 2, 3) if rheads % g == 0]),
                           rng.choice([32, 48, 64, 128]), rng.choice([32, 64, 96]), rng.randint(2, 5))
            layers.append(_parallel(left, right, mlp=mlp))
        else:
            decay = [1.0 - 2.0 ** -rng.uniform(2, 9) for _ in range(heads)]
            dims = rng.choice([0, dim // 2, dim])
            layers.append(_retention(heads, dim, rng.choice([32, 64, 96, 128]), decay,
                                     rot=_rot(dims, rng.choice([1e4, 1e6])) if dims else None, mlp=mlp))
    return _model(width, vocab, rng.choice([1e-5, 1e-6]), rng.choice([1.0, 2.0, 4.0]),
                  rng.choice([1.0, 0.5]), rng.choice([None, 0.5]), rng.choice([None, 25.0]), layers)


def write_model(folder, config, seed, dtype="bfloat16", std=0.08, patch=None):
    """A model folder of ``config`` with seeded random weights; ``patch(tensors)`` may change
    them before they are written.  The router's rows are made large enough for clear choices,
    the corrections partly negative and large enough to change choices, the decays' numbers
    spread from fast to slow, and the layer scales and branch weights given both small and
    large values."""
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
        elif name.endswith("mlp.correction"):
            tensors[name] = (torch.randn(t.shape, generator=g) * 0.6 - 0.4).to(t.dtype)
        elif name.endswith(".A_log"):
            tensors[name] = (torch.rand(t.shape, generator=g) * 4.0 - 4.0).to(t.dtype)
        elif name.endswith(".dt_bias"):
            tensors[name] = (torch.randn(t.shape, generator=g)).to(t.dtype)
        elif name.endswith(".conv"):
            tensors[name] = (torch.randn(t.shape, generator=g) * 0.7).to(t.dtype)
        elif name.endswith((".ls1", ".ls2", ".out")):
            tensors[name] = (torch.rand(t.shape, generator=g) * 1.5 + 0.25).to(t.dtype)
    if patch is not None:
        patch(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def make_folder(tmp, name, seed=0, dtype="bfloat16", patch=None, tag=""):
    folder = os.path.join(str(tmp), f"refolix_{name}_{dtype}_{seed}{tag}")
    if not os.path.isdir(folder):
        write_model(folder, CASES[name], seed, dtype, patch=patch)
    return folder
