"""The Refolix decoder as data: its plan and its checkpoint layout.

Plan: the embedded rows times a constant; the layers ``config.json`` lists, each a block whose
norm stands after the sum (``x <- norm1(alpha x + ls1 * mixer(x))``, ``x <- norm2(alpha x + ls2 *
ff(x))``, layer norms with a weight, the sublayers read the stream itself); the mixer is
"parallel" - windowed attention with normed, partly rotated heads beside the gated delta rule,
the mean of the two results after an RMS norm of each - or "retention", a matrix state per head
with a fixed decay; the feed-forward a mixture of gated experts chosen by corrected sigmoid
scores, with a shared expert behind a gate of one number per token; then the final layer norm
and a scaled, capped head.

Checkpoint layout: ``embed``, ``l<i>.norm1`` / ``.norm2``, ``l<i>.ls1`` / ``.ls2``,
``l<i>.mix.<name>`` (``left.`` / ``right.`` for the two halves of a parallel mixer),
``l<i>.mlp.e<k>.gate`` / ``.up`` / ``.down``, ``l<i>.mlp.router``, ``.correction``,
``l<i>.mlp.shared.gate`` / ``.up`` / ``.down`` / ``.sg``, ``final.norm``, ``head``; linear
weights [out, in].  Projections that read the same input are joined into one matrix when they
are loaded, an expert's gate and up matrices too, and the experts' matrices are stacked.
"""
import torch

from ..config.refolix import ParallelPair, RefolixConfig, Retention
from ..config.registry import Architecture, register_architecture
from ..config.spec import (DecayedMemorySpec, GatedDeltaSpec, LayerSpec, ModelPlan, NormedAttentionSpec,
                           NormSpec, ParallelMixerSpec, PositionSpec, RoutedExpertsSpec, Run)
from ..weights.bindings import Binding, CheckpointLayout, Source


def _position(rot, layout: str):
    if rot is None:
        return None
    scaling = None
    if rot.scaling is not None:
        factor, original, fast, slow = rot.scaling
        scaling = (("rope_type", "yarn"), ("factor", factor), ("original", original),
                   ("fast", fast), ("slow", slow))
    return PositionSpec(kind="rope", rotary_dim=rot.dims, base=rot.base, layout=layout, scaling=scaling)


def _mixer_spec(c: RefolixConfig, m):
    if isinstance(m, ParallelPair):
        l, r = m.left, m.right
        left = NormedAttentionSpec(dim=c.width, n_heads=l.heads, n_kv_heads=l.kv_heads, head_dim=l.dim,
                                   value_dim=l.vdim, position=_position(l.rot, "interleaved"),
                                   scale=l.scale, qk_norm_eps=c.norm_eps, softcap=l.softcap,
                                   window=l.window)
        right = GatedDeltaSpec(dim=c.width, n_heads=r.heads, n_kv_heads=r.kv_heads, key_dim=r.dim,
                               value_dim=r.vdim, conv_taps=r.conv, eps=c.norm_eps, unit_eps=1e-6)
        return ParallelMixerSpec(dim=c.width, branches=(("left", left), ("right", right)), eps=c.norm_eps)
    assert isinstance(m, Retention)
    return DecayedMemorySpec(dim=c.width, n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                             decay=m.decay, eps=c.norm_eps, activation=None,
                             position=_position(m.rot, "half"), key_scale=m.dim ** -0.5,
                             norm="head", norm_weight=False, gate="silu")


def _feed_forward_spec(c: RefolixConfig, mlp):
    return RoutedExpertsSpec(dim=c.width, n_experts=mlp.experts, top=mlp.top, hidden=mlp.ff,
                             n_groups=mlp.groups, keep_groups=mlp.keep, shared_hidden=mlp.shared_ff,
                             activation="silu", weight_eps=1e-20, scoring="sigmoid",
                             choice_correction=True, group_top=2, gated=True,
                             shared_gate=bool(mlp.shared_ff))


def refolix_plan(c: RefolixConfig) -> ModelPlan:
    def layer_norm():
        return NormSpec(c.width, c.norm_eps, kind="layer")

    def none():
        return NormSpec(c.width, c.norm_eps, kind="none")

    layers = []
    for i, l in enumerate(c.layers):
        has_ff = l.mlp is not None
        layers.append(LayerSpec(
            name=f"l{i}", arrangement="post_norm", residual_scale=c.alpha, layer_scale=True,
            mixer=_mixer_spec(c, l.mixer), mixer_norm=none(), mixer_out_norm=layer_norm(),
            feed_forward=_feed_forward_spec(c, l.mlp) if has_ff else None,
            feed_forward_norm=none() if has_ff else None,
            feed_forward_out_norm=layer_norm() if has_ff else None,
            mixer_name="mix", mixer_norm_name="read1", mixer_out_norm_name="norm1",
            mixer_scale_name="ls1", feed_forward_name="mlp", feed_forward_norm_name="read2",
            feed_forward_out_norm_name="norm2", feed_forward_scale_name="ls2"))
    plan = ModelPlan(
        dim=c.width, vocab_size=c.vocab, layers=layers, order=[Run(i) for i in range(len(layers))],
        final_norm=layer_norm(), tie_embeddings=False, max_positions=c.max_positions,
        embedding_name="embed", final_norm_name="final.norm", head_name="head",
        embedding_scale=None if c.embedding_scale == 1.0 else c.embedding_scale,
        logit_scale=c.logit_scale, logit_softcap=c.logit_softcap)
    plan.validate()
    return plan


def refolix_bindings(c: RefolixConfig) -> CheckpointLayout:
    D, V = c.width, c.vocab
    b = [Binding("embed", (Source("embed", (V, D)),))]

    def vector(target, name, shape, init="norm"):
        return Binding(target, (Source(name, shape, init),), role="vector")

    for i, l in enumerate(c.layers):
        p = f"l{i}."
        m = l.mixer
        b += [vector(p + "norm1.weight", p + "norm1", (D,)), vector(p + "ls1.weight", p + "ls1", (D,))]
        if isinstance(m, ParallelPair):
            a, r = m.left, m.right
            H, G, d, dv = a.heads, a.kv_heads, a.dim, a.vdim
            x = p + "mix.left."
            b += [
                Binding(x + "wqkv", (Source(x + "q", (H * d, D)), Source(x + "k", (G * d, D)),
                                     Source(x + "v", (G * dv, D))), combine=torch.cat),
                vector(x + "q_norm", x + "q.norm", (d,)),
                vector(x + "k_norm", x + "k.norm", (d,)),
                Binding(x + "wo", (Source(x + "o", (D, H * dv)),)),
                vector(p + "mix.left_out", x + "out", (D,)),
            ]
            H, G, d, dv = r.heads, r.kv_heads, r.dim, r.vdim
            x = p + "mix.right."
            b += [
                # rows of q, k, v (the convolved channels), beta, the decay, the output gate
                Binding(x + "w_in", (Source(x + "q", (G * d, D)), Source(x + "k", (G * d, D)),
                                     Source(x + "v", (H * dv, D)), Source(x + "b", (H, D)),
                                     Source(x + "a", (H, D)), Source(x + "g", (H * dv, D))),
                        combine=torch.cat),
                Binding(x + "taps", (Source(x + "q.conv", (G * d, r.conv), "unit"),
                                     Source(x + "k.conv", (G * d, r.conv), "unit"),
                                     Source(x + "v.conv", (H * dv, r.conv), "unit")),
                        role="vector", combine=torch.cat),
                vector(x + "A_log", x + "A_log", (H,), "around_zero"),
                vector(x + "dt_bias", x + "dt_bias", (H,), "around_zero"),
                vector(x + "norm", x + "norm", (dv,)),
                Binding(x + "wo", (Source(x + "o", (D, H * dv)),)),
                vector(p + "mix.right_out", x + "out", (D,)),
            ]
        else:
            assert isinstance(m, Retention)
            H, d, dv = m.heads, m.dim, m.vdim
            x = p + "mix."
            b += [
                Binding(x + "w_in", (Source(x + "q", (H * d, D)), Source(x + "k", (H * d, D)),
                                     Source(x + "v", (H * dv, D)), Source(x + "g", (H * dv, D))),
                        combine=torch.cat),
                Binding(x + "wo", (Source(x + "o", (D, H * dv)),)),
            ]
        if l.mlp is not None:
            f = l.mlp
            x = p + "mlp."
            b += [
                vector(p + "norm2.weight", p + "norm2", (D,)), vector(p + "ls2.weight", p + "ls2", (D,)),
                Binding(x + "w_router", (Source(x + "router", (f.experts, D)),)),
                vector(x + "correction", x + "correction", (f.experts,), "around_zero"),
                # an expert's gate rows and then its up rows; the experts stacked
                Binding(x + "w_up", tuple(Source(f"{x}e{e}.{part}", (f.ff, D))
                                          for e in range(f.experts) for part in ("gate", "up")),
                        combine=lambda parts, n=f.experts: torch.cat(parts).view(n, -1, parts[0].shape[1])),
                Binding(x + "w_down", tuple(Source(f"{x}e{e}.down", (D, f.ff)) for e in range(f.experts)),
                        combine=torch.stack),
            ]
            if f.shared_ff:
                b += [Binding(x + "shared_up", (Source(x + "shared.gate", (f.shared_ff, D)),
                                                Source(x + "shared.up", (f.shared_ff, D))),
                              combine=torch.cat),
                      Binding(x + "shared_down", (Source(x + "shared.down", (D, f.shared_ff)),)),
                      Binding(x + "shared_gate", (Source(x + "shared.sg", (1, D)),))]
    b.append(vector("final.norm.weight", "final.norm", (D,)))
    b.append(Binding("head", (Source("head", (V, D)),)))
    # a layer without a feed-forward has no second sum: a norm or scale stored for it is not used
    unused = tuple(rf"^l{i}\.(norm2|ls2)$" for i, l in enumerate(c.layers) if l.mlp is None)
    return CheckpointLayout(tuple(b), ignored=unused)


def refolix_sizes(c: RefolixConfig) -> dict:
    """The sizes that the layers share, flat; per-layer sizes as short strings."""
    letter = {"parallel": "p", "retention": "r"}
    out = {"n_layer": len(c.layers), "dim": c.width, "vocab_size": c.vocab, "norm_eps": c.norm_eps,
           "layer_kinds": "".join(letter[l.type] for l in c.layers), "postln_alpha": c.alpha}
    for l in c.layers:
        m = l.mixer
        if isinstance(m, ParallelPair) and "parallel" not in out:
            a, r = m.left, m.right
            out["parallel"] = (f"attention {a.heads} heads of {a.dim}, {a.kv_heads} kv heads, values "
                               f"{a.vdim}, window {a.window}; delta rule {r.heads} heads of "
                               f"{r.dim} x {r.vdim}, {r.kv_heads} key heads, {r.conv} taps")
        if isinstance(m, Retention) and "retention" not in out:
            out["retention"] = f"{m.heads} heads of {m.dim} x {m.vdim}"
        if l.mlp is not None and "experts" not in out:
            f = l.mlp
            out["experts"] = (f"{f.experts} gated of {f.ff}, top {f.top}, {f.keep} of {f.groups} groups, "
                              f"shared {f.shared_ff}")
            out["intermediate_size"] = f.top * f.ff + f.shared_ff
    return out


REFOLIX = register_architecture(Architecture(
    names=("Refolix", "refolix"),
    read_config=RefolixConfig.from_dict,
    plan=refolix_plan,
    bindings=refolix_bindings,
    config_dict=RefolixConfig.to_dict,
    presets=RefolixConfig.from_name,
    describe=refolix_sizes,
    layer_count_key="layers",
))
