"""The Vusenex decoder as data: its plan and its checkpoint layout.

Plan: the embedded rows get a hashed embedding of the pair (previous token, token) and a
learned position vector; the layers ``config.json`` lists, each a block whose sublayers read
the stream itself and whose results are gated and normed before they join it
(``x + norm1(sigmoid(W1 x + b1) * mixer(x))``, ``x + norm2(sigmoid(W2 x + b2) * ff(x))``, the
norms with one number each); the mixer is attention whose values are its keys, with a bias by
log distance and a sink, or latent attention without positions; the feed-forward a mixture of
experts with a shared expert.

Checkpoint layout: ``embed``, ``bigram``, ``pos``, ``l<i>.norm1``, ``l<i>.rg1`` (+ ``.b``),
``l<i>.mix.<name>``, ``l<i>.mlp.e<k>.up`` / ``.down``, ``l<i>.mlp.router``,
``l<i>.mlp.shared.up`` / ``.down``, ``final.norm``, ``head``; linear weights [out, in]; biases
under the weight's name with ``.b``.  Projections that read the same input are joined into
one matrix when they are loaded, and the experts' matrices are stacked.
"""
import torch

from ..config.registry import Architecture, register_architecture
from ..config.spec import (LatentAttentionSpec, LayerSpec, ModelPlan, NormSpec, PairEmbeddingSpec,
                           PositionSpec, RoutedExpertsSpec, Run, SinkAttentionSpec)
from ..config.vusenex import LatentMixer, SinkMixer, VusenexConfig
from ..weights.bindings import Binding, CheckpointLayout, Source

PAIR_TABLE = "bigram"
POSITION_TABLE = "pos"


def _mixer_spec(c: VusenexConfig, m):
    if isinstance(m, SinkMixer):
        return SinkAttentionSpec(dim=c.width, n_heads=m.heads, n_kv_heads=m.kv_heads,
                                 head_dim=m.dim, value_dim=m.vdim, scale=m.scale, biases=True,
                                 values_are_keys=True, whole_norm_eps=c.norm_eps,
                                 q_temp_coef=m.q_temp_coef, q_temp_every=m.q_temp_every,
                                 log_distance_bias=True, sink=True)
    assert isinstance(m, LatentMixer)
    return LatentAttentionSpec(dim=c.width, n_heads=m.heads, head_dim=m.dim, rot_dim=0,
                               value_dim=m.vdim, q_rank=None, kv_rank=m.kv_rank, scale=m.scale,
                               eps=c.norm_eps, position=PositionSpec(kind="none"), window=None)


def _feed_forward_spec(c: VusenexConfig, mlp):
    return RoutedExpertsSpec(dim=c.width, n_experts=mlp.experts, top=mlp.top, hidden=mlp.ff,
                             n_groups=mlp.groups, keep_groups=mlp.keep, shared_hidden=mlp.shared_ff,
                             activation="gelu", weight_eps=1e-20)


def vusenex_plan(c: VusenexConfig) -> ModelPlan:
    def one_number():
        return NormSpec(c.width, c.norm_eps, kind="rms_scalar")

    def none():
        return NormSpec(c.width, c.norm_eps, kind="none")

    layers = []
    for i, l in enumerate(c.layers):
        has_ff = l.mlp is not None
        layers.append(LayerSpec(
            name=f"l{i}", arrangement="sandwich_norm", result_gate=True,
            mixer=_mixer_spec(c, l.mixer), mixer_norm=none(), mixer_out_norm=one_number(),
            feed_forward=_feed_forward_spec(c, l.mlp) if has_ff else None,
            feed_forward_norm=none() if has_ff else None,
            feed_forward_out_norm=one_number() if has_ff else None,
            mixer_name="mix", mixer_norm_name="read1", mixer_out_norm_name="norm1",
            mixer_gate_name="rg1", feed_forward_name="mlp", feed_forward_norm_name="read2",
            feed_forward_out_norm_name="norm2", feed_forward_gate_name="rg2"))
    plan = ModelPlan(
        dim=c.width, vocab_size=c.vocab, layers=layers, order=[Run(i) for i in range(len(layers))],
        final_norm=one_number(), tie_embeddings=False, max_positions=c.max_positions,
        embedding_name="embed", final_norm_name="final.norm", head_name="head",
        input_adds=(PairEmbeddingSpec(dim=c.width, buckets=c.buckets, mul_prev=c.mul_prev,
                                      mul_cur=c.mul_cur, name=PAIR_TABLE),),
        input_position=PositionSpec(kind="learned", dim=c.width, max_positions=c.max_positions),
        input_position_name=POSITION_TABLE)
    plan.validate()
    return plan


def vusenex_bindings(c: VusenexConfig) -> CheckpointLayout:
    D, V = c.width, c.vocab
    b = [Binding("embed", (Source("embed", (V, D)),)),
         Binding(PAIR_TABLE + ".table", (Source("bigram", (c.buckets + 1, D)),)),
         Binding(POSITION_TABLE + ".table", (Source("pos", (c.max_positions, D)),))]

    def vector(target, name, shape, init="norm"):
        return Binding(target, (Source(name, shape, init),), role="vector")

    for i, l in enumerate(c.layers):
        p = f"l{i}."
        m = l.mixer
        b += [vector(p + "norm1.weight", p + "norm1", ()),
              Binding(p + "rg1.weight", (Source(p + "rg1", (D, D)),)),
              vector(p + "rg1.bias", p + "rg1.b", (D,), "around_zero")]
        if isinstance(m, SinkMixer):
            H, G, d = m.heads, m.kv_heads, m.dim
            b += [
                Binding(p + "mix.w_in", (Source(p + "mix.q", (H * d, D)), Source(p + "mix.k", (G * d, D))),
                        combine=torch.cat),
                Binding(p + "mix.b_in", (Source(p + "mix.q.b", (H * d,), "around_zero"),
                                         Source(p + "mix.k.b", (G * d,), "around_zero")),
                        role="vector", combine=torch.cat),
                vector(p + "mix.q_norm", p + "mix.q.norm", (H * d,)),
                vector(p + "mix.k_norm", p + "mix.k.norm", (G * d,)),
                vector(p + "mix.r1", p + "mix.r1", (H,), "positive"),
                vector(p + "mix.r2", p + "mix.r2", (H,), "positive"),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * m.vdim)),)),
            ]
        else:
            assert isinstance(m, LatentMixer)
            H, d, dv, R = m.heads, m.dim, m.vdim, m.kv_rank
            b += [
                # the kv latent's rows first, then the query's: one product over x serves both
                Binding(p + "mix.w_down", (Source(p + "mix.dkv", (R, D)), Source(p + "mix.q", (H * d, D))),
                        combine=torch.cat),
                vector(p + "mix.kv_norm", p + "mix.dkv.norm", (R,)),
                Binding(p + "mix.w_uk", (Source(p + "mix.uk", (H * d, R)),)),
                Binding(p + "mix.w_uv", (Source(p + "mix.uv", (H * dv, R)),)),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
            ]
        if l.mlp is not None:
            f = l.mlp
            b += [
                vector(p + "norm2.weight", p + "norm2", ()),
                Binding(p + "rg2.weight", (Source(p + "rg2", (D, D)),)),
                vector(p + "rg2.bias", p + "rg2.b", (D,), "around_zero"),
                Binding(p + "mlp.w_router", (Source(p + "mlp.router", (f.experts, D)),)),
                Binding(p + "mlp.w_up", tuple(Source(f"{p}mlp.e{e}.up", (f.ff, D)) for e in range(f.experts)),
                        combine=torch.stack),
                Binding(p + "mlp.w_down", tuple(Source(f"{p}mlp.e{e}.down", (D, f.ff)) for e in range(f.experts)),
                        combine=torch.stack),
            ]
            if f.shared_ff:
                b += [Binding(p + "mlp.shared_up", (Source(p + "mlp.shared.up", (f.shared_ff, D)),)),
                      Binding(p + "mlp.shared_down", (Source(p + "mlp.shared.down", (D, f.shared_ff)),))]
    b.append(vector("final.norm.weight", "final.norm", ()))
    b.append(Binding("head", (Source("head", (V, D)),)))
    return CheckpointLayout(tuple(b))


def vusenex_sizes_from_tensors(c: VusenexConfig, shapes: dict) -> VusenexConfig:
    """Sizes that a configuration may leave to the checkpoint's tensors: the rows of the table
    of learned positions."""
    import dataclasses
    if c.max_positions <= 0 and "pos" in shapes and len(shapes["pos"]) == 2:
        return dataclasses.replace(c, max_positions=int(shapes["pos"][0]))
    return c


def vusenex_sizes(c: VusenexConfig) -> dict:
    """The sizes that the layers share, flat; per-layer sizes as short strings."""
    letter = {"latent_attention": "c", "attention": "a"}
    out = {"n_layer": len(c.layers), "dim": c.width, "vocab_size": c.vocab, "norm_eps": c.norm_eps,
           "layer_kinds": "".join(letter[l.type] for l in c.layers),
           "pair_buckets": c.buckets, "max_positions": c.max_positions}
    for l in c.layers:
        m = l.mixer
        if isinstance(m, LatentMixer) and "latent_attention" not in out:
            out["latent_attention"] = (f"{m.heads} heads of {m.dim}, values {m.vdim}, "
                                       f"latent {m.kv_rank}")
        if isinstance(m, SinkMixer) and "attention" not in out:
            out["attention"] = f"{m.heads} heads of {m.dim}, {m.kv_heads} kv heads, values are keys"
        if l.mlp is not None and "experts" not in out:
            f = l.mlp
            out["experts"] = (f"{f.experts} of {f.ff}, top {f.top}, {f.keep} of {f.groups} groups, "
                              f"shared {f.shared_ff}")
            out["intermediate_size"] = f.top * f.ff + f.shared_ff
    return out


VUSENEX = register_architecture(Architecture(
    names=("Vusenex", "vusenex"),
    read_config=VusenexConfig.from_dict,
    plan=vusenex_plan,
    bindings=vusenex_bindings,
    config_dict=VusenexConfig.to_dict,
    presets=VusenexConfig.from_name,
    describe=vusenex_sizes,
    layer_count_key="layers",
    sizes_from_tensors=vusenex_sizes_from_tensors,
))
