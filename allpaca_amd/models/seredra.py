"""The Seredra decoder described with parts (config.json "architecture": "Seredra").

Token rows times a scale.  A layer is pre-norm, x += mixer(norm1(x)), x += ff(norm2(x)), its norms RMS norms whose
weight is a single number.  Its mixer is one of three: a grouped attention whose q, k and v (with biases) pass a short
causal convolution, q and k normed over the whole projection, a query temperature that grows with the position, a
learned penalty on the distance in the scores, no rotation (optionally reading the keys and values of an earlier
layer); two mixers side by side, a grouped attention whose values are its keys as projected (norm per head, rotation
with a frequency rule for longer contexts, a soft cap on the scores) beside a selective scan, their outputs added with
constant factors; or a retention (linear attention with a fixed decay a head, rotated q and k, every head's output
divided by its root mean square, a silu gate).  Its feed-forward is two matrices around a squared relu, routed experts
(sigmoid scores, the weight on the expert's input), or none.  Final norm and head.  Tensor names: `embed`,
`l<i>.norm1|norm2`, `l<i>.mix.q|k|v|o` (+ `.b`, `.conv`, `.norm`), `l<i>.mix.r1|r2`, `l<i>.mix.left.q|k|o` (+
`.norm`), `l<i>.mix.right.in|conv|conv.b|x|dt|dt.b|A_log|D|o`, `l<i>.mix.g`, `l<i>.mlp.up|down`, `l<i>.mlp.router`,
`l<i>.mlp.e<j>.gate|up|down`, `final.norm`, `head`."""
from __future__ import annotations

from ..config.seredra import SeredraAttention, SeredraConfig, SeredraDense, SeredraParallel, sizes_from_tensors
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture


def _norm(cfg: SeredraConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", dict(size=cfg.width, eps=cfg.eps, name=name, scalar=True))


def seredra_spec(cfg: SeredraConfig) -> ModelSpec:
    D = cfg.width
    blocks, plan = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        cache_of = None
        if isinstance(m, SeredraAttention):
            mixer = PartSpec("conv_attention", dict(
                hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, conv_taps=m.conv, unit_norm=True, norm_eps=cfg.eps, bias=True, mask="causal",
                sink=False, shares_kv=m.kv_from is not None, norm_weights=True, norm_scope="projection",
                q_temp=m.q_temp, distance_bias=True, out_bias=True), "mix.")
            cache_of = m.kv_from
        elif isinstance(m, SeredraParallel):
            l, r = m.left, m.right
            scaling = None
            if l.scaling is not None:
                scaling = dict(rope_type="yarn", factor=l.scaling.factor, original=l.scaling.original,
                               fast=l.scaling.fast, slow=l.scaling.slow)
            mixer = PartSpec("parallel", dict(members=[
                dict(name="left", kind="sink_attention", scale=m.left_scale, params=dict(
                    hidden_size=D, num_heads=l.heads, num_kv_heads=l.kv_heads, key_dim=l.dim, value_dim=l.vdim,
                    scale=l.scale, rotary_dim=l.rot_dims, rope_theta=l.rot_base, rope_scaling=scaling, mask="causal",
                    learned_sink=False, values_are_keys=True, qk_norm=True, norm_eps=cfg.eps, softcap=l.softcap)),
                dict(name="right", kind="selective_scan", scale=m.right_scale, params=dict(
                    hidden_size=D, inner=r.inner, state=r.state, dt_rank=r.dt_rank, conv_taps=r.conv)),
            ]), "mix.")
        else:
            mixer = PartSpec("decay_linear_attention", dict(
                hidden_size=D, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, decay=m.decay, norm_eps=cfg.eps,
                activation="none", gate=True, rotary_dim=m.rot_dims, rope_theta=m.rot_base,
                key_scale=float(m.dim) ** -0.5, norm="heads", gate_act="silu"), "mix.")
        parts = {"mixer_norm": _norm(cfg, "norm1"), "mixer": mixer, "scale": PartSpec("scaled", dict(mult=1.0))}
        f = layer.mlp
        if f is not None:
            parts["ffn_norm"] = _norm(cfg, "norm2")
            if isinstance(f, SeredraDense):
                parts["ffn"] = PartSpec("mlp", dict(hidden_size=D, intermediate_size=f.ff, activation="relu2"), "mlp.")
            else:
                parts["ffn"] = PartSpec("routed_experts", dict(
                    hidden_size=D, intermediate_size=f.ff, experts=f.experts, top=f.top, identity=0, correction=False,
                    renormalize=False, activation="silu", score="sigmoid", weight_on="input"), "mlp.")
        blocks.append(BlockSpec(arrangement="pre_norm", weight_prefix=f"l{i}.", parts=parts))
        plan.append(PlanEntry(i, cache_of=cache_of))
    return ModelSpec(
        hidden_size=D,
        vocab_size=cfg.vocab,
        max_positions=cfg.max_positions,
        embedding=PartSpec("token_table", dict(vocab_size=cfg.vocab, hidden_size=D, name="embed",
                                               scale=cfg.embedding_scale)),
        blocks=blocks,
        plan=plan,
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=D, name="head")),
    )


ARCHITECTURES.register("Seredra", Architecture("seredra", SeredraConfig.from_dict, seredra_spec, sizes_from_tensors))
