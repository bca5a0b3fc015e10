"""The Lesarax decoder described with parts (config.json "architecture": "Lesarax").

Token rows from the table `embed`, which is also the output head.  A layer is pre-norm with a scaled sum:
x += m * mixer(norm1(x)), x += m * ff(norm2(x)).  Its mixer is a grouped attention whose values are the keys as
projected (rotation on the first elements of a head, a learned sink a head), or an attention through low-rank latents
with one rotated key part shared by the heads, a sliding window, a learned sink and a gate a head.  Its feed-forward
is a set of routed experts (clamped gated units, the softmax over the chosen logits), or none.  A range of layers may
run several times in a row with the same weights; every run has a cache of its own (a plan entry each), and ahead of
every pass the stream is mixed with the embedding's output through `loop.in`.  Tensor names: `embed`, `loop.in`,
`l<i>.norm1|norm2`, `l<i>.mix.q|k|sink|o`, `l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|sink|g|o`,
`l<i>.mlp.router`, `l<i>.mlp.e<j>.gate|up|down`, `final.norm`."""
from __future__ import annotations

from ..config.lesarax import LesaraxAttention, LesaraxConfig, sizes_from_tensors
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture

EXPERT_ALPHA = 1.702       # the factor inside the experts' sigmoid: a constant of the design


def lesarax_spec(cfg: LesaraxConfig) -> ModelSpec:
    D = cfg.width
    blocks = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, LesaraxAttention):
            mixer = PartSpec("sink_attention", dict(
                hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, rotary_dim=m.rot_dims, rope_theta=m.rot_base,
                mask="causal" if m.window is None else "window", mask_size=m.window or 0, learned_sink=True,
                values_are_keys=True), "mix.")
        else:
            mixer = PartSpec("latent_attention", dict(
                hidden_size=D, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, q_rank=m.q_rank,
                kv_rank=m.kv_rank, scale=m.scale, rope_theta=m.rot_base, norm_eps=cfg.eps,
                mask="causal" if m.window is None else "window", mask_size=m.window or 0, learned_sink=True,
                head_gate=True), "mix.")
        parts = {"mixer_norm": PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm1")),
                 "mixer": mixer,
                 "scale": PartSpec("scaled", dict(mult=cfg.residual_mult))}
        f = layer.mlp
        if f is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="norm2"))
            parts["ffn"] = PartSpec("routed_experts", dict(
                hidden_size=D, intermediate_size=f.ff, experts=f.experts, top=f.top, identity=0, correction=False,
                renormalize=True, activation="clamped", alpha=EXPERT_ALPHA, limit=f.limit), "mlp.")
        blocks.append(BlockSpec(arrangement="pre_norm", weight_prefix=f"l{i}.", parts=parts))
    links = [PartSpec("reinject", dict(hidden_size=D, name="loop.in"))] if cfg.loop is not None else []
    plan = [PlanEntry(i, enter=0 if enters else None) for i, enters in cfg.order()]
    return ModelSpec(
        hidden_size=D,
        vocab_size=cfg.vocab,
        max_positions=cfg.max_positions,
        embedding=PartSpec("token_table", dict(vocab_size=cfg.vocab, hidden_size=D, name="embed")),
        blocks=blocks,
        plan=plan,
        links=links,
        final_norm=PartSpec("rmsnorm", dict(size=D, eps=cfg.eps, name="final.norm")),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=D, tied=True)),
    )


ARCHITECTURES.register("Lesarax", Architecture("lesarax", LesaraxConfig.from_dict, lesarax_spec, sizes_from_tensors))
