"""``Miberax`` as a list of parts. Tensor names: ``embed``, ``final.norm``, and per layer ``i``
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{left,right}.<name>``, ``l<i>.mix.{left,right}.out`` and
``l<i>.mlp.<name>``; the head is the embedding table. Every layer is the ``pre_norm`` arrangement
around a 32-bit residual stream, with RMS norms in groups; its mixer is a pair of mixers side by
side (rotary attention under a chunked mask; a gated delta rule), its feed-forward dense with a
polynomial activation, a mixture of experts, or absent."""

from __future__ import annotations

from ..config.miberax import MiberaxConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_miberax_spec(cfg: MiberaxConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps

    def norm(name: str, prefix: str) -> PartSpec:
        return PartSpec("group_rms_norm", dict(width=w, eps=eps, groups=cfg.norm_groups, weight_name=name), prefix)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        a, d = layer.left, layer.right
        position = None
        if a.rot_dims:
            position = PartSpec("rotary", dict(dim=a.rot_dims, theta=a.rot_base, pairing="interleaved",
                                               rope_type="linear" if a.rot_factor != 1.0 else "default", factor=a.rot_factor))
        left = PartSpec("scored_attention", dict(
            hidden_size=w, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim, scale=a.scale,
            qk_unit=False, position=position, chunk=a.chunk), p + "mix.left.")
        right = PartSpec("gated_delta", dict(
            hidden_size=w, num_heads=d.heads, num_kv_heads=d.kv_heads, head_dim=d.dim, value_dim=d.vdim, conv_taps=d.conv,
            norm_eps=eps), p + "mix.right.")
        mixer = PartSpec("parallel_mixers", dict(hidden_size=w, branches={"left": left, "right": right}, norm_eps=eps),
                         p + "mix.")
        parts = {"mixer": ("mixer", mixer), "mixer_norm": ("norm", norm("norm1", p))}
        m = layer.mlp
        if m is not None:
            if m.kind == "dense":
                ff = PartSpec("poly_norm_mlp", dict(hidden_size=w, intermediate_size=m.ff, norm_eps=eps), p + "mlp.")
            else:
                ff = PartSpec("routed_experts", dict(
                    hidden_size=w, experts=m.experts, top=m.top, expert_size=m.ff, limit=m.limit, identity=m.identity,
                    groups=m.groups, groups_kept=m.groups_kept, scale=m.scale, shared_size=m.shared_ff,
                    shared_limit=m.shared_limit), p + "mlp.")
            parts["feed_forward"] = ("feed_forward", ff)
            parts["feed_forward_norm"] = ("norm", norm("norm2", p))
        layers.append(LayerSpec(block=PartSpec("pre_norm"), parts=parts))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=w,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=w, weight_name="embed",
                                                   float32_rows=True)),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=norm("norm", "final."),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=w, tied=True)))


register_architecture("Miberax", MiberaxConfig.from_dict, build_miberax_spec, model_types=("miberax",), replace=True)
