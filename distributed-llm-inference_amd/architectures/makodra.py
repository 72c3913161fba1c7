"""``Makodra`` as a list of parts. Tensor names: ``embed``, ``final.norm``, and per layer ``i``
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>`` and ``l<i>.mlp.{gate,up,down}``; the head is the
embedding table. Every layer is the ``output_norm`` arrangement around a 32-bit residual stream;
the first attention layer that mixes values is the one whose values the later ones mix in."""

from __future__ import annotations

from ..config.makodra import MakodraConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_makodra_spec(cfg: MakodraConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    layers = []
    seen_value_source = False
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == "attention":
            value_mix = "none"
            if layer.v_mix:
                value_mix = "mix" if seen_value_source else "source"
                seen_value_source = True
            mixer = PartSpec("scored_attention", dict(
                hidden_size=w, num_heads=layer.heads, num_kv_heads=layer.kv_heads, head_dim=layer.dim,
                value_dim=layer.vdim, scale=layer.scale, qk_unit=True, norm_eps=eps, distance_penalty=True,
                chunk=layer.chunk, sink=True, output_gate=True, value_mix=value_mix), p + "mix.")
        else:
            mixer = PartSpec(layer.type, dict(hidden_size=w, num_heads=layer.heads, head_dim=layer.dim, norm_eps=eps,
                                              decay_rank=layer.rank), p + "mix.")
        parts = {"mixer": ("mixer", mixer),
                 "mixer_norm": ("norm", PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm1"), p))}
        if layer.ff:
            parts["feed_forward"] = ("feed_forward", PartSpec("gated_mlp", dict(
                hidden_size=w, intermediate_size=layer.ff, names={"gate": "gate", "up": "up", "down": "down"},
                few_rows_fused=True), p + "mlp."))
            parts["feed_forward_norm"] = ("norm", PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm2"), p))
        layers.append(LayerSpec(block=PartSpec("output_norm"), parts=parts))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=w,
        embedding=PartSpec("sinusoidal_token_embedding", dict(vocab_size=cfg.vocab, hidden_size=w, weight_name="embed")),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm"), "final."),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=w, tied=True, softcap=cfg.logit_softcap)))


register_architecture("Makodra", MakodraConfig.from_dict, build_makodra_spec, model_types=("makodra",), replace=True)
