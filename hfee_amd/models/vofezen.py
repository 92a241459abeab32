"""The Vofezen decoder as a list of parts.

Every layer is a "sandwich" block: a norm in front of and behind each sub-layer,
x += norm_b(mixer(norm_a(x))), then x += norm_d(feed_forward(norm_c(x))), all norms with weights
stored around zero (multiply by 1 + w).  The mixer of a layer is grouped attention with key and
value sizes of its own, a rotation of the first dims of each head under the "yarn" stretching, a
sink in the softmax and values blended with those of the first blending layer ("kv_attention"), or
latent attention ("latent_attention"); the feed-forward is down(relu(up(h) + b)^2) + b'
("dense_mlp").  Which layer has which, and every size and constant, is config.json's.

What is fixed here is what the design fixes: rotation pairs (i, i + dims/2), the sink in every
"attention" layer, the latents' norms with plain weights and the layer's eps, the square of relu.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.specs import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                            ScheduleEntry, params)
from ..config.vofezen import AttentionConfig, LatentAttentionConfig, VofezenConfig


def _rope(head_dim: int, rot) -> PositionSpec:
    scaling = None if rot.scaling is None else ("yarn",) + tuple(rot.scaling)
    return PositionSpec("rope", params(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, scaling=scaling,
                                       pairing="half"))


def vofezen_model_spec(cfg: VofezenConfig) -> ModelSpec:
    norm = NormSpec("rmsnorm", cfg.width, cfg.norm_eps, params(weight_offset=1.0))
    layers = []
    blend_source_seen = False
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, AttentionConfig):
            blend = None
            if m.v_mix:
                blend = "mix" if blend_source_seen else "source"
                blend_source_seen = True
            mixer = MixerSpec("kv_attention", params(
                hidden=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, sink=True, value_blend=blend,
                names=(("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("sink", "sink"), ("value_blend", "vmix"))),
                position=_rope(m.dim, m.rot))
        elif isinstance(m, LatentAttentionConfig):
            mixer = MixerSpec("latent_attention", params(
                hidden=cfg.width, num_heads=m.heads, plain_dim=m.dim, rotated_dim=m.rot_dim, value_dim=m.vdim,
                q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, norm_eps=cfg.norm_eps,
                names=(("q_down", "dq"), ("q_norm", "dq.norm"), ("q_up", "uq"), ("kv_down", "dkv"),
                       ("kv_norm", "dkv.norm"), ("k_up", "uk"), ("v_up", "uv"), ("o", "o"))),
                position=_rope(m.rot_dim, m.rot))
        else:
            raise ValueError(f"layer {i}: no part for a mixer of type {m.type!r}")
        ffn = None
        if layer.mlp is not None:
            ffn = FeedForwardSpec("dense_mlp", params(
                hidden=cfg.width, intermediate=layer.mlp.ff, activation="relu2", bias=True,
                names=(("up", "up"), ("up_bias", "up.b"), ("down", "down"), ("down_bias", "down.b"))))
        layers.append(LayerSpec(
            arrangement="sandwich", hidden=cfg.width, mixer=mixer, feed_forward=ffn, mixer_norm=norm,
            feed_forward_norm=norm, prefix=f"l{i}.",
            names=(("mixer", "mix."), ("feed_forward", "mlp."), ("mixer_norm", "norm1"), ("mixer_post_norm", "norm1b"),
                   ("feed_forward_norm", "norm2"), ("feed_forward_post_norm", "norm2b"))))
    schedule = tuple(ScheduleEntry(layer=i, cache=i) for i in range(len(layers)))
    return ModelSpec(
        architecture=cfg.architecture, hidden=cfg.width, vocab=cfg.vocab, layers=tuple(layers), schedule=schedule,
        final_norm=norm, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_ids=tuple(cfg.eos_token_ids), bos_token_id=cfg.bos_token_id)


register_architecture("Vofezen", VofezenConfig, vofezen_model_spec)
