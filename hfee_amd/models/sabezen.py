"""The Sabezen decoder as a list of parts.

Every layer is a "parallel" block: one layer norm (a weight, no bias) whose output both the mixer and
the feed-forward read, x += mixer(h) + feed_forward(h).  The mixer of a layer is attention whose
heads' scores are mixed by a learned matrix before a softmax with a sink of score zero, over the keys
of the query's own chunk, with the keys as projected standing in for values ("mixed_attention"); the
gated delta rule with a decay a key channel behind short convolutions ("gated_delta"); or gated linear
attention ("gla").  The feed-forward is down(xielu(up(h))) ("dense_mlp") or experts that a table picks
by the token's id ("table_moe").  The embedding is scaled; the final norm is a layer norm.  Which layer
has which, and every size and constant, is config.json's.

What is fixed here is what the design fixes: rotation pairs (i, i + dims/2), the weightless norm of q
and k behind the rotation, the sink in every attention layer, the unit norm's 1e-6, 1 / top for every
chosen expert.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.sabezen import ChannelDeltaConfig, ChunkedAttentionConfig, DenseConfig, GlaConfig, MoeConfig, SabezenConfig
from ..config.specs import (EmbeddingSpec, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                            ScheduleEntry, params)


def _mixer(cfg: SabezenConfig, m) -> MixerSpec:
    if isinstance(m, ChunkedAttentionConfig):
        position = None
        if m.rot is not None:
            position = PositionSpec("rope", params(head_dim=m.dim, rotary_dim=m.rot.dims, theta=m.rot.base, scaling=None,
                                                   pairing="half"))
        return MixerSpec("mixed_attention", params(
            hidden=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, dim=m.dim, scale=m.scale, chunk=m.chunk,
            sink="zero", head_mix=True, qk_norm="rms_after_rotation", norm_eps=cfg.norm_eps, values="keys",
            names=(("q", "q"), ("k", "k"), ("o", "o"), ("head_mix", "talk"))), position=position)
    if isinstance(m, ChannelDeltaConfig):
        return MixerSpec("gated_delta", params(
            hidden=cfg.width, num_heads=m.heads, num_qk_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, conv=m.conv,
            decay_rank=m.decay_rank, gate_rank=m.gate_rank, unit_eps=1e-6, norm_eps=cfg.norm_eps,
            names=(("q", "q"), ("k", "k"), ("v", "v"), ("q_conv", "q.conv"), ("k_conv", "k.conv"), ("v_conv", "v.conv"),
                   ("b", "b"), ("a_log", "A_log"), ("norm", "norm"), ("a_down", "a1"), ("a_up", "a2"),
                   ("dt_bias", "dt_bias"), ("g_down", "g1"), ("g_up", "g2"), ("o", "o"))))
    if isinstance(m, GlaConfig):
        return MixerSpec("gla", params(
            hidden=cfg.width, num_heads=m.heads, dim=m.dim, vdim=m.vdim, tau=m.tau, decay_rank=m.decay_rank,
            norm_eps=cfg.norm_eps,
            names=(("q", "q"), ("k", "k"), ("v", "v"), ("g", "g"), ("o", "o"), ("norm", "norm"), ("a_down", "a1"),
                   ("a_up", "a2"), ("a_bias", "a2.b"))))
    raise ValueError(f"no part for a mixer of type {m.type!r}")


def _feed_forward(cfg: SabezenConfig, mlp):
    if mlp is None:
        return None
    if isinstance(mlp, DenseConfig):
        return FeedForwardSpec("dense_mlp", params(
            hidden=cfg.width, intermediate=mlp.ff, activation="xielu", bias=False,
            names=(("up", "up"), ("down", "down"), ("activation", "act"))))
    if isinstance(mlp, MoeConfig):
        return FeedForwardSpec("table_moe", params(
            hidden=cfg.width, intermediate=mlp.ff, experts=mlp.experts, top=mlp.top, vocab=cfg.vocab, activation="silu",
            names=(("expert", "e{}."), ("gate", "gate"), ("up", "up"), ("down", "down"), ("table", "table"))))
    raise ValueError(f"no part for a feed-forward of kind {mlp.kind!r}")


def sabezen_model_spec(cfg: SabezenConfig) -> ModelSpec:
    norm = NormSpec("layernorm", cfg.width, cfg.norm_eps)
    layers = tuple(
        LayerSpec(arrangement="parallel", hidden=cfg.width, mixer=_mixer(cfg, layer.mixer),
                  feed_forward=_feed_forward(cfg, layer.mlp), mixer_norm=norm, feed_forward_norm=norm, prefix=f"l{i}.",
                  names=(("mixer", "mix."), ("feed_forward", "mlp."), ("mixer_norm", "norm1")))
        for i, layer in enumerate(cfg.layers))
    schedule = tuple(ScheduleEntry(layer=i, cache=i) for i in range(len(layers)))
    return ModelSpec(
        architecture=cfg.architecture, hidden=cfg.width, vocab=cfg.vocab, layers=layers, schedule=schedule,
        final_norm=norm, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_ids=tuple(cfg.eos_token_ids), bos_token_id=cfg.bos_token_id,
        embedding=EmbeddingSpec("lookup", params(scale=cfg.embedding_scale)))


register_architecture("Sabezen", SabezenConfig, sabezen_model_spec)
