"""SabezenConfig: the Sabezen decoder's configuration, read from config.json.

The file lists the layers one by one: each entry names its mixer (`type`: "attention",
"channel_delta" or "gla") with that mixer's sizes and constants (`mixer`), and its feed-forward
(`mlp`: {"kind": "dense", "ff"}, {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}, or
null for a layer without one).  Beside the list it gives the vocabulary, the width, the norms' eps
and the embedding's scale.  The ranks of the low-rank projections are not in the file: they are the
shapes of their tensors, so the configuration takes them from the checkpoint's header when it is
read from a folder (`tensor_shapes`), or from `decay_rank` / `gate_rank` where a caller gives them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .base import ConfigError, KeyReader
from .vofezen import RotaryConfig


def _positive(r: KeyReader, **values):
    for name, v in values.items():
        r.require(v is None or v > 0, f"{name} must be positive")


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int                      # 0: no chunks
    rot: Optional[RotaryConfig]
    type: str = "attention"

    @staticmethod
    def read(data: dict, where: str, ranks=None) -> "ChunkedAttentionConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        kv_heads, vdim = r.int("kv_heads", heads), r.int("vdim", dim)
        scale = r.float("scale")
        # (a layer whose entry names no mask sees every earlier position; one that names no rotation is not rotated)
        rot, mask = r.object("rot", None), r.object("mask", None)
        r.require(not heads or not kv_heads or (heads > 0 and kv_heads > 0 and heads % kv_heads == 0),
                  f"{heads} heads are not a multiple of {kv_heads} kv_heads")
        _positive(r, dim=dim, vdim=vdim)
        r.require(dim is None or vdim == dim, f"the values are the keys: vdim {vdim} must equal dim {dim}")
        r.finish()
        chunk = 0
        if mask is not None:
            rm = KeyReader(mask, where + ".mask")
            chunk = rm.int("size")
            _positive(rm, size=chunk)
            rm.finish()
        rc = None
        if rot is not None:
            rc = RotaryConfig.read(rot, where + ".rot")
            if rc.scaling is not None:
                raise ConfigError(f"{where}.rot: this design's rotation is not stretched")
            if rc.dims > dim:
                raise ConfigError(f"{where}: {rc.dims} rotated dims do not fit a head of {dim}")
        return ChunkedAttentionConfig(heads, kv_heads, dim, vdim, scale, chunk, rc)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int
    type: str = "channel_delta"

    @staticmethod
    def read(data: dict, where: str, ranks=None) -> "ChannelDeltaConfig":
        r = KeyReader(data, where)
        heads, dim, conv = r.int("heads"), r.int("dim"), r.int("conv")
        kv_heads, vdim = r.int("kv_heads", heads), r.int("vdim", dim)
        ranks = ranks or {}
        decay_rank = r.int("decay_rank", ranks.get("a1", None))
        gate_rank = r.int("gate_rank", ranks.get("g1", None))
        r.require(not heads or not kv_heads or (heads > 0 and kv_heads > 0 and heads % kv_heads == 0),
                  f"{heads} heads are not a multiple of {kv_heads} kv_heads")
        _positive(r, dim=dim, vdim=vdim, conv=conv)
        r.require(decay_rank is not None and gate_rank is not None,
                  "the ranks of the decay's and the gate's projections are given by their tensors' shapes "
                  "(or by decay_rank and gate_rank)")
        r.finish()
        return ChannelDeltaConfig(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
                "decay_rank": self.decay_rank, "gate_rank": self.gate_rank}


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int
    type: str = "gla"

    @staticmethod
    def read(data: dict, where: str, ranks=None) -> "GlaConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        vdim, tau = r.int("vdim", dim), r.float("tau")
        decay_rank = r.int("decay_rank", (ranks or {}).get("a1", None))
        _positive(r, heads=heads, dim=dim, vdim=vdim, tau=tau)
        r.require(decay_rank is not None, "the rank of the decay's projections is given by their tensors' shapes (or by decay_rank)")
        r.finish()
        return GlaConfig(heads, dim, vdim, tau, decay_rank)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau, "decay_rank": self.decay_rank}


MIXERS = {"attention": ChunkedAttentionConfig, "channel_delta": ChannelDeltaConfig, "gla": GlaConfig}


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    kind: str = "dense"

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class MoeConfig:
    ff: int
    experts: int
    top: int
    kind: str = "moe"

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


def _read_mlp(mlp: dict, where: str):
    r = KeyReader(mlp, where)
    kind = r.str("kind", "dense")
    if kind == "dense":
        ff = r.int("ff")
        _positive(r, ff=ff)
        r.finish()
        return DenseConfig(ff)
    if kind == "moe":
        expert, router = r.object("expert"), r.object("router")
        r.finish()
        re_, rr = KeyReader(expert, where + ".expert"), KeyReader(router, where + ".router")
        ff, experts, top = re_.int("ff"), rr.int("experts"), rr.int("top")
        _positive(re_, ff=ff)
        _positive(rr, experts=experts, top=top)
        rr.require(not experts or not top or top <= experts, f"a token cannot use {top} of {experts} experts")
        re_.finish()
        rr.finish()
        return MoeConfig(ff, experts, top)
    raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: dense, moe)")


@dataclass(frozen=True)
class LayerConfig:
    mixer: object                   # one of MIXERS' classes
    mlp: object                     # DenseConfig, MoeConfig or None


@dataclass(frozen=True)
class SabezenConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: tuple                   # of LayerConfig
    max_positions: int
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None

    # the design names no longest context; the engine's tables are made for what a caller asks
    # for (its num_ctx or a trace's max_tokens), up to this
    DEFAULT_MAX_POSITIONS = 1 << 20
    reads_tensor_shapes = True

    @staticmethod
    def from_dict(data: dict, where: str = "config.json", tensor_shapes=None) -> "SabezenConfig":
        """tensor_shapes: name -> shape of the checkpoint's tensors, where there is one: the ranks of
        the low-rank projections are read from it."""
        r = KeyReader(data, where)
        arch = r.str("architecture", "Sabezen")
        vocab, width = r.int("vocab"), r.int("width")
        norm = r.object("norm")
        embedding = r.object("embedding", {})
        layers = data.get("layers")
        r.require(isinstance(layers, list) and len(layers) > 0, "key 'layers' must be a non-empty list")
        _positive(r, vocab=vocab, width=width)
        max_positions = r.int("max_positions", SabezenConfig.DEFAULT_MAX_POSITIONS)
        eos = r.int_or_list("eos_token_id", None)
        bos = r.int("bos_token_id", None)
        r.finish()
        rn = KeyReader(norm, where + ".norm")
        eps = rn.float("eps")
        rn.require(eps is None or eps >= 0, "eps must not be negative")
        rn.finish()
        rs = KeyReader(embedding, where + ".embedding")
        scale = rs.float("scale", 1.0)
        rs.finish()
        out = []
        for i, layer in enumerate(layers):
            at = f"{where}.layers[{i}]"
            rl = KeyReader(layer, at)
            kind = rl.str("type")
            mixer = rl.object("mixer")
            mlp = rl.object("mlp", None)
            rl.require(kind is None or kind in MIXERS, f"unknown mixer type {kind!r} (known: {', '.join(sorted(MIXERS))})")
            rl.finish()
            ranks = {}
            for low in ("a1", "g1"):
                shape = (tensor_shapes or {}).get(f"l{i}.mix.{low}")
                if shape is not None and len(shape) == 2:
                    ranks[low] = int(shape[0])
            m = MIXERS[kind].read(mixer, at + ".mixer", ranks)
            out.append(LayerConfig(m, None if mlp is None else _read_mlp(mlp, at + ".mlp")))
        return SabezenConfig(arch, vocab, width, eps, scale, tuple(out), max_positions, tuple(eos), bos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
               "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                          for l in self.layers]}
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out
