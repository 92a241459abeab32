"""VofezenConfig: the Vofezen decoder's configuration, read from config.json.

The file lists the layers one by one: each entry names its mixer (`type`: "attention" or
"latent_attention") with that mixer's sizes and constants (`mixer`), and its feed-forward
(`mlp`, or null for a layer without one).  Beside the list it gives the vocabulary, the width
and the norms' eps.  Nothing else is read, and nothing that the file gives stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[tuple]       # (factor, original, fast, slow) or None

    @staticmethod
    def read(data: dict, where: str, dims_default=None) -> "RotaryConfig":
        r = KeyReader(data, where)
        base = r.float("base")
        dims = r.int("dims") if dims_default is None else r.int("dims", dims_default)
        sc = r.object("scaling", None)
        scaling = None
        if sc is not None:
            rs = KeyReader(sc, where + ".scaling")
            scaling = (rs.float("factor"), rs.float("original"), rs.float("fast"), rs.float("slow"))
            rs.finish()
            r.require(scaling[0] > 0 and scaling[1] > 0 and scaling[2] > 0 and scaling[3] > 0,
                      "the scaling's factor, original, fast and slow must be positive")
        r.require(base is None or base > 1, "the rotation's base must exceed 1")
        r.require(dims is None or (dims > 0 and dims % 2 == 0), "the rotated dims must be even and positive")
        r.finish()
        return RotaryConfig(base, dims, scaling)

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return out


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    v_mix: bool
    rot: RotaryConfig
    type: str = "attention"

    @staticmethod
    def read(data: dict, where: str) -> "AttentionConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        kv_heads, vdim = r.int("kv_heads", heads), r.int("vdim", dim)
        scale, v_mix = r.float("scale"), r.bool("v_mix", False)
        rot = r.object("rot")
        r.require(not heads or not kv_heads or (heads > 0 and kv_heads > 0 and heads % kv_heads == 0),
                  f"{heads} heads are not a multiple of {kv_heads} kv_heads")
        r.require((dim or 1) > 0 and (vdim or 1) > 0, "dim and vdim must be positive")
        r.finish()
        rc = RotaryConfig.read(rot, where + ".rot")
        if rc.dims > dim:
            raise ConfigError(f"{where}: {rc.dims} rotated dims do not fit a head of {dim}")
        return AttentionConfig(heads, kv_heads, dim, vdim, scale, v_mix, rc)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "scale": self.scale, "v_mix": self.v_mix, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int           # unrotated query/key dims a head
    rot_dim: int       # rotated dims a head (the key's are shared by all heads)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: RotaryConfig
    type: str = "latent_attention"

    @staticmethod
    def read(data: dict, where: str) -> "LatentAttentionConfig":
        r = KeyReader(data, where)
        heads, dim, rot_dim = r.int("heads"), r.int("dim"), r.int("rot_dim")
        vdim, q_rank, kv_rank = r.int("vdim", dim), r.int("q_rank"), r.int("kv_rank")
        scale = r.float("scale")
        rot = r.object("rot")
        for name, v in (("heads", heads), ("dim", dim), ("rot_dim", rot_dim), ("vdim", vdim), ("q_rank", q_rank),
                        ("kv_rank", kv_rank)):
            r.require(v is None or v > 0, f"{name} must be positive")
        r.finish()
        rc = RotaryConfig.read(rot, where + ".rot", dims_default=rot_dim)
        if rc.dims != rot_dim:
            raise ConfigError(f"{where}: the rotation covers {rc.dims} dims, the rotated part has {rot_dim}")
        return LatentAttentionConfig(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rc)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}


MIXERS = {"attention": AttentionConfig, "latent_attention": LatentAttentionConfig}


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class LayerConfig:
    mixer: object                   # one of MIXERS' classes
    mlp: Optional[DenseConfig]


@dataclass(frozen=True)
class VofezenConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    layers: tuple                   # of LayerConfig
    max_positions: int
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None

    # the design names no longest context; the engine's tables are made for what a caller asks
    # for (its num_ctx or a trace's max_tokens), up to this
    DEFAULT_MAX_POSITIONS = 1 << 20

    @staticmethod
    def from_dict(data: dict, where: str = "config.json") -> "VofezenConfig":
        r = KeyReader(data, where)
        arch = r.str("architecture", "Vofezen")
        vocab, width = r.int("vocab"), r.int("width")
        norm = r.object("norm")
        layers = data.get("layers")
        r.require(isinstance(layers, list) and len(layers) > 0, "key 'layers' must be a non-empty list")
        r.require((vocab or 1) > 0 and (width or 1) > 0, "vocab and width must be positive")
        max_positions = r.int("max_positions", VofezenConfig.DEFAULT_MAX_POSITIONS)
        eos = r.int_or_list("eos_token_id", None)
        bos = r.int("bos_token_id", None)
        r.finish()
        rn = KeyReader(norm, where + ".norm")
        eps = rn.float("eps")
        rn.require(eps is None or eps >= 0, "eps must not be negative")
        rn.finish()
        out = []
        for i, layer in enumerate(layers):
            at = f"{where}.layers[{i}]"
            rl = KeyReader(layer, at)
            kind = rl.str("type")
            mixer = rl.object("mixer")
            mlp = rl.object("mlp", None)
            rl.require(kind is None or kind in MIXERS, f"unknown mixer type {kind!r} (known: {', '.join(sorted(MIXERS))})")
            rl.finish()
            m = MIXERS[kind].read(mixer, at + ".mixer")
            ff = None
            if mlp is not None:
                rm = KeyReader(mlp, at + ".mlp")
                mk, f = rm.str("kind", "dense"), rm.int("ff")
                rm.require(mk == "dense", f"unknown feed-forward kind {mk!r} (known: dense)")
                rm.require(f is None or f > 0, "ff must be positive")
                rm.finish()
                ff = DenseConfig(f, mk)
            out.append(LayerConfig(m, ff))
        blending = [l.mixer for l in out if isinstance(l.mixer, AttentionConfig) and l.mixer.v_mix]
        if any((b.kv_heads, b.vdim) != (blending[0].kv_heads, blending[0].vdim) for b in blending):
            raise ConfigError(f"{where}: layers that blend their values must agree on kv_heads and vdim")
        return VofezenConfig(arch, vocab, width, eps, tuple(out), max_positions, tuple(eos), bos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps},
               "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(),
                           "mlp": None if l.mlp is None else {"kind": l.mlp.kind, "ff": l.mlp.ff}}
                          for l in self.layers]}
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out
