"""Typed configuration of the Safurax decoder, read from config.json.

A pre-norm decoder: x <- x + mixer(ln(x)), x <- x + ff(ln(x)), the norms being layer norms with a weight and no
bias; the embedding is scaled.  Three mixers, chosen per layer by ``type``:

* ``latent_attention``: attention over one cached latent per token, the queries through a normed latent of their
  own, no positions, all earlier keys.
* ``latent_attention_2``: the same with direct queries whose last ``rot_dim`` numbers are rotated (half-split pairs)
  and meet one rotated key part that all heads share, a sliding window, a learned sink per head in the softmax's
  denominator and a sigmoid gate per head; with ``kv_from: j`` the layer has no latent of its own and reads layer
  j's cache.
* ``attention``: differential attention over grouped heads, q and k normed per head and map, rotated with linearly
  scaled positions, a sigmoid gate per head.

The feed-forward is a dense gated one or a mixture of gated experts whose router picks the largest biased logits
and weighs them by the softmax over those alone, with a shared expert behind a sigmoid gate of one number a token.

Keys: architecture, vocab, width, embedding.scale, norm.eps, layers[i].type, layers[i].mixer {heads, dim, vdim,
scale, and by type: kv_rank, q_rank | kv_rank, rot_dim, rot {base, dims}, mask {size}, kv_from | kv_heads, diff,
rot {base, dims, scaling {factor}}}, layers[i].mlp (null | {kind: dense, ff} | {kind: moe, expert {ff},
router {experts, top}, shared {ff}}).  No size has a default.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional

from .qwen3 import ConfigError
from .spec import (BareLayerNormSpec, DiffAttentionSpec, LatentAttentionSpec, LayerSpec, ModelSpec, RopeHalfAnglesSpec,
                   ScheduleEntry, StreamScaleSpec, SwiGLUSpec, TopSoftmaxMoESpec)

ARCHITECTURE = "Safurax"
MIXER_TYPES = ("latent_attention", "latent_attention_2", "attention")
MAX_POSITIONS = 1 << 20      # the design names no limit; positions stay exact in 32-bit floats far beyond this
PART_NAMES = ("norm1", "mix", "norm2", "mlp")


def _get(d: Dict[str, Any], path: str, where: str):
    cur: Any = d
    for key in path.split("."):
        if not isinstance(cur, dict) or key not in cur:
            raise ConfigError(f"config.json lacks {where}{path}")
        cur = cur[key]
    return cur


class SafuraxConfig:
    architecture = ARCHITECTURE

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_get(d, "vocab", ""))
        self.width = int(_get(d, "width", ""))
        self.embedding_scale = float(_get(d, "embedding.scale", ""))
        self.eps = float(_get(d, "norm.eps", ""))
        self.layers: List[Dict[str, Any]] = list(_get(d, "layers", ""))
        self.max_positions = int(d.get("max_positions", MAX_POSITIONS))
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "SafuraxConfig":
        return cls(d)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not self.layers:
            raise ConfigError("the model has no layers")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            if layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"{where}type is {layer.get('type')!r}; known: {list(MIXER_TYPES)}")
            self._source(i)
        for i, layer in enumerate(self.layers):
            self._mixer(i)
            self._ffn(layer, f"layers[{i}].")

    # ---- a layer that reads another layer's cache -------------------------------------------------------------
    def _source(self, i: int) -> Optional[int]:
        """The layer whose latent layer i reads, None if it keeps its own."""
        layer = self.layers[i]
        m = _get(layer, "mixer", f"layers[{i}].")
        src = m.get("kv_from")
        if src is None:
            return None
        where = f"layers[{i}].mixer."
        if layer["type"] != "latent_attention_2":
            raise ConfigError(f"{where}kv_from goes with latent_attention_2 layers")
        if not (isinstance(src, int) and not isinstance(src, bool) and 0 <= src < i):
            raise ConfigError(f"{where}kv_from names layer {src!r}, which does not run before layer {i}")
        other = self.layers[src]
        om = other.get("mixer") or {}
        if other.get("type") != layer["type"] or om.get("kv_from") is not None:
            raise ConfigError(f"{where}kv_from names layer {src}, which keeps no latent of this kind of its own")
        for key in ("kv_rank", "rot_dim"):
            if int(_get(om, key, f"layers[{src}].mixer.")) != int(_get(m, key, where)):
                raise ConfigError(f"{where}{key} differs from that of layer {src}, whose cache the layer reads")
        if (om.get("rot") or {}) != (m.get("rot") or {}):
            raise ConfigError(f"{where}rot differs from that of layer {src}, whose cache the layer reads")
        return int(src)

    @staticmethod
    def _window(m: Dict[str, Any], where: str) -> Optional[int]:
        if m.get("mask") is None:
            return None
        size = int(_get(m, "mask.size", where))
        if size <= 0:
            raise ConfigError(f"{where}mask.size must be positive")
        return size

    def _kept(self, i: int) -> Optional[int]:
        """How many keys layer i's cache keeps: the widest window of the layer and of the layers that read its cache
        (None: all keys)."""
        widths = [self._window(self.layers[i]["mixer"], f"layers[{i}].mixer.")]
        for j in range(i + 1, len(self.layers)):
            if (self.layers[j].get("mixer") or {}).get("kv_from") == i:
                widths.append(self._window(self.layers[j]["mixer"], f"layers[{j}].mixer."))
        return None if any(w is None for w in widths) else max(widths)

    # ---- one layer's parts --------------------------------------------------------------------------------------
    def _rot(self, m: Dict[str, Any], where: str, most: int) -> Optional[RopeHalfAnglesSpec]:
        rot = m.get("rot")
        if rot is None:
            return None
        dims = int(_get(rot, "dims", where + "rot."))
        if dims == 0:
            return None
        if dims % 2 or not 0 < dims <= most:
            raise ConfigError(f"{where}rot.dims = {dims} must be even and at most {most}")
        factor = 1.0
        if rot.get("scaling") is not None:
            factor = float(_get(rot, "scaling.factor", where + "rot."))
            if not factor > 0:
                raise ConfigError(f"{where}rot.scaling.factor must be positive")
        return RopeHalfAnglesSpec(theta=float(_get(rot, "base", where + "rot.")), rotary_dim=dims, scaling_factor=factor)

    def _mixer(self, i: int):
        layer = self.layers[i]
        w = f"layers[{i}].mixer."
        m = _get(layer, "mixer", f"layers[{i}].")
        kind = layer["type"]
        heads, dim, vdim = int(_get(m, "heads", w)), int(_get(m, "dim", w)), int(_get(m, "vdim", w))
        scale = float(_get(m, "scale", w))
        if heads <= 0 or vdim <= 0 or dim < 0:
            raise ConfigError(f"{w}heads and vdim must be positive")
        if kind == "attention":
            kv_heads = int(_get(m, "kv_heads", w))
            if kv_heads <= 0 or heads % kv_heads or dim <= 0:
                raise ConfigError(f"{w}{heads} heads are no multiple of {kv_heads} key/value heads")
            return DiffAttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=dim, v_head_dim=vdim, scale=scale,
                                     diff=float(_get(m, "diff", w)), norm_eps=self.eps, qk_norm_eps=self.eps,
                                     output_gate=True, position=self._rot(m, w, dim))
        rank = int(_get(m, "kv_rank", w))
        if rank <= 0:
            raise ConfigError(f"{w}kv_rank must be positive")
        if kind == "latent_attention":
            if dim <= 0:
                raise ConfigError(f"{w}dim must be positive")
            return LatentAttentionSpec(num_heads=heads, head_dim=dim, rot_dim=0, v_head_dim=vdim, kv_rank=rank, scale=scale,
                                       norm_eps=self.eps, q_rank=int(_get(m, "q_rank", w)))
        rot_dim = int(_get(m, "rot_dim", w))
        if rot_dim < 0 or dim + rot_dim <= 0:
            raise ConfigError(f"{w}dim and rot_dim leave no query")
        position = self._rot(m, w, rot_dim) if rot_dim else None
        src = self._source(i)
        window = self._window(m, w)
        kept = self._kept(i) if src is None else window
        return LatentAttentionSpec(num_heads=heads, head_dim=dim, rot_dim=rot_dim, v_head_dim=vdim, kv_rank=rank,
                                   scale=scale, norm_eps=self.eps, q_rank=None, output_gate=True, gate_per_head=True,
                                   position=position, window=window, keep_window=kept if kept != window else None,
                                   sink=True, own_latent=src is None)

    def _ffn(self, layer: Dict[str, Any], where: str):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        w = where + "mlp."
        kind = _get(mlp, "kind", w)
        if kind == "dense":
            ff = int(_get(mlp, "ff", w))
            if ff <= 0:
                raise ConfigError(f"{w}ff must be positive")
            return SwiGLUSpec(intermediate_size=ff, names=("gate", "up", "down"))
        if kind == "moe":
            experts, top = int(_get(mlp, "router.experts", w)), int(_get(mlp, "router.top", w))
            ff = int(_get(mlp, "expert.ff", w))
            if not 1 <= top <= experts or ff <= 0:
                raise ConfigError(f"{w}router: top {top} of {experts} experts of width {ff}")
            shared = mlp.get("shared")
            shared_ff = int(_get(shared, "ff", w + "shared.")) if shared is not None else None
            if shared_ff is not None and shared_ff <= 0:
                raise ConfigError(f"{w}shared.ff must be positive")
            return TopSoftmaxMoESpec(num_experts=experts, top=top, intermediate_size=ff, router_bias=True,
                                     shared_intermediate_size=shared_ff, shared_gate=shared_ff is not None)
        raise ConfigError(f"{w}kind is {kind!r}; known: dense, moe")

    # ---- the model this configuration describes -------------------------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        norm = BareLayerNormSpec(eps=self.eps)
        layers, schedule = [], []
        for i, layer in enumerate(self.layers):
            ffn = self._ffn(layer, f"layers[{i}].")
            layers.append(LayerSpec(prefix=f"l{i}", mixer_norm=norm, mixer=self._mixer(i),
                                    ffn_norm=norm if ffn is not None else None, ffn=ffn, part_names=PART_NAMES))
            schedule.append(ScheduleEntry(layer=i, cache_from=self._source(i)))
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden_size=self.width,
            layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
            embed_name="embed", final_norm_name="final.norm", head_name="head", tie_head=False,
            max_positions=self.max_positions,
            stream_prologue=StreamScaleSpec(scale=self.embedding_scale) if self.embedding_scale != 1.0 else None)
        spec.validate()
        return spec
