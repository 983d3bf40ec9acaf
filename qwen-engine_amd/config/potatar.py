"""Typed configuration of the Potatar decoder, read from config.json.

A decoder whose layers norm after the sum: x <- n1(alpha x + mixer(x)), x <- n2(alpha x + ff(x)), with RMS norms
that carry a weight per coordinate.  A layer's mixer is one of
  attention   grouped-query attention inside chunks of positions, biased projections, q and k normed over the whole
              projection, a half-split rotation of the first numbers of every q and k head, value heads divided by
              their root mean square and, where a layer says so, blended with the values of the first such layer;
  wkv         a recurrence per head with a decay per key channel, fed by blends of a token with the token before it;
  parallel    two mixers side by side, added with weights: attention inside chunks whose values are the projected
              keys, with q and k normed per head, a learned bias by distance and scores mixed across heads; and
              linear attention with one decay per head.
The feed-forward is down(gelu(up x)) or absent.  The last norm, the head and a soft cap give the logits.

Keys: architecture, vocab, width, norm.eps, postln_alpha, logit_softcap, layers[i].type, layers[i].mlp
(null | {kind: dense, ff}), layers[i].mixer:
  attention   {heads, kv_heads, dim, vdim, scale, mask {size}, rot {base, dims}, v_mix}
  wkv         {heads, dim} (+ decay_rank, else the rows of the layer's tensor mix.w1)
  parallel    {left {heads, kv_heads, dim, vdim, scale, mask {size}, bias_max} (+ bias_rows, else the rows of
              mix.left.rel), right {heads, dim, vdim, decay [heads]}, left_scale, right_scale}
The two sizes that only a tensor's shape gives are taken from the model folder's tensor shapes when config.json
does not name them, and are written into the dictionary that ``to_dict`` returns.
"""
from __future__ import annotations

import copy
from typing import Any, Callable, Dict, List, Optional, Tuple

from .qwen3 import ConfigError
from .spec import (BareRMSNormSpec, ChunkAttentionSpec, DecayedLinearSpec, GeluMLPSpec, LogitSoftcapSpec, ModelSpec,
                   PostNormLayerSpec, RopeHalfAnglesSpec, ScheduleEntry, ShiftedDecaySpec, SideBySideMixerSpec)

ARCHITECTURE = "Potatar"
MAX_POSITIONS = 1 << 20      # the design names no limit; positions stay exact in 32-bit floats far beyond this
MIXERS = ("attention", "wkv", "parallel")


def _get(d: Dict[str, Any], path: str, where: str):
    cur: Any = d
    for key in path.split("."):
        if not isinstance(cur, dict) or key not in cur:
            raise ConfigError(f"config.json lacks {where}{path}")
        cur = cur[key]
    return cur


class PotatarConfig:
    architecture = ARCHITECTURE

    def __init__(self, d: Dict[str, Any], shapes: Optional[Dict[str, Tuple[int, ...]]] = None):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_get(d, "vocab", ""))
        self.width = int(_get(d, "width", ""))
        self.eps = float(_get(d, "norm.eps", ""))
        self.alpha = float(_get(d, "postln_alpha", ""))
        cap = d.get("logit_softcap")
        self.softcap = float(cap) if cap else 0.0
        _get(d, "layers", "")
        self.layers: List[Dict[str, Any]] = self.raw["layers"]      # (sizes found in tensor shapes are written here)
        self.max_positions = int(d.get("max_positions", MAX_POSITIONS))
        self._sizes_from_shapes(shapes or {})
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any], shapes: Optional[Dict[str, Tuple[int, ...]]] = None) -> "PotatarConfig":
        return cls(d, shapes)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)

    def _sizes_from_shapes(self, shapes) -> None:
        """The sizes that config.json may leave to the tensors' shapes."""
        for i, layer in enumerate(self.layers):
            m = layer.get("mixer")
            if not isinstance(m, dict):
                continue
            if layer.get("type") == "wkv" and "decay_rank" not in m and f"l{i}.mix.w1" in shapes:
                m["decay_rank"] = int(shapes[f"l{i}.mix.w1"][0])
            left = m.get("left") if layer.get("type") == "parallel" else None
            if isinstance(left, dict) and "bias_rows" not in left and f"l{i}.mix.left.rel" in shapes:
                left["bias_rows"] = int(shapes[f"l{i}.mix.left.rel"][0])

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.softcap < 0:
            raise ConfigError("logit_softcap must be positive (or absent)")
        if not self.layers:
            raise ConfigError("the model has no layers")
        blended = None
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            kind = layer.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}type is {kind!r}; known: {', '.join(MIXERS)}")
            spec = self._mixer(layer, where, first_blend=True)
            if kind == "attention" and spec.value_blend is not None:
                size = spec.num_kv_heads * spec.v_head_dim
                if blended is not None and blended != size:
                    raise ConfigError(f"{where}mixer: values of {size} numbers cannot be blended with the first "
                                      f"blending layer's {blended}")
                blended = size
            self._ffn(layer, where)

    # ---- one layer's parts ---------------------------------------------------------------------------------
    @staticmethod
    def _heads(m, w, kv: bool = True):
        heads = int(_get(m, "heads", w))
        kv_heads = int(_get(m, "kv_heads", w)) if kv else heads
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise ConfigError(f"{w}{heads} heads over {kv_heads} key/value heads")
        return heads, kv_heads

    @staticmethod
    def _chunk(m, w) -> Optional[int]:
        mask = m.get("mask")
        if not mask or mask.get("size") is None:
            return None
        size = int(mask["size"])
        if size <= 0:
            raise ConfigError(f"{w}mask.size = {size}")
        return size

    def _attention(self, m, w, first_blend: bool) -> ChunkAttentionSpec:
        heads, kv_heads = self._heads(m, w)
        dim, vdim = int(_get(m, "dim", w)), int(_get(m, "vdim", w))
        if dim <= 0 or vdim <= 0:
            raise ConfigError(f"{w}dim and vdim must be positive")
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", 0) or 0)
        if dims % 2 or not 0 <= dims <= dim:
            raise ConfigError(f"{w}rot.dims = {dims} must be even and at most dim = {dim}")
        blend = None
        if m.get("v_mix"):
            blend = "source" if first_blend else "blend"
        return ChunkAttentionSpec(
            num_heads=heads, num_kv_heads=kv_heads, head_dim=dim, v_head_dim=vdim, scale=float(_get(m, "scale", w)),
            chunk=self._chunk(m, w), bias=True, qk_norm="whole", qk_norm_eps=self.eps, value_norm_eps=self.eps,
            value_blend=blend,
            position=RopeHalfAnglesSpec(theta=float(_get(rot, "base", w + "rot.")), rotary_dim=dims) if dims else None)

    def _left(self, m, w) -> ChunkAttentionSpec:
        heads, kv_heads = self._heads(m, w)
        dim = int(_get(m, "dim", w))
        if int(m.get("vdim", dim)) != dim:
            raise ConfigError(f"{w}vdim = {m.get('vdim')}: the values are the keys, of dim = {dim} numbers")
        rows = m.get("bias_rows")
        if rows is None:
            raise ConfigError(f"config.json lacks {w}bias_rows, and no tensor's shape was at hand to give it")
        rows, far = int(rows), float(_get(m, "bias_max", w))
        if rows < 2 or not far > rows // 2:
            raise ConfigError(f"{w}a distance bias of {rows} rows up to a distance of {far}")
        return ChunkAttentionSpec(
            num_heads=heads, num_kv_heads=kv_heads, head_dim=dim, v_head_dim=dim, scale=float(_get(m, "scale", w)),
            chunk=self._chunk(m, w), bias=True, qk_norm="head", qk_norm_eps=self.eps, values_from_keys=True,
            distance_bias_rows=rows, distance_bias_far=far, talking_heads=True)

    def _right(self, m, w) -> DecayedLinearSpec:
        heads, _ = self._heads(m, w, kv=False)
        decay = tuple(float(v) for v in _get(m, "decay", w))
        if len(decay) != heads:
            raise ConfigError(f"{w}decay has {len(decay)} entries for {heads} heads")
        dim, vdim = int(_get(m, "dim", w)), int(_get(m, "vdim", w))
        if dim <= 0 or vdim <= 0:
            raise ConfigError(f"{w}dim and vdim must be positive")
        return DecayedLinearSpec(num_heads=heads, head_dim=dim, v_head_dim=vdim, decay=decay, norm_eps=self.eps)

    def _mixer(self, layer: Dict[str, Any], where: str, first_blend: bool):
        m = _get(layer, "mixer", where)
        w = where + "mixer."
        kind = layer["type"]
        if kind == "attention":
            return self._attention(m, w, first_blend)
        if kind == "wkv":
            heads, _ = self._heads(m, w, kv=False)
            rank = m.get("decay_rank")
            if rank is None:
                raise ConfigError(f"config.json lacks {w}decay_rank, and no tensor's shape was at hand to give it")
            dim = int(_get(m, "dim", w))
            if dim <= 0 or int(rank) <= 0:
                raise ConfigError(f"{w}dim and decay_rank must be positive")
            return ShiftedDecaySpec(num_heads=heads, head_dim=dim, decay_rank=int(rank), norm_eps=self.eps)
        return SideBySideMixerSpec(left=self._left(_get(m, "left", w), w + "left."),
                                   right=self._right(_get(m, "right", w), w + "right."),
                                   left_scale=float(_get(m, "left_scale", w)), right_scale=float(_get(m, "right_scale", w)))

    def _ffn(self, layer: Dict[str, Any], where: str):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        w = where + "mlp."
        kind = _get(mlp, "kind", w)
        if kind != "dense":
            raise ConfigError(f"{w}kind is {kind!r}; known: dense")
        ff = int(_get(mlp, "ff", w))
        if ff <= 0:
            raise ConfigError(f"{w}ff must be positive")
        return GeluMLPSpec(intermediate_size=ff)

    # ---- the model this configuration describes --------------------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        norm = BareRMSNormSpec(eps=self.eps)
        layers = []
        seen_blend = False
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            mixer = self._mixer(layer, where, first_blend=not seen_blend)
            if layer["type"] == "attention" and mixer.value_blend is not None:
                seen_blend = True
            ffn = self._ffn(layer, where)
            layers.append(PostNormLayerSpec(prefix=f"l{i}", mixer=mixer, mixer_norm=norm, ffn=ffn,
                                            ffn_norm=norm if ffn is not None else None, alpha=self.alpha))
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden_size=self.width,
            layers=tuple(layers), schedule=tuple(ScheduleEntry(layer=i) for i in range(len(layers))),
            final_norm=norm, embed_name="embed", final_norm_name="final.norm", head_name="head", tie_head=False,
            max_positions=self.max_positions,
            logit_epilogue=LogitSoftcapSpec(cap=self.softcap) if self.softcap else None)
        spec.validate()
        return spec
