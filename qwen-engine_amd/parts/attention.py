"""Grouped-query attention over the paged cache.

Order of operations as in src/models/qwen3/model.py:200-213: q, k, v projections
(here one product with the three weights stacked), per-head q/k RMSNorm when the
spec asks for it, position encoding of q and k, write of k and v into the cache,
attention of the new tokens over the cache, output projection without bias.
Scores, mask and softmax follow src/layers/fused_ops/attn.py:236-267.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

from ..cache.plan import KVNeed
from ..kernels import ops
from .base import CacheBinding, Runtime, StreamInput, TensorInfo
from .registry import build_part, register_part


# Up to this many single new tokens in a step, the decode attention kernel norms, rotates and
# writes the cache itself; above, the separate kernel is quicker (every wave of the attention
# kernel repeats the preparation of q, which then outweighs the kernel saved).
FUSED_DECODE_MAX_TOKENS = 16


def prefill_tiles(portions, rows_per_tile: int) -> List[int]:
    """(first row, rows) pairs, flat, for portions given as (first row, number of rows): tiles of
    at most rows_per_tile rows, in groups of four per portion, padded with (first row, 0): what the
    prefill attention kernel takes."""
    flat: List[int] = []
    for start, n in portions:
        tiles = [(start + r, min(rows_per_tile, n - r)) for r in range(0, n, rows_per_tile)]
        while len(tiles) % 4:
            tiles.append((start, 0))
        for t in tiles:
            flat.extend(t)
    return flat


class PagedAttention:
    takes_stream = True       # forward may get a StreamInput: residual sum and norm are then the q|k|v product's prologue

    # ---- what the step function prepares for this part (parts.base) --------------------------
    @staticmethod
    def step_extras(seqs) -> dict:
        """The rows that are the single new token of their request (they go to the decode kernel, the
        largest of their positions fixing its number of key splits) and all other rows."""
        dec = [s.q_start for s in seqs if s.q_len == 1]
        other = [np.arange(s.q_start, s.q_start + s.q_len, dtype=np.int32) for s in seqs if s.q_len > 1]
        return {"dec_tokens": np.asarray(dec, dtype=np.int32),
                "other_tokens": np.concatenate(other) if other else np.zeros(0, dtype=np.int32),
                "max_dec_position": max([s.kv_before for s in seqs if s.q_len == 1], default=0),
                "max_other_keys": max([s.kv_before + s.q_len for s in seqs if s.q_len > 1], default=0)}

    GRAPH_SPLIT_BUCKET = 8      # a recorded decode step serves positions up to the next multiple of this many key splits

    @classmethod
    def graph_key(cls, max_position: int) -> int:
        """The decode kernel's grid and workspace follow the number of key splits: recorded steps are
        kept per bucket of splits."""
        splits = int(max_position) // ops.DECODE_SPLIT_KEYS + 1
        b = cls.GRAPH_SPLIT_BUCKET
        return (splits + b - 1) // b * b

    @staticmethod
    def graph_extras(rows: int, key: int, device) -> dict:
        return {"dec_tokens": torch.arange(rows, dtype=torch.int32, device=device), "other_tokens": None,
                "max_dec_position": key * ops.DECODE_SPLIT_KEYS - 1}

    @staticmethod
    def portion_graph_key(tokens: int, keys: int) -> bool:
        """Beyond a number of keys the prefill kernel cuts long walks into segments and a second kernel
        merges them; how long a segment is the kernels take from the last row's position themselves."""
        return keys > ops.prefill_uncut_keys()

    @staticmethod
    def portion_graph_extras(tokens: int, device, key: bool = False) -> dict:
        """For a recorded step that is one prompt portion of ``tokens`` rows: no single new tokens, all
        rows in order; the last row sees the most keys."""
        return {"dec_tokens": torch.zeros(0, dtype=torch.int32, device=device),
                "other_tokens": torch.arange(tokens, dtype=torch.int32, device=device), "max_dec_position": 0,
                "max_other_keys": 0, "other_keys_row": tokens - 1 if key else None}

    # A recorded step of single new tokens beside one prompt portion (parts.base): the rows of the
    # single tokens come first, then rows that fill the portion up to a round length (a portion of the
    # tables' spare row that writes nowhere), then the portion, whose last row is the step's last.
    mixed_graph_dynamic_size = 4

    @classmethod
    def mixed_graph_key(cls, max_dec_position: int, portion_keys: int):
        return cls.graph_key(max_dec_position), portion_keys > ops.prefill_uncut_keys()

    @staticmethod
    def mixed_graph_dynamic(rows: int, pad: int, tokens: int) -> List[int]:
        """What changes from replay to replay: the two portions (first row, rows) that the prefill
        kernel's tiles are cut from, on the device."""
        return [rows, pad, rows + pad, tokens - pad]

    @staticmethod
    def mixed_graph_extras(rows: int, tokens: int, key, device, dynamic: torch.Tensor) -> dict:
        splits, cut = key
        return {"dec_tokens": torch.arange(rows, dtype=torch.int32, device=device),
                "other_tokens": torch.arange(rows, rows + tokens, dtype=torch.int32, device=device),
                "max_dec_position": splits * ops.DECODE_SPLIT_KEYS - 1, "max_other_keys": 0,
                "other_keys_row": rows + tokens - 1 if cut else None,
                "portions": dynamic.view(2, 2), "portion_rows": int(tokens)}

    def _extras(self, ctx) -> dict:
        """What the step function prepared for this part's class (a class derived from this one finds
        its own entry: the step function files them under the class of the part it met)."""
        for cls in type(self).__mro__:
            if cls in ctx.extras:
                return ctx.extras[cls]
        return {"dec_tokens": None, "other_tokens": None, "max_dec_position": 0, "max_other_keys": 0}

    def _other_tiles(self, ctx) -> Optional[torch.Tensor]:
        """The rows of requests that bring several tokens, cut into tiles for the prefill kernel: built
        and sent to the device once per step and tile size, shared by the layers."""
        rows_per_tile = ops.prefill_tile_rows(self.hq, self.hkv)
        if rows_per_tile <= 0:
            return None
        key = ("paged_attention.tiles", rows_per_tile)
        ex = self._extras(ctx)
        if key not in ctx.memo and ex.get("portions") is not None:
            # a recorded step: the portions' lengths are known on the device only
            portions = ex["portions"]
            groups = -(-ex["portion_rows"] // (4 * rows_per_tile)) + portions.shape[0]
            ctx.memo[key] = ops.prefill_tiles_on_device(portions, rows_per_tile, groups)
        if key not in ctx.memo:
            flat = prefill_tiles([(s.q_start, s.q_len) for s in ctx.seqs if s.q_len > 1], rows_per_tile)
            ctx.memo[key] = torch.tensor(flat, dtype=torch.int32).view(-1, 2).to(ctx.rt.device) if flat else None
        return ctx.memo[key]

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.hq, self.hkv, self.d = int(spec.num_heads), int(spec.num_kv_heads), int(spec.head_dim)
        if self.hq % self.hkv:
            raise ValueError(f"{self.hq} query heads are no multiple of {self.hkv} key/value heads")
        self.scale = float(spec.scale)
        self.window = int(spec.window) if spec.window else 0
        self.qk_eps = spec.qk_norm_eps
        self.position = build_part(spec.position, hidden_size) if spec.position is not None else None
        self.w_qkv = self.b_qkv = self.w_o = self.q_norm = self.k_norm = None

    @property
    def graph_safe(self) -> bool:
        return getattr(self.position, "graph_safe", True)

    # ---- what it needs ----------------------------------------------------------
    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        hq, hkv, d = spec.num_heads, spec.num_kv_heads, spec.head_dim
        t = {
            "q_proj.weight": TensorInfo((hq * d, hidden)),
            "k_proj.weight": TensorInfo((hkv * d, hidden)),
            "v_proj.weight": TensorInfo((hkv * d, hidden)),
            "o_proj.weight": TensorInfo((hidden, hq * d)),
        }
        if spec.qkv_bias:
            t["q_proj.bias"] = TensorInfo((hq * d,), "zeros", "vector")
            t["k_proj.bias"] = TensorInfo((hkv * d,), "zeros", "vector")
            t["v_proj.bias"] = TensorInfo((hkv * d,), "zeros", "vector")
        if spec.qk_norm_eps is not None:
            t["q_norm.weight"] = TensorInfo((d,), "ones", "vector")
            t["k_norm.weight"] = TensorInfo((d,), "ones", "vector")
        return t

    @staticmethod
    def cache_need(spec) -> Optional[KVNeed]:
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim, window=spec.window)

    @staticmethod
    def state_need(spec, hidden: int):
        return None

    # ---- weights ------------------------------------------------------------------
    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        mats = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_qkv = rt.place_matrix(torch.cat(mats, dim=0))
        self.w_o = rt.place_matrix(tensors["o_proj.weight"])
        if self.spec.qkv_bias:
            self.b_qkv = rt.place_vector(torch.cat(
                [tensors["q_proj.bias"].float(), tensors["k_proj.bias"].float(), tensors["v_proj.bias"].float()]))
        if self.qk_eps is not None:
            self.q_norm = rt.place_vector(tensors["q_norm.weight"])
            self.k_norm = rt.place_vector(tensors["k_norm.weight"])
        if self.position is not None:
            self.position.load({}, rt)

    # ---- one step -------------------------------------------------------------------
    def forward(self, x, ctx, binding: CacheBinding) -> torch.Tensor:
        """Returns the mixer's output [T, H], or float32 partial products [S, T, H] of it.
        x: the normed rows, or a StreamInput."""
        if binding.kv is None:
            raise RuntimeError("attention was given no cache")
        lazy = None
        if isinstance(x, StreamInput):
            if x.prefers_prologue(ops, self.w_qkv):
                lazy, x = x, x.stream.h
            else:
                x = x.materialize()
        T = x.shape[0]
        g = binding.group
        eps = self.qk_eps if self.qk_eps is not None else 0.0
        slots = ctx.slots[g] if binding.write else None
        cache = binding.kv
        pos = self.position
        fused_position = pos is None or getattr(pos, "fused", False)
        table = pos.table() if (pos is not None and fused_position) else None
        if table is not None and ctx.max_position >= table.shape[0]:
            raise RuntimeError(f"position {ctx.max_position} is beyond the rotation table "
                               f"({table.shape[0]} positions)")
        if lazy is None and fused_position and ops.gemm_qkv_supported(x, self.w_qkv, cache, self.hq, table):
            # many rows (portions of prompts): norm, rotation and cache write are the epilogue of the
            # q|k|v product, which never stores its result
            q = ops.gemm_qkv(x, self.w_qkv, self.b_qkv, self.hq, cache, ctx.positions if table is not None else None,
                             self.q_norm, self.k_norm, eps, table, slots)
            return self._attend(q, ctx, cache, g, T)
        if (lazy is None and fused_position and cache.dtype == torch.bfloat16 and ops.gemm_partial_preferred(x, self.w_qkv) and
                ops.qk_rope_store_parts_supported(self.d, table)):
            # 17 to 64 rows against a large matrix: the product is cut along K to fill the chip, and
            # the kernel that norms, rotates and writes the cache adds the parts up as it reads them
            parts = ops.gemm(x, self.w_qkv, epilogue=ops.EPI_PARTIAL)
            q = ops.qk_rope_store_parts(parts, self.b_qkv, self.hq, self.hkv, self.d,
                                        ctx.positions if table is not None else None, self.q_norm, self.k_norm,
                                        eps, table, slots, cache, ctx.page_size)
            return self._attend(q, ctx, cache, g, T)
        if lazy is not None:    # few rows: the norm before the part is the product's prologue
            qkv = lazy.gemm(ops, self.w_qkv, self.b_qkv)
        else:
            qkv = ops.gemm(x, self.w_qkv, self.b_qkv)
        if fused_position:
            ex = self._extras(ctx)
            only_new_tokens = (ex["dec_tokens"] is not None and ex["dec_tokens"].shape[0] == T and
                               (ex["other_tokens"] is None or ex["other_tokens"].shape[0] == 0))
            if (only_new_tokens and T <= FUSED_DECODE_MAX_TOKENS and binding.write and
                    ops.attention_decode_fused_supported(qkv, cache, self.hq, table)):
                # every row is the one new token of its request: norm, rotation and cache write
                # happen inside the attention kernel
                o = ops.attention_decode_fused(qkv, self.hq, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g],
                                               self.scale, self.window, None, ex["max_dec_position"],
                                               self.q_norm, self.k_norm, eps, table, slots,
                                               shared_keys=ctx.shared_keys)
                return self._project_out(o.view(T, self.hq * self.d))
            q = ops.qk_rope_store(qkv, self.hq, self.hkv, self.d, ctx.positions, self.q_norm, self.k_norm,
                                  eps, table, slots, cache, ctx.page_size)
        else:
            # another position encoding: norm into a packed q|k|v tensor, let the part
            # change it in place, then write the cache from it
            packed = ops.qk_rope_store(qkv, self.hq, self.hkv, self.d, None, self.q_norm, self.k_norm,
                                       eps, None, None, None, ctx.page_size, packed=True)
            pos.apply(packed, ctx.positions, self.hq, self.hkv)
            q = ops.qk_rope_store(packed.view(T, -1), self.hq, self.hkv, self.d, None, None, None, 0.0,
                                  None, slots, cache, ctx.page_size)
        return self._attend(q, ctx, cache, g, T)

    def _attend(self, q: torch.Tensor, ctx, cache: torch.Tensor, g: int, T: int) -> torch.Tensor:
        ex = self._extras(ctx)
        o = ops.attention(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, self.window,
                          dec_tokens=ex["dec_tokens"], max_dec_position=ex["max_dec_position"],
                          other_tokens=ex["other_tokens"],
                          other_tiles=self._other_tiles(ctx) if ex["other_tokens"] is not None else None,
                          max_other_keys=ex.get("max_other_keys", 0), other_keys_row=ex.get("other_keys_row"),
                          shared_keys=ctx.shared_keys)
        return self._project_out(o.view(T, self.hq * self.d))

    def _project_out(self, o: torch.Tensor) -> torch.Tensor:
        splits = ops.gemm_branch_splits(o, self.w_o)
        if splits:
            # the product is cut along K (few rows: to fill the chip; a narrow matrix: to give every
            # compute unit blocks to overlap); the norm that follows adds the parts
            return ops.gemm(o, self.w_o, epilogue=ops.EPI_PARTIAL, splits=splits)
        return ops.gemm(o, self.w_o)


def common_head_dim(k_dim: int, v_dim: int) -> int:
    """The one head size under which keys and values of different sizes share the paged cache and the attention
    kernels (zeros beyond a head's own numbers): 64 or 128, which the matrix-unit kernels take, else the next
    multiple of 16."""
    m = max(int(k_dim), int(v_dim))
    if m <= 64:
        return 64
    if m <= 128:
        return 128
    return (m + 15) // 16 * 16


class ConvAttention(PagedAttention):
    """Grouped-query attention with a short causal convolution over time on every channel of the projected q, k
    and v (``ConvAttentionSpec``): one product for q | k | v with the biases, then one kernel that convolves (a
    request's last ``conv_taps - 1`` projected rows are its state), rotates the first numbers of every q and k head
    and writes q and the cache, then the attention kernels of PagedAttention with the window's kept first keys and
    the sink, then the output projection.  Keys and values of different sizes share the cache under one head size
    (``common_head_dim``), and the output projection's columns beyond a value head's own numbers are zeros."""
    takes_stream = False

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.hq, self.hkv = int(spec.num_heads), int(spec.num_kv_heads)
        self.dk, self.dv = int(spec.head_dim), int(spec.v_head_dim)
        self.d = common_head_dim(self.dk, self.dv)
        if self.hq % self.hkv:
            raise ValueError(f"{self.hq} query heads are no multiple of {self.hkv} key/value heads")
        self.scale = float(spec.scale)
        self.window = int(spec.window) if spec.window else 0
        self.keep_first = int(spec.keep_first) if self.window else 0
        self.sink = bool(spec.sink)
        self.taps = int(spec.conv_taps)
        self.position = build_part(spec.position, hidden_size) if spec.position is not None else None
        self.w_qkv = self.b_qkv = self.w_o = self.conv_w = self.conv_w_t = None

    graph_safe = True        # every launch's grid follows the rows alone; the state is device memory

    @staticmethod
    def _channels(spec) -> int:
        return spec.num_heads * spec.head_dim + spec.num_kv_heads * (spec.head_dim + spec.v_head_dim)

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        nq, nk, nv, no = spec.names
        rows = {nq: spec.num_heads * spec.head_dim, nk: spec.num_kv_heads * spec.head_dim,
                nv: spec.num_kv_heads * spec.v_head_dim}
        t = {}
        for name, n in rows.items():
            t[name] = TensorInfo((n, hidden))
            if spec.qkv_bias:
                t[name + spec.bias_suffix] = TensorInfo((n,), "zeros", "vector")
            if spec.conv_taps >= 1:
                t[name + spec.conv_suffix] = TensorInfo((n, int(spec.conv_taps)), "normal", "vector")
        t[no] = TensorInfo((hidden, spec.num_heads * spec.v_head_dim))
        return t

    @staticmethod
    def cache_need(spec) -> Optional[KVNeed]:
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=common_head_dim(spec.head_dim, spec.v_head_dim),
                      window=spec.window, keep_first=int(spec.keep_first) if spec.window else 0)

    @staticmethod
    def state_need(spec, hidden: int):
        from ..cache.plan import StateNeed
        taps = int(spec.conv_taps)
        return StateNeed(shape=(taps - 1, ConvAttention._channels(spec)), dtype="float32") if taps > 1 else None

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        s = self.spec
        nq, nk, nv, no = s.names
        mats = [tensors[nq], tensors[nk], tensors[nv]]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_qkv = rt.place_matrix(torch.cat(mats, dim=0))
        if s.qkv_bias:
            self.b_qkv = rt.place_vector(torch.cat([tensors[n + s.bias_suffix].float() for n in (nq, nk, nv)]))
        if self.taps >= 1:
            self.conv_w = rt.place_vector(torch.cat([tensors[n + s.conv_suffix].float() for n in (nq, nk, nv)], dim=0))
        else:                                              # no convolution: one tap of weight 1
            self.conv_w = torch.ones((self._channels(s), 1), dtype=torch.float32, device=rt.device)
        self.conv_w_t = self.conv_w.t().contiguous()      # [taps, channels]: what the kernel for many rows reads
        # the output projection against heads of the common size: zero columns beyond a value head's own numbers
        w_o = tensors[no]
        padded = torch.zeros((self.hidden, self.hq, self.d), dtype=w_o.dtype)
        padded[:, :, :self.dv] = w_o.view(self.hidden, self.hq, self.dv)
        self.w_o = rt.place_matrix(padded.view(self.hidden, self.hq * self.d))
        if self.position is not None:
            self.position.load({}, rt)

    def output_parts(self, rows: int, dtype: torch.dtype) -> int:
        """Into how many 32-bit partial products the output projection of ``rows`` rows is cut (0: not at all):
        forward can leave them in a tensor it is given (``parts_out``)."""
        return ops.gemm_branch_splits_for(rows, self.w_o, dtype)

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding, parts_out: Optional[torch.Tensor] = None,
                add_to: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """x [T, H] in the activation type.  Returns the mixer's output [T, H], or float32 partial products
        [S, T, H] of it (in ``parts_out`` [S, T, H], S = output_parts(T, type), if given).  ``add_to``: the 32-bit
        stream [T, H]; where the output projection can add its result into it itself (its residual epilogue, and
        no cut along K wanted) it does, and None is returned: nothing is left to add."""
        if binding.kv is None:
            raise RuntimeError("attention was given no cache")
        if self.taps > 1 and binding.state is None:
            raise RuntimeError("the convolution was given no state")
        T, g, cache = x.shape[0], binding.group, binding.kv
        qkv = ops.gemm(x, self.w_qkv, self.b_qkv)
        # (a step in which every request brings one token: convolution and the state's shift in one launch)
        single = all(s.q_len == 1 for s in ctx.seqs) and len(ctx.seqs) == T
        q = ops.qkv_conv_rope_store(qkv, self.conv_w, binding.state, ctx.tok_seq, ctx.positions,
                                    self.position.inv_freq() if self.position is not None else None,
                                    ctx.slots[g] if binding.write else None, cache, self.hq, self.hkv, self.dk, self.dv,
                                    single_rows=single, conv_w_t=self.conv_w_t)
        ex = self._extras(ctx)
        o = ops.attention(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, self.window,
                          dec_tokens=ex["dec_tokens"], max_dec_position=ex["max_dec_position"],
                          other_tokens=ex["other_tokens"],
                          other_tiles=self._other_tiles(ctx) if ex["other_tokens"] is not None else None,
                          max_other_keys=ex.get("max_other_keys", 0), other_keys_row=ex.get("other_keys_row"),
                          shared_keys=ctx.shared_keys, keep_first=self.keep_first, sink=self.sink)
        o = o.view(T, self.hq * self.d)
        if parts_out is not None:
            return ops.gemm(o, self.w_o, epilogue=ops.EPI_PARTIAL, splits=parts_out.shape[0], out=parts_out)
        if add_to is not None and not ops.gemm_branch_splits(o, self.w_o) and ops.gemm_fused_supported(o, self.w_o):
            ops.gemm(o, self.w_o, epilogue=ops.EPI_RESIDUAL, out=add_to)
            return None
        return self._project_out(o)


def distance_bias_rows(table: torch.Tensor, far: float, max_distance: Optional[int] = None) -> torch.Tensor:
    """A learned bias by distance as one row per distance: ``table`` [B, heads] holds a row each for the distances
    below B // 2 and logarithmic steps up to ``far`` for the rest; distance n reads row n for n < B // 2, else
    min(B - 1, B // 2 + floor(log(n / (B // 2)) / log(far / (B // 2)) * (B - B // 2))).  Returns float32
    [ceil(far) + 1, heads]: row n for distance n, the last row for every distance beyond (it is the table's last).
    With ``max_distance`` (the largest distance a query ever has to a key it sees, a chunk's length less one) the
    rows end there.  The rows are looked up in 64-bit on the host, once."""
    import math
    B = table.shape[0]
    half = B // 2
    if half < 1 or not far > half:
        raise ValueError(f"a distance bias of {B} rows up to {far}")
    rows = []
    count = int(math.ceil(far)) + 1
    if max_distance is not None and max_distance + 1 < count:
        count = int(max_distance) + 1
        far_row = None
    else:
        far_row = B - 1
    for n in range(count):
        if n < half:
            rows.append(n)
        else:
            rows.append(min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half)))))
    if far_row is not None:
        rows[-1] = far_row
    return table.float()[torch.tensor(rows)].contiguous()


class ChunkAttention(PagedAttention):
    """Grouped-query attention inside chunks of positions (``ChunkAttentionSpec``): one product for q | k (| v) with
    the biases; one kernel that norms q and k (per head or over the whole projection), takes the values from their
    projection or from the keys, norms and blends them, rotates q and k and writes q and the cache; then either the
    attention kernels of PagedAttention with the chunk as their mask (keys and values of different sizes share the
    cache under one head size, ``common_head_dim``), or, with a bias by distance or talking heads, the kernel
    that handles all heads of a token together; then the output projection, whose result stays 32-bit.
    The values that a layer leaves for later layers of the step travel in ``ctx.memo``."""
    takes_stream = False
    graph_safe = True        # every launch's grid follows the rows alone

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.hq, self.hkv = int(spec.num_heads), int(spec.num_kv_heads)
        self.dk, self.dv = int(spec.head_dim), int(spec.v_head_dim)
        if self.hq % self.hkv:
            raise ValueError(f"{self.hq} query heads are no multiple of {self.hkv} key/value heads")
        if spec.values_from_keys and self.dk != self.dv:
            raise ValueError("values that are the keys have the keys' size")
        if spec.qk_norm not in (None, "head", "whole"):
            raise ValueError(f"unknown q/k norm {spec.qk_norm!r}")
        if spec.value_blend not in (None, "source", "blend"):
            raise ValueError(f"unknown value blend {spec.value_blend!r}")
        self.talks = self._talks(spec)
        self.d = self._cache_head_dim(spec)
        self.scale = float(spec.scale)
        self.chunk = int(spec.chunk) if spec.chunk else 0
        self.window = 0
        self.position = build_part(spec.position, hidden_size) if spec.position is not None else None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.q_norm = self.k_norm = None
        self.blend = self.dist_bias = self.talk = None

    @staticmethod
    def _talks(spec) -> bool:
        return bool(spec.distance_bias_rows) or bool(spec.talking_heads)

    @staticmethod
    def _cache_head_dim(spec) -> int:
        if ChunkAttention._talks(spec):
            return (max(int(spec.head_dim), int(spec.v_head_dim)) + 3) // 4 * 4
        return common_head_dim(spec.head_dim, spec.v_head_dim)

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        nq, nk, nv, no = spec.names
        rows = {nq: spec.num_heads * spec.head_dim, nk: spec.num_kv_heads * spec.head_dim}
        if not spec.values_from_keys:
            rows[nv] = spec.num_kv_heads * spec.v_head_dim
        t = {}
        for name, n in rows.items():
            t[name] = TensorInfo((n, hidden))
            if spec.bias:
                t[name + spec.bias_suffix] = TensorInfo((n,), "zeros", "vector")
        if spec.qk_norm is not None:
            for name in (nq, nk):
                t[name + spec.norm_suffix] = TensorInfo((rows[name] if spec.qk_norm == "whole" else spec.head_dim,),
                                                        "ones", "vector")
        if spec.value_blend is not None:
            t[spec.blend_name] = TensorInfo((), "zeros", "vector")
        if spec.distance_bias_rows:
            t[spec.distance_bias_name] = TensorInfo((int(spec.distance_bias_rows), spec.num_heads), "normal", "vector")
        if spec.talking_heads:
            t[spec.talk_name] = TensorInfo((spec.num_heads, spec.num_heads), "normal", "vector")
        t[no] = TensorInfo((hidden, spec.num_heads * spec.v_head_dim))
        if spec.bias:
            t[no + spec.bias_suffix] = TensorInfo((hidden,), "zeros", "vector")
        return t

    @staticmethod
    def cache_need(spec) -> Optional[KVNeed]:
        # (every key stays held: a chunk's first keys are read until the chunk ends)
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=ChunkAttention._cache_head_dim(spec), window=None)

    @staticmethod
    def state_need(spec, hidden: int):
        return None

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        s = self.spec
        nq, nk, nv, no = s.names
        proj = [nq, nk] if s.values_from_keys else [nq, nk, nv]
        mats = [tensors[n] for n in proj]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_qkv = rt.place_matrix(torch.cat(mats, dim=0))
        if s.bias:
            self.b_qkv = rt.place_vector(torch.cat([tensors[n + s.bias_suffix].float() for n in proj]))
            self.b_o = rt.place_vector(tensors[no + s.bias_suffix])
        if s.qk_norm is not None:
            self.q_norm = rt.place_vector(tensors[nq + s.norm_suffix])
            self.k_norm = rt.place_vector(tensors[nk + s.norm_suffix])
        if s.value_blend == "blend":
            self.blend = rt.place_vector(tensors[s.blend_name].reshape(1))
        if s.distance_bias_rows:
            self.dist_bias = rt.place_vector(distance_bias_rows(tensors[s.distance_bias_name], float(s.distance_bias_far),
                                                                max_distance=self.chunk - 1 if self.chunk else None))
        if s.talking_heads:
            self.talk = rt.place_vector(tensors[s.talk_name])
        w_o = tensors[no]
        if self.talks:               # (that kernel writes a head's own values only)
            self.w_o = rt.place_matrix(w_o)
        else:                        # heads of the common size: zero columns beyond a value head's own numbers
            padded = torch.zeros((self.hidden, self.hq, self.d), dtype=w_o.dtype)
            padded[:, :, :self.dv] = w_o.view(self.hidden, self.hq, self.dv)
            self.w_o = rt.place_matrix(padded.view(self.hidden, self.hq * self.d))
        if self.position is not None:
            self.position.load({}, rt)

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        """x [T, H] in the activation type.  Returns the mixer's output, float32 [T, H]."""
        if binding.kv is None:
            raise RuntimeError("attention was given no cache")
        s = self.spec
        T, g, cache = x.shape[0], binding.group, binding.kv
        qkv = ops.gemm(x, self.w_qkv, self.b_qkv)
        v_first = None
        if s.value_blend is not None:
            key = ("chunk_attention.values", self.hkv * self.dv)
            if s.value_blend == "source":
                v_first = ctx.memo[key] = torch.empty((T, self.hkv * self.dv), dtype=torch.float32, device=x.device)
            else:
                v_first = ctx.memo.get(key)
                if v_first is None:
                    raise RuntimeError("values to blend with: no layer before this one has left any")
        mode = {None: ops.QK_NORM_NONE, "head": ops.QK_NORM_HEAD, "whole": ops.QK_NORM_WHOLE}[s.qk_norm]
        q = ops.qkv_norm_store(qkv, self.hq, self.hkv, self.dk, self.dv, cache, ctx.slots[g] if binding.write else None,
                               qk_norm=mode, q_weight=self.q_norm, k_weight=self.k_norm, qk_eps=float(s.qk_norm_eps),
                               values_from_keys=bool(s.values_from_keys), value_norm_eps=s.value_norm_eps,
                               v_first=v_first, v_blend=self.blend if s.value_blend == "blend" else None,
                               positions=ctx.positions,
                               inv_freq=self.position.inv_freq() if self.position is not None else None,
                               value_rows=self.talks)
        if self.talks:
            o = ops.attention_talk(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, self.dk,
                                   self.dv, chunk=self.chunk, bias=self.dist_bias, talk=self.talk)
        else:
            ex = self._extras(ctx)
            o = ops.attention(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, 0,
                              dec_tokens=ex["dec_tokens"], max_dec_position=ex["max_dec_position"],
                              other_tokens=ex["other_tokens"],
                              other_tiles=self._other_tiles(ctx) if ex["other_tokens"] is not None else None,
                              max_other_keys=ex.get("max_other_keys", 0), other_keys_row=ex.get("other_keys_row"),
                              shared_keys=ctx.shared_keys, chunk=self.chunk).view(T, self.hq * self.d)
        return ops.gemm(o, self.w_o, self.b_o, out_dtype=torch.float32)


register_part("paged_attention", PagedAttention)
register_part("conv_attention", ConvAttention)
register_part("chunk_attention", ChunkAttention)
