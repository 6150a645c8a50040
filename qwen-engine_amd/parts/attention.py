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


register_part("paged_attention", PagedAttention)
