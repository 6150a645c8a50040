"""Grouped-query attention over the paged cache.

Order of operations as in src/models/qwen3/model.py:200-213: q, k, v projections
(here one product with the three weights stacked), per-head q/k RMSNorm when the
spec asks for it, position encoding of q and k, write of k and v into the cache,
attention of the new tokens over the cache, output projection without bias.
Scores, mask and softmax follow src/layers/fused_ops/attn.py:236-267.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.plan import KVNeed
from ..kernels import ops
from .base import CacheBinding, Runtime, TensorInfo
from .registry import build_part, register_part


# Up to this many single new tokens in a step, the decode attention kernel norms, rotates and
# writes the cache itself; above, the separate kernel is quicker (every wave of the attention
# kernel repeats the preparation of q, which then outweighs the kernel saved).
FUSED_DECODE_MAX_TOKENS = 16


class PagedAttention:
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
    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        """Returns the mixer's output [T, H], or float32 partial products [S, T, H] of it."""
        if binding.kv is None:
            raise RuntimeError("attention was given no cache")
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
        if fused_position and ops.gemm_qkv_supported(x, self.w_qkv, cache, self.hq, table):
            # many rows (portions of prompts): norm, rotation and cache write are the epilogue of the
            # q|k|v product, which never stores its result
            q = ops.gemm_qkv(x, self.w_qkv, self.b_qkv, self.hq, cache, ctx.positions if table is not None else None,
                             self.q_norm, self.k_norm, eps, table, slots)
            return self._attend(q, ctx, cache, g, T)
        if (fused_position and cache.dtype == torch.bfloat16 and ops.gemm_partial_preferred(x, self.w_qkv) and
                ops.qk_rope_store_parts_supported(self.d, table)):
            # 17 to 64 rows against a large matrix: the product is cut along K to fill the chip, and
            # the kernel that norms, rotates and writes the cache adds the parts up as it reads them
            parts = ops.gemm(x, self.w_qkv, epilogue=ops.EPI_PARTIAL)
            q = ops.qk_rope_store_parts(parts, self.b_qkv, self.hq, self.hkv, self.d,
                                        ctx.positions if table is not None else None, self.q_norm, self.k_norm,
                                        eps, table, slots, cache, ctx.page_size)
            return self._attend(q, ctx, cache, g, T)
        qkv = ops.gemm(x, self.w_qkv, self.b_qkv)
        if fused_position:
            only_new_tokens = (ctx.dec_tokens is not None and ctx.dec_tokens.shape[0] == T and
                               (ctx.other_tokens is None or ctx.other_tokens.shape[0] == 0))
            if (only_new_tokens and T <= FUSED_DECODE_MAX_TOKENS and binding.write and
                    ops.attention_decode_fused_supported(qkv, cache, self.hq, table)):
                # every row is the one new token of its request: norm, rotation and cache write
                # happen inside the attention kernel
                o = ops.attention_decode_fused(qkv, self.hq, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g],
                                               self.scale, self.window, None, ctx.max_dec_position,
                                               self.q_norm, self.k_norm, eps, table, slots)
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
        o = ops.attention(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, self.window,
                          dec_tokens=ctx.dec_tokens, max_dec_position=ctx.max_dec_position,
                          other_tokens=ctx.other_tokens,
                          other_tiles=ctx.other_tiles(ops.prefill_tile_rows(self.hq, self.hkv)))
        return self._project_out(o.view(T, self.hq * self.d))

    def _project_out(self, o: torch.Tensor) -> torch.Tensor:
        splits = ops.gemm_branch_splits(o, self.w_o)
        if splits:
            # the product is cut along K (few rows: to fill the chip; a narrow matrix: to give every
            # compute unit blocks to overlap); the norm that follows adds the parts
            return ops.gemm(o, self.w_o, epilogue=ops.EPI_PARTIAL, splits=splits)
        return ops.gemm(o, self.w_o)


register_part("paged_attention", PagedAttention)
