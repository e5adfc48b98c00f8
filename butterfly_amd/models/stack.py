"""What the heterogeneous layer stacks (models/nesizen.py, models/zinesun.py) share: unsharded
single-rank models whose steps are packed rows (decoded rows first, then prompt chunks) that
always attend through the paged cache."""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from ..engine.batch import ForwardBatch


def pad128(n: int) -> int:
    """Fused projections carry zero rows up to a multiple of 128 (the MFMA GEMMs' N tiling)."""
    return (n + 127) // 128 * 128


class PackedStack:
    """Mixin: expects self.p (parameter dict), self.cfg, self.device, self.dtype, self.specs,
    self.has_state."""
    paged_prefill_only = True     # the runner builds block tables for every prompt chunk
    supports_f32 = True           # every kernel of the family has a true 32-bit form
    attention_types = ("attention",)

    def local_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.p.values() if t is not None)

    def packed_decode_bytes(self, kinds=None) -> int:
        return 0

    def pack_decode_weights(self, budget_bytes=None, kinds=None) -> int:
        return 0

    def kv_bytes_per_token(self, dtype: Optional[torch.dtype] = None) -> int:
        es = torch.empty((), dtype=dtype or self.dtype).element_size()
        return max(1, self.cfg.kv_bytes_per_token(es))

    def gemm_shapes(self) -> list:
        return sorted({tuple(w.shape) for k, w in self.p.items()
                       if w is not None and w.dim() == 2 and w.dtype == torch.bfloat16 and k != "embed"
                       and w.shape[0] % 128 == 0 and w.shape[1] % 64 == 0})

    def _iota(self, n: int) -> torch.Tensor:
        t = self._arange.get(n)
        if t is None:
            t = self._arange[n] = torch.arange(n, dtype=torch.int32, device=self.device)
        return t

    def _step_meta(self, fb: ForwardBatch) -> dict:
        """Packed-row description shared by the mixers: row_cu [nseq + 1] (decode rows are
        one-row sequences, then the prompt chunks), one block table per sequence, state slots."""
        T = fb.num_tokens
        name = type(self).__name__
        if not fb.is_prefill:
            row_cu, tables = self._iota(T + 1), fb.block_tables
        else:
            nd = fb.num_decode
            if fb.cu_seqlens.numel() > 1 and fb.prefix_tables is None:
                raise RuntimeError(f"{name}: prompt chunks need their block tables (mixed scheduling)")
            if nd:
                row_cu = torch.cat([self._iota(nd), fb.cu_seqlens + nd])
                tables = fb.block_tables[:nd] if fb.prefix_tables is None else torch.cat([fb.block_tables[:nd], fb.prefix_tables])
            else:
                row_cu, tables = fb.cu_seqlens, fb.prefix_tables
        m = {"row_cu": row_cu, "tables": tables, "state_slots": fb.state_slots, "row_map": None}
        if self.has_state and fb.state_slots is None and T:
            raise RuntimeError(f"{name}: the batch carries no per-sequence state slots")
        if self.device.type == "cuda" and T and any(sp["type"] in self.attention_types for sp in self.specs):
            m["row_map"] = ops.row_seq(row_cu, T)
        return m
