"""Per-iteration forward metadata threaded through every decoder block.

One ForwardMeta describes either a (chunked-)prefill batch or a decode batch —
the equivalent of the reference's batch formation output (sglang/batch_info.py)
re-designed around our paged layout. All tensors live on the model's device.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import TYPE_CHECKING, Optional

import torch

if TYPE_CHECKING:
    from ..server.kv_cache import LinearStateCache, MLAKVCache, PagedKVCache


@dataclass
class ForwardMeta:
    is_prefill: bool
    positions: torch.Tensor          # [T] int32 — absolute position of each token
    slot_mapping: torch.Tensor       # [T] int64 — flat KV slot per token
    block_tables: torch.Tensor       # [B, max_blocks] int32
    seq_lens: torch.Tensor           # [B] int32 — total ctx len incl. this step
    query_lens: Optional[torch.Tensor] = None   # [B] int32, prefill only
    kv_cache: Optional["PagedKVCache"] = None
    mla_cache: Optional["MLAKVCache"] = None
    linear_cache: Optional["LinearStateCache"] = None
    linear_slots: Optional[torch.Tensor] = None  # [B] int32 slot ids (hybrid stacks)
    # indices of the last token of each request within the packed token dim
    # (where logits are needed; for decode this is arange(B))
    logits_indices: Optional[torch.Tensor] = None
    # host-side max of seq_lens (avoids a device sync when picking the
    # flash-decoding partition count)
    max_seq_len: int = 0
    # [T] int64: the token before each token in its own sequence, -1 for a
    # sequence's first token (filled for models that set `uses_prev_tokens`:
    # their embedding reads the pair)
    prev_ids: Optional[torch.Tensor] = None
    # derived per-token tables for packed-sequence kernels (built on first
    # use, shared by every layer of the forward)
    _token_seq: Optional[torch.Tensor] = None
    _query_bounds: Optional[torch.Tensor] = None

    def token_seq(self) -> Optional[torch.Tensor]:
        """[T] int32: the batch row each packed token belongs to. None for a
        decode batch (token i is row i)."""
        if not self.is_prefill:
            return None
        if self._token_seq is None:
            B = self.query_lens.shape[0]
            self._token_seq = torch.repeat_interleave(
                torch.arange(B, dtype=torch.int32, device=self.query_lens.device),
                self.query_lens.long(), output_size=self.num_tokens,
            )
        return self._token_seq

    def query_bounds(self) -> Optional[torch.Tensor]:
        """[B+1] int32 prefix sums of query_lens (None for a decode batch)."""
        if not self.is_prefill:
            return None
        if self._query_bounds is None:
            self._query_bounds = torch.nn.functional.pad(
                torch.cumsum(self.query_lens, 0), (1, 0)
            ).to(torch.int32)
        return self._query_bounds

    @property
    def num_tokens(self) -> int:
        return self.positions.shape[0]

    @property
    def batch_size(self) -> int:
        return self.seq_lens.shape[0]
