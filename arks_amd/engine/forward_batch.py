"""Device-side batch metadata handed to the model forward."""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class ForwardBatch:
    is_prefill: bool
    input_ids: torch.Tensor  # [total_tokens] int64
    positions: torch.Tensor  # [total_tokens] int64
    slot_mapping: torch.Tensor  # [total_tokens] int64 (KV write slots)
    # prefill only:
    cu_seqlens: torch.Tensor | None = None  # [num_seqs+1] int32 (device)
    seq_lens_list: list[int] | None = None  # host copy for tile building
    # decode only:
    block_tables: torch.Tensor | None = None  # [num_seqs, max_blocks] int32
    seq_lens: torch.Tensor | None = None  # [num_seqs] int32 (device)
    # prefill-extend only: precomputed work-sorted (tiles64, tiles256) for
    # the paged extend kernels, shared by every layer of the forward
    ext_tiles: tuple | None = None
    # rows of the hidden states from which logits are needed (last token of
    # each sequence for prefill; everything for decode)
    logits_indices: torch.Tensor | None = None
    # models with per-sequence state (recurrent mixers, token shift): the
    # slot of every sequence in the slot-addressed state tensors (-1 =
    # padding row), each row's sequence index, and the longest run of rows
    # of one sequence (host int, sizes the kernels' grids). For these
    # models cu_seqlens / seq_lens / block_tables are set for decode
    # batches too, so one set of kernels serves prompt portions, single
    # tokens and mixes of both.
    state_slots: torch.Tensor | None = None  # [num_seqs] int32
    token_seq: torch.Tensor | None = None  # [total_tokens] int32
    max_q_len: int = 0
    # host copies of the per-sequence total lengths (None inside a captured
    # decode graph) and the per-step cache of kernel work lists built from
    # them, keyed by head layout
    kv_lens_list: list[int] | None = None
    tile_cache: dict = field(default_factory=dict)

    @property
    def num_tokens(self) -> int:
        return self.input_ids.shape[0]
