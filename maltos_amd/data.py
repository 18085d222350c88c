"""Token-shard reader and deterministic pretraining loader: the data format on the input side of the train step.

Same interface and stream semantics as the reference's `TokenShardDataset` / `PretrainingDataLoader`
(data/pretrain.py:22-146): shards are raw little-endian uint32 token ids, memory-mapped; the loader walks them as one
cyclic stream in samples of seq_len + 1 tokens, data-parallel rank r taking samples r, r + W, r + 2W, ...;
`input_ids` are the first seq_len tokens of a sample, `labels` the last seq_len; the position in the stream is a
(shard, offset) pair that can be saved and restored.  Host-side code only: batches are int64 CPU tensors.
"""
from __future__ import annotations

import dataclasses
from pathlib import Path
from typing import Any, Iterable, Iterator

import numpy as np
import torch

INPUT_IDS_KEY = "input_ids"  # utils/constants.py
LABELS_KEY = "labels"


def _require(ok: bool, message: str) -> None:
    if not ok:
        raise ValueError(message)


@dataclasses.dataclass(frozen=True)
class PretrainingDataState:
    shard_idx: int
    token_offset: int
    consumed_tokens: int
    seed: int


class TokenShardDataset:
    """Memory-mapped token shards read as one cyclic stream."""

    def __init__(self, paths: Iterable[str | Path], *, dtype: np.dtype = np.dtype("<u4")) -> None:
        self.paths = [Path(p) for p in paths]
        _require(bool(self.paths), "TokenShardDataset requires at least one token shard")
        self.dtype = np.dtype(dtype)
        self.shards = [np.memmap(p, mode="r", dtype=self.dtype) for p in self.paths]
        for p, shard in zip(self.paths, self.shards):
            _require(shard.size > 0, f"token shard is empty: {p}")

    def __len__(self) -> int:
        return sum(int(s.size) for s in self.shards)

    def _pieces(self, shard: int, offset: int, length: int) -> Iterator[tuple[int, int, int]]:
        """(shard, lo, hi) slices that make up `length` tokens from (shard, offset) on; a position at the end of a shard
        moves to the start of the next one only when more tokens are wanted."""
        while length > 0:
            size = int(self.shards[shard].size)
            if offset >= size:
                shard, offset = (shard + 1) % len(self.shards), 0
                continue
            hi = min(size, offset + length)
            yield shard, offset, hi
            length -= hi - offset
            offset = hi

    def read(self, shard_idx: int, token_offset: int, length: int) -> tuple[np.ndarray, int, int]:
        """`length` tokens and the position after them (which may be the end of a shard)."""
        _require(length >= 1, f"length must be >= 1, got {length}")
        pieces = list(self._pieces(shard_idx % len(self.shards), int(token_offset), int(length)))
        tokens = np.concatenate([self.shards[s][lo:hi] for s, lo, hi in pieces]).astype(self.dtype, copy=False)
        last_shard, _, last_hi = pieces[-1]
        return tokens, last_shard, last_hi


class PretrainingDataLoader:
    """Next-token-prediction batches from the token stream.  `cp_batch_sharder` is the seam for the context-parallel
    split of a batch: any object with `shard(batch, rank=...)`."""

    def __init__(self, dataset: TokenShardDataset, *, seq_len: int, micro_batch_size: int, dp_rank: int = 0,
                 dp_world_size: int = 1, seed: int = 1234, start_state: PretrainingDataState | None = None,
                 cp_batch_sharder: Any | None = None) -> None:
        _require(seq_len >= 1, f"seq_len must be >= 1, got {seq_len}")
        _require(micro_batch_size >= 1, f"micro_batch_size must be >= 1, got {micro_batch_size}")
        _require(dp_world_size >= 1, f"dp_world_size must be >= 1, got {dp_world_size}")
        _require(0 <= dp_rank < dp_world_size, f"dp_rank must be in [0, {dp_world_size}), got {dp_rank}")
        self.dataset, self.seq_len, self.micro_batch_size = dataset, seq_len, micro_batch_size
        self.dp_rank, self.dp_world_size, self.seed = dp_rank, dp_world_size, seed
        self._sample = seq_len + 1                      # tokens per sample: inputs plus the last label
        self._stride_rest = (dp_world_size - 1) * self._sample  # the other ranks' samples between two of ours
        self.shard_idx, self.token_offset, self.consumed_tokens = 0, dp_rank * self._sample, 0
        self._cp_batch_sharder = cp_batch_sharder
        if start_state is not None:
            self.load_state_dict(dataclasses.asdict(start_state))

    def _take(self, n: int) -> np.ndarray:
        tokens, self.shard_idx, self.token_offset = self.dataset.read(self.shard_idx, self.token_offset, n)
        return tokens

    def next_batch(self, cp_rank: int | None = None) -> dict[str, torch.Tensor]:
        rows = np.empty((self.micro_batch_size, self._sample), dtype=np.int64)
        for row in rows:
            row[:] = self._take(self._sample)
            if self._stride_rest:
                self._take(self._stride_rest)
        self.consumed_tokens += self.micro_batch_size * self.seq_len
        tokens = torch.from_numpy(rows)
        batch = {INPUT_IDS_KEY: tokens[:, :-1].contiguous(), LABELS_KEY: tokens[:, 1:].contiguous()}
        if cp_rank is None:
            return batch
        if self._cp_batch_sharder is None:
            raise RuntimeError("CP-local next_batch(cp_rank) requires constructor cp_batch_sharder")
        return self._cp_batch_sharder.shard(batch, rank=cp_rank)

    def state_dict(self) -> PretrainingDataState:
        return PretrainingDataState(self.shard_idx, self.token_offset, self.consumed_tokens, self.seed)

    def load_state_dict(self, state: dict[str, Any]) -> None:
        st = PretrainingDataState(**state)
        _require(0 <= st.shard_idx < len(self.dataset.shards), f"invalid shard_idx={st.shard_idx}")
        _require(0 <= st.token_offset <= self.dataset.shards[st.shard_idx].size, f"invalid token_offset={st.token_offset}")
        self.shard_idx, self.token_offset, self.consumed_tokens, self.seed = st.shard_idx, st.token_offset, st.consumed_tokens, st.seed
