"""Token-shard reader and pretraining loader (maltos_amd/data.py) against the reference's own shard fixtures
(tests/golden/tokens_0000{0,1}.bin = tests/testdata of the reference: 128 little-endian uint32 tokens each, the
values 0..127).  Both shards hold the same ramp, so the token at position t of the cyclic stream is t mod 128: every
expected batch below is a closed form of the loader's parameters, not a second implementation of its loop.
"""
import dataclasses
from pathlib import Path

import numpy as np
import pytest
import torch

from maltos_amd.data import INPUT_IDS_KEY, LABELS_KEY, PretrainingDataLoader, PretrainingDataState, TokenShardDataset

GOLDEN = Path(__file__).parent / "golden"
SHARDS = [GOLDEN / "tokens_00000.bin", GOLDEN / "tokens_00001.bin"]


def test_fixture_format():
    for path in SHARDS:
        raw = path.read_bytes()
        assert len(raw) == 512 and raw[:8] == bytes([0, 0, 0, 0, 1, 0, 0, 0])  # little-endian uint32
    ds = TokenShardDataset(SHARDS)
    assert len(ds) == 256 and all(np.array_equal(s, np.arange(128)) for s in ds.shards)


def test_read_crosses_shards_and_wraps():
    ds = TokenShardDataset(SHARDS)
    tok, shard, off = ds.read(0, 120, 20)
    assert tok.tolist() == [*range(120, 128), *range(12)] and (shard, off) == (1, 12)
    tok, shard, off = ds.read(1, 100, 60)   # end of the last shard -> back to the first
    assert tok.tolist() == [*range(100, 128), *range(32)] and (shard, off) == (0, 32)
    tok, shard, off = ds.read(0, 0, 128)    # ends exactly at a shard boundary: the position stays there
    assert (shard, off) == (0, 128) and ds.read(shard, off, 3)[0].tolist() == [0, 1, 2]
    assert ds.read(5, 0, 2)[1] == 1         # shard index taken modulo the number of shards
    with pytest.raises(ValueError):
        ds.read(0, 0, 0)
    with pytest.raises(ValueError):
        TokenShardDataset([])


@pytest.mark.parametrize("seq_len,mb,world", [(7, 3, 1), (16, 2, 2), (31, 4, 4), (127, 1, 3)])
def test_batches_are_the_ranks_interleaved_samples_of_the_stream(seq_len, mb, world):
    per = seq_len + 1
    loaders = [PretrainingDataLoader(TokenShardDataset(SHARDS), seq_len=seq_len, micro_batch_size=mb, dp_rank=r, dp_world_size=world)
               for r in range(world)]
    for it in range(5):
        for r, loader in enumerate(loaders):
            batch = loader.next_batch()
            assert batch[INPUT_IDS_KEY].dtype == torch.int64 and batch[INPUT_IDS_KEY].shape == (mb, seq_len)
            for m in range(mb):
                start = ((it * mb + m) * world + r) * per  # sample index in the stream times its length
                want = torch.arange(start, start + per) % 128
                assert torch.equal(batch[INPUT_IDS_KEY][m], want[:-1]) and torch.equal(batch[LABELS_KEY][m], want[1:])
            assert loader.consumed_tokens == (it + 1) * mb * seq_len


def test_state_round_trip_resumes_the_stream():
    mk = lambda **kw: PretrainingDataLoader(TokenShardDataset(SHARDS), seq_len=9, micro_batch_size=2, dp_rank=1, dp_world_size=2, **kw)
    a = mk()
    for _ in range(7):
        a.next_batch()
    state = a.state_dict()
    assert isinstance(state, PretrainingDataState) and state.consumed_tokens == 7 * 2 * 9 and state.seed == 1234
    b = mk(start_state=state)
    c = mk()
    c.load_state_dict(dataclasses.asdict(state))
    for _ in range(4):
        want = a.next_batch()
        for other in (b.next_batch(), c.next_batch()):
            assert all(torch.equal(want[k], other[k]) for k in want)
    with pytest.raises(ValueError, match="invalid shard_idx"):
        c.load_state_dict(dict(shard_idx=2, token_offset=0, consumed_tokens=0, seed=0))
    with pytest.raises(ValueError, match="invalid token_offset"):
        c.load_state_dict(dict(shard_idx=0, token_offset=129, consumed_tokens=0, seed=0))


def test_argument_errors_and_cp_seam():
    ds = TokenShardDataset(SHARDS)
    for kw in (dict(seq_len=0, micro_batch_size=1), dict(seq_len=4, micro_batch_size=0), dict(seq_len=4, micro_batch_size=1, dp_world_size=0),
               dict(seq_len=4, micro_batch_size=1, dp_rank=2, dp_world_size=2)):
        with pytest.raises(ValueError):
            PretrainingDataLoader(ds, **kw)
    with pytest.raises(RuntimeError, match="cp_batch_sharder"):
        PretrainingDataLoader(ds, seq_len=4, micro_batch_size=1).next_batch(cp_rank=0)

    class Halves:
        def shard(self, batch, *, rank):
            return {k: v[:, rank * 2:(rank + 1) * 2] for k, v in batch.items()}

    got = PretrainingDataLoader(ds, seq_len=4, micro_batch_size=1, cp_batch_sharder=Halves()).next_batch(cp_rank=1)
    assert got[INPUT_IDS_KEY].tolist() == [[2, 3]] and got[LABELS_KEY].tolist() == [[3, 4]]
