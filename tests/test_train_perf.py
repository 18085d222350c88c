"""Step harness (maltos_amd/train_perf.py): synthetic batches on the CPU, the timed runner on the GPU."""
import json

import pytest
import torch

from maltos_amd import train_perf as tp
from maltos_amd.losses import IGNORE_INDEX


@pytest.mark.parametrize("layout", ["dense", "packed"])
def test_synthetic_batches_are_valid_causal_lm_batches(layout):
    B, S, V = 5, 96, 50
    batch = tp.make_synthetic_batch(batch_size=B, seq_len=S, vocab_size=V, layout=layout, seed=3, device=torch.device("cpu"))
    again = tp.make_synthetic_batch(batch_size=B, seq_len=S, vocab_size=V, layout=layout, seed=3, device=torch.device("cpu"))
    assert all(torch.equal(batch[k], again[k]) for k in batch)  # deterministic
    ids, labels = batch[tp.INPUT_IDS_KEY], batch[tp.LABELS_KEY]
    assert ids.shape == labels.shape == (B, S) and ids.min() >= 0 and ids.max() < V
    sup = labels != IGNORE_INDEX
    assert torch.equal(labels[:, :-1][sup[:, :-1]], ids[:, 1:][sup[:, :-1]]) and not sup[:, -1].any()
    if layout == "dense":
        assert sup[:, :-1].all() and set(batch) == {tp.INPUT_IDS_KEY, tp.LABELS_KEY}
        return
    pos, seq = batch[tp.POSITION_IDS_KEY], batch[tp.SEQUENCE_IDS_KEY]
    for row in range(B):
        active = int((seq[row] != tp.PAD_SEQUENCE_ID).sum())
        assert (seq[row, active:] == tp.PAD_SEQUENCE_ID).all() and (seq[row, :active] >= 0).all() and active >= S * 0.9 - 1
        docs = seq[row, :active].unique_consecutive(return_counts=True)
        assert 2 <= len(docs[0]) <= 8 and docs[1].min() >= 2 and len(set(docs[0].tolist())) == len(docs[0])
        start = 0
        for n in docs[1].tolist():
            assert torch.equal(pos[row, start:start + n], torch.arange(n))
            assert labels[row, start + n - 1] == IGNORE_INDEX  # no target across a document boundary
            start += n
        assert not sup[row, active:].any()
    # sequence ids of different rows never collide
    assert len({int(s) for r in range(B) for s in seq[r].unique() if s >= 0}) == sum(len(seq[r][seq[r] >= 0].unique()) for r in range(B))
    with pytest.raises(ValueError):
        tp.make_synthetic_batch(batch_size=1, seq_len=8, vocab_size=9, layout="ragged", seed=0, device=torch.device("cpu"))


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--layout", "dense"], ["--layout", "packed", "--optimizer-layout", "zero1"],
                                   ["--shards", "tests/golden/tokens_0000*.bin", "--seq-len", "31", "--batch-size", "4"],
                                   ["--layout", "packed", "--graph"], ["--layout", "dense", "--graph", "--optimizer-layout", "zero1"]],
                         ids=["dense", "packed-zero1", "shards", "packed-graph", "dense-graph-zero1"])
def test_runner_steps_and_reports(dev, tmp_path, extra):
    out = tmp_path / "summary.json"
    argv = ["--model", "llama-tiny", "--batch-size", "2", "--seq-len", "256", "--steps", "3", "--warmup", "1", "--out", str(out), *extra]
    assert tp.main(argv) == 0
    s = json.loads(out.read_text())
    assert s["steps"] == 3 and s["tokens_per_sec"] > 0 and s["step_ms_min"] <= s["step_ms_median"]
    assert 0 < s["loss_last"] < 12 and s["grad_norm_last"] > 0
    if "zero1" in extra:
        assert s["buckets"] >= 1
    assert s["graph"] == ("--graph" in extra)
    if "--graph" in extra:      # the same run without the graph gives the same loss (the steps are deterministic)
        eager = tmp_path / "eager.json"
        assert tp.main([a for a in argv if a != "--graph"] + ["--out", str(eager)]) == 0   # the later --out wins
        e = json.loads(eager.read_text())
        assert abs(e["loss_last"] - s["loss_last"]) <= 1e-6 * abs(e["loss_last"])
        assert abs(e["grad_norm_last"] - s["grad_norm_last"]) <= 1e-5 * abs(e["grad_norm_last"])


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--shards", "tests/golden/tokens_0000*.bin", "--seq-len", "31", "--batch-size", "4"],
                                   ["--layout", "packed", "--batch-size", "2", "--seq-len", "256"]], ids=["shards", "packed"])
def test_first_step_loss_equals_the_oracle_forward(dev, tmp_path, extra):
    """The first step of the harness (initial weights, first batch of the loader / the synthetic batch) against the
    oracle's forward on the same weights and batch: 1e-3 relative, the bf16 loss bar."""
    import glob
    from collections import OrderedDict

    from maltos_amd.data import PretrainingDataLoader, TokenShardDataset
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM
    from oracle import llama as ol

    out = tmp_path / "summary.json"
    assert tp.main(["--model", "llama-tiny", "--steps", "2", "--warmup", "0", "--out", str(out), *extra]) == 0
    summary = json.loads(out.read_text())
    # the harness's initial weights: torch.manual_seed(seed), default construction, matrices redrawn N(0, 0.02)
    torch.manual_seed(1234)
    model = LlamaForCausalLM(LlamaConfig(**tp.MODELS["llama-tiny"]))
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0.0, 0.02)
    params = OrderedDict((n, p.detach().to(torch.bfloat16).float().to(dev)) for n, p in model.named_parameters())
    if "--shards" in extra:
        loader = PretrainingDataLoader(TokenShardDataset(sorted(glob.glob("tests/golden/tokens_0000*.bin"))), seq_len=31,
                                       micro_batch_size=4, seed=1234)
        batch = {k: v.to(dev) for k, v in loader.next_batch().items()}
    else:
        batch = tp.make_synthetic_batch(batch_size=2, seq_len=256, vocab_size=8192, layout="packed", seed=1234, device=dev)
    cfg = ol.OracleLlamaConfig(**tp.MODELS["llama-tiny"])
    want = ol.forward(params, cfg, batch[tp.INPUT_IDS_KEY], batch[tp.LABELS_KEY], position_ids=batch.get(tp.POSITION_IDS_KEY),
                      sequence_ids=batch.get(tp.SEQUENCE_IDS_KEY))
    assert abs(summary["loss_first"] - float(want)) <= 1e-3 * float(want), (summary["loss_first"], float(want))
