"""Synthetic train-step runner: the caller side of the hot path, for throughput runs of a recipe on one GPU.

    python -m maltos_amd.train_perf --model llama-50m --layout dense  --steps 20 --out summary.json
    python -m maltos_amd.train_perf --model llama-50m --layout packed --optimizer-layout zero1
    python -m maltos_amd.train_perf --model llama-50m --layout dense  --graph
    python -m maltos_amd.train_perf --model llama-tiny --shards tests/golden/tokens_0000*.bin --seq-len 31

What it does is what the reference's `tools/profile_train_perf.py` does around its timed region (:470-548 synthetic
dense / packed batches built outside the timed steps, :962-1096 warm-up, timed steps, a `summary.json`): build the
model and the optimizer, make deterministic batches (random token ids; the packed layout adds per-row documents with
`position_ids` / `sequence_ids` and a padded tail), or read them from token shards, then time full steps (forward,
backward, global-norm clip, AdamW) between device synchronisations and write the figures as JSON.
"""
from __future__ import annotations

import argparse
import glob
import json
import statistics
import sys
import time

import torch

from .data import INPUT_IDS_KEY, LABELS_KEY, PretrainingDataLoader, TokenShardDataset
from .losses import IGNORE_INDEX

POSITION_IDS_KEY = "position_ids"   # utils/constants.py
SEQUENCE_IDS_KEY = "sequence_ids"
PAD_SEQUENCE_ID = -1

MODELS = {
    # configs/llama_50m.yaml of the reference; the tiny one is the CPU-runnable check configuration
    "llama-50m": dict(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=8, num_attention_heads=8,
                      max_position_embeddings=2048, rms_norm_eps=1e-5),
    "llama-tiny": dict(vocab_size=8192, hidden_size=256, intermediate_size=688, num_hidden_layers=4, num_attention_heads=4,
                       max_position_embeddings=2048, rms_norm_eps=1e-5),
}


def make_synthetic_batch(*, batch_size: int, seq_len: int, vocab_size: int, layout: str, seed: int, device: torch.device,
                         segments: tuple[int, int] = (2, 8), max_padding_fraction: float = 0.1) -> dict[str, torch.Tensor]:
    """A valid causal-LM batch: labels are the inputs shifted by one with the last position ignored.  `packed` cuts every
    row into documents (positions restart, sequence ids differ, the last label of a document is ignored) and pads the
    tail with sequence id -1."""
    if batch_size < 1 or seq_len < 2 or vocab_size < 2:
        raise ValueError("synthetic batch requires batch_size >= 1, seq_len >= 2 and vocab_size >= 2")
    gen = torch.Generator().manual_seed(seed)
    input_ids = torch.randint(0, vocab_size, (batch_size, seq_len), generator=gen)
    labels = torch.full_like(input_ids, IGNORE_INDEX)
    labels[:, :-1] = input_ids[:, 1:]
    batch = {INPUT_IDS_KEY: input_ids, LABELS_KEY: labels}
    if layout == "packed":
        lo, hi = segments
        if not 2 <= lo <= hi <= seq_len // 2:
            raise ValueError(f"segment counts must satisfy 2 <= min <= max <= seq_len / 2, got {segments}")
        position_ids = torch.zeros_like(input_ids)
        sequence_ids = torch.full_like(input_ids, PAD_SEQUENCE_ID)
        for row in range(batch_size):
            count = int(torch.randint(lo, hi + 1, (), generator=gen))
            active = seq_len - int(torch.randint(int(seq_len * max_padding_fraction) + 1, (), generator=gen))
            active = max(active, 2 * count)
            # every document two tokens plus its share of the rest, the shares being the gaps between sorted cut points
            spare = active - 2 * count
            cuts = torch.randint(0, spare + 1, (count - 1,), generator=gen).sort().values
            shares = torch.diff(torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([spare])]))
            bounds = [0, *torch.cumsum(shares + 2, 0).tolist()]
            for doc, (start, end) in enumerate(zip(bounds[:-1], bounds[1:])):
                position_ids[row, start:end] = torch.arange(end - start)
                sequence_ids[row, start:end] = row * hi + doc
                labels[row, end - 1] = IGNORE_INDEX
            input_ids[row, active:] = 0
            labels[row, active:] = IGNORE_INDEX
        batch[POSITION_IDS_KEY] = position_ids
        batch[SEQUENCE_IDS_KEY] = sequence_ids
    elif layout != "dense":
        raise ValueError(f"unsupported synthetic layout={layout!r}")
    return {k: v.to(device) for k, v in batch.items()}


def run(args: argparse.Namespace) -> dict:
    from .grad_clip import clip_grad_norm_
    from .llama import LlamaConfig, LlamaForCausalLM, set_grad_accumulation_into_buffers
    from .optim import FusedAdamW, MasterWeightsOptimizer
    from .zero1 import Zero1FlatBuffers

    if not torch.cuda.is_available():
        raise RuntimeError("maltos_amd.train_perf needs a GPU: the HIP path has no CPU fallback")
    dev = torch.device("cuda:0")
    cfg = LlamaConfig(**MODELS[args.model])
    torch.manual_seed(args.seed)
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    model = LlamaForCausalLM(cfg)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0.0, 0.02)
    model = model.to(dev).to(dtype)
    set_grad_accumulation_into_buffers(model)   # weight gradients add into bound gradient buffers where there are any
    adamw = lambda ps: FusedAdamW(ps, lr=args.lr, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    factory = (lambda ps: MasterWeightsOptimizer(ps, optimizer_factory=adamw)) if dtype == torch.bfloat16 else adamw
    zero = None
    if args.optimizer_layout == "zero1":
        zero = Zero1FlatBuffers(model, optimizer_factory=factory, bucket_mb_size=args.bucket_mb)
    elif args.optimizer_layout == "zero2":
        from .zero2 import Zero2FlatBuffers
        zero = Zero2FlatBuffers(model, optimizer_factory=factory, bucket_mb_size=args.bucket_mb)
    gemm_shapes = 0
    if not args.library_gemm_choice:
        from .gemm_tuning import use_tuned_gemms
        gemm_shapes = use_tuned_gemms()   # 0: the shipped selection does not fit this GEMM library version and is not used
    opt = None if zero else factory(list(model.parameters()))

    if args.shards:
        paths = sorted(p for pattern in args.shards for p in glob.glob(pattern))
        loader = PretrainingDataLoader(TokenShardDataset(paths), seq_len=args.seq_len, micro_batch_size=args.batch_size, seed=args.seed)
        next_batch = lambda: {k: v.to(dev) for k, v in loader.next_batch().items()}
        source = {"shards": paths}
    else:
        fixed = make_synthetic_batch(batch_size=args.batch_size, seq_len=args.seq_len, vocab_size=cfg.vocab_size, layout=args.layout,
                                     seed=args.seed, device=dev)
        next_batch = lambda: fixed
        source = {"synthetic": args.layout}

    losses, norms, times = [], [], []
    captured = None
    if args.graph:
        from .graph_step import CapturedForwardBackward
        if zero:
            zero.reset_grads()
        clear = zero.reset_grads if zero else (lambda: opt.zero_grad(set_to_none=True))
        captured = CapturedForwardBackward(model, next_batch(), embed=model.embed_tokens, clear_grads=clear)

    def step() -> None:
        batch = next_batch()
        if zero:
            zero.reset_grads()
        if captured is not None:
            loss = captured(batch).clone()
        else:
            loss = model(batch)
            loss.backward()
        if zero:
            norm = zero.step(args.max_grad_norm)
        else:
            norm = clip_grad_norm_(opt, args.max_grad_norm)
            opt.step()
            opt.zero_grad(set_to_none=True)
        losses.append(loss.detach())
        norms.append(norm)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    del losses[:], norms[:]
    for _ in range(args.steps):
        t0 = time.perf_counter()
        step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    tokens = args.batch_size * args.seq_len
    mean = sum(times) / len(times)
    return {
        "model": args.model, "dtype": args.dtype, "batch_size": args.batch_size, "seq_len": args.seq_len, "data": source,
        "optimizer_layout": args.optimizer_layout, "graph": bool(args.graph), "buckets": len(zero.buckets) if zero else None,
        "gemm_shapes_selected_from_file": gemm_shapes,
        "params": sum(p.numel() for p in model.parameters()), "steps": args.steps, "warmup": args.warmup,
        "step_ms_mean": mean * 1e3, "step_ms_median": statistics.median(times) * 1e3, "step_ms_min": min(times) * 1e3,
        "tokens_per_sec": tokens / mean, "model_tflops": tokens * model.flops_per_token() / mean / 1e12,
        "loss_first": float(losses[0]), "loss_last": float(losses[-1]), "grad_norm_last": float(norms[-1]),
    }


def parse_args(argv: list[str] | None = None) -> argparse.Namespace:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", choices=sorted(MODELS), default="llama-50m")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--layout", choices=["dense", "packed"], default="dense")
    ap.add_argument("--optimizer-layout", choices=["flat", "zero1", "zero2"], default="flat")
    ap.add_argument("--library-gemm-choice", action="store_true",
                    help="leave the choice of GEMM kernels to hipBLASLt / rocBLAS instead of the per-shape selection "
                         "shipped for gfx950 (maltos_amd.gemm_tuning)")
    ap.add_argument("--graph", action="store_true",
                    help="replay forward + backward from one HIP graph (bf16, fixed batch shapes; see maltos_amd.graph_step)")
    ap.add_argument("--bucket-mb", type=int, default=25)
    ap.add_argument("--shards", nargs="*", default=[], help="token shard files (raw little-endian uint32) instead of synthetic ids")
    ap.add_argument("--batch-size", type=int, default=8)
    ap.add_argument("--seq-len", type=int, default=2048)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--lr", type=float, default=3e-4)
    ap.add_argument("--max-grad-norm", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--out", default=None, help="write the summary to this JSON file as well as to stdout")
    return ap.parse_args(argv)


def main(argv: list[str] | None = None) -> int:
    args = parse_args(argv)
    summary = run(args)
    text = json.dumps(summary, indent=1)
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
