"""Which vendor GEMM kernel serves which product of the linear layers.

The projections and the lm_head of the decoder run on the vendor libraries (hipBLASLt / rocBLAS) through torch; for
every product shape those libraries hold hundreds of kernels and pick one by a heuristic.  At the LLaMA-50M shapes
(16384 tokens against 512 .. 2752 wide weights, contraction length 512) the heuristic's pick is often not the fastest:
timing the candidates once and keeping the winner per shape (torch's TunableOp does the timing) takes 5 % off the
whole train step on MI355X.  This module ships such a selection for gfx950 (`tuned/gemm_gfx950.csv`, one line per
product shape) and the two switches around it:

    use_tuned_gemms()            look the shapes of the file up from now on; unknown shapes keep the library's pick
    record_gemm_tuning(path)     time the candidates of every new shape that runs from now on and write the winners

The file names the torch, HIP, hipBLASLt and rocBLAS versions and the GPU architecture it was recorded with; torch
refuses it when they differ, and `use_tuned_gemms` then leaves everything as it was and says so in its return value.
Nothing here touches the hand-written kernels, and nothing changes unless one of the two functions is called.

`python -m maltos_amd.gemm_tuning [path]` records the selection for the LLaMA-50M step (B=8, S=2048, bf16) on the
current GPU: a few eager train steps in the flat optimizer layout, with the q/k/v and gate/up projections as one
product each and as separate ones.
"""
from __future__ import annotations

import sys
from pathlib import Path

import torch

TUNED_FILE = Path(__file__).with_name("tuned") / "gemm_gfx950.csv"


def use_tuned_gemms(path: "str | Path | None" = None) -> int:
    """Turn the per-shape GEMM selection of `path` (default: the file shipped for gfx950) on for this process.
    Returns the number of product shapes now selected; 0 means the file was refused (recorded with other library
    versions or another GPU) or missing, and the libraries' own choices stay in force."""
    if not torch.cuda.is_available():
        raise RuntimeError("use_tuned_gemms needs a GPU: the selection names kernels of the GPU GEMM libraries")
    path = Path(path) if path is not None else TUNED_FILE
    tunable = torch.cuda.tunable
    if not path.is_file():
        return 0
    tunable.enable(True)
    tunable.tuning_enable(False)   # look up only: a shape the file does not list keeps the library's pick
    if not tunable.read_file(str(path)):
        tunable.enable(False)
        return 0
    return len(tunable.get_results())


def tuned_gemms_off() -> None:
    """Back to the libraries' own choice for every product."""
    torch.cuda.tunable.tuning_enable(False)
    torch.cuda.tunable.enable(False)


def record_gemm_tuning(path: "str | Path", max_tuning_ms: int = 100) -> None:
    """From now on every GEMM shape that runs for the first time has its candidate kernels timed (up to `max_tuning_ms`
    each) and the winner written to `path`; call `tuned_gemms_off()` or `use_tuned_gemms(path)` when the shapes of
    interest have run.  Timing runs the product many times: do this in a warm-up, outside graph capture."""
    if not torch.cuda.is_available():
        raise RuntimeError("record_gemm_tuning needs a GPU")
    tunable = torch.cuda.tunable
    Path(path).parent.mkdir(parents=True, exist_ok=True)
    tunable.set_filename(str(path), insert_device_ordinal=False)
    tunable.set_max_tuning_duration(int(max_tuning_ms))
    tunable.enable(True)
    tunable.tuning_enable(True)


def _record_llama50m(path: Path) -> None:
    from .llama import LlamaConfig, LlamaForCausalLM, set_grad_accumulation_into_buffers
    from .optim import FusedAdamW, MasterWeightsOptimizer

    dev = torch.device("cuda:0")
    record_gemm_tuning(path)
    for fuse in (True, False):
        cfg = LlamaConfig(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=2,
                          num_attention_heads=8, max_position_embeddings=2048, rms_norm_eps=1e-5, fuse_projections=fuse)
        torch.manual_seed(0)
        model = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
        set_grad_accumulation_into_buffers(model)
        opt = MasterWeightsOptimizer(model.parameters(), optimizer_factory=lambda ps: FusedAdamW(ps, lr=3e-4))
        ids = torch.randint(0, cfg.vocab_size, (8, 2049), generator=torch.Generator().manual_seed(0)).to(dev)
        batch = {"input_ids": ids[:, :-1].contiguous(), "labels": ids[:, 1:].contiguous()}
        for _ in range(2):
            model(batch).backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
            torch.cuda.synchronize()
            print(f"[gemm_tuning] step done (fuse_projections={fuse}), {len(torch.cuda.tunable.get_results())} shapes", flush=True)
    tuned_gemms_off()
    print(f"[gemm_tuning] wrote {path}", flush=True)


if __name__ == "__main__":
    _record_llama50m(Path(sys.argv[1]) if len(sys.argv) > 1 else TUNED_FILE)
