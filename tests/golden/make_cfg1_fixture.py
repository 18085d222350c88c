"""Writes tests/golden/cfg1_tiny_llama_step.json: the tiny-LLaMA fp32 train step of the first benchmark
configuration, evaluated by the CPU oracle (oracle/llama.py) in this container.

    python tests/golden/make_cfg1_fixture.py

Inputs come from ONE CPU generator seeded with 1234, drawn in this order: every >=2-D parameter in
named_parameters() order (randn * 0.02; norm weights stay 1), then ids = randint(0, 8192, (8, 257)).
Labels use the pre-training loader's alignment: input = ids[:, :-1], labels = ids[:, 1:] (all 2048 positions
supervised).  One AdamW step: lr 3e-4, betas (0.9, 0.95), eps 1e-8, weight decay 0.1 on every parameter,
no clipping.  The fixture stores the loss, the global grad norm and, per parameter, the sum, the sum of
absolute values and the first four entries of the post-step value.
"""
import json
import sys
from collections import OrderedDict
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import llama as ol  # noqa: E402

CFG1 = dict(vocab_size=8192, hidden_size=256, intermediate_size=688, num_hidden_layers=4, num_attention_heads=4,
            max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=10000.0)
SEED = 1234


def cfg1_inputs():
    cfg = ol.OracleLlamaConfig(**CFG1)
    gen = torch.Generator().manual_seed(SEED)
    params = OrderedDict()
    for name, shape in ol.param_shapes(cfg).items():
        params[name] = torch.randn(shape, generator=gen) * 0.02 if len(shape) >= 2 else torch.ones(shape)
    ids = torch.randint(0, cfg.vocab_size, (8, 257), generator=gen)
    return cfg, params, ids[:, :-1].contiguous(), ids[:, 1:].contiguous()


def main() -> None:
    torch.set_num_threads(8)
    cfg, params, input_ids, labels = cfg1_inputs()
    loss, grad_norm, new_params = ol.train_step(params, cfg, input_ids, labels)
    out = {
        "config": CFG1, "seed": SEED, "label_alignment": "loader (ids[:, :-1] -> ids[:, 1:], 2048 targets)",
        "optimizer": {"lr": 3e-4, "betas": [0.9, 0.95], "eps": 1e-8, "weight_decay": 0.1, "steps": 1},
        "loss": loss, "grad_norm": grad_norm,
        "params": {n: {"sum": float(p.double().sum()), "abs_sum": float(p.double().abs().sum()),
                       "head": [float(x) for x in p.flatten()[:4]]} for n, p in new_params.items()},
    }
    path = Path(__file__).with_name("cfg1_tiny_llama_step.json")
    path.write_text(json.dumps(out, indent=1))
    print(f"wrote {path}: loss={loss:.6f} grad_norm={grad_norm:.6f}")


if __name__ == "__main__":
    main()
