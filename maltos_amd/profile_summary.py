"""Short text summaries of rocprofv3 runs of bench.py, written under profiles/.

    python -m maltos_amd.profile_summary RAW_DIR [--out profiles]

RAW_DIR holds the raw output of these runs (each its own rocprofv3 invocation on one MI355X, from the repository
root after `export TMPDIR=/tmp`; only the sub-directories that exist are summarised):

    stats      rocprofv3 --kernel-trace --stats -f csv -d RAW_DIR/stats -- python3 bench.py --steps 40 --warmup 10 --skip-cpu --skip-extra
    llama      rocprofv3 --kernel-trace --stats -f csv -d RAW_DIR/llama -- python3 bench.py --steps 10 --warmup 3 --skip-cpu --only llama50m_train_step
    fetch      rocprofv3 --pmc FETCH_SIZE -f csv -d RAW_DIR/fetch -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra
    write      rocprofv3 --pmc WRITE_SIZE -f csv -d RAW_DIR/write -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra
    fetch_cal  rocprofv3 --pmc FETCH_SIZE -f csv -d RAW_DIR/fetch_cal -- python3 bench.py --calibrate-traffic
    write_cal  rocprofv3 --pmc WRITE_SIZE -f csv -d RAW_DIR/write_cal -- python3 bench.py --calibrate-traffic
    pmc_a      rocprofv3 --pmc SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA SQ_INSTS_VALU SQ_ACTIVE_INST_VALU
                   SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT SQ_WAIT_INST_LDS -f csv -d RAW_DIR/pmc_a -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra
    pmc_b      rocprofv3 --pmc SQ_WAVE_CYCLES SQ_ACTIVE_INST_ANY SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS SQ_ACTIVE_INST_SCA
                   SQ_INSTS_SALU -f csv -d RAW_DIR/pmc_b -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra

Outputs: attn_cfg2_kernel_stats.md, llama50m_step_kernel_stats.md, attn_cfg2_hbm_traffic.md and .json (the .json is
what bench.py reads for `roofline.traffic`), attn_cfg2_mfma_util.md.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import sys

CFG2 = dict(B=4, H=16, S=4096, D=128)
KERNELS = {  # kernel-name fragment -> bench.py's timer name
    "attn_fwd_dma_kernel": "attn_fwd",
    "attn_bwd_dkdv_split_kernel": "attn_bwd_dkdv",
    "attn_bwd_dq_tr_kernel": "attn_bwd_dq",
    "attn_bwd_dq_ds_kernel": "attn_bwd_dq_ds",
    "attn_delta_vec_kernel": "attn_delta",
}


def short(name: str, width: int = 84) -> str:
    name = name.replace("(anonymous namespace)::", "").replace("void ", "")
    return name if len(name) <= width else name[: width - 3] + "..."


def find(raw: str, sub: str, pattern: str) -> str | None:
    hits = glob.glob(os.path.join(raw, sub, "**", pattern), recursive=True)
    return max(hits, key=os.path.getsize) if hits else None


def kernel_stats(raw: str, sub: str, out_path: str, title: str, command: str, note: str, top: int = 24) -> bool:
    path = find(raw, sub, "*kernel_stats.csv")
    if not path:
        return False
    rows = list(csv.DictReader(open(path)))
    with open(out_path, "w") as f:
        f.write(f"# {title}\n\nCommand (from the repository root on one MI355X, after `export TMPDIR=/tmp`):\n\n    {command}\n\n")
        f.write(note + "\n\n| kernel | calls | avg us | min us | max us | % of GPU time |\n|---|---:|---:|---:|---:|---:|\n")
        for r in rows[:top]:
            f.write(f"| `{short(r['Name'])}` | {r['Calls']} | {float(r['AverageNs']) / 1e3:.1f} | {float(r['MinNs']) / 1e3:.1f} | "
                    f"{float(r['MaxNs']) / 1e3:.1f} | {r['Percentage']} |\n")
    return True


def counters(raw: str, sub: str) -> tuple[dict, dict]:
    """Per kernel name: {counter: mean value per dispatch}, and mean dispatch duration in ns."""
    path = find(raw, sub, "*counter_collection.csv")
    if not path:
        return {}, {}
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    dur = collections.defaultdict(dict)
    for r in csv.DictReader(open(path)):
        acc[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
        dur[r["Kernel_Name"]][r["Dispatch_Id"]] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
    mean = {k: {c: sum(v) / len(v) for c, v in cs.items()} for k, cs in acc.items()}
    return mean, {k: sum(v.values()) / len(v) for k, v in dur.items()}


def pick(table: dict, fragment: str):
    """The entry of the kernel whose name contains `fragment`, the head_dim 128 instance when there are several."""
    cands = [n for n in table if fragment in n]
    pref = [n for n in cands if "<128" in n]
    return table[(pref or cands)[0]] if cands else None


def hbm_traffic(raw: str, out_dir: str) -> bool:
    fe, _ = counters(raw, "fetch")
    wr, _ = counters(raw, "write")
    fc, _ = counters(raw, "fetch_cal")
    wc, _ = counters(raw, "write_cal")
    if not (fe and wr and fc and wc):
        return False
    cal_f = pick(fc, "scale_vec_kernel")["FETCH_SIZE"]
    cal_w = pick(wc, "scale_vec_kernel")["WRITE_SIZE"]
    kf, kw = 1048576.0 / cal_f, 1048576.0 / cal_w   # the calibration kernel reads and writes 1 GiB = 1048576 KiB
    B, H, S, D = (CFG2[k] for k in "BHSD")
    t = B * H * S * D * 2 / 1e6            # one bf16 tensor, MB
    stat = B * H * S * 4 / 1e6             # one fp32 row statistic, MB
    ds = B * H * S * S / 2 * 2 / 1e6       # handed-over dS: 2 bytes per visible (query, key) pair
    alg = {"attn_fwd_dma_kernel": (3 * t, t + stat), "attn_bwd_dkdv_split_kernel": (4 * t + 2 * stat, 2 * t),
           # the recomputing dQ kernel also reads O and writes the two row statistics (delta, LSE in base 2)
           "attn_bwd_dq_tr_kernel": (5 * t + stat, t + 2 * stat), "attn_bwd_dq_ds_kernel": (t + ds, t), "attn_delta_vec_kernel": (2 * t, stat)}
    rec = {}
    with open(os.path.join(out_dir, "attn_cfg2_hbm_traffic.md"), "w") as f:
        f.write("# HBM traffic of the attention kernels, causal B=4 H=16 S=4096 D=128 bf16 (rocprofv3 --pmc)\n\n")
        f.write("Commands (each its own run, from the repository root on one MI355X after `export TMPDIR=/tmp`):\n\n")
        for c, a in (("FETCH_SIZE", "--steps 3 --warmup 1 --skip-cpu --skip-extra"), ("WRITE_SIZE", "--steps 3 --warmup 1 --skip-cpu --skip-extra"),
                     ("FETCH_SIZE", "--calibrate-traffic"), ("WRITE_SIZE", "--calibrate-traffic")):
            f.write(f"    rocprofv3 --pmc {c} -f csv -d <raw dir> -- python3 bench.py {a}\n")
        f.write("    python -m maltos_amd.profile_summary <raw dir>\n")
        f.write("\nCalibration: `bench.py --calibrate-traffic` launches `scale_vec_kernel` over 1 GiB of fp32 in place (1 GiB read, 1 GiB "
                f"written).\nThe counters read FETCH_SIZE = {cal_f:.0f} KiB and WRITE_SIZE = {cal_w:.0f} KiB per launch for it, so the scale "
                f"factors are\n{kf:.3f} (fetch) and {kw:.3f} (write).\n\n")
        f.write("| kernel | FETCH_SIZE KiB/launch | WRITE_SIZE KiB/launch | HBM read MB (scaled) | HBM written MB (scaled) | total MB | "
                "algorithmic read MB | algorithmic written MB | total / algorithmic |\n|---|---:|---:|---:|---:|---:|---:|---:|---:|\n")
        for key, (ar, aw) in alg.items():
            fk, wk = pick(fe, key), pick(wr, key)
            if fk is None or wk is None:
                continue
            rd, wt = fk["FETCH_SIZE"] * kf * 1024 / 1e6, wk["WRITE_SIZE"] * kw * 1024 / 1e6
            rec[KERNELS[key]] = {"kernel": key, "hbm_bytes_per_launch": (rd + wt) * 1e6, "read_bytes": rd * 1e6, "written_bytes": wt * 1e6,
                                 "algorithmic_bytes": (ar + aw) * 1e6}
            f.write(f"| `{key}` | {fk['FETCH_SIZE']:.0f} | {wk['WRITE_SIZE']:.0f} | {rd:.0f} | {wt:.0f} | {rd + wt:.0f} | {ar:.0f} | {aw:.0f} | "
                    f"{(rd + wt) / (ar + aw):.2f} |\n")
        f.write("\nAlgorithmic = every operand read once and every result written once.  The excess reads are K/V (forward, dQ) and Q/dO\n"
                "(dK/dV) tiles fetched again by the workgroups that share a head after they fell out of the 4 MiB per-XCD L2.  All of these\n"
                "kernels stay far from the 8 TB/s HBM roof: they are bound by the matrix and vector pipelines.\n")
    with open(os.path.join(out_dir, "attn_cfg2_hbm_traffic.json"), "w") as f:
        json.dump({"workload": "causal attention fwd+bwd B=4 H=16 S=4096 D=128 bf16", "fetch_scale": kf, "write_scale": kw, "kernels": rec}, f, indent=1)
        f.write("\n")
    return True


def mfma_util(raw: str, out_dir: str) -> bool:
    a, dur_a = counters(raw, "pmc_a")
    b, _ = counters(raw, "pmc_b")
    if not a:
        return False
    B, H, S, D = (CFG2[k] for k in "BHSD")
    unit = 2.0 * B * H * S * S * D / 2.0   # flop of one GEMM of the causal problem
    executed = {"attn_fwd_dma_kernel": 2, "attn_bwd_dkdv_split_kernel": 4, "attn_bwd_dq_tr_kernel": 3, "attn_bwd_dq_ds_kernel": 1}
    with open(os.path.join(out_dir, "attn_cfg2_mfma_util.md"), "w") as f:
        f.write("# Matrix-pipe utilisation of the attention kernels, causal B=4 H=16 S=4096 D=128 bf16 (rocprofv3 --pmc)\n\n")
        f.write("Commands (each its own run, from the repository root on one MI355X after `export TMPDIR=/tmp`):\n\n")
        f.write("    rocprofv3 --pmc SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_INSTS_LDS "
                "SQ_LDS_BANK_CONFLICT SQ_WAIT_INST_LDS -f csv -d <raw dir>/pmc_a -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra\n")
        f.write("    rocprofv3 --pmc SQ_WAVE_CYCLES SQ_ACTIVE_INST_ANY SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS SQ_ACTIVE_INST_SCA "
                "SQ_INSTS_SALU -f csv -d <raw dir>/pmc_b -- python3 bench.py --steps 3 --warmup 1 --skip-cpu --skip-extra\n")
        f.write("    python -m maltos_amd.profile_summary <raw dir>\n\n")
        f.write("Per dispatch, mean over the dispatches of the run.  `SQ_VALU_MFMA_BUSY_CYCLES` counts matrix-pipe busy cycles summed over\n"
                "the 1024 SIMDs; `SQ_BUSY_CU_CYCLES` counts busy cycles summed over the 256 CUs, so the matrix pipes were busy for\n"
                "MFMA_BUSY / (4 x BUSY_CU) of the kernel's cycles.  `SQ_ACTIVE_INST_VALU`, `SQ_WAVE_CYCLES`, `SQ_ACTIVE_INST_*` and `SQ_WAIT_*`\n"
                "count in units of four cycles per wavefront.  Clock = BUSY_CU / 256 / duration (the chip lowers it under matrix load).\n\n")
        f.write("| kernel | us | clock GHz | MFMA pipe busy | MFMA rate TFLOP/s (executed) | fraction of 2.5 PFLOP/s | VALU port busy | "
                "VALU instr per MFMA | LDS instr per MFMA | LDS bank-conflict / LDS wait (M quad-cycles) |\n|---|---:|---:|---:|---:|---:|---:|---:|---:|---:|\n")
        for key, units in executed.items():
            ca, us = pick(a, key), pick(dur_a, key)
            if ca is None:
                continue
            us = us / 1e3
            busy_cu = ca["SQ_BUSY_CU_CYCLES"]
            clock = busy_cu / 256 / (us * 1e-6) / 1e9
            duty = ca["SQ_VALU_MFMA_BUSY_CYCLES"] / (4 * busy_cu)
            rate = units * unit / (us * 1e-6) / 1e12
            port = 4 * ca["SQ_ACTIVE_INST_VALU"] / (4 * busy_cu)
            f.write(f"| `{key}` | {us:.1f} | {clock:.2f} | {100 * duty:.1f} % | {rate:.0f} | {100 * rate / 2500:.1f} % | {100 * port:.1f} % | "
                    f"{(ca['SQ_INSTS_VALU'] - ca['SQ_INSTS_MFMA']) / ca['SQ_INSTS_MFMA']:.2f} | {ca['SQ_INSTS_LDS'] / ca['SQ_INSTS_MFMA']:.2f} | "
                    f"{ca['SQ_LDS_BANK_CONFLICT'] / 1e6:.1f} / {ca['SQ_WAIT_INST_LDS'] / 1e6:.1f} |\n")
        if b:
            f.write("\nWhere a wavefront's time goes (fractions of `SQ_WAVE_CYCLES`): an instruction of it executing, waiting at an `s_waitcnt`,\n"
                    "waiting for an instruction to issue (matrix pipe or issue port taken, dependency):\n\n")
            f.write("| kernel | executing | of which LDS | of which scalar | waiting at s_waitcnt | waiting to issue | scalar instr per MFMA |\n"
                    "|---|---:|---:|---:|---:|---:|---:|\n")
            for key in executed:
                cb, ca = pick(b, key), pick(a, key)
                if cb is None:
                    continue
                w = cb["SQ_WAVE_CYCLES"]
                f.write(f"| `{key}` | {100 * cb['SQ_ACTIVE_INST_ANY'] / w:.1f} % | {100 * cb['SQ_ACTIVE_INST_LDS'] / w:.1f} % | "
                        f"{100 * cb['SQ_ACTIVE_INST_SCA'] / w:.1f} % | {100 * cb['SQ_WAIT_ANY'] / w:.1f} % | {100 * cb['SQ_WAIT_INST_ANY'] / w:.1f} % | "
                        f"{cb['SQ_INSTS_SALU'] / ca['SQ_INSTS_MFMA']:.2f} |\n")
        f.write("\nA pure `v_mfma_f32_32x32x16_bf16` loop on all 256 CUs sustains 2.4-2.5 PFLOP/s on operands of zeros or ones and 1.7-1.8 PFLOP/s on\n"
                "normally distributed operands (the clock drops from 2.4 to about 1.7 GHz: the matrix cores' power depends on the data),\n"
                "and hipBLASLt's 8192^3 bf16 GEMM reaches 1.36 PFLOP/s at 1.92 GHz on this chip; the attention inputs of this workload are\n"
                "normally distributed.\n")
    return True


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("raw")
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "profiles"))
    args = ap.parse_args()
    os.makedirs(args.out, exist_ok=True)
    done = []
    if kernel_stats(args.raw, "stats", os.path.join(args.out, "attn_cfg2_kernel_stats.md"),
                    "rocprofv3 kernel statistics of the headline step (causal attention fwd+bwd, B=4 H=16 S=4096 D=128 bf16)",
                    "rocprofv3 --kernel-trace --stats -f csv -d <raw dir>/stats -- python3 bench.py --steps 40 --warmup 10 --skip-cpu --skip-extra",
                    "Source: `*_kernel_stats.csv` of that run.  `attn_fwd_dma_kernel` = `attn_fwd`, `attn_bwd_dkdv_split_kernel` = `attn_bwd_dkdv`,\n"
                    "`attn_bwd_dq_tr_kernel` = `attn_bwd_dq` (the recomputing dQ kernel of the default backward; it runs first and also\n"
                    "forms the row statistics delta and LSE in base 2, so no separate delta pass appears) in bench.py's `kernels` block,\n"
                    "whose HIP-event averages these agree with.", top=8):
        done.append("attn_cfg2_kernel_stats.md")
    if kernel_stats(args.raw, "llama", os.path.join(args.out, "llama50m_step_kernel_stats.md"),
                    "rocprofv3 kernel statistics of the LLaMA-50M bf16 train step (B=8, S=2048; configuration 5)",
                    "rocprofv3 --kernel-trace --stats -f csv -d <raw dir>/llama -- python3 bench.py --steps 10 --warmup 3 --skip-cpu --only llama50m_train_step",
                    "Source: `*_kernel_stats.csv` of that run (it also contains the headline attention step, whose `<128, 1>` kernels appear\n"
                    "with few calls).  The `<64, 1>` attention kernels, the layer / loss / optimizer kernels are the hand-written path;\n"
                    "`Cijk_*` are hipBLASLt GEMMs of the linear layers (library code).", top=30):
        done.append("llama50m_step_kernel_stats.md")
    if hbm_traffic(args.raw, args.out):
        done += ["attn_cfg2_hbm_traffic.md", "attn_cfg2_hbm_traffic.json"]
    if mfma_util(args.raw, args.out):
        done.append("attn_cfg2_mfma_util.md")
    print("wrote: " + (", ".join(done) if done else "nothing (no raw runs found)"))
    return 0 if done else 1


if __name__ == "__main__":
    sys.exit(main())
