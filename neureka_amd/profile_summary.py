"""Turns the CSV output of four ``rocprofv3`` runs of ``bench.py`` into the tables under ``profiles/``.

    python3 -m neureka_amd.profile_summary --trace DIR --fetch DIR --write DIR --sq DIR --out profiles

``DIR`` are the ``-d`` directories of a ``--kernel-trace --stats`` run and of one ``--pmc`` run per counter group (FETCH_SIZE;
WRITE_SIZE; the SQ group), all of the same ``bench.py`` command with ``--calibrate`` (which adds one plain 1 GiB copy to
the run: the scale of the two traffic counters is what they read for it).  Written: one Markdown table per kernel family
(text below a ``## Notes`` line of an existing file is kept), and ``rows_binary_lean_kernel_broadcast_c2.json``, the
counter-measured traffic of the headline kernel that ``bench.py`` reports as ``roofline.traffic``.

A (kernel, grid) pair is summarised over its *settled* dispatches: the later half in launch order where the pair has 20
dispatches or more (the first launches of a process and of each workload run at a lower clock), all of them otherwise.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import hashlib
import json
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
HEADLINE_KERNEL = "rows_binary_lean_kernel<float, 4, 2, 0, true>"
HEADLINE_PATH = "rows_vec_binary_lean"
HEADLINE_SOURCES = ("nk_eltwise.h", "nk_eltwise_family.inc", "nk_eltwise.hip", "nk_internal.h", "Makefile")
COPY_KERNEL, COPY_BYTES = "__amd_rocclr_copyBuffer", 1 << 30
FAMILIES = (      # file, title, pattern of kernel names
    ("rows_binary_lean_kernel_broadcast_c2.md",
     "rows_binary_lean_kernel -- broadcast add / multiply, f32 [1024,1,512] o [1,2048,512] -> [1024,2048,512] and its neighbours", r"rows_binary_lean"),
    ("elementwise_kernels_chain_c3.md",
     "rows_kernel, fused_kernel, strided and literal elementwise kernels -- tanh(sig(a)*b+c) on 2^26 elements, its parts, derivatives and views", r"^(rows_kernel|rows_binary_kernel|fused|strided|literal|perm|int_|tile_kernel|canon)"),
    ("matmul_mfma_kernels_c4.md",
     "matmul kernels -- [4096,4096] @ [4096,4096] (f32, f64), [65536,256] @ [256,256], 1024^3 to 4000^3 and the small-batch products", r"^matmul"),
    ("convolution_kernels_c1_c5.md",
     "conv2d_direct, conv2d_window, conv_chan_fwd_tiles, conv_chan_dx, conv_chan_dk -- [64,64] x [3,3], large images, [64,256,256] x [64,5,5]", r"^conv"),
    ("other_kernels_backward_reductions_f64_int.md",
     "reducing broadcast backward, whole-tensor reductions, fills", r"^(broadcast_bwd|tile_reduce|tail_reduce|tile_index|tail_index|tile_dot|fill|__amd)"),
    ("hardware_counters_all_bench_kernels.md", "every kernel of a bench.py run", r"."),
)


def kernel_sources_digest() -> str:
    """sha256 over the sources the headline kernel is built from (and the flags it is built with)."""
    h = hashlib.sha256()
    for name in HEADLINE_SOURCES:
        with open(os.path.join(_HERE, "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    return h.hexdigest()


def short(name: str) -> str:
    return re.sub(r"\(.*$", "", name).replace("void ", "").replace("nk::", "").strip()


def one_file(directory: str, suffix: str) -> str:
    found = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not found:
        raise SystemExit(f"no *{suffix} under {directory}")
    return found[-1]


def settled(values):
    return values[len(values) // 2:] if len(values) >= 20 else values


def mean(values):
    return sum(values) / len(values) if values else None


def read_trace(directory):
    """(kernel, blocks, class) -> durations in launch order; class "long" separates a second workload of one (kernel,
    grid) pair whose launches take more than four times as long (the reductions run over 2^26 and 2^30 elements)."""
    rows = sorted(csv.DictReader(open(one_file(directory, "kernel_trace.csv"))), key=lambda r: int(r["Start_Timestamp"]))
    raw = collections.OrderedDict()
    for r in rows:
        blocks = 1
        for ax in "XYZ":
            blocks *= int(r["Grid_Size_" + ax]) // max(1, int(r["Workgroup_Size_" + ax]))
        raw.setdefault((short(r["Kernel_Name"]), blocks), []).append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    out, split_keys = collections.OrderedDict(), set()
    for key, durs in raw.items():
        split = max(durs) > 6 * min(durs)
        if split:
            split_keys.add(key)
        for d in durs:
            out.setdefault(key + ("long" if split and d > 4 * min(durs) else "",), []).append(d)
    return out, split_keys


def read_counters(directory, split_keys, into, meta):
    per = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in csv.DictReader(open(one_file(directory, "counter_collection.csv"))):
        key = (short(r["Kernel_Name"]), int(r["Grid_Size"]) // max(1, int(r["Workgroup_Size"])))
        per[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
        for c in ("", "long"):
            meta[key + (c,)] = (r["VGPR_Count"], r["Accum_VGPR_Count"], r["LDS_Block_Size"])
    for key, by_name in per.items():
        for name, vals in by_name.items():
            pos = [v for v in vals if v > 0]
            lo = min(pos) if pos else 0.0
            two = key in split_keys and lo > 0 and max(pos) > 6 * lo       # told by the counter's own value
            if key in split_keys and name == "SQ_WAVES":
                continue
            for v in vals:
                into[key + ("long" if two and v > 4 * lo else "",)][name].append(v)


def num(x, fmt="{:,.0f}"):
    return "" if x is None else fmt.format(x).replace(",", " ")


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--trace", required=True); ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True); ap.add_argument("--sq", required=True)
    ap.add_argument("--out", required=True)
    ap.add_argument("--rows-json", help="also write every row as JSON to this file")
    ap.add_argument("--bench-args", default="--no-cpu --no-ops --calibrate --steps 20 --warmup 5")
    ap.add_argument("--sq-counters", default="SQ_INSTS_VALU SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES SQ_WAVES SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS GRBM_GUI_ACTIVE")
    args = ap.parse_args()

    trace, split_keys = read_trace(args.trace)
    ctr = collections.defaultdict(lambda: collections.defaultdict(list))
    meta = {}
    for d in (args.fetch, args.write, args.sq):
        read_counters(d, split_keys, ctr, meta)

    copy_key = next((k for k in ctr if k[0] == COPY_KERNEL and ctr[k].get("FETCH_SIZE") and ctr[k].get("WRITE_SIZE")), None)
    if copy_key is None:
        raise SystemExit("the runs hold no plain copy to scale FETCH_SIZE / WRITE_SIZE by (bench.py --calibrate)")
    copy_fetch, copy_write = mean(ctr[copy_key]["FETCH_SIZE"]), mean(ctr[copy_key]["WRITE_SIZE"])
    fetch_scale, write_scale = COPY_BYTES / (copy_fetch * 1024), COPY_BYTES / (copy_write * 1024)

    rows = []
    for key, durs in trace.items():
        c = {name: settled(vals) for name, vals in ctr.get(key, {}).items()}
        s = settled(durs)
        f, w = mean(c.get("FETCH_SIZE", [])), mean(c.get("WRITE_SIZE", []))
        rows.append(dict(kernel=key[0] + (" (the larger workload)" if key[2] else ""), blocks=key[1], calls=len(durs), settled_calls=len(s),
                         avg=mean(s), median=sorted(s)[len(s) // 2], mn=min(s), mx=max(s), avg_all=mean(durs), fetch=f, write=w,
                         hbm=None if f is None or w is None else (fetch_scale * f + write_scale * w) * 1024,
                         valu=mean(c.get("SQ_INSTS_VALU", [])), lds=mean(c.get("SQ_INSTS_LDS", [])), mfma=mean(c.get("SQ_INSTS_MFMA", [])),
                         mfma_busy=mean(c.get("SQ_VALU_MFMA_BUSY_CYCLES", [])), gui=mean(c.get("GRBM_GUI_ACTIVE", [])),
                         conflict=mean(c.get("SQ_LDS_BANK_CONFLICT", [])), waves=mean(c.get("SQ_WAVES", [])), regs=meta.get(key)))

    head = f"""MI355X (gfx950, 256 CUs, 1 024 SIMDs), one GPU.  Four runs of one command from the repository root after `cd /tmp && export TMPDIR=/tmp`
(kernel trace; then one counter group per run), and the summary of their CSV files:

    rocprofv3 --kernel-trace --stats --output-format csv -d {args.trace} -o all -- python3 bench.py {args.bench_args}
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d {args.fetch} -o fetch -- python3 bench.py {args.bench_args}
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d {args.write} -o write -- python3 bench.py {args.bench_args}
    rocprofv3 --pmc {args.sq_counters} --output-format csv -d {args.sq} -o sq -- python3 bench.py {args.bench_args}
    python3 -m neureka_amd.profile_summary --trace {args.trace} --fetch {args.fetch} --write {args.write} --sq {args.sq} --out {args.out}

Per (kernel, grid): "Calls" = every dispatch of the trace; the durations are of the *settled* dispatches, the later half in launch order where there are
20 or more (the first launches of a process and of each workload run at a lower clock), "Avg ns, all" is over every dispatch for comparison.  FETCH_SIZE and
WRITE_SIZE are KiB per dispatch as rocprofv3 reports them, averaged over the settled dispatches of the counter runs; **HBM bytes = ({fetch_scale:.3f} x FETCH_SIZE +
{write_scale:.3f} x WRITE_SIZE) x 1024**, the factors that make a plain copy of 1 GiB read 1 GiB and write 1 GiB (`{COPY_KERNEL}` in the same runs: FETCH_SIZE
{num(copy_fetch, '{:,.1f}')}, WRITE_SIZE {num(copy_write, '{:,.1f}')}).  SQ counters are sums over the chip per dispatch.  "VGPRs / LDS B" are VGPR_Count (+ Accum_VGPR_Count) and LDS_Block_Size.
"""
    cols = ("| Kernel | Blocks | Calls | Avg ns | Median ns | Min ns | Max ns | Avg ns, all | FETCH KiB | WRITE KiB | HBM bytes | SQ_INSTS_VALU | SQ_INSTS_MFMA | SQ_INSTS_LDS | VGPRs / LDS B |\n"
            "|---|---|---|---|---|---|---|---|---|---|---|---|---|---|---|\n")
    os.makedirs(args.out, exist_ok=True)
    for fname, title, pat in FAMILIES:
        body = ""
        for r in rows:
            if not re.search(pat, r["kernel"]):
                continue
            regs = "" if not r["regs"] else f"{r['regs'][0]}{' + ' + r['regs'][1] + ' acc' if r['regs'][1] != '0' else ''} / {r['regs'][2]}"
            body += (f"| `{r['kernel']}` | {num(r['blocks'])} | {r['calls']} | {num(r['avg'])} | {num(r['median'])} | {num(r['mn'])} | {num(r['mx'])} | {num(r['avg_all'])} | "
                     f"{num(r['fetch'], '{:,.1f}')} | {num(r['write'], '{:,.1f}')} | {num(r['hbm'])} | {num(r['valu'])} | {num(r['mfma'])} | {num(r['lds'])} | {regs} |\n")
        path = os.path.join(args.out, fname)
        notes = ""
        if os.path.exists(path):
            old = open(path).read()
            at = old.find("\n## Notes")
            notes = old[at:] if at >= 0 else ""
        with open(path, "w") as f:
            f.write(f"# {title}\n\n{head}\n## Kernel time and counters\n\n{cols}{body}{notes if notes else chr(10) + '## Notes' + chr(10)}")

    hl = next((r for r in rows if r["kernel"] == HEADLINE_KERNEL and r["hbm"] is not None), None)
    if hl is None:
        raise SystemExit(f"the runs hold no {HEADLINE_KERNEL} with both traffic counters")
    with open(os.path.join(args.out, "rows_binary_lean_kernel_broadcast_c2.json"), "w") as f:
        json.dump({"kernel": "nk::" + HEADLINE_KERNEL, "path": HEADLINE_PATH, "traffic_bytes": round(hl["hbm"]),
                   "fetch_KiB": round(hl["fetch"], 1), "write_KiB": round(hl["write"], 1), "fetch_scale": round(fetch_scale, 4), "write_scale": round(write_scale, 4),
                   "dispatches": hl["settled_calls"], "settled_avg_ns": round(hl["avg"]), "settled_median_ns": hl["median"], "avg_ns_all_dispatches": round(hl["avg_all"]),
                   "sources_sha256": kernel_sources_digest(), "sources": list(HEADLINE_SOURCES),
                   "made_by": f"python3 -m neureka_amd.profile_summary --trace {args.trace} --fetch {args.fetch} --write {args.write} --sq {args.sq} --out {args.out}"},
                  f, indent=1)
        f.write("\n")
    if args.rows_json:
        with open(args.rows_json, "w") as f:
            json.dump(rows, f, indent=1)


if __name__ == "__main__":
    main()
