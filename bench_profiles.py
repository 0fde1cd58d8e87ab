#!/usr/bin/env python3
"""rocprofv3 runs behind the summaries under profiles/, and the summaries themselves.

  python bench_profiles.py run [--sets cfg3,cfg5,prod,nodct,bench,matrix] [--phases encode,aggregate,...]
      on a box with an MI355X: for every (set, phase) a kernel trace of `bench.py --profile <phase>` (50 timed
      launches after the settle phase and 10 warm-up ones), and one run each for the FETCH_SIZE, WRITE_SIZE and
      (encode, aggregate) SQ_* counters.  Raw CSVs go to gpurun_out/prof/<set>_<phase>_<what>/, trimmed to this
      library's rows.  Every profiler run is a child process with a time limit of its own; the first failure
      ends the script.
  python bench_profiles.py summarise [--out profiles]
      turns those CSVs into profiles/*.md and profiles/traffic.json (the HBM bytes per launch that bench.py
      quotes as `roofline.traffic`).

Counters are scaled by what the same counter reads for the library's 1 GiB calibration copy (set cfg3, phase
copy): FETCH_SIZE and WRITE_SIZE are reported in units that the copy pins down.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
RAW = os.path.join(ROOT, "gpurun_out", "prof")


def traffic_key(workload, k, use_dct, peers, kernel):
    """Key of a launch in profiles/traffic.json (bench.py looks its own launches up with it)."""
    return f"{workload}/k{k}/{'dct' if use_dct else 'nodct'}/{peers}peers/{kernel}"


SQ = ("SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS "
      "SQ_INSTS_VALU SQ_INSTS_LDS").split()
PRE = "cd /tmp && export TMPDIR=/tmp && cd <repo> && "

SETS = {
    "cfg3": dict(args=[], workload="cfg3_llama1b", chunks=294144, k=32, P=15, dct=True, name="cfg3_llama1b",
                 what="the 1B gradient set (294 144 chunks of 64x64, k = 32)",
                 phases=["copy", "linfill", "encode", "read", "aggregate", "calib", "fill", "miner", "outer"]),
    "cfg5": dict(args=["--workload", "cfg5_72b_block"], workload="cfg5_72b_block", chunks=214272, k=64, P=15, dct=True, name="cfg5_72b_block",
                 what="the 72B-class block (214 272 chunks, k = 64)",
                 phases=["encode", "read", "aggregate", "calib", "fill"]),
    "prod": dict(args=["--topk", "64", "--peers", "20", "--no-dct"], workload="cfg3_llama1b", chunks=294144, k=64, P=20, dct=False,
                 name="cfg3_llama1b_templar_hparams",
                 what="the 1B gradient set at templar's own settings (hparams.json: top-k 64, use_dct false, 20 peers)",
                 phases=["encode", "read", "aggregate", "calib", "fill"]),
    # the same launches with the transform taken out: what any faster transform could gain at most
    "nodct": dict(args=["--no-dct"], workload="cfg3_llama1b", chunks=294144, k=32, P=15, dct=False, name="cfg3_llama1b_no_transform",
                  what="the 1B gradient set, k = 32, chunks not transformed", phases=["encode", "aggregate"]),
}
COUNTED = {"copy", "encode", "aggregate", "calib", "outer"}   # phases whose HBM traffic is counted
WITH_SQ = {"encode", "aggregate"}
# the measurement build with half of the forward transform on the matrix cores (`TPLR_BUILD_MATRIX_VARIANT=1` makes
# __graft_entry__.build() write it beside the product library): the set `matrix` profiles its encode launch
MATRIX_LIB = os.path.join(ROOT, "templar_amd", "libtplr_hip_matrix_variant.so")
MFMA = "SQ_INSTS_VALU_MFMA_MOPS_F32 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES GRBM_GUI_ACTIVE".split()


# ------------------------------------------------------------------------------------------------ run
def _trim(directory):
    for f in glob.glob(os.path.join(directory, "**", "*agent_info*"), recursive=True):
        os.remove(f)
    for pat in ("*kernel_trace.csv", "*counter_collection.csv"):
        for f in glob.glob(os.path.join(directory, "**", pat), recursive=True):
            with open(f) as fh:
                lines = fh.readlines()
            keep = [ln for ln in lines[1:] if "tplr" in ln or "FillFunctor<float>" in ln]
            if pat == "*kernel_trace.csv":  # the last launches of every kernel are the timed ones: 120 rows of each
                col = lines[0].strip().split(",").index('"Kernel_Name"')
                seen = collections.Counter()
                last = []
                for ln in reversed(keep):
                    name = next(csv.reader([ln]))[col]
                    seen[name] += 1
                    if seen[name] <= 120:
                        last.append(ln)
                keep = last[::-1]
            with open(f, "w") as fh:
                fh.writelines([lines[0]] + keep)


def _profile(tag, what, prof_args, bench_args, limit, lib=None):
    out = os.path.join(RAW, f"{tag}_{what}")
    cmd = ["rocprofv3", *prof_args, "--output-format", "csv", "-d", out, "-o", "p", "--", "python3",
           os.path.join(ROOT, "bench.py"), *bench_args]
    print("==", tag, what, flush=True)
    env = dict(os.environ, TMPDIR="/tmp")
    if lib:
        env["TPLR_HIP_LIB"] = lib
    with open(out + ".log", "w") as log:
        try:
            rc = subprocess.run(cmd, cwd="/tmp", env=env, stdout=log, stderr=subprocess.STDOUT, timeout=limit).returncode
        except subprocess.TimeoutExpired:
            rc = 124
    if rc != 0:
        print(f"profiler run failed ({rc}): {' '.join(cmd)}; see {out}.log", file=sys.stderr)
        sys.exit(3)
    _trim(out)


def run(sets, phases):
    os.makedirs(RAW, exist_ok=True)
    for tag in sets:
        if tag == "bench":  # the default benchmark run as a whole: every kernel of the library once
            _profile("bench_default", "kt", ["--kernel-trace", "--stats"], ["--no-cpu-baseline"], 400)
            continue
        if tag == "matrix":
            if not os.path.exists(MATRIX_LIB):
                sys.exit(f"{MATRIX_LIB} is not built: TPLR_BUILD_MATRIX_VARIANT=1 python -c 'import __graft_entry__ as g; g.build()'")
            base = ["--profile", "encode"]
            _profile("matrix_encode", "kt", ["--kernel-trace", "--stats"], base + ["--steps", "50", "--warmup", "10"], 300, MATRIX_LIB)
            for what, counters in (("SQ", SQ), ("MFMA", MFMA)):
                _profile("matrix_encode", what, ["--kernel-include-regex", "tplr", "--pmc", *counters],
                         base + ["--steps", "3", "--warmup", "1"], 240, MATRIX_LIB)
            _profile("cfg3_encode", "MFMA", ["--kernel-include-regex", "tplr", "--pmc", *MFMA], base + ["--steps", "3", "--warmup", "1"], 240)
            continue
        S = SETS[tag]
        for ph in S["phases"]:
            if phases and ph not in phases:
                continue
            base = ["--profile", ph, *S["args"]]
            _profile(f"{tag}_{ph}", "kt", ["--kernel-trace", "--stats"], base + ["--steps", "50", "--warmup", "10"], 300)
            if ph in COUNTED and tag != "nodct":
                for c in ("FETCH_SIZE", "WRITE_SIZE"):
                    _profile(f"{tag}_{ph}", c, ["--kernel-include-regex", "tplr", "--pmc", c],
                             base + ["--steps", "3", "--warmup", "1"], 240)
            if ph in WITH_SQ and tag != "nodct":
                _profile(f"{tag}_{ph}", "SQ", ["--kernel-include-regex", "tplr", "--pmc", *SQ],
                         base + ["--steps", "3", "--warmup", "1"], 240)


# ------------------------------------------------------------------------------------------------ summarise
def _csv(tag, what, pattern):
    found = glob.glob(os.path.join(RAW, f"{tag}_{what}", "**", pattern), recursive=True)
    return found[0] if found else None


def _have(tag, what="kt"):
    return _csv(tag, what, "*kernel_stats.csv" if what == "kt" else "*counter_collection.csv") is not None


def _short(name):
    return name.replace("void ", "").split("(")[0]


def _stats_table(tag, also=None):
    rows = [r for r in csv.DictReader(open(_csv(tag, "kt", "*kernel_stats.csv"))) if "tplr" in r["Name"] or (also and also in r["Name"])]
    out = ["| kernel | calls | total ms | avg us | min us | max us |", "|---|---|---|---|---|---|"]
    for r in rows:
        out.append(f"| `{_short(r['Name'])[:110]}` | {r['Calls']} | {int(r['TotalDurationNs']) / 1e6:.3f} | "
                   f"{float(r['AverageNs']) / 1e3:.1f} | {int(r['MinNs']) / 1e3:.1f} | {int(r['MaxNs']) / 1e3:.1f} |")
    return "\n".join(out)


def _trace(tag, kern):
    rows = [r for r in csv.DictReader(open(_csv(tag, "kt", "*kernel_trace.csv"))) if kern in r["Kernel_Name"]]
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    dur = [(int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3 for r in rows]
    return rows, dur


def _pmc(tag, counter, kern):
    f = _csv(tag, counter, "*counter_collection.csv")
    v = [float(r["Counter_Value"]) for r in csv.DictReader(open(f)) if kern in r["Kernel_Name"] and r["Counter_Name"] == counter]
    return sum(v) / len(v), len(v)


def _sq(tag, kern, chunks, waves, note):
    acc = collections.defaultdict(list)
    for r in csv.DictReader(open(_csv(tag, "SQ", "*counter_collection.csv"))):
        if kern in r["Kernel_Name"]:
            acc[r["Counter_Name"]].append(float(r["Counter_Value"]))
    m = {k: sum(v) / len(v) for k, v in acc.items()}
    out = ["| counter | mean per dispatch |", "|---|---|"] + [f"| {n} | {m[n]:,.0f} |" for n in SQ]
    out += ["", f"Per chunk: {m['SQ_INSTS_VALU'] / chunks:.0f} vector-ALU instructions, {m['SQ_INSTS_LDS'] / chunks:.0f} LDS instructions.",
            f"Vector ALU active {m['SQ_ACTIVE_INST_VALU'] / m['SQ_WAVE_CYCLES'] * 100:.1f} % of a wave's resident time with up to "
            f"{waves} waves on a SIMD; waves wait on counters {m['SQ_WAIT_ANY'] / m['SQ_WAVE_CYCLES'] * 100:.0f} % and for an issue "
            f"slot {m['SQ_WAIT_INST_ANY'] / m['SQ_WAVE_CYCLES'] * 100:.0f} % of their time; LDS instructions are active "
            f"{m['SQ_ACTIVE_INST_LDS'] / m['SQ_WAVE_CYCLES'] * 100:.1f} %.  {note}"]
    return "\n".join(out)


def _cmd(tag, ph, what, args):
    a = (" " + " ".join(args)) if args else ""
    if what == "kt":
        return (f"    {PRE}rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof/{tag}_{ph}_kt -o p -- "
                f"python3 bench.py --profile {ph}{a} --steps 50 --warmup 10")
    counters = " ".join(SQ) if what == "SQ" else what
    return (f"    {PRE}rocprofv3 --kernel-include-regex tplr --pmc {counters} --output-format csv -d "
            f"gpurun_out/prof/{tag}_{ph}_{what} -o p -- python3 bench.py --profile {ph}{a} --steps 3 --warmup 1")


def _geometry(r0):
    return (f"grid {r0['Grid_Size_X']} threads, workgroup {r0['Workgroup_Size_X']}, {r0['VGPR_Count']} VGPRs + "
            f"{r0['Accum_VGPR_Count']} AGPRs as the profiler counts them (half of the allocation: the code object's "
            f"`.vgpr_count`, rounded up to a multiple of 8, is {2 * int(r0['VGPR_Count'])} registers per lane), "
            f"{r0['SGPR_Count']} SGPRs, LDS {r0['LDS_Block_Size']} B, scratch {r0['Scratch_Size']} B")


def summarise(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    traffic = {}
    note = ("every run goes through bench.py's settle phase (0.25 s of the same launches) and 10 warm-up launches first; "
            "the figures below are those of the last 50 launches of the trace, the timed ones")

    def write(name, text):
        with open(os.path.join(out_dir, name), "w") as fh:
            fh.write(text)
        print("wrote", name)

    # ---- counter scale from the calibration copy
    sf = sw = None
    if _have("cfg3_copy", "FETCH_SIZE") and _have("cfg3_copy", "WRITE_SIZE"):
        cf, _ = _pmc("cfg3_copy", "FETCH_SIZE", "k_calib_copy")
        cw, _ = _pmc("cfg3_copy", "WRITE_SIZE", "k_calib_copy")
        sf, sw = (1 << 20) / cf, (1 << 20) / cw
        _, dur = _trace("cfg3_copy", "k_calib_copy")
        t50 = dur[-50:]
        us = sum(t50) / len(t50)
        write("k_calib_copy_1GiB.md", f"""# k_calib_copy, 1 GiB device-to-device copy: scale of the HBM traffic counters

Commands (one counter per run; {note}):

{_cmd('cfg3', 'copy', 'FETCH_SIZE', [])}
{_cmd('cfg3', 'copy', 'WRITE_SIZE', [])}
{_cmd('cfg3', 'copy', 'kt', [])}

The kernel reads 1 GiB = 1 048 576 KiB and writes the same amount.

| counter | mean per dispatch | true KiB | scale factor (true / reported) |
|---|---|---|---|
| FETCH_SIZE | {cf:.1f} | 1048576 | {sf:.4f} |
| WRITE_SIZE | {cw:.1f} | 1048576 | {sw:.4f} |

Every FETCH_SIZE / WRITE_SIZE figure quoted for the codec kernels is the reported value times these factors.  The
copy itself takes {us:.1f} us on average over the 50 timed launches: {2 * (1 << 30) / us / 1e3:.0f} GB/s of traffic, half
of it each way.
""")
        traffic["counter_scale"] = {"FETCH_SIZE": sf, "WRITE_SIZE": sw, "source": "k_calib_copy_1GiB.md"}

    def counted(tag, kern):
        if sf is None or not (_have(tag, "FETCH_SIZE") and _have(tag, "WRITE_SIZE")):
            return None
        f, nf = _pmc(tag, "FETCH_SIZE", kern)
        w, nw = _pmc(tag, "WRITE_SIZE", kern)
        return f, nf, f * sf * 1024, w, nw, w * sw * 1024

    # ---- linear fills (cfg3 only)
    if _have("cfg3_linfill"):
        n_out = 294144 * 16384
        rows = []
        for kern, label in (("k_calib_fill<0>", "library fill, 16 B per lane, grid-stride over a linear range"),
                            ("k_calib_fill<2>", "library fill, 16 B per lane, every wave a contiguous span"),
                            ("FillFunctor<float>", "`torch.Tensor.fill_`: one 16 B store per thread, workgroups dispatched in address "
                                                   "order (torch cuts a tensor of more than 2 GiB into several launches)")):
            tr, dur = _trace("cfg3_linfill", kern)
            if not dur:
                continue
            if kern.startswith("k_calib_fill"):
                t = dur[-50:]
                us, lo, nbytes, per = sum(t) / len(t), min(t), n_out, "launch"
            else:  # launches of grid x 16 bytes each; the last 200 make 50 fills of the whole buffer
                t, g = dur[-200:], [int(r["Grid_Size_X"]) * 16 for r in tr[-200:]]
                us, lo, nbytes, per = sum(t) / len(t), min(t), sum(g) / len(g), f"launch of {sum(g) / len(g) / 1e6:.0f} MB"
            rows.append(f"| {label} | `{kern}` | {len(dur)} | {us:.1f} per {per} | {lo:.1f} | {nbytes / us / 1e3:.0f} | {nbytes / us / 1e3 / 80:.1f} % |")
        write("k_calib_fill_linear.md", f"""# Writes of the aggregate's output size (4 819 255 296 B) over a linear address range: the write ceiling of this memory system

{_cmd('cfg3', 'linfill', 'kt', [])}

({note}.)  `p_kernel_stats.csv`:

{_stats_table('cfg3_linfill', also='FillFunctor<float>')}

The timed launches of each kernel, `p_kernel_trace.csv`:

| what | kernel | launches in the trace | avg us | min us | GB/s written | of 8 TB/s |
|---|---|---|---|---|---|---|
{chr(10).join(rows)}

`torch.Tensor.copy_` between two such buffers is a device-to-device copy of the runtime, not a kernel: it does not
appear in a kernel trace; its event timing is `roofline_aggregate.attainable` in the bench line (4.3-4.5 TB/s of
traffic, half of it each way).

The aggregate's own store pattern (64 rows of 256 B per chunk, a tensor row apart) is in
k_decode_aggregate_cfg3_llama1b_15peers.md (`--profile fill`), beside the launch's loads and stores together.
""")

    for tag, S in SETS.items():
        n, k, Pn, a = S["chunks"], S["k"], S["P"], S["args"]
        two = "true" if k > 32 else "false"
        dct = "true" if S["dct"] else "false"
        # ---------------- encode
        if _have(f"{tag}_encode"):
            kern = f"k_encode_topk_pack<{two}, {dct}, false>"
            tr, dur = _trace(f"{tag}_encode", kern)
            t50 = dur[-50:]
            avg = sum(t50) / len(t50)
            alg_r, alg_w = n * 16384, n * 11 * k // 2
            alg = alg_r + alg_w
            text = f"""# {_short(tr[-1]['Kernel_Name'])}: {S['what']}, one persistent launch

## Kernel trace

{_cmd(tag, 'encode', 'kt', a)}

({note}.)  `p_kernel_stats.csv`, rows of this library's kernels:

{_stats_table(f'{tag}_encode')}

Launch geometry of the dominant kernel: {_geometry(tr[-1])}.

Durations of its last 60 launches in order (us), `p_kernel_trace.csv`:
{', '.join(f'{d:.0f}' for d in dur[-60:])}

The 50 timed launches average **{avg:.1f} us** (min {min(t50):.1f}); algorithmic bytes per launch
{alg:,} -> **{alg / avg / 1e3:.0f} GB/s = {alg / avg / 1e3 / 80:.1f} % of 8 TB/s**.
"""
            c = counted(f"{tag}_encode", kern)
            if c:
                f, nf, fb, w, nw, wb = c
                traffic[traffic_key(S["workload"], k, S["dct"], Pn, "encode")] = round(fb + wb)
                text += f"""
## HBM traffic (hardware counters)

{_cmd(tag, 'encode', 'FETCH_SIZE', a)}
{_cmd(tag, 'encode', 'WRITE_SIZE', a)}

| counter | mean per dispatch ({nf} dispatches) | scale (k_calib_copy_1GiB.md) | bytes per launch | algorithmic bytes | ratio |
|---|---|---|---|---|---|
| FETCH_SIZE | {f:.1f} | {sf:.4f} | {fb:,.0f} | {alg_r:,} | {fb / alg_r:.3f} |
| WRITE_SIZE | {w:.1f} | {sw:.4f} | {wb:,.0f} | {alg_w:,} | {wb / alg_w:.3f} |

Total HBM traffic per launch {fb + wb:,.0f} B = {(fb + wb) / alg:.3f} x the algorithmic bytes.
"""
            if _have(f"{tag}_encode", "SQ"):
                text += f"""
## Vector ALU and LDS activity (hardware counters)

{_cmd(tag, 'encode', 'SQ', a)}

{_sq(f'{tag}_encode', kern, n, 3, 'The kernel issues no matrix-core instruction: the 64-point transform is generated vector code.')}
"""
            if _have(f"{tag}_read"):
                _, rd = _trace(f"{tag}_read", "k_calib_encode")
                r50 = rd[-50:]
                ravg = sum(r50) / len(r50)
                text += f"""
## The memory side alone

`k_calib_encode` (`tplr_calib_encode`) runs the same grid over the same chunk ranges and issues the same 64 streaming row
loads per chunk, and nothing else.

{_cmd(tag, 'read', 'kt', a)}

| launch | avg us (50 timed) | min us | GB/s of the bytes read | of 8 TB/s |
|---|---|---|---|---|
| row loads only (`--profile read`) | {ravg:.1f} | {min(r50):.1f} | {alg_r / ravg / 1e3:.0f} | {alg_r / ravg / 1e3 / 80:.1f} % |

The encode launch takes {avg / ravg:.2f} x its memory-only form.
"""
            write(f"k_encode_topk_pack_{S['name']}.md", text)
        # ---------------- aggregate
        if _have(f"{tag}_aggregate"):
            units = 8 if Pn <= 8 else 16 if Pn <= 15 else 24
            bits = 4 if Pn <= 15 else 5
            kern = f"k_decode_aggregate<{dct}, {units}, {bits}, false, true, false, 0>"
            tr, dur = _trace(f"{tag}_aggregate", kern)
            t50 = dur[-50:]
            avg = sum(t50) / len(t50)
            alg_r, alg_w = n * Pn * 11 * k // 2, n * 16384
            alg = alg_r + alg_w
            text = f"""# {_short(tr[-1]['Kernel_Name'])}: {Pn} peers' payloads of {S['what']}, one persistent launch

## Kernel trace

{_cmd(tag, 'aggregate', 'kt', a)}

({note}; a step of this phase is the whole aggregate pass: the clip factors from the row figures noted on arrival, the
fused launch, the norm vectors.)  `p_kernel_stats.csv`, rows of this library's kernels (the {Pn} `k_encode_topk_pack`
launches build the peers' payloads):

{_stats_table(f'{tag}_aggregate')}

Launch geometry of the dominant kernel: {_geometry(tr[-1])}.

Durations of its last 60 launches in order (us), `p_kernel_trace.csv`:
{', '.join(f'{d:.0f}' for d in dur[-60:])}

The 50 timed launches average **{avg:.1f} us** (min {min(t50):.1f}); algorithmic bytes per launch
{alg:,} -> **{alg / avg / 1e3:.0f} GB/s = {alg / avg / 1e3 / 80:.1f} % of 8 TB/s**.
"""
            c = counted(f"{tag}_aggregate", kern)
            if c:
                f, nf, fb, w, nw, wb = c
                traffic[traffic_key(S["workload"], k, S["dct"], Pn, "aggregate")] = round(fb + wb)
                text += f"""
## HBM traffic (hardware counters)

{_cmd(tag, 'aggregate', 'FETCH_SIZE', a)}
{_cmd(tag, 'aggregate', 'WRITE_SIZE', a)}

| counter | mean per dispatch ({nf} dispatches) | scale (k_calib_copy_1GiB.md) | bytes per launch | algorithmic bytes | ratio |
|---|---|---|---|---|---|
| FETCH_SIZE | {f:.1f} | {sf:.4f} | {fb:,.0f} | {alg_r:,} | {fb / alg_r:.3f} |
| WRITE_SIZE | {w:.1f} | {sw:.4f} | {wb:,.0f} | {alg_w:,} | {wb / alg_w:.3f} |

Total HBM traffic per launch {fb + wb:,.0f} B = {(fb + wb) / alg:.3f} x the algorithmic bytes.
"""
            if _have(f"{tag}_calib") and _have(f"{tag}_fill"):
                _, cd = _trace(f"{tag}_calib", "k_calib_aggregate")
                _, fd = _trace(f"{tag}_fill", "k_calib_aggregate")
                c50, f50 = cd[-50:], fd[-50:]
                cavg, favg = sum(c50) / len(c50), sum(f50) / len(f50)
                cc = counted(f"{tag}_calib", "k_calib_aggregate")
                cbytes = f"{cc[2]:,.0f} read + {cc[5]:,.0f} written" if cc else ""
                kbytes = f"{c[2]:,.0f} read + {c[5]:,.0f} written" if c else ""
                text += f"""
## What the memory system alone needs: the kernel's loads and stores without the scatter and the transform

`k_calib_aggregate` (`tplr_calib_aggregate`) runs the same grid over the same chunk ranges (teams of four waves that
meet at a barrier before their stores where the launch itself runs them: `k_calib_aggregate_team`) and issues the same
payload loads and the same 64 row stores per chunk, and nothing else; with no peers it is the pure fill of the outputs.

{_cmd(tag, 'calib', 'kt', a)}
{_cmd(tag, 'fill', 'kt', a)}

| launch | avg us (50 timed) | min us | algorithmic GB/s | of 8 TB/s | HBM bytes (counters) |
|---|---|---|---|---|---|
| stores only (`--profile fill`) | {favg:.1f} | {min(f50):.1f} | {alg_w / favg / 1e3:.0f} | {alg_w / favg / 1e3 / 80:.1f} % | |
| loads + stores (`--profile calib`) | {cavg:.1f} | {min(c50):.1f} | {alg / cavg / 1e3:.0f} | {alg / cavg / 1e3 / 80:.1f} % | {cbytes} |
| `k_decode_aggregate` | {avg:.1f} | {min(t50):.1f} | {alg / avg / 1e3:.0f} | {alg / avg / 1e3 / 80:.1f} % | {kbytes} |

The memory-only launch takes {cavg / favg:.2f} x the pure fill although the payload is {alg_r / alg * 100:.0f} % of the bytes.  The
kernel runs at **{cavg / avg * 100:.1f} %** of its own memory-only form ({avg / cavg:.3f} x its duration).
"""
            if _have(f"{tag}_aggregate", "SQ"):
                text += f"""
## Vector ALU and LDS activity (hardware counters)

{_cmd(tag, 'aggregate', 'SQ', a)}

{_sq(f'{tag}_aggregate', kern, n, 2, 'No matrix-core instruction is issued.')}
"""
            write(f"k_decode_aggregate_{S['name']}_{Pn}peers.md", text)
        # ---------------- outer step
        if _have(f"{tag}_outer"):
            kern = "k_decode_aggregate<true, 16, 4, true, true, false, 0>"
            tr, dur = _trace(f"{tag}_outer", kern)
            t50 = dur[-50:]
            avg = sum(t50) / len(t50)
            alg = n * (Pn * 11 * k // 2 + 2 * 16384)
            text = f"""# {_short(tr[-1]['Kernel_Name'])}: the outer step, p <- p - lr * decode(aggregate of {Pn} peers), over {S['what']}

{_cmd(tag, 'outer', 'kt', a)}

({note}.)  `p_kernel_stats.csv`, rows of this library's kernels:

{_stats_table(f'{tag}_outer')}

Launch geometry: {_geometry(tr[-1])}.

The 50 timed launches average **{avg:.1f} us** (min {min(t50):.1f}); algorithmic bytes per launch (payload read, every
parameter chunk read and written) {alg:,} -> **{alg / avg / 1e3:.0f} GB/s = {alg / avg / 1e3 / 80:.1f} % of 8 TB/s**.
"""
            c = counted(f"{tag}_outer", kern)
            if c:
                f, nf, fb, w, nw, wb = c
                traffic[traffic_key(S["workload"], k, S["dct"], Pn, "outer_step")] = round(fb + wb)
                text += f"""
HBM traffic by the counters ({nf} dispatches; FETCH_SIZE {f:.1f}, WRITE_SIZE {w:.1f}, scaled as in k_calib_copy_1GiB.md):
{fb:,.0f} B read + {wb:,.0f} B written = {(fb + wb) / alg:.3f} x the algorithmic bytes.

{_cmd(tag, 'outer', 'FETCH_SIZE', a)}
{_cmd(tag, 'outer', 'WRITE_SIZE', a)}
"""
            write(f"k_outer_step_{S['name']}_{Pn}peers.md", text)

    # ---- miner step
    if _have("cfg3_miner"):
        rows = []
        for kern, label, b in (("k_ef_step<false>", "the whole step in one launch (no quantiser between its halves)", 294144 * (3 * 16384 + 176)),
                               ("k_encode_topk_pack<false, true, true>", "update + encode", 294144 * (3 * 16384 + 176)),
                               ("k_decode_aggregate<true, 8, 4, true, true, false, 0>", "subtract decoded", 294144 * (2 * 16384 + 176))):
            _, dur = _trace("cfg3_miner", kern)
            if not dur:
                continue
            t = dur[-50:]
            us = sum(t) / len(t)
            rows.append(f"| `{kern}` | {label} | {len(dur)} | {us:.1f} | {min(t):.1f} | {b:,} | {b / us / 1e3:.0f} | {b / us / 1e3 / 80:.1f} % |")
        write("error_feedback_step_cfg3_llama1b.md", f"""# Miner-side error-feedback step on the 1B gradient set (294 144 chunks, k=32): one persistent launch, or two where a quantiser sits between its halves

{_cmd('cfg3', 'miner', 'kt', [])}

`p_kernel_stats.csv`, rows of this library's kernels:

{_stats_table('cfg3_miner')}

From `p_kernel_trace.csv` (the last 50 launches of each kernel):

| kernel | step | launches in the trace | avg us | min us | algorithmic bytes | GB/s | of 8 TB/s |
|---|---|---|---|---|---|---|---|
{chr(10).join(rows)}
""")
    if _have("bench_default"):
        write("bench_default_cfg3_llama1b.md", f"""# bench.py (default arguments), 1B gradient set: all kernels of this library

    {PRE}rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof/bench_default_kt -o p -- python3 bench.py --no-cpu-baseline

`p_kernel_stats.csv`, rows of this library's kernels (the run also times the one-launch-per-tensor paths, the
calibration launches and the settle phases, so the fused kernels appear with many launches of several sizes; their
whole-set launches are profiled alone in k_encode_topk_pack_cfg3_llama1b.md and
k_decode_aggregate_cfg3_llama1b_15peers.md):

{_stats_table('bench_default')}
""")
    # ---------------- the measurement build with half of the forward transform on the matrix cores
    if _have("matrix_encode") and _have("matrix_encode", "MFMA") and _have("cfg3_encode", "MFMA") and _have("cfg3_encode"):
        kern = "k_encode_topk_pack<false, true, false>"
        n = SETS["cfg3"]["chunks"]
        alg = n * 16384 + n * 11 * 32 // 2
        tr, dur = _trace("matrix_encode", kern)
        avg = sum(dur[-50:]) / 50
        _, dur0 = _trace("cfg3_encode", kern)
        avg0 = sum(dur0[-50:]) / 50

        def mfma(tag):
            acc = collections.defaultdict(list)
            for r in csv.DictReader(open(_csv(tag, "MFMA", "*counter_collection.csv"))):
                if kern in r["Kernel_Name"]:
                    acc[r["Counter_Name"]].append(float(r["Counter_Value"]))
            return {k_: sum(v) / len(v) for k_, v in acc.items()}

        m1, m0 = mfma("matrix_encode"), mfma("cfg3_encode")
        mops, busy = m1.get("SQ_INSTS_VALU_MFMA_MOPS_F32", 0), m1.get("SQ_VALU_MFMA_BUSY_CYCLES", 0)
        n_mfma, simds, cyc = mops / 8, 1024, m1.get("GRBM_GUI_ACTIVE", 8) / 8   # (a 32x32x2 instruction is 4 096 operations)
        m_sq = collections.defaultdict(list)
        for r in csv.DictReader(open(_csv("matrix_encode", "SQ", "*counter_collection.csv"))):
            if kern in r["Kernel_Name"]:
                m_sq[r["Counter_Name"]].append(float(r["Counter_Value"]))
        m_sq = {k_: sum(v) / len(v) for k_, v in m_sq.items()}
        m_sq0 = 0.0
        if _have("cfg3_encode", "SQ"):
            v0 = [float(r["Counter_Value"]) for r in csv.DictReader(open(_csv("cfg3_encode", "SQ", "*counter_collection.csv")))
                  if kern in r["Kernel_Name"] and r["Counter_Name"] == "SQ_INSTS_VALU"]
            m_sq0 = sum(v0) / len(v0) / n
        rows = ["| counter | vector code (the product) | odd half on the matrix cores |", "|---|---|---|"]
        rows += [f"| {c} | {m0.get(c, 0):,.0f} | {m1.get(c, 0):,.0f} |" for c in MFMA]
        pre = PRE + "TPLR_HIP_LIB=templar_amd/libtplr_hip_matrix_variant.so "
        write("k_encode_topk_pack_cfg3_llama1b_matrix_cores.md", f"""# The forward transform's odd half on the matrix cores against the generated vector code: encode launch of the 1B set

The product computes the 64-point transform as factorised vector code (535 instructions per 64-vector).  A
measurement build of the same sources (`-DTPLR_DCT_MATRIX_CORES=1`, `templar_amd/csrc/tplr_device.h`:
`dct64_fwd_matrix`) computes the odd half of the forward transform - a 32-point DCT-IV, 250 of those instructions -
as a dense 32x32x64 product with 32 `v_mfma_f32_32x32x2_f32` per pass, operands formed with `v_permlane32_swap`, and
keeps everything else.  Built beside the product library by

    TPLR_BUILD_MATRIX_VARIANT=1 python -c 'import __graft_entry__ as g; g.build()'

and profiled with the commands below (`python bench_profiles.py run --sets matrix` runs all of them).

## Kernel trace

    {pre}rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof/matrix_encode_kt -o p -- python3 bench.py --profile encode --steps 50 --warmup 10

{_stats_table('matrix_encode')}

Launch geometry: {_geometry(tr[-1])}.

The 50 timed launches average **{avg:.1f} us** against **{avg0:.1f} us** for the product's vector code
(k_encode_topk_pack_cfg3_llama1b.md): {alg / avg / 1e3:.0f} GB/s = {alg / avg / 1e3 / 80:.1f} % of 8 TB/s against
{alg / avg0 / 1e3:.0f} GB/s = {alg / avg0 / 1e3 / 80:.1f} %.

## Matrix-core and vector-ALU activity (hardware counters)

    {pre}rocprofv3 --kernel-include-regex tplr --pmc {' '.join(MFMA)} --output-format csv -d gpurun_out/prof/matrix_encode_MFMA -o p -- python3 bench.py --profile encode --steps 3 --warmup 1
    {PRE}rocprofv3 --kernel-include-regex tplr --pmc {' '.join(MFMA)} --output-format csv -d gpurun_out/prof/cfg3_encode_MFMA -o p -- python3 bench.py --profile encode --steps 3 --warmup 1

{chr(10).join(rows)}

`SQ_INSTS_VALU_MFMA_MOPS_F32` counts 512 floating-point operations each: {mops * 512 / n:,.0f} per chunk (two passes of
a dense 32x32x64 product are 262 144), in {n_mfma / n:.0f} matrix instructions per chunk.  `SQ_VALU_MFMA_BUSY_CYCLES` is
{busy / n_mfma:.1f} cycles per instruction: the matrix pipelines of the {simds} SIMDs are busy {busy / simds / cyc * 100:.0f} % of the
launch's {cyc / 1e6:.2f} M cycles (`GRBM_GUI_ACTIVE` over 8 XCDs) - far from saturated - and yet the launch takes
{avg / avg0:.2f} x as long as with vector code although it issues {m_sq['SQ_INSTS_VALU'] / n:.0f} vector instructions per chunk instead of
{m_sq0:.0f}: the vector ALU is active {m_sq['SQ_ACTIVE_INST_VALU'] / m_sq['SQ_WAVE_CYCLES'] * 100:.0f} % of a wave's time (31 % in the product) and the waves wait
for an issue slot {m_sq['SQ_WAIT_INST_ANY'] / m_sq['SQ_WAVE_CYCLES'] * 100:.0f} % of it.  A SIMD that is working on a matrix instruction issues next to nothing
else here, so the 64 cycles of each instruction come on top of the vector work instead of beside it - 4 096
cycles per chunk against the 1 000 the factorised odd half takes.  The transform stays vector code.

    {pre}rocprofv3 --kernel-include-regex tplr --pmc {' '.join(SQ)} --output-format csv -d gpurun_out/prof/matrix_encode_SQ -o p -- python3 bench.py --profile encode --steps 3 --warmup 1

{_sq('matrix_encode', kern, n, 3, 'Here the transform is half vector code, half matrix-core instructions.')}
""")
    if traffic:
        traffic["what"] = ("HBM bytes per launch of the whole-set kernels (FETCH_SIZE + WRITE_SIZE, each scaled by the calibration "
                           "copy), keyed workload/peers/kernel; written by bench_profiles.py summarise from the rocprofv3 runs whose "
                           "commands the summaries in this folder give")
        with open(os.path.join(out_dir, "traffic.json"), "w") as fh:
            json.dump(traffic, fh, indent=1, sort_keys=True)
            fh.write("\n")
        print("wrote traffic.json")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=["run", "summarise"])
    ap.add_argument("--sets", default=",".join(SETS) + ",bench")
    ap.add_argument("--phases", default="")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    args = ap.parse_args()
    sets = [s for s in args.sets.split(",") if s]
    for s in sets:
        if s not in SETS and s not in ("bench", "matrix"):
            ap.error(f"unknown set {s}")
    if args.what == "run":
        run(sets, [p for p in args.phases.split(",") if p])
    else:
        summarise(args.out)


if __name__ == "__main__":
    main()
