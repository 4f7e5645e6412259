"""Summaries of rocprofv3 output for bench.py's workloads: per-kernel durations from a kernel trace, raw counter
averages from a --pmc run, and the HBM bytes per launch of every bench leg (FETCH_SIZE and WRITE_SIZE, each scaled by
what the same counter reads for bench.py's calibration copy of 256 MiB).  bench.py prints them (`--summarise ...`) and
reads the traffic figures back from the summary kept with the other profiler summaries.
"""
from __future__ import annotations

import collections
import csv
import ctypes
import re

CALIBRATION_KIB = 262144.0          # bench.py --counter-calibration: torch.mul(src, 1.0, out=dst) on 256 MiB reads and writes this much
TRAFFIC_LINE = re.compile(r"^traffic\s+(\S+)\s+(\d+)\b")


def short_name(kernel_name: str) -> str:
    return re.sub(r"\(.*", "", kernel_name).replace("void ", "").replace("ttmi::", "")[:72]


def summarise_trace(path: str) -> str:
    """Per (kernel, grid): launches, average / minimum / maximum duration, registers and LDS, longest total first."""
    groups = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        key = (short_name(r["Kernel_Name"]), int(r["Grid_Size_X"]) // int(r["Workgroup_Size_X"]), int(r["Workgroup_Size_X"]),
               r["VGPR_Count"], r["Accum_VGPR_Count"], r["LDS_Block_Size"], r["Scratch_Size"])
        groups[key].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    rows = sorted(((sum(v), k, v) for k, v in groups.items()), reverse=True)
    out = [f"{'kernel':72s} {'WGs':>7s} {'wg':>4s} {'vgpr':>4s} {'agpr':>4s} {'lds':>6s} {'scr':>4s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s}"]
    for _, k, v in rows:
        out.append(f"{k[0]:72s} {k[1]:7d} {k[2]:4d} {k[3]:>4s} {k[4]:>4s} {k[5]:>6s} {k[6]:>4s} {len(v):6d} "
                   f"{sum(v) / len(v) / 1e3:9.2f} {min(v) / 1e3:9.2f} {max(v) / 1e3:9.2f}")
    return "\n".join(out)


def counter_rows(path: str):
    """{(kernel, workgroups, counter): [value per launch]} of a --pmc run."""
    groups = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        groups[(short_name(r["Kernel_Name"]), int(r["Grid_Size"]) // int(r["Workgroup_Size"]), r["Counter_Name"])].append(float(r["Counter_Value"]))
    return groups


def summarise_pmc(path: str, only: str | None = None) -> str:
    out = [f"{'kernel':72s} {'WGs':>7s} {'counter':>32s} {'calls':>6s} {'avg':>14s} {'min':>14s} {'max':>14s}"]
    for k, v in sorted(counter_rows(path).items(), key=lambda kv: (kv[0][0], kv[0][1], kv[0][2])):
        if only and only not in k[0]:
            continue
        out.append(f"{k[0]:72s} {k[1]:7d} {k[2]:>32s} {len(v):6d} {sum(v) / len(v):14.1f} {min(v):14.1f} {max(v):14.1f}")
    return "\n".join(out)


def leg_kernels():
    """bench leg -> [(kernel name prefix, workgroups or None)]: the launches that make up one step of that leg.  The
    grids of the decode GEMMs come from the library's own decomposition; None = the grid launched most often."""
    from . import capi, workloads

    L = capi.lib()
    legs = {}
    for name, m, k, n, fmt, batch in workloads.DECODE_FALCON + workloads.DECODE_MISTRAL:
        plan = (ctypes.c_uint32 * 4)()
        L.ttmi_matmul_bfp_plan(batch or 1, m, k, n, capi.BFLOAT16, capi.BFLOAT8_B if fmt == "bfp8_b" else capi.BFLOAT4_B, capi.BFLOAT16, plan)
        w = 7 if fmt == "bfp8_b" else 3
        # the grid of an MI355X (output groups dealt out to its XCDs)
        legs[name] = [(f"matmul_wide_kernel<{w}, 0, 1, 1, false>" if plan[0] == 2 else f"matmul_stream_kernel<{w}, 0>", int(plan[3]))]
    legs["prefill_ff1"] = [("expand_kernel<7>", None), ("matmul_expanded_kernel<0>", None)]
    legs["prefill_ff1_256"] = [("matmul_wide_kernel<7, 0, 1, 2, false>", None)]
    legs["bert_bmm"] = [("matmul_tall_kernel<7, 0", None)]
    legs["pack_bfp4_4k_pack"] = [("pack_whole_kernel<3,", None)]
    legs["pack_bfp4_4k_unpack"] = [("unpack_whole_kernel<3,", None)]
    legs["pack_bfp8_1k_pack"] = [("pack_kernel<7,", None)]
    legs["pack_bfp8_1k_unpack"] = [("unpack_kernel<7,", None)]
    return legs


def _average_for(rows, counter, prefix, workgroups):
    """Average raw counter value of the launches of kernel `prefix` on `workgroups` workgroups (None: the grid launched most often)."""
    matching = {k: v for k, v in rows.items() if k[2] == counter and k[0].startswith(prefix)}
    if workgroups is not None:
        matching = {k: v for k, v in matching.items() if k[1] == workgroups}
    if not matching:
        return None, None
    key = max(matching, key=lambda k: len(matching[k]))
    v = matching[key]
    return sum(v) / len(v), key


def traffic_lines(fetch_csv: str, write_csv: str) -> str:
    """One line per bench leg: `traffic <leg> <HBM bytes per launch> ...`, from a FETCH_SIZE run and a WRITE_SIZE run
    of `bench.py --counter-calibration`; each counter is scaled so that the calibration copy reads / writes 256 MiB."""
    fetch, write = counter_rows(fetch_csv), counter_rows(write_csv)

    def calibration(rows, counter):
        # torch.mul(src, 1.0, out=dst) on fp32: vectorized_elementwise_kernel<4, AUnaryFunctor<.. MulFunctor ..>>, every workgroup
        # of which reads 4 KiB and writes 4 KiB (the calibration copy of 256 MiB is 65536 of them); bench.py's copy-ceiling
        # leg launches the same kernel on 512 MiB and calibrates as well
        moved = raw = 0.0
        for k, v in rows.items():
            if k[2] == counter and "vectorized_elementwise_kernel<4" in k[0] and "AUnaryFunctor" in k[0] and k[1] >= 65536:
                moved += 4.0 * k[1] * len(v)
                raw += sum(v)
        if not raw:
            raise SystemExit(f"no calibration launch (torch.mul on 256 MiB) found for {counter}: run bench.py with --counter-calibration")
        return moved / raw

    f_scale, w_scale = calibration(fetch, "FETCH_SIZE"), calibration(write, "WRITE_SIZE")
    out = [f"scale FETCH_SIZE x{f_scale:.3f}  WRITE_SIZE x{w_scale:.3f}  (calibration copy = {CALIBRATION_KIB:.0f} KiB each way)"]
    for leg, kernels in leg_kernels().items():
        total, parts = 0.0, []
        for prefix, workgroups in kernels:
            f, fkey = _average_for(fetch, "FETCH_SIZE", prefix, workgroups)
            w, wkey = _average_for(write, "WRITE_SIZE", prefix, workgroups)
            if f is None or w is None:
                total = None
                break
            total += (f * f_scale + w * w_scale) * 1024
            parts.append(f"{fkey[0]} on {fkey[1]} WGs: fetch {f * f_scale:.0f} KiB write {w * w_scale:.0f} KiB")
        if total is not None:
            out.append(f"traffic {leg} {int(round(total))}   # " + "; ".join(parts))
    return "\n".join(out)


def read_traffic(summary_path: str) -> dict:
    """{leg: HBM bytes per launch} from the `traffic` lines of a summary written with traffic_lines()."""
    found = {}
    try:
        for line in open(summary_path):
            m = TRAFFIC_LINE.match(line.strip())
            if m:
                found[m.group(1)] = int(m.group(2))
    except OSError:
        pass
    return found
