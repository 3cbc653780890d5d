"""Condense rocprofv3 CSV output into a few lines per kernel of this library.

    python3 profile_summary.py <rocprofv3 output dir> [more dirs...]

Prints, for every kernel of this library (and the totals row of --stats), the call count and
average duration, and the per-dispatch average of every hardware counter
collected. Raw CSVs hold every torch kernel of the run and are large; this is
the part worth keeping.

The `launch` lines repeat rocprofv3's own columns. Its VGPR_Count is not the
kernel's register allocation on this device (it reads 80 for lookup_kernel,
whose code object allocates 157 vector registers, 3 waves per SIMD): take
register counts from the code object's notes, not from here.
"""
import csv
import glob
import os
import sys
from collections import defaultdict

OURS = ("lookup_lean_wide4_redo_kernel", "lookup_lean_wide4_kernel", "lookup_lean_kernel", "split_offsets_kernel", "combine_segments_kernel", "gather_lines_lds_kernel", "gather_lines_kernel", "stream_read_kernel", "remap_rank_build", "inplace_update_kernel", "remap_row_idx_kernel", "sequence_lookup_kernel", "row_lookup_kernel", "pruned_array_lookup", "pruned_hashmap_lookup", "lookup_kernel",
        "calibration_copy_kernel", "float_to_hfp8_kernel", "hfp8_to_float_kernel", "prune_count", "prune_carry", "prune_remap",
        "prune_gather", "remap_count", "remap_move", "remap_offsets",
        "bag_order_kernel", "lengths_to_offsets", "bounds_partial_max", "bounds_carry", "bounds_fix_offsets",
        "bounds_check_bags", "dequantize_rowwise", "quantize_rowwise")


def short(name):
    for k in OURS:
        if k in name:
            return k + ("<int64>" if "IlE" in name else "<int32>" if "IiE" in name else
                        "<16>" if ("ILi16E" in name or "<16>" in name) else "<8>" if ("ILi8E" in name or "<8>" in name) else "")
    return None


def summarize(d):
    lines = []
    for f in sorted(glob.glob(os.path.join(d, "**", "*kernel_stats.csv"), recursive=True)):
        with open(f) as fh:
            for row in csv.DictReader(fh):
                s = short(row.get("Name", ""))
                if s:
                    lines.append(f"stats  {s}: calls={row.get('Calls')} avg_ns={row.get('AverageNs')} "
                                 f"min_ns={row.get('MinNs')} max_ns={row.get('MaxNs')} pct={row.get('Percentage')}")
    for f in sorted(glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)):
        acc = defaultdict(lambda: [0.0, 0])
        grid = {}
        with open(f) as fh:
            for row in csv.DictReader(fh):
                s = short(row.get("Kernel_Name", ""))
                if not s:
                    continue
                key = (s, row.get("Counter_Name"))
                acc[key][0] += float(row.get("Counter_Value", 0))
                acc[key][1] += 1
                grid[s] = (row.get("Grid_Size"), row.get("Workgroup_Size"), row.get("VGPR_Count"),
                           row.get("Accum_VGPR_Count"), row.get("SGPR_Count"), row.get("LDS_Block_Size"),
                           row.get("Scratch_Size"))
        for (s, c), (tot, n) in sorted(acc.items()):
            lines.append(f"pmc    {s}: {c} avg_per_dispatch={tot / n:.6g} dispatches={n}")
        for s, g in sorted(grid.items()):
            lines.append(f"launch {s}: grid={g[0]} wg={g[1]} rocprof_vgpr_column={g[2]} agpr={g[3]} sgpr={g[4]} lds={g[5]} scratch={g[6]}")
    return lines


if __name__ == "__main__":
    for d in sys.argv[1:]:
        print(f"# {d}")
        for l in summarize(d):
            print(l)
