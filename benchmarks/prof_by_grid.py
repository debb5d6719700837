"""Per (kernel, grid size) call counts and median durations from a rocprofv3 --kernel-trace CSV: the
grid separates a kernel's prefill dispatches from its decode dispatches.
python benchmarks/prof_by_grid.py <dir> [top]"""
import collections, csv, glob, re, statistics, sys

d = sys.argv[1]
top = int(sys.argv[2]) if len(sys.argv) > 2 else 40
f = glob.glob(d + "/*/*kernel_trace.csv")[0]
by = collections.defaultdict(list)
for r in csv.DictReader(open(f)):
    n = r["Kernel_Name"]
    m = re.search(r"(\w+_kernel\w*)(<[^>]*>)?", n)
    grid = "x".join(str(r.get(k, "?")) for k in ("Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"))
    by[((m.group(0) if m else n)[:60], grid)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
print("%-60s %-18s %6s %10s %10s" % ("kernel", "grid (threads)", "calls", "median_us", "total_ms"))
for (k, g), v in sorted(by.items(), key=lambda kv: -sum(kv[1]))[:top]:
    print("%-60s %-18s %6d %10.1f %10.1f" % (k, g, len(v), statistics.median(v), sum(v) / 1e3))
