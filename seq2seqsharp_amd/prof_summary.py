"""Turn a rocprofv3 result database (--kernel-trace [--pmc ...]) into the short text summaries kept under profiles/.

    python -m seq2seqsharp_amd.prof_summary gpurun_out/prof/decode_results.db "<command that produced it>" > profiles/<name>.txt
"""
import re
import sqlite3
import statistics
import sys


def main():
    db_path, cmd = sys.argv[1], (sys.argv[2] if len(sys.argv) > 2 else "")
    cur = sqlite3.connect(db_path).cursor()
    print("command:", cmd)
    rows = list(cur.execute("select name, count(*), sum(duration), avg(duration), min(duration), max(duration) from kernels "
                            "group by name order by sum(duration) desc"))
    tot = sum(r[2] for r in rows) or 1
    print("\nkernel-trace statistics (durations from dispatch begin/end timestamps)")
    print("%-78s %8s %12s %10s %9s %9s %6s" % ("kernel", "calls", "total_ms", "avg_us", "min_us", "max_us", "%"))
    for n, c, s, a, mn, mx in rows:
        n = re.sub(r"tship::", "", n)
        print("%-78s %8d %12.3f %10.2f %9.2f %9.2f %6.1f" % (n[:78], c, s / 1e6, a / 1e3, mn / 1e3, mx / 1e3, 100.0 * s / tot))
    ks = list(cur.execute("select start, end from kernels order by start"))
    if len(ks) > 200:
        sub = ks[-min(len(ks) // 2, 4000):]
        gaps = [max(0, sub[i + 1][0] - sub[i][1]) for i in range(len(sub) - 1)]
        busy = sum(e - s for s, e in sub)
        span = sub[-1][1] - sub[0][0]
        print("\nlast %d dispatches: busy %.1f %% of the span, mean gap between consecutive kernels %.2f us (median %.2f us)"
              % (len(sub), 100.0 * busy / span, sum(gaps) / len(gaps) / 1e3, statistics.median(gaps) / 1e3))
    try:
        pmc = list(cur.execute("select name, counter_name, count(*), avg(counter_value), sum(counter_value) from pmc_events "
                               "group by name, counter_name order by name, counter_name"))
    except Exception:
        pmc = []
    if pmc:
        print("\ncounters (per dispatch averages)")
        print("%-78s %-18s %8s %16s" % ("kernel", "counter", "calls", "avg"))
        for n, cn, c, a, s in pmc:
            print("%-78s %-18s %8d %16.1f" % (re.sub(r"tship::", "", n)[:78], cn, c, a))


if __name__ == "__main__":
    main()
