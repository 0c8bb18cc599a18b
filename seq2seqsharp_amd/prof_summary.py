"""Turn a rocprofv3 result database (--kernel-trace [--pmc ...]) into the short text summaries kept under profiles/.

    python -m seq2seqsharp_amd.prof_summary <rocprofv3 output dir>/decode_results.db "<command that produced it>" > <summary>.txt
"""
import re
import sqlite3
import statistics
import sys


def _avg(db_path, counter, like):
    cur = sqlite3.connect(db_path).cursor()
    r = list(cur.execute("select count(*), avg(counter_value) from pmc_events where counter_name = ? and name like ?", (counter, like)))
    return (r[0][0], r[0][1]) if r and r[0][0] else (0, None)


def traffic(fetch_db, write_db, kernel_like, copy_like, copy_bytes, out_json):
    """HBM bytes per launch of one kernel from a FETCH_SIZE run and a WRITE_SIZE run (KiB per dispatch), each scaled by
    what the same counter reads for a plain copy kernel that reads and writes `copy_bytes`."""
    import json
    nf, f = _avg(fetch_db, "FETCH_SIZE", kernel_like)
    nw, w = _avg(write_db, "WRITE_SIZE", kernel_like)
    _, cf = _avg(fetch_db, "FETCH_SIZE", copy_like)
    _, cw = _avg(write_db, "WRITE_SIZE", copy_like)
    fs, ws = copy_bytes / (cf * 1024.0), copy_bytes / (cw * 1024.0)
    out = {"kernel_like": kernel_like, "dispatches": nf, "fetch_kib_per_dispatch": f, "write_kib_per_dispatch": w,
           "copy_kernel_like": copy_like, "copy_bytes": copy_bytes, "copy_fetch_kib": cf, "copy_write_kib": cw,
           "fetch_scale": fs, "write_scale": ws,
           "traffic_bytes_per_launch": round((f * fs + (w or 0.0) * ws) * 1024.0)}
    json.dump(out, open(out_json, "w"), indent=1)
    print(json.dumps(out, indent=1))


def main():
    if sys.argv[1] == "--traffic":
        traffic(sys.argv[2], sys.argv[3], sys.argv[4], sys.argv[5], int(sys.argv[6]), sys.argv[7])
        return
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
        # a counter has one row per hardware instance (XCD, shader engine ...) and dispatch: add the instances of a
        # dispatch, then average over the dispatches of a kernel
        pmc = list(cur.execute(
            "select name, counter_name, count(*), avg(v), avg(d) from (select name, counter_name, dispatch_id, sum(counter_value) as v, "
            "max(duration) as d from pmc_events group by name, counter_name, dispatch_id) group by name, counter_name order by name, counter_name"))
    except Exception:
        pmc = []
    if pmc:
        print("\ncounters (sum over hardware instances, average per dispatch)")
        print("%-78s %-30s %8s %16s" % ("kernel", "counter", "calls", "per_dispatch"))
        per = {}
        top = set(r[0] for r in rows[:12])           # the twelve kernels with the largest total time
        for n, cn, c, a, d in pmc:
            if n in top:
                print("%-78s %-30s %8d %16.1f" % (re.sub(r"tship::", "", n)[:78], cn, c, a))
            per.setdefault(n, {})[cn] = (a, d)
        # MFMA utilisation: busy cycles of the matrix pipes over (4 SIMDs x CUs x kernel cycles); SQ_BUSY_CYCLES counts
        # the kernel's cycles once per shader engine (32 on MI355X), MFMA busy cycles once per SIMD
        mrows = [(n, v) for n, v in per.items() if "SQ_VALU_MFMA_BUSY_CYCLES" in v and "SQ_BUSY_CYCLES" in v and v["SQ_BUSY_CYCLES"][0] > 0]
        if mrows:
            print("\nMFMA utilisation = SQ_VALU_MFMA_BUSY_CYCLES / (SQ_BUSY_CYCLES / 32 shader engines x 256 CUs x 4 SIMDs)")
            for n, v in mrows:
                cyc = v["SQ_BUSY_CYCLES"][0] / 32.0
                util = v["SQ_VALU_MFMA_BUSY_CYCLES"][0] / (cyc * 256 * 4)
                extra = ""
                if "SQ_INSTS_VALU_MFMA_MOPS_F16" in v and v["SQ_BUSY_CYCLES"][1]:
                    tflops = v["SQ_INSTS_VALU_MFMA_MOPS_F16"][0] * 512.0 / (v["SQ_BUSY_CYCLES"][1] * 1e-9) / 1e12
                    extra = "  %.0f TFLOP/s issued" % tflops
                if util > 0.001:
                    print("%-78s %6.1f %%%s" % (re.sub(r"tship::", "", n)[:78], 100.0 * util, extra))


if __name__ == "__main__":
    main()
