"""Text summary of a rocprofv3 result database (rocpd SQLite):

    python -m triteia_amd.profile_summary <results.db> [--top N] [--match SUBSTR]

Prints per-kernel dispatch statistics (from --kernel-trace) and, when the run collected
hardware counters (--pmc), the mean counter value per dispatch for every kernel.
"""
import argparse
import sqlite3


def kernel_stats(con, top, match):
    rows = con.execute(
        "select name, count(*), avg(duration), min(duration), max(duration), sum(duration) "
        "from kernels group by name order by sum(duration) desc").fetchall()
    total = sum(r[5] for r in rows) or 1
    out = [f"{'kernel':78s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'total_ms':>9s} {'%':>6s}"]
    for n, cnt, avg, mn, mx, sm in rows:
        if match and match not in n:
            continue
        out.append(f"{n[:78]:78s} {cnt:6d} {avg / 1e3:9.2f} {mn / 1e3:9.2f} {mx / 1e3:9.2f} {sm / 1e6:9.3f} {100 * sm / total:6.1f}")
        if len(out) > top:
            break
    return out


def counter_stats(con, top, match):
    try:
        rows = con.execute(
            "select kernel_name, counter_name, count(*), avg(value), min(value), max(value) "
            "from counters_collection group by kernel_name, counter_name order by avg(value) desc").fetchall()
    except sqlite3.Error:
        return []
    out = [f"{'kernel':78s} {'counter':14s} {'n':>5s} {'avg':>14s} {'min':>14s} {'max':>14s}"]
    for n, cn, cnt, avg, mn, mx in rows:
        if match and match not in n:
            continue
        out.append(f"{n[:78]:78s} {cn:14s} {cnt:5d} {avg:14.1f} {mn:14.1f} {mx:14.1f}")
        if len(out) > top:
            break
    return out if len(out) > 1 else []


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("db")
    ap.add_argument("--top", type=int, default=12)
    ap.add_argument("--match", default=None, help="only kernels whose name contains this text")
    a = ap.parse_args()
    con = sqlite3.connect(a.db)
    print("\n".join(kernel_stats(con, a.top, a.match)))
    cs = counter_stats(con, a.top, a.match)
    if cs:
        print()
        print("\n".join(cs))


if __name__ == "__main__":
    main()
