"""Per-kernel timing of the path, in the shape of the reference's profiler
(python/jittor/__init__.py:235-263 profile_scope;
python/jittor/src/profiler/profiler.cc:374-470 report): every launch of the
executor is bracketed by device events on the library's stream and
accumulated per kernel name with the bytes of the group's external inputs
and outputs (the reference's byte accounting, fused_op.cc:149-156).

    with jt.profile_scope(warmup=1, rerun=9) as report:
        y = (a * b).sum(1); y.sync()
    for row in report: print(row)

Rows: Name, FileName, Count, TotalTime, AvgTime, MinTime, MaxTime (ns),
Input, Output, InOut (bytes/s), Compute (empty: no flop model).
"""
from . import _lib

HEADER = ["Name", "FileName", "Count", "TotalTime", "AvgTime", "MinTime", "MaxTime", "Input", "Output", "InOut", "Compute"]


class _Recorder:
    def __init__(self, warmup, rerun):
        self.warmup, self.rerun = int(warmup), int(rerun)
        self.pending = []          # (name, kind, start event, stop event, in bytes, out bytes)

    def run(self, call, kind, in_bytes, out_bytes):
        """Runs the launch (warmup + 1 + rerun times; the extra runs rewrite the same outputs)."""
        result = None
        for i in range(self.warmup + 1 + self.rerun):
            if i < self.warmup:
                result = call()
                continue
            e0, e1 = _lib.Event(), _lib.Event()
            e0.record()
            result = call()
            e1.record()
            if result is not False:                    # False: the library declined this form, nothing ran
                self.pending.append((_lib.last_kernel(), kind, e0, e1, in_bytes, out_bytes))
        return result

    def report(self):
        _lib.sync()
        acc = {}
        for name, kind, e0, e1, ib, ob in self.pending:
            ns = e1.elapsed_ms_since(e0) * 1e6
            a = acc.setdefault(name, [kind, 0, 0.0, float("inf"), 0.0, 0, 0])
            a[1] += 1
            a[2] += ns
            a[3] = min(a[3], ns)
            a[4] = max(a[4], ns)
            a[5] += ib
            a[6] += ob
        rows = [list(HEADER)]
        total_ns = sum(a[2] for a in acc.values())
        total_in = sum(a[5] for a in acc.values())
        total_out = sum(a[6] for a in acc.values())
        rows.append(["total", "", str(sum(a[1] for a in acc.values())), "%.0f" % total_ns, "", "", "",
                     _rate(total_in, total_ns), _rate(total_out, total_ns), _rate(total_in + total_out, total_ns), ""])
        for name, a in sorted(acc.items(), key=lambda kv: -kv[1][2]):
            kind, count, tot, mn, mx, ib, ob = a
            rows.append([name, kind, str(count), "%.0f" % tot, "%.0f" % (tot / count), "%.0f" % mn, "%.0f" % mx,
                         _rate(ib, tot), _rate(ob, tot), _rate(ib + ob, tot), ""])
        return rows


def _rate(nbytes, ns):
    return "%.4g" % (nbytes / (ns * 1e-9)) if ns > 0 else "0"


_active = [None]


def active():
    return _active[0]


class profile_scope:
    def __init__(self, warmup=0, rerun=0):
        self.warmup, self.rerun = warmup, rerun

    def __enter__(self):
        if _active[0] is not None:
            raise RuntimeError("profile_scope does not nest")
        self.report = []
        _active[0] = _Recorder(self.warmup, self.rerun)
        return self.report

    def __exit__(self, *exc):
        rec, _active[0] = _active[0], None
        self.report.extend(rec.report())
        return False
