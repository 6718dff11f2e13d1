"""`bench.py --summarize-profile`: per-kernel figures over the LAST dispatches of each kernel in rocprofv3's CSV output (the timed
launches of a configuration come last, its warm-up launches first).  Host logic only: synthetic CSV files, no GPU."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_summary_takes_last_dispatches_only(tmp_path, capsys):
    d = tmp_path / "run" / "host"
    d.mkdir(parents=True)
    # kernel "k": five slow warm-up dispatches (100 us), then three timed ones (10, 12, 14 us); rows deliberately out of order
    rows = [(i * 1000000, i * 1000000 + 100000) for i in range(5)] + [(9000000, 9010000), (9100000, 9112000), (9200000, 9214000)]
    rows = rows[::-1]
    with open(d / "bench_kernel_trace.csv", "w") as f:
        f.write('"Kind","Kernel_Name","Start_Timestamp","End_Timestamp"\n')
        for s, e in rows:
            f.write('"KERNEL_DISPATCH","k(int)",%d,%d\n' % (s, e))
    with open(d / "bench_counter_collection.csv", "w") as f:
        f.write('"Kernel_Name","Counter_Name","Counter_Value"\n')
        for v in (900.0, 900.0, 100.0, 102.0, 104.0):
            f.write('"k(int)","FETCH_SIZE",%r\n' % v)
    assert _bench()._summarize_profile(str(tmp_path / "run"), 3) == 0
    out = capsys.readouterr().out
    assert "calls=8 last=3 avg=12.00 min=10.00 max=14.00" in out
    assert "(all calls avg 67.00)" in out
    assert "FETCH_SIZE=102 (n=5)" in out
