"""bench.py carries the HBM-side traffic of each kernel as constants, because counters cannot be read inside a timed
run. Every constant is tied to the kernel sources it was measured on: this test fails when one of those sources has
changed (comments and white space aside) since the counters were last read, so that a stale figure cannot be
reported as a measurement, and checks that every constant has a summary under profiles/ that holds it."""
import glob
import types
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    # (compiled from the source text: no bytecode cache between the file and the test)
    path = os.path.join(ROOT, "bench.py")
    mod = types.ModuleType("bench_under_test")
    mod.__file__ = path
    exec(compile(open(path).read(), path, "exec"), mod.__dict__)
    return mod


def test_traffic_constants_were_measured_on_the_current_kernel_sources():
    bench = load_bench()
    used = set()
    for key, (value, sources) in bench.MEASURED_TRAFFIC_BYTES.items():
        assert value > 0 and sources, key
        used.update(sources)
        assert bench.measured_traffic(key) == value, (
            "%s: a kernel source changed since its counters were read; run the two counter passes named in "
            "profiles/ again, then update the constant and MEASURED_SOURCE_DIGEST" % key)
    assert used == set(bench.MEASURED_SOURCE_DIGEST)
    for name in used:
        assert bench.source_digest(name) == bench.MEASURED_SOURCE_DIGEST[name], name


def test_digest_ignores_comments_and_layout_only(tmp_path, monkeypatch):
    bench = load_bench()
    monkeypatch.setattr(bench, "CSRC", str(tmp_path))
    (tmp_path / "a.hip").write_text("int f(int x) {\n  return x + 1;  // one more\n}\n")
    (tmp_path / "b.hip").write_text("/* header */\nint f(int x) { return x + 1; }\n")
    (tmp_path / "c.hip").write_text("int f(int x) { return x + 2; }\n")
    assert bench.source_digest("a.hip") == bench.source_digest("b.hip") != bench.source_digest("c.hip")
    monkeypatch.setattr(bench, "MEASURED_TRAFFIC_BYTES", {"k": (5.0, ("a.hip", ))})
    monkeypatch.setattr(bench, "MEASURED_SOURCE_DIGEST", {"a.hip": bench.source_digest("c.hip")})
    assert bench.measured_traffic("k") is None
    monkeypatch.setattr(bench, "MEASURED_SOURCE_DIGEST", {"a.hip": bench.source_digest("b.hip")})
    assert bench.measured_traffic("k") == 5.0


def test_every_traffic_constant_is_in_a_committed_profile():
    bench = load_bench()
    text = "".join(open(p).read() for p in glob.glob(os.path.join(ROOT, "profiles", "*.md")))
    for key, (value, _) in bench.MEASURED_TRAFFIC_BYTES.items():
        shown = "%.1f MB" % (value / 1e6)
        assert re.search(re.escape(shown), text), "%s: %s is in no summary under profiles/" % (key, shown)
