"""Host-side logic of bench.py that needs no GPU: the trace / counter summarisers and the
traffic record keyed by the kernel sources."""
import importlib
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)
bench = importlib.import_module("bench")


def _write(path, header, rows):
  with open(path, "w") as f:
    f.write(",".join(header) + "\n")
    for r in rows:
      f.write(",".join(f'"{v}"' if "," in str(v) or "(" in str(v) else str(v) for v in r) + "\n")


def test_step_trace_summary_takes_the_last_complete_step(tmp_path, capsys):
  # three commits = two complete steps; the summary covers the one between the last two but one
  rows, t = [], 0
  def k(name, dur, gap=1000):
    nonlocal t
    rows.append((name, t, t + dur))
    t += dur + gap
  for step in range(3):
    k("void (anonymous namespace)::qgemm128_kernel<2, 2, 8>((anonymous namespace)::QLArgs)", 20000 + step)
    k("(anonymous namespace)::lora_down_kernel(unsigned short const*, long)", 5000)
    k("void (anonymous namespace)::qgemm128_kernel<2, 2, 8>((anonymous namespace)::QLArgs)", 30000)
    k("(anonymous namespace)::sample_commit_kernel(int const*)", 3000)
  p = tmp_path / "t.csv"
  _write(p, ["Kernel_Name", "Start_Timestamp", "End_Timestamp"], rows)
  bench.summarize_step_trace(str(p))
  out = capsys.readouterr().out
  assert "4 kernels" in out
  line = [l for l in out.splitlines() if l.startswith("| qgemm128_kernel<2, 2, 8>")][0].split("|")
  assert int(line[2]) == 2                       # two GEMM launches in the step
  assert abs(float(line[3]) - 50.0) < 0.01       # 20.001 + 30.000 us: the second step's durations
  assert abs(float(line[5]) - 26.0) < 0.01       # start-to-start includes the 1 us gaps


def test_counter_summary_means_and_ratios(tmp_path, capsys):
  name = "void (anonymous namespace)::attn_kernel<128, 2, true>((anonymous namespace)::AttnArgs)"
  rows = []
  for d in range(2):
    rows += [(name, "TCP_TCC_READ_REQ_sum", 1000 + 1000 * d), (name, "TCP_TCC_READ_REQ_LATENCY_sum", 300000 + 900000 * d),
             (name, "TCP_UTCL1_TRANSLATION_HIT_sum", 9990), (name, "TCP_UTCL1_TRANSLATION_MISS_sum", 10)]
  p = tmp_path / "c.csv"
  _write(p, ["Kernel_Name", "Counter_Name", "Counter_Value"], rows)
  bench.summarize_counters(str(p))
  out = capsys.readouterr().out
  assert "attn_kernel<128, 2, true>" in out and "dispatches     2" in out
  assert "500 cycles per read request" in out    # mean latency 750000 / mean requests 1500
  assert "translation miss rate 0.1000%" in out


def test_traffic_record_is_dropped_when_the_kernel_sources_change(tmp_path, monkeypatch):
  t = bench.measured_traffic()
  rec = json.load(open(os.path.join(ROOT, "profiles", "qgemm128_kernel_llama8b_decode_b128.json")))
  if rec["kernel_source_sha256_16"] == bench.kernel_source_hash():
    assert t is not None and t["read"] == rec["read_bytes_per_launch"] and t["write"] == rec["write_bytes_per_launch"]
  else:
    assert t is None
  monkeypatch.setattr(bench, "kernel_source_hash", lambda: "0" * 16)
  assert bench.measured_traffic() is None
