"""Decode throughput of the quantized rollout path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` builds the Llama-3.1-8B-shaped NF4 QLoRA model
(random-init weights, synthetic prompts), prefills batch 128 x prompt 512, runs W untimed decode
steps and times exactly K decode steps (one captured HIP graph replayed K times), then prints ONE
JSON line.  A "step" is one decode step of the whole batch: embedding -> 32 layers -> lm_head ->
greedy sampling -> token commit.  The workload is a 512-step rollout whose context grows from
512 to 1024: when K is smaller than the rollout, the K steps are taken in equal groups spread
evenly over that range (the device step counter is moved between groups, over a cache filled
beforehand; each group is bracketed by a synchronisation and only the groups are timed), so
that `value` speaks for the whole rollout (mean context 768) whatever K is; the figure over the
first K steps alone is reported beside it (`first_steps`).

Extra objects on the line:
  roofline      the kernel with the largest share of a step (the quantised GEMM), timed in
                isolation with events on its launch stream; roofline_hbm prices the same
                launches against the HBM roof
  kernels_isolated  the same measurement for every kernel family of the step, each alone in its own
                replayed graph (the linears with their LoRA down-projection and a finishing pass):
                not a breakdown of ms_per_step -- the step's kernel trace is under profiles/
  fused_logps   the standalone per-token log-probability workload at training scale
  cpu_baseline  the CPU oracle (a port of the reference's JAX path) timed on this host on a
                bounded sample and scaled linearly

`--config c1|c2|c4` measures the other rollout workloads through the public Sampler call
(their own JSON line), `--fused-logps` the standalone log-probability workload alone.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def log(*a):
  print(*a, file=sys.stderr, flush=True)


def time_loop(fn, iters, warm=2, per_graph=10):
  """Mean duration (ms) of one fn() on the GPU: `per_graph` launches are captured in one HIP graph
  (host launch overhead would otherwise floor a ~20 us kernel) and the graph is replayed between
  two events recorded on the stream it runs on."""
  import torch
  for _ in range(warm):
    fn()
  graph = torch.cuda.CUDAGraph()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
      for _ in range(per_graph):
        fn()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  graph.replay()
  reps = max(1, iters // per_graph)
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  torch.cuda.synchronize()
  e0.record()
  for _ in range(reps):
    graph.replay()
  e1.record()
  torch.cuda.synchronize()
  return e0.elapsed_time(e1) / (reps * per_graph)  # ms


def kernel_breakdown(model, runner, st, ctx, iters):
  """Times each kernel family of one layer in isolation (events on the launch stream)."""
  import torch

  from tunix_amd import _lib as L
  from tunix_amd import ops
  cfg = model.cfg
  B, S = runner.B, runner.S
  ly = model.layers[0]
  col = torch.tensor([ctx - 1], dtype=torch.int32, device=model.device)
  out = {}

  def attn():
    ad = L.AttnDesc()
    ad.B, ad.T, ad.S = B, 1, S
    ad.Hq, ad.Hkv, ad.dh = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
    ad.scale, ad.window, ad.pad_id = cfg.head_dim ** -0.5, 0, runner.pad_id
    ad.q, ad.kcache, ad.vcache = runner.q.data_ptr(), st.kcache[0].data_ptr(), st.vcache[0].data_ptr()
    ad.tokens, ad.tok_ld, ad.col_ptr = st.token_buffer.data_ptr(), st.token_buffer.shape[1], col.data_ptr()
    ad.kv_chunk, ad.ws, ad.out = runner.kv_chunk, runner.attn_ws.data_ptr(), runner.attn.data_ptr()
    ops.gqa_attn(ad)

  kv_bytes = B * cfg.num_kv_heads * ctx * cfg.head_dim * 2 * 2
  out["gqa_attn"] = {"ms": time_loop(attn, iters), "bytes": kv_bytes, "flops": 0, "per_step": cfg.num_layers}

  def lin(key, x, y, epi=L.TNX_EPI_STORE, residual=None):
    """One fused linear as the decode step runs it (LoRA down-projection + GEMM + split-k sum)
    and, separately, its main GEMM launch alone (`kernel_ms`)."""
    import ctypes

    f = ly[key]
    nbytes = f.codes.numel() * 4 + f.scales.numel() * 2
    if f.has_lora:
      nbytes += (f.K * f.r * len(f.names) + f.N * f.r) * 2
    nbytes += B * f.K * 2 + B * (f.N // (2 if f.interleave2 else 1)) * 2
    ms = time_loop(lambda: runner.linear(f, x, y, B, epilogue=epi, residual=residual), iters)
    split = runner._split_k(f, B)
    d = ops.make_qlinear_desc(
        M=B, K=f.K, N=f.N, group=f.group, qtype=f.qtype, x=x, codes=f.codes, scales=f.scales, y=y,
        epilogue=epi, residual=residual, lora_rank=f.rp,
        lora_nseg=(-1 if f.interleave2 else len(f.names)), lora_seg_end=f.seg_end,
        lora_seg_toff=f.seg_toff, t=runner.t if f.has_lora else None, t_ld=runner.t.shape[1],
        lora_b=f.b_t if f.has_lora else None, lora_scale=f.lora_scale, split_k=split,
        ws=runner.splitk_ws if split > 1 else None)
    stream = torch.cuda.current_stream

    def gemm_only():
      L.check(L.lib().tnx_qlinear_lora(stream().cuda_stream, ctypes.byref(d)), "tnx_qlinear_lora")

    kms = time_loop(gemm_only, iters)
    return {"ms": ms, "kernel_ms": kms, "bytes": nbytes, "flops": 2.0 * B * f.K * f.N,
            "per_step": cfg.num_layers, "split_k": split}

  out["qlinear_qkv"] = lin("qkv", runner.xn, runner.qkv)
  out["qlinear_o"] = lin("o", runner.attn, runner.tmp)
  out["qlinear_gate_up"] = lin("gu", runner.xn, runner.act, L.TNX_EPI_SILU_MUL)
  out["qlinear_down"] = lin("down", runner.act, runner.tmp)
  head_bytes = model.weight_bytes()["head"] + B * cfg.embed_dim * 2
  ms = time_loop(lambda: runner.run_head(runner.xn, B, best_id=runner.best_id,
                                         best_logp=runner.best_logp), iters)
  out["lmhead_logp"] = {"ms": ms, "bytes": head_bytes, "flops": 2.0 * B * cfg.embed_dim * cfg.vocab_size,
                        "per_step": 1}
  for v in out.values():
    v["gbs"] = v["bytes"] / (v["ms"] * 1e-3) / 1e9
    v["tflops"] = v["flops"] / (v["ms"] * 1e-3) / 1e12
    v["step_ms"] = v["ms"] * v["per_step"]
  return out


def many_rows_breakdown(model, rows, iters):
  """The four linears of a layer at `rows` activation rows (one prefill / per-token-logps chunk):
  the regime of the 128 x 256-tile GEMM kernel, bound by the matrix pipe.  Returns per-linear
  microseconds and TFLOP/s and their mean as a fraction of the dense bf16 MFMA peak."""
  import torch

  from tunix_amd import _lib as L
  from tunix_amd import ops
  dev, ly = model.device, model.layers[0]
  bf = torch.bfloat16
  out = {}
  for key, epi in (("qkv", L.TNX_EPI_STORE), ("o", L.TNX_EPI_STORE), ("gu", L.TNX_EPI_SILU_MUL),
                   ("down", L.TNX_EPI_STORE)):
    f = ly[key]
    x = torch.randn(rows, f.K, device=dev).to(bf)
    y = torch.empty(rows, f.N // (2 if f.interleave2 else 1), dtype=bf, device=dev)
    t = torch.randn(rows, max(f.rp * len(f.names), 32), device=dev).to(bf) if f.has_lora else None
    d = ops.make_qlinear_desc(
        M=rows, K=f.K, N=f.N, group=f.group, qtype=f.qtype, x=x, codes=f.codes, scales=f.scales, y=y,
        epilogue=epi, lora_rank=f.rp, lora_nseg=(-1 if f.interleave2 else len(f.names)),
        lora_seg_end=f.seg_end, lora_seg_toff=f.seg_toff, t=t, t_ld=t.shape[1] if t is not None else 0,
        lora_b=f.b_t if f.has_lora else None, lora_scale=f.lora_scale, w_expanded=f.expanded)
    ms = time_loop(lambda: ops.qlinear(d), iters, per_graph=2, warm=1)
    flops = 2.0 * rows * f.K * f.N
    out[key] = {"us": round(ms * 1e3, 1), "TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1)}
    del x, y, t
  tot_flops = sum(2.0 * rows * ly[k].K * ly[k].N for k in out)
  tot_s = sum(v["us"] for v in out.values()) * 1e-6
  tf = tot_flops / tot_s / 1e12
  return {"kernel": "qgemm_wide_kernel", "rows": rows, "bound": "mfma", "achieved": round(tf, 1),
          "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
          "linears": out}


# HBM bytes of one qgemm128 launch on the default workload come from counter runs of this script
# (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over `--kernels-only`), kept in a tracked summary next
# to a hash of the kernel's sources: the figure is reported only while the sources are the ones it
# was measured on.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qgemm128_kernel_llama8b_decode_b128.json")
# everything that decides what a GEMM launch reads and writes: the kernel and its tile loop, the
# store-policy helpers, the dispatch, and the host's choice of the k split
KERNEL_SOURCES = ("csrc/qgemm128.h", "csrc/gemm_tile.h", "csrc/common.h", "csrc/qlinear.hip", "model.py")


def kernel_source_hash():
  return source_hash(KERNEL_SOURCES)


def measured_traffic():
  """{"traffic": bytes per launch, "read": ..., "write": ...} from the tracked counter summary, or
  None when there is none for the current kernel sources."""
  try:
    with open(TRAFFIC_PROFILE) as f:
      prof = json.load(f)
  except (OSError, ValueError):
    return None
  if prof.get("kernel_source_sha256_16") != kernel_source_hash():
    return None
  return {"traffic": int(prof["read_bytes_per_launch"] + prof["write_bytes_per_launch"]),
          "read": int(prof["read_bytes_per_launch"]), "write": int(prof["write_bytes_per_launch"])}


def write_traffic_profile(fetch_csv, write_csv):
  """Rebuilds the tracked traffic record from two `rocprofv3 --pmc` runs of
  `bench.py --kernels-only` (FETCH_SIZE in one, WRITE_SIZE in the other; KiB per dispatch).  The
  GEMM's dispatches come in four runs, in the order the breakdown launches them (qkv, o, gate|up,
  down); the 1 GiB `stream_read_kernel` launches of the same runs give the scale of FETCH_SIZE
  for the 8- / 16-byte-per-lane buffer loads every streaming kernel here uses, a 1002 MiB torch
  copy the scale of both counters for plain copies."""
  import csv

  def runs(path, counter):
    rows = [r for r in csv.DictReader(open(path)) if r["Counter_Name"] == counter]
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    gemm, stream, copy = [], {}, []
    for r in rows:
      name, grid, val = r["Kernel_Name"], r.get("Grid_Size", "?"), float(r["Counter_Value"])
      if "qgemm128_kernel" in name:
        if gemm and gemm[-1][0] == grid:
          gemm[-1][1].append(val)
        else:
          gemm.append((grid, [val]))
      elif "stream_read_kernel" in name:
        stream.setdefault("stream_read_kernel<16>" if "<16>" in name else "stream_read_kernel<8>", []).append(val)
      elif "copy" in name.lower() and val > 1000000:
        copy.append(val)
    gemm = [(g, v) for g, v in gemm if len(v) >= 5]
    if len(gemm) != 4:
      raise SystemExit(f"expected four runs of qgemm128 dispatches in {path}, found {len(gemm)}")
    return [sum(v) / len(v) for _, v in gemm], {k: sum(v) / len(v) for k, v in stream.items()}, copy

  f_shapes, f_stream, f_copy = runs(fetch_csv, "FETCH_SIZE")
  w_shapes, _, w_copy = runs(write_csv, "WRITE_SIZE")
  true_kib = (1 << 30) / 1024.0
  factors = [true_kib / v for v in f_stream.values()]
  if not factors or max(factors) - min(factors) > 0.02 * max(factors):
    raise SystemExit(f"no consistent stream_read yardstick in {fetch_csv}: {f_stream}")
  fetch_factor = round(sum(factors) / len(factors), 3)
  names = ["qkv", "o", "gate_up", "down"]
  rec = {
      "kernel": "qgemm128_kernel<2,2,8>",
      "workload": "Llama-3.1-8B NF4(g64)+LoRA r64 decode, batch 128: mean over the qkv / o / gate|up / down "
                  "launches of a layer",
      "kernel_source_sha256_16": kernel_source_hash(),
      "kernel_sources": list(KERNEL_SOURCES),
      "fetch_counter_factor": fetch_factor,
      "write_counter_factor": 1.0,
      "yardsticks": {**{f"{k} over 1 GiB": {"FETCH_SIZE_kib": round(v, 1), "true_kib": int(true_kib)}
                        for k, v in f_stream.items()},
                     "largest torch copies": {"FETCH_SIZE_kib": [round(v) for v in f_copy[:3]],
                                              "WRITE_SIZE_kib": [round(v) for v in w_copy[:3]]}},
      "per_shape_counter_kib": {n: {"fetch_kib": round(f, 1), "write_kib": round(w, 1)}
                                for n, f, w in zip(names, f_shapes, w_shapes)},
      "read_bytes_per_launch": int(sum(f_shapes) / 4 * 1024 * fetch_factor),
      "write_bytes_per_launch": int(sum(w_shapes) / 4 * 1024),
  }
  with open(TRAFFIC_PROFILE, "w") as f:
    json.dump(rec, f, indent=1)
    f.write("\n")
  print(json.dumps(rec, indent=1))


# The same for the many-row kernel on the standalone log-probability pass (one launch = 16384 rows
# x 128256 columns): counter runs of `bench.py --fused-logps`.
FUSED_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qgemm_wide_kernel_fused_logps_131072rows.json")
FUSED_KERNEL_SOURCES = ("csrc/qgemm_wide.h", "csrc/gemm_tile.h", "csrc/common.h", "csrc/qlinear.hip",
                        "csrc/lmhead.hip")


def source_hash(names):
  import hashlib
  h = hashlib.sha256()
  for name in names:
    with open(os.path.join(ROOT, "tunix_amd", name), "rb") as f:
      h.update(f.read())
  return h.hexdigest()[:16]


def fused_measured_traffic():
  try:
    with open(FUSED_TRAFFIC_PROFILE) as f:
      prof = json.load(f)
  except (OSError, ValueError):
    return None
  if prof.get("kernel_source_sha256_16") != source_hash(FUSED_KERNEL_SOURCES):
    return None
  return int(prof["read_bytes_per_launch"] + prof["write_bytes_per_launch"])


def write_fused_traffic_profile(fetch_csv, write_csv):
  """Rebuilds the tracked traffic record of the log-probability pass from two `rocprofv3 --pmc`
  runs of `bench.py --fused-logps` (FETCH_SIZE in one, WRITE_SIZE in the other; KiB per dispatch of
  qgemm_wide_kernel).  FETCH_SIZE is scaled with the factor the decode GEMM's record holds for
  buffer loads (its 1 GiB yardstick reads)."""
  import csv

  def mean(path, counter):
    v = [float(r["Counter_Value"]) for r in csv.DictReader(open(path))
         if r["Counter_Name"] == counter and "qgemm_wide_kernel" in r["Kernel_Name"]]
    if not v:
      raise SystemExit(f"no qgemm_wide_kernel dispatches with {counter} in {path}")
    return sum(v) / len(v), len(v)

  with open(TRAFFIC_PROFILE) as f:
    factor = float(json.load(f)["fetch_counter_factor"])
  fk, nf = mean(fetch_csv, "FETCH_SIZE")
  wk, nw = mean(write_csv, "WRITE_SIZE")
  rows, D, V, r = 16384, 4096, 128256, 64
  rec = {
      "kernel": "qgemm_wide_kernel (head-statistics epilogue)",
      "workload": "one launch of the standalone log-probability pass: 16384 rows x 4096 -> 128256, int4 g128 + LoRA r64, "
                  "the head read from its expanded bf16 copy",
      "kernel_source_sha256_16": source_hash(FUSED_KERNEL_SOURCES),
      "kernel_sources": list(FUSED_KERNEL_SOURCES),
      "fetch_counter_factor": factor, "write_counter_factor": 1.0,
      "dispatches": {"fetch_run": nf, "write_run": nw},
      "counter_kib_per_launch": {"FETCH_SIZE": round(fk, 1), "WRITE_SIZE": round(wk, 1)},
      "read_bytes_per_launch": int(fk * 1024 * factor), "write_bytes_per_launch": int(wk * 1024),
      # what one launch must move: hidden rows + the head's bf16 copy + adapter once, statistics out
      "algorithmic_bytes_per_launch": int(rows * D * 2 + D * V * 2 + V * r * 2 + rows * r * 2 + rows * (V // 128) * 16),
  }
  with open(FUSED_TRAFFIC_PROFILE, "w") as f:
    json.dump(rec, f, indent=1)
    f.write("\n")
  print(json.dumps(rec, indent=1))


def rooflines(kern, default_workload=False):
  """The dominant kernel of a step is the quantised GEMM (one kernel, launched for the four
  linears of every layer).  One launch = the mean over those four shapes.  At 128 rows its
  arithmetic intensity (2 * 128 flop per 0.53 B of packed weight = 483 flop/B) is past the
  machine's ridge (2.5 PFLOP/s / 8 TB/s = 312 flop/B), so the bounding roof is the bf16 MFMA
  peak; the same launches priced against the HBM roof are reported beside it."""
  names = [k for k in kern if k.startswith("qlinear")]
  flops = sum(kern[k]["flops"] for k in names) / len(names)
  nbytes = sum(kern[k]["bytes"] for k in names) / len(names)
  us = sum(kern[k]["kernel_ms"] for k in names) / len(names) * 1e3
  tf = flops / (us * 1e-6) / 1e12
  gbs = nbytes / (us * 1e-6) / 1e9
  meas = measured_traffic() if default_workload else None
  roofline = {"kernel": "qgemm128_kernel", "bound": "mfma", "achieved": round(tf, 1),
              "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
              "traffic": meas["traffic"] if meas else None,
              "traffic_read": meas["read"] if meas else None, "traffic_write": meas["write"] if meas else None,
              "us_per_launch": round(us, 2), "algorithmic_flops": flops,
              "algorithmic_bytes": nbytes,
              "launch_shapes_us": {k: round(kern[k]["kernel_ms"] * 1e3, 2) for k in names}}
  roofline_hbm = {"kernel": "qgemm128_kernel", "bound": "hbm", "achieved": round(gbs, 1),
                  "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)}
  return roofline, roofline_hbm


def cpu_baseline(cfg_full, B, ctx, S, threads):
  """CPU oracle on a bounded sample: 1 layer x 2 decode steps at context `ctx` + the lm_head,
  scaled linearly to the full depth."""
  import dataclasses

  import numpy as np
  import torch

  from oracle import model_ref
  from oracle import utils_ref
  from tunix_amd import dummy_model
  torch.set_num_threads(threads)
  cfg = dataclasses.replace(cfg_full, num_layers=1, vocab_size=1024)
  w = dummy_model.create_dummy_weights(cfg, seed=3)
  ref = model_ref.RefModel(cfg, w, bf16=True, acc=torch.float32)
  cache = ref.init_cache(B, S)
  for k, v in cache:
    k.normal_()
    v.normal_()
  tokens = torch.randint(1, cfg.vocab_size, (B, 1))
  positions = torch.full((B, 1), ctx - 1, dtype=torch.int64)
  mask = torch.from_numpy(utils_ref.compute_attention_masks(ctx - 1, S, np.zeros((B, S), dtype=bool)))
  x = ref.embed(tokens)
  ref.layer(0, x, positions, cache, mask, ctx - 1)  # warm
  t0 = time.perf_counter()
  n = 2
  for _ in range(n):
    ref.layer(0, x, positions, cache, mask, ctx - 1)
  t_layer = (time.perf_counter() - t0) / n
  D, V = cfg_full.embed_dim, cfg_full.vocab_size
  head = (torch.randn(D, V // 8) * 0.02).to(torch.bfloat16).float()
  h = torch.randn(B, D).to(torch.bfloat16).float()
  t0 = time.perf_counter()
  for _ in range(2):
    lg = (h @ head).to(torch.bfloat16).float()
    lg.argmax(-1)
  t_head = (time.perf_counter() - t0) / 2 * 8
  t_step = cfg_full.num_layers * t_layer + t_head
  return {"value": B / t_step, "unit": "tokens/s", "cores": threads, "kind": "port",
          "sample": (f"1 of {cfg_full.num_layers} layers x {n} decode steps at context {ctx} "
                     f"(dense mask over the {S}-slot cache, fp32 torch matmuls) + 1/8 of the lm_head "
                     "columns, scaled linearly (extrapolated)"),
          "layer_s": t_layer, "head_s": t_head}


def summarize_step_trace(path):
  """Prints the kernels of the last complete decode step found in a `rocprofv3 --kernel-trace`
  csv of this script (a step = the dispatches between two sample_commit kernels): count, total
  and mean duration per kernel, start-to-start time included (the dependent-launch gaps)."""
  import collections
  import csv
  rows = sorted(csv.DictReader(open(path)), key=lambda r: int(r["Start_Timestamp"]))
  commits = [i for i, r in enumerate(rows) if "sample_commit" in r["Kernel_Name"]]
  if len(commits) < 3:
    raise SystemExit("the trace holds fewer than two decode steps")
  step = rows[commits[-3] + 1: commits[-2] + 1]
  t0, t1 = int(step[0]["Start_Timestamp"]), int(step[-1]["End_Timestamp"])
  agg = collections.OrderedDict()
  for r, nxt in zip(step, step[1:] + [None]):
    name = r["Kernel_Name"].replace("(anonymous namespace)::", "").replace("void ", "").split("(")[0]
    busy = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
    span = (int(nxt["Start_Timestamp"]) if nxt else t1) - int(r["Start_Timestamp"])
    e = agg.setdefault(name, [0, 0, 0])
    e[0] += 1
    e[1] += busy
    e[2] += span
  print(f"one decode step: {(t1 - t0) / 1e3:.1f} us, {len(step)} kernels")
  print(f"| {'kernel':34s} | calls | total us | mean us | mean start-to-start us |")
  print(f"|{'-' * 36}|-------|----------|---------|------------------------|")
  for name, (n, busy, span) in agg.items():
    print(f"| {name:34s} | {n:5d} | {busy / 1e3:8.1f} | {busy / n / 1e3:7.2f} | {span / n / 1e3:22.2f} |")


def summarize_counters(path, by_grid=False):
  """Prints, per kernel (by_grid: per kernel and grid size, which keeps a kernel's decode-sized
  launches apart from its many-row ones), the mean of every counter in a `rocprofv3 --pmc ...`
  counter-collection csv of this script (one row per dispatch and counter), and, where the
  counters are there, the L1 -> L2 read latency per request and the address-translation miss rate."""
  import collections
  import csv
  import re
  agg = collections.defaultdict(lambda: collections.defaultdict(list))
  for row in csv.DictReader(open(path)):
    name = row["Kernel_Name"].replace("(anonymous namespace)::", "")
    m = re.search(r"([A-Za-z_0-9]+(<[^(]*>)?)\(", name)
    key = (m.group(1) if m else name)[:48]
    if by_grid:
      key = f"{key[:34]} grid {row.get('Grid_Size', '?')}"
    agg[key][row["Counter_Name"]].append(float(row["Counter_Value"]))
  for name, counters in sorted(agg.items()):
    mean = {c: sum(v) / len(v) for c, v in counters.items()}
    n = max(len(v) for v in counters.values())
    line = f"{name:48s} dispatches {n:5d}  " + "  ".join(f"{c} {v:.0f}" for c, v in sorted(mean.items()))
    req, lat = mean.get("TCP_TCC_READ_REQ_sum"), mean.get("TCP_TCC_READ_REQ_LATENCY_sum")
    if req and lat is not None:
      line += f"  | {lat / req:.0f} cycles per read request"
    hit, miss = mean.get("TCP_UTCL1_TRANSLATION_HIT_sum"), mean.get("TCP_UTCL1_TRANSLATION_MISS_sum")
    if hit is not None and miss is not None and hit + miss > 0:
      line += f"  | translation miss rate {miss / (hit + miss):.4%}"
    print(line)


def fused_logps_workload(rows, chunk, iters, expanded=True):
  """The standalone per-token log-probability case at training scale: hidden states
  [rows, 4096] bf16 N(0,1) x an int4 (group 128) + LoRA r64 lm_head of 128256 columns ->
  log-softmax -> gather at random targets -> GRPO clipped ratio; logits never reach HBM.
  expanded: the kernel reads the frozen head from its converted copy (tnx_qw_expand, what
  QLoRAModel keeps for its many-row calls; same bits as converting the codes in the loop, which
  expanded=False measures).  Timed with HIP events around `iters` passes after one warm-up pass."""
  import torch
  from tunix_amd import _lib as L
  from tunix_amd import ops
  dev = torch.device("cuda:0")
  D, V, r, group = 4096, 128256, 64, 128
  g = torch.Generator(device=dev).manual_seed(20254)
  x = torch.randn(rows, D, generator=g, device=dev).to(torch.bfloat16)
  w = (torch.randn(D, V, generator=g, device=dev) * 0.02).to(torch.bfloat16)
  a_t = (torch.randn(r, D, generator=g, device=dev) * 0.02).to(torch.bfloat16)
  b_t = (torch.randn(V, r, generator=g, device=dev) * 0.01).to(torch.bfloat16)
  targets = torch.randint(0, V, (rows,), generator=g, device=dev, dtype=torch.int32)
  codes, scales = ops.quantize_pack(w, group, 0)
  del w
  w_exp = ops.qw_expand(codes, scales, D, V, group, 0) if expanded else None
  t = torch.zeros(rows, r, dtype=torch.bfloat16, device=dev)
  nvb = ops.lmhead_nblocks(V)
  part = torch.empty(chunk * nvb * 4, dtype=torch.float32, device=dev)
  logp = torch.empty(rows, dtype=torch.float32, device=dev)
  ref = torch.empty(rows, dtype=torch.float32, device=dev)
  adv = torch.randn(max(rows // 4096, 1), generator=g, device=dev)
  ratio, loss = torch.empty(rows, device=dev), torch.empty(rows, device=dev)

  def one_pass():
    ops.lora_down(x, a_t, t)
    for r0 in range(0, rows, chunk):
      d = L.LmHeadDesc()
      d.M, d.D, d.V = min(chunk, rows - r0), D, V
      d.x, d.codes, d.scales, d.group, d.qtype = x[r0:].data_ptr(), codes.data_ptr(), scales.data_ptr(), group, 0
      d.lora_rank, d.t, d.t_ld, d.lora_b, d.lora_scale = r, t[r0:].data_ptr(), r, b_t.data_ptr(), 1.0
      d.temperature = 1.0
      if w_exp is not None:
        d.w_expanded = w_exp.data_ptr()
      d.targets, d.part, d.target_logp = targets[r0:].data_ptr(), part.data_ptr(), logp[r0:].data_ptr()
      ops.lmhead(d)
    ops.grpo_ratio(logp, ref, adv, min(4096, rows), 0.2, 0.2, ratio=ratio, loss=loss)

  one_pass()
  ref.copy_(logp + 0.05 * torch.randn(rows, generator=g, device=dev))
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(iters):
    one_pass()
  e1.record()
  torch.cuda.synchronize()
  ms = e0.elapsed_time(e1) / iters
  flops = 2.0 * rows * D * V + 2.0 * rows * r * (D + V)
  assert bool(torch.isfinite(logp).all()) and bool(torch.isfinite(loss).all())
  del x, codes, scales, b_t, part, w_exp
  torch.cuda.empty_cache()
  return {
      "metric": "fused per-token logps rows/sec @1 MI355X (int4 g128 + LoRA r64 head, 4096 x 128256)",
      "value": round(rows / (ms * 1e-3), 1), "unit": "rows/s", "n_gpus": 1, "steps": iters, "warmup": 1,
      "ms_per_step": round(ms, 3), "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
      "config": {"workload": "standalone fused lm_head -> log-softmax -> gather -> GRPO ratio", "rows": rows,
                 "rows_per_launch": chunk,
                 "head_operand": "expanded bf16 copy of the int4 head" if expanded else "int4 codes converted in the loop"},
      "roofline": {"kernel": "qgemm_wide_kernel (statistics epilogue)", "bound": "mfma",
                   "achieved": round(flops / (ms * 1e-3) / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                   "frac": round(flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                   # HBM bytes of one 16384-row launch, from the tracked counter record
                   "traffic": fused_measured_traffic() if chunk == 16384 and expanded else None}}


def config_workload(name, steps):
  """The other rollout workloads, through the public Sampler call: two rollouts of different
  length, so that prefill, graph capture and host work cancel; ms per decode step from the
  difference.  c1: tiny Qwen3-style decoder, batch 8, prompt 64, greedy.  c2: Gemma3-1B shape,
  batch 64, prompt 256, temperature 1.0 / top-k 50.  c4: Qwen3-30B-A3B shape (128 experts, top-8),
  batch 64, prompt 1024, greedy."""
  import numpy as np
  import torch

  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  dev = torch.device("cuda:0")
  spec = {
      "c1": (config.tiny_qwen3(), 8, 64, 64, dict(), "tiny Qwen3-style decoder (2 layers, D512, V32000, int4 g64 + LoRA r8), greedy"),
      "c2": (config.gemma3_1b(), 64, 256, 256, dict(temperature=1.0, top_p=1.0, top_k=50, seed=7),
             "Gemma3-1B-shaped (26 layers, V262144 tied head, int4 g128 + LoRA r16), temperature 1.0 top-k 50"),
      "c4": (config.qwen3_30b_a3b(), 64, 1024, 256, dict(),
             "Qwen3-30B-A3B-shaped MoE (48 layers, 128 experts top-8, int4 g128, LoRA r16 on attention), greedy"),
  }[name]
  cfg, B, P, T, kw, label = spec
  t0 = time.time()
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20250 + int(name[1]), device=dev), dev)
  torch.cuda.empty_cache()
  log(f"{name}: model built in {time.time() - t0:.1f}s; bytes per step {model.weight_bytes()}")
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(P + T, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  ids = np.random.Generator(np.random.PCG64(20250)).integers(1, cfg.vocab_size, size=(B, P)).astype(np.int32)
  prompts = [ids[b] for b in range(B)]
  steps = max(1, min(steps, T - 8))
  times, stats = [], []
  for n in (4, 4, 4 + steps):     # the first call also pays the lazy module loads
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sampler(prompts, n, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1], **kw)
    torch.cuda.synchronize()
    times.append(time.perf_counter() - t0)
    stats.append(dict(sampler.last_stats))
  ms = (times[2] - times[1]) / steps * 1e3
  wb = model.weight_bytes()
  mean_ctx = P + 4 + steps / 2.0
  window = cfg.sliding_window or 0
  kv = 0
  for i in range(cfg.num_layers):
    ctx = min(mean_ctx, window) if (window and cfg.is_local_layer(i)) else mean_ctx
    kv += B * cfg.num_kv_heads * ctx * cfg.head_dim * 4
  step_bytes = wb["quantized"] + wb["lora"] + wb["head"] + kv
  return {
      "metric": f"decode tokens/sec @1 MI355X ({name})", "value": round(B / (ms * 1e-3), 1), "unit": "tokens/s",
      "n_gpus": 1, "steps": steps, "warmup": 4, "ms_per_step": round(ms, 4), "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
      "config": {"workload": label, "layers": cfg.num_layers, "global_batch": B, "prompt_len": P, "gen_len": T,
                 "context_range": [P + 4, P + 4 + steps], "parallelism": "single GPU"},
      "prefill_s": round(stats[2]["prefill_ms"] * 1e-3, 3),
      "hbm_roofline_frac_step": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "step_bytes": int(step_bytes)}


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=508)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--batch", type=int, default=128)
  ap.add_argument("--prompt", type=int, default=512)
  ap.add_argument("--gen", type=int, default=512)
  ap.add_argument("--layers", type=int, default=0, help="debug only: fewer layers (invalidates the metric)")
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--kernel-iters", type=int, default=20)
  ap.add_argument("--sampling-steps", type=int, default=64,
                  help="decode steps of the extra temperature-1.0 measurement (0: skip it)")
  ap.add_argument("--kernels-only", action="store_true",
                  help="profiling aid: one layer, no prefill / decode; only the per-kernel loops at "
                       "context prompt + gen / 2 (prints the kernel table, not the metric)")
  ap.add_argument("--fused-logps", action="store_true",
                  help="instead of the decode benchmark: the standalone fused per-token log-probability "
                       "workload (32 x 4096 rows, quantised 128256-column head), its own JSON line")
  ap.add_argument("--fused-logps-rows", type=int, default=131072)
  ap.add_argument("--fused-logps-codes", action="store_true",
                  help="the log-probability workload converts the head's int4 codes in its loop "
                       "instead of reading the head's expanded copy")
  ap.add_argument("--no-fused-logps", action="store_true",
                  help="leave the standalone log-probability workload out of the default run's line")
  ap.add_argument("--config", choices=["c1", "c2", "c3", "c4"], default="c3",
                  help="c3 (default): the headline workload; c1 / c2 / c4: the other rollout workloads through "
                       "the public Sampler call, their own JSON line")
  ap.add_argument("--contiguous", action="store_true",
                  help="time the K steps that follow the prefill directly instead of K steps spread over the "
                       "rollout's context range")
  ap.add_argument("--summarize-trace", metavar="CSV", default=None,
                  help="no GPU work: tabulate one decode step of a rocprofv3 kernel-trace csv of this script")
  ap.add_argument("--write-fused-traffic-profile", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), default=None,
                  help="rebuild profiles/qgemm_wide_kernel_fused_logps_131072rows.json from the counter csv files "
                       "of two `rocprofv3 --pmc FETCH_SIZE | WRITE_SIZE -- python3 bench.py --fused-logps` runs")
  ap.add_argument("--write-traffic-profile", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), default=None,
                  help="no GPU work: rebuild profiles/qgemm128_kernel_llama8b_decode_b128.json from the counter csvs "
                       "of two `rocprofv3 --pmc FETCH_SIZE | WRITE_SIZE -- python3 bench.py --kernels-only` runs")
  ap.add_argument("--summarize-counters", metavar="CSV", default=None,
                  help="no GPU work: per-kernel means of a rocprofv3 --pmc counter-collection csv of this script")
  ap.add_argument("--by-grid", action="store_true", help="with --summarize-counters: one line per kernel and grid size")
  args = ap.parse_args()
  if args.fused_logps:
    if args.gpus != 1:
      sys.exit("bench.py measures one GPU; --gpus must be 1")
    print(json.dumps(fused_logps_workload(args.fused_logps_rows, 16384, max(1, args.kernel_iters // 10),
                                          expanded=not args.fused_logps_codes)), flush=True)
    return
  if args.summarize_trace:
    summarize_step_trace(args.summarize_trace)
    return
  if args.summarize_counters:
    summarize_counters(args.summarize_counters, args.by_grid)
    return
  if args.write_fused_traffic_profile:
    write_fused_traffic_profile(*args.write_fused_traffic_profile)
    return
  if args.write_traffic_profile:
    write_traffic_profile(*args.write_traffic_profile)
    return
  if args.gpus != 1:
    print("bench.py measures one GPU: this build has no multi-GPU path (the decode path shards "
          "by batch rows with no exchange); run with --gpus 1", file=sys.stderr)
    sys.exit(2)

  if args.config != "c3":
    print(json.dumps(config_workload(args.config, args.steps if args.steps != 508 else 200)), flush=True)
    return

  import numpy as np
  import torch

  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.sampler import _SamplingState
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel, Runner

  assert torch.cuda.is_available(), "bench.py needs a GPU"
  dev = torch.device("cuda:0")
  cfg = config.llama31_8b()
  if args.layers:
    cfg = config.llama31_8b(num_layers=args.layers)
  B, P, T = args.batch, args.prompt, args.gen
  S = P + T
  if args.kernels_only:
    cfg = config.llama31_8b(num_layers=1)
    model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20253, device=dev), dev)
    ids = np.random.Generator(np.random.PCG64(20253)).integers(1, cfg.vocab_size, size=(B, P)).astype(np.int32)
    st = _SamplingState(model, ids, S, S, 0, False, False)
    st.token_buffer.fill_(5)
    for kc, vc in zip(st.kcache, st.vcache):
      kc.normal_()
      vc.normal_()
    runner = Runner(model, B, 1, S, 0)
    for buf in (runner.xn, runner.attn, runner.act, runner.q):
      buf.normal_()
    kern = kernel_breakdown(model, runner, st, P + T // 2, args.kernel_iters)
    roofline, roofline_hbm = rooflines(kern, default_workload=(B == 128))
    # a plain device copy of known size (256 MiB read + 256 MiB written): the yardstick that
    # scales the FETCH_SIZE / WRITE_SIZE counters of a counter-collection run of this command
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
      dst.copy_(src)
    # and a second yardstick for reads: 1 GiB fetched once with the 16-byte-per-lane buffer loads
    # the GEMM, attention and head kernels stream their operands with (stream_read_kernel)
    # (a probe of this benchmark, in its own shared object: not part of the product library)
    import ctypes
    probe = ctypes.CDLL(os.path.join(ROOT, "tunix_amd", "libtunix_probe.so"))
    probe.tnx_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int,
                                            ctypes.c_void_p]
    big = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(64, dtype=torch.int32, device=dev)
    for width in (16, 8, 16, 8):      # 8 bytes per lane: the GEMM's packed-code loads
      rc = probe.tnx_probe_stream_read(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
                                       ctypes.c_void_p(big.data_ptr()), big.numel(), width,
                                       ctypes.c_void_p(sink.data_ptr()))
      assert rc == 0, "stream-read probe failed"
    torch.cuda.synchronize()
    del big
    many = many_rows_breakdown(model, 8192, max(2, args.kernel_iters // 5))
    print(json.dumps({"kernels_only": True, "context": P + T // 2, "roofline": roofline,
                      "roofline_hbm": roofline_hbm, "roofline_many_rows": many,
                      "kernels": {k: {"us": round(v["ms"] * 1e3, 2),
                                      "gemm_us": round(v.get("kernel_ms", v["ms"]) * 1e3, 2)}
                                  for k, v in kern.items()}}), flush=True)
    return
  W = max(1, args.warmup)
  K = args.steps
  if W + K > T - 1:
    K = T - 1 - W
    log(f"steps clamped to {K}: a rollout of {T} tokens has {T - 1} decode steps")

  t0 = time.time()
  weights = dummy_model.create_dummy_weights(cfg, seed=20253, device=dev)
  model = QLoRAModel(cfg, weights, dev)
  del weights
  torch.cuda.empty_cache()
  log(f"model built in {time.time() - t0:.1f}s; bytes per step {model.weight_bytes()}")

  pad = 0
  tok = IdTokenizer(cfg.vocab_size, pad_id=pad, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(S, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  rng = np.random.Generator(np.random.PCG64(20253))
  ids = rng.integers(1, cfg.vocab_size, size=(B, P)).astype(np.int32)
  st = _SamplingState(model, ids, S, S, pad, False, False)
  mode = {"name": "greedy", "forbidden": None, "eos": torch.tensor([-1], dtype=torch.int32, device=dev)}
  runner = Runner(model, B, 1, S, pad)
  torch.cuda.synchronize()
  t0 = time.time()
  sampler._prefill(st, runner, mode, False)
  torch.cuda.synchronize()
  prefill_s = time.time() - t0
  log(f"prefill {B}x{P}: {prefill_s:.2f}s")

  for _ in range(W):
    sampler._decode_step(runner, st, mode)
  graph = torch.cuda.CUDAGraph()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
      sampler._decode_step(runner, st, mode)
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  step_first = int(st.step.item())
  last_step = P + T - 2          # the step counter's value before the rollout's last decode step

  def timed(n):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
      graph.replay()
    torch.cuda.synchronize()
    return time.perf_counter() - t0

  first_steps = None
  if args.contiguous or K >= last_step - step_first:
    dt = timed(K)
    step_last = int(st.step.item())
    assert step_last - step_first == K, (step_first, step_last, K)
    contexts = [step_first + 1 + i for i in range(K)]
    groups = 1
  else:
    # K steps in `groups` equal groups whose starting points are spread evenly from the step after
    # the warm-up to the end of the rollout.  The part of the rollout that is skipped must look
    # like a rollout to the kernels: the cache slots and token columns between the groups are
    # filled with values of the kind a decode step writes (copies of the prompt's keys and values,
    # random non-pad token ids: every key is attended).
    groups = max(g for g in (8, 5, 4, 2, 1) if K % g == 0 and K // g >= 1)
    per = K // groups
    gen = torch.Generator(device=dev).manual_seed(20253)
    st.token_buffer[:, step_first + 1:] = torch.randint(1, cfg.vocab_size, (B, S - step_first - 1), generator=gen,
                                                        device=dev, dtype=torch.int32)
    n_fill = S - step_first - 1
    for kc, vc in zip(st.kcache, st.vcache):   # keys / values of the kind the model writes: the prompt's own
      kc[:, :, step_first + 1:] = kc[:, :, :n_fill]
      vc[:, :, step_first + 1:] = vc[:, :, :n_fill]
    starts = [step_first + round(g * (last_step + 1 - per - step_first) / max(groups - 1, 1)) for g in range(groups)]
    dt, contexts = 0.0, []
    first_dt = None
    for s0 in starts:
      st.step.fill_(s0)
      dt_g = timed(per)
      assert int(st.step.item()) == s0 + per
      contexts += [s0 + 1 + i for i in range(per)]
      dt += dt_g
      if first_dt is None:
        first_dt = dt_g
    first_steps = {"steps": per, "ms_per_step": round(first_dt / per * 1e3, 4),
                   "tokens_per_s": round(B * per / first_dt, 1), "context_range": [starts[0] + 1, starts[0] + per]}
    step_last = starts[-1] + per
  ms_per_step = dt / K * 1e3
  value = B * K / dt
  mean_ctx = sum(contexts) / len(contexts) + 0.5
  log(f"decode: {K} steps in {groups} group(s), {ms_per_step:.3f} ms/step, {value:.0f} tokens/s, "
      f"mean context {mean_ctx:.1f} (contexts {contexts[0]}..{contexts[-1]})")

  # The workload's other variant: temperature 1.0, top_p 1.0, no top-k (the reference's default
  # rollout sampling: one categorical draw over the whole vocabulary per row and step), through
  # the public Sampler call; two rollouts of different length, so that prefill, graph capture
  # and host work cancel.  Reported beside the headline (greedy) number, never instead of it.
  sampling = recipe = None
  if args.sampling_steps > 0:
    prompts = [ids[b] for b in range(B)]

    def variant(label, **kw):
      # two rollouts of different length; the decode phases' own clocks (events behind the prefill
      # and behind the last step), so that neither the prefill nor the capture enters the difference
      times = []
      for n in (4, 4 + args.sampling_steps):
        sampler(prompts, n, max_prompt_length=P, seed=7, return_logprobs=True, eos_tokens=[-1], **kw)
        times.append(sampler.last_stats["decode_ms"])
      s_ms = (times[1] - times[0]) / args.sampling_steps
      log(f"sampling variant ({label}): {s_ms:.3f} ms/step over {args.sampling_steps} steps from context {P + 4}")
      return {"mode": label, "steps": args.sampling_steps, "ms_per_step": round(s_ms, 4),
              "tokens_per_s": round(B / (s_ms * 1e-3), 1), "context_range": [P + 4, P + 4 + args.sampling_steps]}

    sampling = variant("temperature 1.0, top_p 1.0, no top-k (categorical over the vocabulary)",
                       temperature=1.0, top_p=1.0, top_k=None)
    # the sampling settings of the reference's own Llama-3.1-8B GRPO recipe
    # (examples/rl/grpo/gsm8k/configs/llama3.1_8b.yaml: temperature 0.9, top_p 1.0, top_k 50)
    recipe = variant("temperature 0.9, top_p 1.0, top-k 50 (the reference's Llama-3.1-8B GRPO recipe)",
                     temperature=0.9, top_p=1.0, top_k=50)

  kern = kernel_breakdown(model, runner, st, int(round(mean_ctx)), args.kernel_iters)
  for name, v in kern.items():
    log(f"  {name:16s} {v['ms'] * 1e3:8.1f} us/launch  {v['gbs']:7.0f} GB/s  {v['tflops']:7.1f} TFLOP/s"
        f"  x{v['per_step']} = {v['step_ms']:.3f} ms/step")
  roofline, roofline_linears = rooflines(kern, default_workload=(B == 128 and not args.layers))
  many = many_rows_breakdown(model, 8192, max(2, args.kernel_iters // 5))
  log(f"  linears at 8192 rows (prefill / logps chunk): {many['achieved']} TFLOP/s, {many['linears']}")
  wb = model.weight_bytes()
  step_bytes = (wb["quantized"] + wb["lora"] + wb["head"]
                + B * cfg.num_kv_heads * mean_ctx * cfg.head_dim * 4 * cfg.num_layers)
  result = {
      "metric": "decode tokens/sec @1 MI355X (8B NF4 QLoRA, bs128); % HBM roofline",
      "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
      "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
      "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
      "config": {"workload": "Llama-3.1-8B-shaped NF4(g64)+LoRA r64 greedy rollout decode",
                 "layers": cfg.num_layers, "global_batch": B, "prompt_len": P, "gen_len": T,
                 "context_range": [contexts[0], contexts[-1]], "mean_context": round(mean_ctx, 1),
                 "timed_groups": groups, "parallelism": "single GPU"},
      "hbm_roofline_frac_step": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
      "step_bytes": int(step_bytes), "prefill_s": round(prefill_s, 3),
      "roofline": roofline, "roofline_hbm": roofline_linears, "roofline_many_rows": many,
      # each family alone in its own replayed graph at the mean context -- the linears with their
      # LoRA down-projection and a finishing pass that the decode chain folds into its consumers --
      # so these do NOT add up to ms_per_step; the step's own kernel trace is in profiles/
      "kernels_isolated": {k: {"us": round(v["ms"] * 1e3, 2), "launches_per_step": v["per_step"],
                               "GBps": round(v["gbs"], 1), "TFLOPs": round(v["tflops"], 1)}
                           for k, v in kern.items()},
  }
  if first_steps is not None:
    result["first_steps"] = first_steps
  if sampling is not None:
    result["sampling_variant"] = sampling
    result["sampling_recipe"] = recipe
  if not args.no_fused_logps:
    del sampler, st, runner, graph
    torch.cuda.empty_cache()
    fl = fused_logps_workload(args.fused_logps_rows, 16384, 2, expanded=not args.fused_logps_codes)
    result["fused_logps"] = {k: fl[k] for k in ("metric", "value", "unit", "ms_per_step", "config", "roofline")}
    log(f"fused logps: {fl['ms_per_step']} ms per pass over {args.fused_logps_rows} rows, {fl['roofline']['achieved']} TFLOP/s")
  if not args.no_cpu_baseline:
    threads = min(16, os.cpu_count() or 1)
    t0 = time.time()
    result["cpu_baseline"] = cpu_baseline(cfg, B, int(round(mean_ctx)), S, threads)
    log(f"cpu baseline took {time.time() - t0:.1f}s: {result['cpu_baseline']['value']:.2f} tokens/s")
  print(json.dumps(result), flush=True)


if __name__ == "__main__":
  main()
