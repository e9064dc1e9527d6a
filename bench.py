#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

A "step" is one call of torch.ops.xla.quantized_matmul on the decode-GEMV
configuration (x bf16 [16,4096], w int8 [14336,4096], scaler bf16 [14336]),
with every input already resident in HBM.  The weight rotates over enough
distinct copies (> 512 MB) that neither L2 nor the 256 MB Infinity Cache can
hold it, so the reported bandwidth is HBM bandwidth.  The K timed steps are
captured once into a HIP graph and replayed (a decode step is launch-bound
otherwise); `--no-graph` times eager calls instead.  Before every timed
replay the graph is replayed untimed for PREWARM_MS, so that the chip is at
the clocks it sustains under the workload, not in the low power state the
host-side set-up leaves it in.

Prints ONE JSON line.  `value` is algorithmic GB/s of the whole timed region
(wall clock between device synchronisations); `roofline` is the same kernel
measured with HIP events on its stream; `cpu_baseline` is the CPU oracle timed
on this host; `extra` carries the other configurations (M=1/4, hot cache,
a vocabulary projection, blockwise int4, W8A8 prefill GEMM with its own MFMA
roofline, the weight-only prefill GEMMs, the 7 linears of a Llama-3-8B layer).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA (5.0 POP/s)
BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA (2.5 PFLOP/s)
PREWARM_MS = 50.0  # untimed graph replays before each timed region (sustained clocks)

N_OUT, K_IN = 14336, 4096
TRAFFIC_PROFILE = "profiles/skinny_gemv_cfg2_m16_hbm_traffic.md"


def profile_traffic_bytes():
  """HBM bytes per launch of the decode GEMV kernel as the rocprofv3 counter summary under profiles/ states it
  (the figure in bold there: scaled FETCH_SIZE + WRITE_SIZE), or None when the file or the figure is missing."""
  import re
  try:
    text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
  except OSError:
    return None
  m = re.search(r"\*\*([0-9.]+) MB\*\*", text)
  return float(m.group(1)) * 1e6 if m else None


def gemv_bytes(m, n, k, w_bytes_per_elem=1.0, x_b=2, s_b=2, out_b=2, n_scale_rows=1, zp=False):
  """Algorithmic bytes: weight + activations + scale(+zp) + output."""
  scale_bytes = n * s_b * n_scale_rows * (2 if zp else 1)
  return int(n * k * w_bytes_per_elem + m * k * x_b + scale_bytes + m * n * out_b)


def timeline(torch, _lib, qmm, cases, dev, m, hot, config=2):
  """In-kernel timeline of the decode GEMV (x bf16 [m,4096], w int8 [14336,4096]), or with config=3 of the
  blockwise int4 + zero point matmul (x bf16 [m,4096], w int4 [32,128,4096]).

  The diagnostic build of the streaming kernel notes, per wave, the chip-wide 100 MHz
  counter at fixed points (entry, first weights requested / landed, first x chunk in
  LDS, every step, exit) and the shader clock counter at entry and exit.  The launch
  that is read back is the last node of a HIP graph of launches over rotating weight
  copies (cold weights, as in the benchmark), replayed until the clocks have settled.
  """
  import ctypes
  import numpy as np
  lib = _lib.load()
  raw = ctypes.CDLL(_lib.lib_path())
  raw.xla_amd_qmm_timeline_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
  raw.xla_amd_qmm_timeline_read.restype = ctypes.c_int
  if config == 3:
    n_out, k_in, row_bytes = 4096, 4096, 2048
    x, w3, s3, z3, _ = cases.blockwise(m, n_out, k_in, 128, 4, torch.bfloat16, symmetric=False, seed=4)
    x, s_d, z_d = x.to(dev), s3.to(dev), z3.to(dev)
    n_rot = 1 if hot else 40  # 40 x 8.4 MB: more than the Infinity Cache
    wts = [w3.to(dev) for _ in range(n_rot)]
    op = torch.ops.xla.quantized_matmul
    what = f"blockwise int4 + zero point x bf16 [{m},{k_in}] x w int4 [{k_in // 128},128,{n_out}]"

    def run(wt):
      op(x, wt, s_d, z_d, block_size=128, int4_weight=True)
  else:
    n_out, k_in, row_bytes = N_OUT, K_IN, K_IN
    x, w_cpu, s_cpu, _ = cases.per_channel_int8(m, N_OUT, K_IN, torch.bfloat16, torch.bfloat16, seed=2)
    x, s_d, w0 = x.to(dev), s_cpu.to(dev), w_cpu.to(dev)
    wt0 = qmm._tiled_weight(w0, 8, _lib.W_NK)
    n_rot = 1 if hot else 12
    wts = [wt0] + [wt0.clone() for _ in range(n_rot - 1)]
    out = torch.empty(m, N_OUT, dtype=torch.bfloat16, device=dev)
    bf = _lib.DT_BF16
    what = f"decode GEMV x bf16 [{m},{K_IN}] x w int8 [{N_OUT},{K_IN}]"

    def run(wt):
      _lib.check(lib.xla_amd_qmm_weight_only_skinny(x.data_ptr(), wt.data_ptr(), s_d.data_ptr(), None, out.data_ptr(), m,
                                                    N_OUT, K_IN, K_IN, 8, bf, bf, bf, bf, bf, bf,
                                                    torch.cuda.current_stream().cuda_stream), "weight_only_skinny")

  for wt in wts:
    run(wt)
  torch.cuda.synchronize()
  g = torch.cuda.CUDAGraph()
  with torch.cuda.graph(g):
    for i in range(max(24, n_rot)):
      run(wts[i % n_rot])
  t_pre = time.perf_counter()
  while (time.perf_counter() - t_pre) * 1e3 < PREWARM_MS:
    g.replay()
    torch.cuda.synchronize()
  n_blocks, n_waves, n_notes = 2048, 12, 32
  host = np.zeros(n_blocks * n_waves * n_notes, dtype=np.uint64)
  rc = raw.xla_amd_qmm_timeline_read(host.ctypes.data_as(ctypes.c_void_p), host.size)
  assert rc == 0, "timeline_read failed"
  t = host.reshape(n_blocks, n_waves, n_notes).astype(np.int64)
  live = t[:, :, 0] > 0
  nb, nwv = int(live.any(axis=1).sum()), int(live[0].sum())
  ncomp = nwv - 4  # the last four waves of a workgroup copy x
  t0 = t[:, :, 0][live].min()
  rel = np.where(t > 0, (t - t0) * 0.01, np.nan)  # 100 MHz ticks -> us since the first wave's entry
  print(f"{what}, {'one weight copy (cache-resident)' if hot else f'{n_rot} rotating weight copies (cold)'}: "
        f"{nb} workgroups x ({ncomp} computing + {nwv - ncomp} copying waves)")

  def table(title, waves, names):
    print(f"{title}: min / median / max over waves, us since the first wave's entry")
    for i, name in names:
      v = rel[:nb, waves, i].ravel()
      v = v[~np.isnan(v)]
      if v.size:
        print(f"  {name:34s} {v.min():7.2f} {np.median(v):7.2f} {v.max():7.2f}")

  n_steps = row_bytes // 512
  table("computing waves", slice(0, ncomp),
        [(0, "entry"), (1, "first weights requested"), (2, "first weights landed"), (3, "first x chunk in LDS (met)")] +
        [(4 + i, f"step {i} done") for i in range(min(n_steps - 1, 22))] +
        [(28, "all steps done"), (29, "k-split sums in LDS"), (30, "results stored, leaves")])
  table("copying waves", slice(ncomp, nwv),
        [(0, "entry"), (1, "first chunk requested"), (2, "first chunk landed"), (3, "first meeting passed")] +
        [(4 + i, f"chunk {i + 1} landed") for i in range(8)] + [(30, "leaves")])
  end = np.nanmax(rel[:nb, :nwv, 30], axis=1)
  print(f"first entry to last exit: {end.max():.2f} us; exit of a workgroup's last wave: min {end.min():.2f}, "
        f"median {np.median(end):.2f}, max {end.max():.2f}")
  steps = rel[:nb, :ncomp, 4:4 + min(n_steps - 1, 22)]
  d = np.diff(steps, axis=2).reshape(-1, steps.shape[2] - 1)
  print("duration of steps 1.., median over waves (us):", " ".join(f"{v:.2f}" for v in np.nanmedian(d, axis=0)))
  clk = (t[:nb, :ncomp, 27] - t[:nb, :ncomp, 26]).astype(np.float64)
  dur = (t[:nb, :ncomp, 30] - t[:nb, :ncomp, 0]).astype(np.float64) * 0.01
  print(f"shader clock over the computing waves' lifetime: median {np.median(clk / dur):.0f} MHz")


def stream_probe(torch, _lib, dev):
  """Kernels that only read the decode GEMV's weight bytes (14336 x 4096 = 58.7 MB), shaped like its memory side:
  `grid` workgroups of `waves` waves, each wave keeping `depth` 1 KB loads in flight over its own region.
  Per-launch time as a node of a HIP graph over 12 rotating buffers (cold) and over one buffer (cache-resident)."""
  import ctypes
  raw = ctypes.CDLL(_lib.lib_path())
  fn = raw.xla_amd_qmm_diag_stream
  fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 4 + [ctypes.c_void_p]
  fn.restype = ctypes.c_int
  total = N_OUT * K_IN
  bufs = [torch.ones(total + (1 << 20), dtype=torch.uint8, device=dev) for _ in range(12)]
  sink = torch.zeros(4, dtype=torch.int32, device=dev)
  print(f"streaming {total / 1e6:.1f} MB: us per launch (graph node), cold = 12 rotating buffers, hot = one buffer")
  print(f"{'grid':>5} {'waves':>5} {'KB in flight/wave':>18} {'cold us':>8} {'TB/s':>5} {'hot us':>7}")
  for grid, waves, depth in [(224, 4, 8), (256, 4, 8), (256, 4, 4), (256, 4, 16), (256, 8, 4), (256, 8, 8), (512, 4, 8),
                             (1024, 4, 8)]:
    kb = -(-total // 1024 // (grid * waves))
    times = []
    for hot in (False, True):
      def launch(b):
        rc = fn(b.data_ptr(), sink.data_ptr(), grid, waves, depth, kb, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
      for b in bufs:
        launch(b)
      torch.cuda.synchronize()
      g = torch.cuda.CUDAGraph()
      with torch.cuda.graph(g):
        for i in range(48):
          launch(bufs[0 if hot else i % 12])
      t_pre = time.perf_counter()
      while (time.perf_counter() - t_pre) * 1e3 < PREWARM_MS:
        g.replay()
        torch.cuda.synchronize()
      best = 1e9
      for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
          g.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / (5 * 48))
      times.append(best)
    print(f"{grid:5d} {waves:5d} {depth:18d} {times[0]:8.2f} {total / times[0] / 1e6:5.2f} {times[1]:7.2f}")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=240)
  ap.add_argument("--warmup", type=int, default=48)
  ap.add_argument("--no-graph", action="store_true", help="time eager calls instead of a HIP graph replay")
  ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
  ap.add_argument("--no-sclk", action="store_true",
                  help="do not sample the shader clock (it starts rocm-smi as a child process, which a counter-collecting "
                       "profiler run must not do)")
  ap.add_argument("--timeline", action="store_true",
                  help="instead of the benchmark: in-kernel timeline of the decode GEMV (diagnostic build of the "
                       "streaming kernel, libxla_amd_qmm_timeline.so); prints a table, not the JSON line")
  ap.add_argument("--stream-probe", action="store_true",
                  help="instead of the benchmark: time kernels that only read the decode GEMV's 58.7 MB, for several "
                       "launch shapes (diagnostic library); prints a table")
  ap.add_argument("--timeline-hot", action="store_true", help="with --timeline: one weight copy (cache-resident) instead of rotating ones")
  ap.add_argument("--timeline-m", type=int, default=16, help="with --timeline: rows of x")
  ap.add_argument("--timeline-config", type=int, default=2, choices=(2, 3),
                  help="with --timeline: 2 = decode GEMV (int8 per channel), 3 = blockwise int4 + zero point 4096 x 4096")
  ap.add_argument("--calibrate-copy", action="store_true",
                  help="also run a plain 256 MiB device copy (known traffic, for scaling rocprof byte counters)")
  args = ap.parse_args()
  if args.gpus != 1:
    print("bench.py: this build measures one GPU; --gpus must be 1 (the kernels are not sharded: a "
          "tensor-parallel run would give each GPU its own slice of the output channels)", file=sys.stderr)
    sys.exit(2)

  import torch
  if not torch.cuda.is_available():
    print("bench.py: no GPU visible", file=sys.stderr)
    sys.exit(3)
  from xla_amd import _lib
  if args.timeline or args.stream_probe:
    # the diagnostic build of the library takes the place of the regular one for this process
    _lib._LIB_PATH = os.path.join(os.path.dirname(_lib._LIB_PATH), "libxla_amd_qmm_timeline.so")
  _lib.load()  # no fallback: fail here if the HIP library is missing
  import xla_amd.experimental.custom_kernel  # noqa: F401
  import xla_amd.experimental.xla_quantized_matmul as qmm
  from tests import cases

  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  op = torch.ops.xla.quantized_matmul

  def time_calls(fns, steps, warmup, graph=True):
    """fns: list of zero-arg callables used round-robin.  Returns (wall_ms_per_step, event_ms_per_step, graphed).

    Every callable runs once before the warm-up, whatever `warmup` is: one-time work of a first
    call (the tiled copy of a weight) must be done before anything is captured or timed, and the
    count of such re-layouts is checked not to move afterwards."""
    for f in fns:
      f()
    torch.cuda.synchronize()
    relayouts = qmm.counters["pack"]
    for i in range(warmup):
      fns[i % len(fns)]()
    torch.cuda.synchronize()
    g = None
    if graph:
      try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
          for i in range(steps):
            fns[i % len(fns)]()
        g.replay()  # untimed: first replay uploads the graph
        torch.cuda.synchronize()
        # untimed: keep the GPU busy for PREWARM_MS before the timed replay.  After the host-side set-up
        # above the chip sits in a low power state and takes tens of milliseconds of work to reach its
        # sustained clocks (measured: the int8 GEMM of config 4 takes 125 us per launch in a burst of 20
        # after 1 s of idling and 115 us sustained; the decode GEMV 12.8 against 12.3 us)
        t_pre = time.perf_counter()
        while (time.perf_counter() - t_pre) * 1e3 < PREWARM_MS:
          g.replay()
          torch.cuda.synchronize()
      except Exception as e:  # capture unsupported for some reason: time eager calls
        print(f"bench.py: graph capture failed ({e}); timing eager calls", file=sys.stderr)
        g = None
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    if g is not None:
      g.replay()
    else:
      for i in range(steps):
        fns[i % len(fns)]()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert qmm.counters["pack"] == relayouts, "a weight was re-laid out inside the captured / timed region"
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps, g is not None

  def observed_sclk_mhz(fn, seconds=1.0):
    """Shader clock reported by rocm-smi while `fn` runs back to back (None if it cannot be read)."""
    import re
    import subprocess
    import threading
    found = []
    if args.no_sclk:
      return None

    def sample():
      time.sleep(seconds * 0.4)
      try:
        text = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
        m = re.search(r"sclk clock level:\s*\d+:\s*\((\d+)Mhz\)", text)
        if m:
          found.append(int(m.group(1)))
      except Exception:
        pass

    th = threading.Thread(target=sample)
    th.start()
    t_begin = time.perf_counter()
    while th.is_alive() or time.perf_counter() - t_begin < seconds:
      for _ in range(50):
        fn()
      torch.cuda.synchronize()
    th.join()
    return found[0] if found else None

  use_graph = not args.no_graph

  if args.timeline:
    timeline(torch, _lib, qmm, cases, dev, args.timeline_m, args.timeline_hot, args.timeline_config)
    return
  if args.stream_probe:
    stream_probe(torch, _lib, dev)
    return

  if args.calibrate_copy:
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(4):
      torch.add(src, 1, out=dst)  # elementwise kernel: 256 MiB read + 256 MiB written per launch
    torch.cuda.synchronize()
    del src, dst

  # ---- headline: decode GEMV, M = 16, rotating (cold) weights -----------------
  x16, w_cpu, s_cpu, _ = cases.per_channel_int8(16, N_OUT, K_IN, torch.bfloat16, torch.bfloat16, seed=2)
  n_rot = 12  # 12 x 58.7 MB = 704 MB > 512 MB
  w0 = w_cpu.to(dev)
  ws = [w0] + [w0.clone() for _ in range(n_rot - 1)]
  s_d = s_cpu.to(dev)
  xs = {m: x16[:m].contiguous().to(dev) for m in (1, 4, 16)}

  def gemv_fns(m, weights):
    return [(lambda w=w: op(xs[m], w, s_d)) for w in weights]

  wall_ms, ev_ms, graphed = time_calls(gemv_fns(16, ws), args.steps, args.warmup, use_graph)
  bytes16 = gemv_bytes(16, N_OUT, K_IN)
  value = bytes16 / (wall_ms * 1e-3) / 1e9
  achieved = bytes16 / (ev_ms * 1e-3) / 1e9

  result = {
      "metric": "quantized_matmul HBM GB/s & TOPS (% roofline): int8 decode GEMV + W8A8 GEMM",
      "value": round(value, 1),
      "unit": "GB/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": round(wall_ms, 6),
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "bf16 x int8 -> f32 accumulate -> bf16",
      "data": "synthetic",
      "config": {
          "workload": "decode GEMV, per-channel int8 weight-only: x bf16 [16,4096], w int8 [14336,4096], scaler bf16 [14336]",
          "weights": f"{n_rot} rotating copies (cold: > Infinity Cache)",
          "launch": "HIP graph replay" if graphed else "eager calls",
          "untimed_before_the_timed_steps": f"{args.warmup} warm-up steps, then {PREWARM_MS:.0f} ms of graph replays (sustained clocks)",
          "algorithmic_bytes_per_step": bytes16,
      },
      "roofline": {
          "bound": "hbm",
          "achieved": round(achieved, 1),
          "peak": HBM_PEAK_GBPS,
          "unit": "GB/s",
          "frac": round(achieved / HBM_PEAK_GBPS, 4),
          # HBM bytes per launch measured with rocprofv3 (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, factors from an
          # elementwise kernel of known size); it is a profile result, not re-measured by this script
          "traffic": profile_traffic_bytes(),
          "traffic_source": TRAFFIC_PROFILE,
          "kernel": "qmm_skinny_kernel<bf16, int8, MT=1> (4 computing + 4 copying waves)",
          "avg_launch_us": round(ev_ms * 1e3, 3),
      },
  }

  extra = {}
  if not args.no_extra:
    steps2 = max(24, args.steps // 2)
    # decode GEMV at M = 1, 4 (cold) and M = 16 hot (single weight buffer: cache resident)
    for m in (1, 4):
      _, ev, _ = time_calls(gemv_fns(m, ws), steps2, 12, use_graph)
      b = gemv_bytes(m, N_OUT, K_IN)
      extra[f"gemv_M{m}_cold"] = {"us": round(ev * 1e3, 3), "GBps": round(b / ev / 1e6, 1),
                                  "frac_hbm": round(b / ev / 1e6 / HBM_PEAK_GBPS, 4)}
    _, ev, _ = time_calls(gemv_fns(16, ws[:1]), steps2, 12, use_graph)
    extra["gemv_M16_hot"] = {"us": round(ev * 1e3, 3), "GBps": round(bytes16 / ev / 1e6, 1),
                             "note": "one weight buffer, served from Infinity Cache; not HBM bandwidth"}
    del ws[1:]

    # a launch long enough to amortise its fixed cost: the Llama-3 vocabulary projection (128256 x 4096, 525 MB) at M = 1;
    # two weight copies in turn (1.05 GB: nothing of a copy is left in the 256 MB Infinity Cache when its turn comes)
    gv = cases.gen(9)
    wv = [torch.randint(-127, 128, (128256, K_IN), generator=gv, dtype=torch.int32).to(torch.int8).to(dev)]
    wv.append(wv[0].clone())
    sv = (torch.rand(128256, generator=gv) * 0.01).bfloat16().to(dev)
    _, ev, _ = time_calls([(lambda w=w: op(xs[1], w, sv)) for w in wv], 24, 4, use_graph)
    bv = gemv_bytes(1, 128256, K_IN)
    extra["gemv_vocabulary_projection_128256x4096_M1_cold"] = {
        "us": round(ev * 1e3, 2), "GBps": round(bv / ev / 1e6, 1), "frac_hbm": round(bv / ev / 1e6 / HBM_PEAK_GBPS, 4)}
    for w in wv:
      qmm.invalidate_weight_cache(w)  # frees the tiled copies too
    del wv, sv, w

    # config 1: fp32 activations, 1 MB of weights (latency-bound: reported only)
    x1, w1, s1 = [t.to(dev) for t in cases.uniform_int8(8, 1024, 1024, torch.float32, torch.float32, seed=1)]
    _, ev, _ = time_calls([lambda: op(x1, w1, s1)], steps2, 12, use_graph)
    b1 = gemv_bytes(8, 1024, 1024, x_b=4, s_b=4, out_b=4)
    extra["cfg1_fp32_M8_1024x1024"] = {"us": round(ev * 1e3, 3), "GBps": round(b1 / ev / 1e6, 1),
                                       "frac_hbm": round(b1 / ev / 1e6 / HBM_PEAK_GBPS, 4),
                                       "note": "1.1 MB per call: launch latency, not bandwidth"}

    # blockwise int4 (config 3)
    x3, w3, s3, z3, _ = cases.blockwise(16, 4096, 4096, 128, 4, torch.bfloat16, symmetric=False, seed=4)
    x3d, s3d, z3d = x3.to(dev), s3.to(dev), z3.to(dev)
    w3s = [w3.to(dev) for _ in range(40)]  # packed copies: 40 x 8.4 MB
    fns = [(lambda w=w: op(x3d, w, s3d, z3d, block_size=128, int4_weight=True)) for w in w3s]
    _, ev, _ = time_calls(fns, steps2, 80, use_graph)
    b3 = gemv_bytes(16, 4096, 4096, 0.5, n_scale_rows=32, zp=True)
    extra["blockwise_int4_M16"] = {"us": round(ev * 1e3, 3), "GBps": round(b3 / ev / 1e6, 1),
                                   "frac_hbm": round(b3 / ev / 1e6 / HBM_PEAK_GBPS, 4),
                                   "algorithmic_bytes": b3}
    # the same weights against a prefill-sized M: the tiled GEMM with per-block rounding points
    x3p = torch.randn(2048, 4096, generator=cases.gen(4)).bfloat16().to(dev)
    w3d = w3s[0]
    _, ev, _ = time_calls([lambda: op(x3p, w3d, s3d, z3d, block_size=128, int4_weight=True)], 20, 5, use_graph)
    f3 = 2.0 * 2048 * 4096 * 4096
    extra["blockwise_int4_prefill_M2048"] = {
        "us": round(ev * 1e3, 2),
        "roofline": {"bound": "mfma", "achieved": round(f3 / ev / 1e9, 1), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(f3 / ev / 1e9 / BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "qmm_wo_bw_gemm_kernel<bf16, int4, zero point> (64 x 128 tiles)"}}
    del w3s, fns, x3p, w3d

    # W8A8 prefill GEMM (config 4)
    m4 = 2048
    x4 = cases.outlier_activations(m4, K_IN, torch.bfloat16, seed=1234).to(dev)
    s4 = s_cpu.float().to(dev)
    xq, xsc, _ = qmm.quantize_per_token_gpu(x4)
    steps4 = 20
    _, ev_q, _ = time_calls([lambda: qmm.quantize_per_token_gpu(x4)], steps4, 5, use_graph)
    _, ev_g, _ = time_calls([lambda: qmm.w8a8_gemm_gpu(xq, w0, xsc, s4, None, None, cvt_dtype=torch.float32,
                                                       mid_dtype=torch.float32, out_dtype=torch.float32)],
                            steps4, 5, use_graph)
    _, ev_gb, _ = time_calls([lambda: qmm.w8a8_gemm_gpu(xq, w0, xsc, s4, None, None, cvt_dtype=torch.float32,
                                                        mid_dtype=torch.float32, out_dtype=torch.bfloat16)],
                             steps4, 5, use_graph)
    _, ev_e2e, _ = time_calls([lambda: op(x4, w0, s4, quantize_activation=True)], steps4, 5, use_graph)
    ops4 = 2.0 * m4 * N_OUT * K_IN
    # the shader clock the chip holds under this kernel (it is power-limited with operands that toggle): rocm-smi
    # sampled while the GEMM runs back to back for about a second; the paper peak assumes 2400 MHz
    sclk = observed_sclk_mhz(lambda: qmm.w8a8_gemm_gpu(xq, w0, xsc, s4, None, None, cvt_dtype=torch.float32,
                                                       mid_dtype=torch.float32, out_dtype=torch.bfloat16))
    extra["w8a8_prefill_M2048"] = {
        "gemm_us_f32_out": round(ev_g * 1e3, 2),
        "gemm_us_bf16_out": round(ev_gb * 1e3, 2),
        "quantize_us": round(ev_q * 1e3, 2),
        "end_to_end_us": round(ev_e2e * 1e3, 2),
        "roofline": {"bound": "mfma", "achieved": round(ops4 / ev_gb / 1e9, 1), "peak": INT8_PEAK_TOPS,
                     "unit": "TOP/s", "frac": round(ops4 / ev_gb / 1e9 / INT8_PEAK_TOPS, 4),
                     "traffic": None, "kernel": "qmm_w8a8_gemm_kernel (bf16 out)"},
        "sclk_mhz_observed": sclk,
        "frac_of_peak_at_observed_clock": None if not sclk else round(ops4 / ev_gb / 1e9 / (INT8_PEAK_TOPS * sclk / 2400.0), 4),
        "tops_f32_out": round(ops4 / ev_g / 1e9, 1),
        "tops_end_to_end": round(ops4 / ev_e2e / 1e9, 1),
    }
    # weight-only prefill at the same shape (config 2's weight, M = 2048): the tiled bf16 GEMM with int8 weights
    s2 = s_cpu.to(dev)
    x4b = torch.randn(m4, K_IN, generator=cases.gen(2)).bfloat16().to(dev)  # config 2's activations: N(0, 1)
    _, ev_wo, _ = time_calls([lambda: op(x4b, w0, s2)], steps4, 5, use_graph)
    sclk_wo = observed_sclk_mhz(lambda: op(x4b, w0, s2))
    _, ev_wo_sustained, _ = time_calls([lambda: op(x4b, w0, s2)], 4 * steps4, 5, use_graph)
    extra["weight_only_prefill_M2048"] = {
        "us": round(ev_wo * 1e3, 2),
        "us_sustained": round(ev_wo_sustained * 1e3, 2),
        "sclk_mhz_observed": sclk_wo,
        "roofline": {"bound": "mfma", "achieved": round(ops4 / ev_wo / 1e9, 1), "peak": BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(ops4 / ev_wo / 1e9 / BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "qmm_wo_gemm_kernel<bf16, 128 x 256 tile> (persistent, 4 computing + 4 copying waves)"},
        "vs_w8a8_end_to_end": round(ev_wo / ev_e2e, 2),
    }
    # the same shape with f32 activations: split into three bf16 parts, the same GEMM at three times the arithmetic
    x4f = torch.randn(m4, K_IN, generator=cases.gen(2)).to(dev)
    s2f = s2.float()
    _, ev_f32, _ = time_calls([lambda: op(x4f, w0, s2f)], 10, 3, use_graph)
    extra["weight_only_prefill_M2048_f32_rows"] = {
        "us": round(ev_f32 * 1e3, 1),
        "note": "x f32 [2048,4096]: xla_amd_qmm_weight_only_gemm_f32 (split kernel + bf16 GEMM over 3 K columns, f32 results; "
                "workspace allocation included); the streaming kernel's 128 passes take 3.8 ms"}
    del x4, x4b, x4f, xq, xsc

    # Llama-3-8B decoder layer, 7 linears (config 5)
    shapes = {"q": (4096, 4096), "k": (1024, 4096), "v": (1024, 4096), "o": (4096, 4096),
              "gate": (14336, 4096), "up": (14336, 4096), "down": (4096, 14336)}
    g5 = cases.gen(5)
    layer = {}
    for name, (n, k) in shapes.items():
      w = torch.randint(-127, 128, (n, k), generator=g5, dtype=torch.int32).to(torch.int8).to(dev)
      layer[name] = (w, (torch.rand(n, generator=g5) * 0.01).to(dev))
    # two more copies of the layer's weights: with three sets (654 MB) used in turn no weight is
    # still in the 256 MB Infinity Cache when its turn comes again ("cold", what a model with many layers sees)
    layer_sets = [layer] + [{k_: (v[0].clone(), v[1]) for k_, v in layer.items()} for _ in range(2)]
    for tag, m, qa in (("decode_M32", 32, False), ("prefill_M512", 512, True)):
      x_in = {4096: torch.randn(m, 4096, generator=g5).bfloat16().to(dev),
              14336: torch.randn(m, 14336, generator=g5).bfloat16().to(dev)}

      layer_s = {k_: (v[0], v[1] if qa else v[1].bfloat16()) for k_, v in layer.items()}
      sets_s = [{k_: (v[0], v[1] if qa else v[1].bfloat16()) for k_, v in ls.items()} for ls in layer_sets]

      def run_layer():
        for name, (w, s) in layer_s.items():
          op(x_in[w.shape[1]], w, s, quantize_activation=qa)

      _, ev, _ = time_calls([run_layer], 20, 5, use_graph)
      extra[f"llama3_8b_layer_linears_{tag}"] = {
          "us_one_weight_set": round(ev * 1e3, 2),
          "note": "us_one_weight_set: the same 218 MB of weights every iteration (they do not stay in the 256 MB Infinity "
                  "Cache next to the activations and outputs: close to cold); us_cold: three sets in turn; per_linear: "
                  "each projection alone over the three sets in turn (cold), with its share of the roofline that bounds it"}

      def run_set(ls):
        for name, (w, s) in ls.items():
          op(x_in[w.shape[1]], w, s, quantize_activation=qa)

      _, ev, _ = time_calls([(lambda ls=ls: run_set(ls)) for ls in sets_s], 21, 6, use_graph)
      extra[f"llama3_8b_layer_linears_{tag}"]["us_cold"] = round(ev * 1e3, 2)
      per = {}
      for name in ("q", "k", "o", "gate", "down"):  # (v is k's shape, up is gate's)
        n_, k_ = shapes[name]
        _, ev1, _ = time_calls([(lambda ls=ls: op(x_in[k_], ls[name][0], ls[name][1], quantize_activation=qa)) for ls in sets_s],
                               21, 6, use_graph)
        if qa:
          per[name] = {"us": round(ev1 * 1e3, 2), "frac_mfma": round(2.0 * m * n_ * k_ / ev1 / 1e9 / INT8_PEAK_TOPS, 4)}
        else:
          per[name] = {"us": round(ev1 * 1e3, 2), "frac_hbm": round(gemv_bytes(m, n_, k_) / ev1 / 1e6 / HBM_PEAK_GBPS, 4)}
      extra[f"llama3_8b_layer_linears_{tag}"]["per_linear"] = per

      # the same layer with q/k/v and gate/up concatenated along N: 4 launches instead of 7
      def cat(names):
        return (torch.cat([layer_s[n][0] for n in names]).contiguous(),
                torch.cat([layer_s[n][1] for n in names]).contiguous())

      fused_s = {"qkv": cat(("q", "k", "v")), "o": layer_s["o"], "gate_up": cat(("gate", "up")),
                 "down": layer_s["down"]}

      def run_fused():
        for name, (w, s) in fused_s.items():
          op(x_in[w.shape[1]], w, s, quantize_activation=qa)

      _, ev, _ = time_calls([run_fused], 20, 5, use_graph)
      extra[f"llama3_8b_layer_linears_{tag}"]["us_qkv_and_gate_up_fused"] = round(ev * 1e3, 2)
      del fused_s, sets_s
    del layer_sets[1:]
    # W8A8 GEMM with few output tiles: the down projection (4096 x 14336) at decode-sized M
    wd, sd = layer["down"]
    small = {}
    for m in (32, 128, 512):
      xq_s, xs_s, _ = qmm.quantize_per_token_gpu(torch.randn(m, 14336, generator=g5).bfloat16().to(dev))
      _, ev, _ = time_calls([lambda: qmm.w8a8_gemm_gpu(xq_s, wd, xs_s, sd, None, None, cvt_dtype=torch.float32,
                                                       mid_dtype=torch.float32, out_dtype=torch.bfloat16)],
                            20, 5, use_graph)
      small[f"M{m}_us"] = round(ev * 1e3, 2)
    small["note"] = "GEMM alone, bf16 output, weights (59 MB) cache-warm; M=32: 32x32 tiles, M=128: 64x32, M=512: 64x64"
    extra["w8a8_gemm_4096x14336_small_M"] = small
    # quantized_decomposed quantize / dequantize of a weight-sized tensor (HBM-bound elementwise)
    import xla_amd.experimental.quantized  # noqa: F401
    qd = torch.ops.quantized_decomposed
    wf = [torch.randn(N_OUT, K_IN, generator=g5).bfloat16().to(dev) for _ in range(6)]  # 6 x 117 MB, rotating
    _, ev_qt, _ = time_calls([(lambda t=t: qd.quantize_per_tensor(t, 0.05, 0, -128, 127, torch.int8)) for t in wf],
                             24, 6, False)
    qs = [qd.quantize_per_tensor(t, 0.05, 0, -128, 127, torch.int8) for t in wf]
    _, ev_dq, _ = time_calls([(lambda t=t: qd.dequantize_per_tensor(t, 0.05, 0, -128, 127, torch.int8)) for t in qs],
                             24, 6, False)
    nel = N_OUT * K_IN
    extra["quantized_decomposed_per_tensor_14336x4096"] = {
        "quantize_bf16_to_int8_us": round(ev_qt * 1e3, 2),
        "quantize_frac_hbm": round(nel * 3 / ev_qt / 1e6 / HBM_PEAK_GBPS, 4),
        "dequantize_int8_to_f32_us": round(ev_dq * 1e3, 2),
        "dequantize_frac_hbm": round(nel * 5 / ev_dq / 1e6 / HBM_PEAK_GBPS, 4),
        "note": "eager calls (allocation and host-side parameter tensors included); bytes = read + written per element",
    }
    del wf, qs
    result["extra"] = extra

  # ---- CPU baseline: the oracle (reference's eager CPU semantics) on this host ----
  if not args.no_cpu:
    from oracle import quantized_matmul_oracle as oracle
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)

    def cpu_time(fn, budget_s, max_runs=50, min_runs=5):
      """(min, median, runs) of the wall time of fn over at least min_runs calls (one untimed call first)."""
      fn()
      runs, t_begin = [], time.perf_counter()
      while len(runs) < min_runs or (time.perf_counter() - t_begin < budget_s and len(runs) < max_runs):
        t0 = time.perf_counter()
        fn()
        runs.append(time.perf_counter() - t0)
      runs.sort()
      return runs[0], runs[len(runs) // 2], len(runs)

    def cpu_entry(t_min, t_med, n, amount, unit, scale, what):
      return {"value": round(amount / t_med / scale, 4), "value_best_run": round(amount / t_min / scale, 4), "unit": unit,
              "cores": cores, "kind": "port", "runs": n, "ms_median": round(t_med * 1e3, 2), "ms_min": round(t_min * 1e3, 2),
              "sample": what}

    t_min, t_med, n_runs = cpu_time(lambda: oracle.quantized_matmul(x16, w_cpu, s_cpu), 8.0)
    result["cpu_baseline"] = cpu_entry(
        t_min, t_med, n_runs, bytes16, "GB/s", 1e9,
        f"{n_runs} full calls of the same M=16 workload through the CPU oracle (torch {torch.__version__} eager ops, the "
        f"reference's CPU-tensor semantics); value from the median, value_best_run from the fastest call")
    # the other configurations (bounded samples), next to their GPU entries where there is one
    if extra:
      per_config = {}
      x1, w1, s1 = cases.uniform_int8(8, 1024, 1024, torch.float32, torch.float32, seed=1)[:3]
      t = cpu_time(lambda: oracle.quantized_matmul(x1, w1, s1), 1.0)
      per_config["cfg1_fp32_8x1024x1024"] = cpu_entry(*t, gemv_bytes(8, 1024, 1024, x_b=4, s_b=4, out_b=4), "GB/s", 1e9,
                                                      "full calls of config 1")
      for m in (1, 4):
        xm = x16[:m].contiguous()
        t = cpu_time(lambda: oracle.quantized_matmul(xm, w_cpu, s_cpu), 2.0)
        per_config[f"cfg2_decode_gemv_M{m}"] = cpu_entry(*t, gemv_bytes(m, N_OUT, K_IN), "GB/s", 1e9, f"full calls of config 2, M={m}")
      per_config["cfg2_decode_gemv_M16"] = result["cpu_baseline"]
      x3, w3, s3, z3, _ = cases.blockwise(16, 4096, 4096, 128, 4, torch.bfloat16, symmetric=False, seed=4)
      t = cpu_time(lambda: oracle.quantized_matmul(x3, w3, s3, z3, block_size=128, int4_weight=True), 3.0)
      b3 = gemv_bytes(16, 4096, 4096, 0.5, n_scale_rows=32, zp=True)
      per_config["cfg3_blockwise_int4_M16"] = cpu_entry(*t, b3, "GB/s", 1e9, "full calls of config 3 (algorithmic bytes of the packed int4 weight)")
      if "blockwise_int4_M16" in extra:
        extra["blockwise_int4_M16"]["cpu_baseline"] = per_config["cfg3_blockwise_int4_M16"]
      rows4 = 128  # of the 2048 rows: the CPU's int32 matmul takes seconds for all of them
      x4c = cases.outlier_activations(2048, K_IN, torch.bfloat16, seed=1234)[:rows4].contiguous()
      s4c = s_cpu.float()
      t = cpu_time(lambda: oracle.quantized_matmul(x4c, w_cpu, s4c, quantize_activation=True), 6.0, max_runs=10)
      per_config["cfg4_w8a8_prefill"] = cpu_entry(
          *t, 2.0 * rows4 * N_OUT * K_IN, "TOP/s", 1e12,
          f"calls on the first {rows4} of the 2048 rows (quantize + int32 matmul + scales) through the CPU oracle")
      if "w8a8_prefill_M2048" in extra:
        extra["w8a8_prefill_M2048"]["cpu_baseline"] = per_config["cfg4_w8a8_prefill"]
      # config 5, decode step: the seven linears at M = 32 (218 MB of int8 weights converted to bf16 per call)
      g5c = cases.gen(5)
      shapes5 = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]
      lin5 = [(torch.randint(-127, 128, (n, k), generator=g5c, dtype=torch.int32).to(torch.int8),
               (torch.rand(n, generator=g5c) * 0.01).bfloat16(), torch.randn(32, k, generator=g5c).bfloat16()) for n, k in shapes5]

      def layer_cpu():
        for w_, s_, x_ in lin5:
          oracle.quantized_matmul(x_, w_, s_)

      t = cpu_time(layer_cpu, 4.0, max_runs=10)
      bytes5 = sum(gemv_bytes(32, n, k) for n, k in shapes5)
      per_config["cfg5_layer_decode_M32"] = cpu_entry(*t, bytes5, "GB/s", 1e9, "the seven linears of config 5 at M=32, one after the other")
      extra["cpu_baseline_per_config"] = per_config
  print(json.dumps(result))


if __name__ == "__main__":
  main()
