"""Benchmark of the octree hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

Workload (BASELINE.json configs[3], the configuration the metric is quoted on): a
synthetic 5 m x 5 m x 3 m room sampled to 250 000 points, built on the GPU into an
octree of depth 9 (full_depth 2).  One step = one 3x3x3 stride-1 octree convolution
with Cin = Cout = 64 in fp32 over all depth-9 octants, inputs resident in HBM.
`value` = octants/s of that step.  Sub-measurements of the other kernels of the path
(bf16 conv, stride-2 conv, depth-7 batch, octree build, neighbour table, pooling) go
to `extra`, each timed with HIP events on the stream the kernels run on.
Prints ONE JSON line.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_MFMA_TFLOPS = {"f32": 157.3, "bf16": 2500.0}

# HBM bytes per launch of the headline kernel, from two `rocprofv3 --pmc` runs (FETCH_SIZE,
# WRITE_SIZE) scaled by a 1-GiB device copy: see
# profiles/conv_s1_f32_lds_kernel__scene_depth9__hbm_traffic.md.  Counters cannot be read from
# inside this process, so the recorded figure is reported for the workload it was taken on, and
# only while the kernel's source file is the one it was taken from (first 16 hex digits of the
# SHA-256 of o-cnn_amd/csrc/conv.hip); after any change to that file `traffic` is null until
# the counters have been read again.
RECORDED_TRAFFIC = {("conv_s1_f32_lds_kernel", 1494168, 64, 64): (1.0183e9, "e85dd11c2cd5af18")}


def recorded_traffic(key):
  import hashlib
  entry = RECORDED_TRAFFIC.get(key)
  if entry is None:
    return None
  try:
    with open(os.path.join(ROOT, "o-cnn_amd", "csrc", "conv.hip"), "rb") as fh:
      digest = hashlib.sha256(fh.read()).hexdigest()[:16]
  except OSError:
    return None
  return entry[0] if digest == entry[1] else None


def oc_points_blob(cloud):
  from oracle.checker import make_points_blob
  return make_points_blob(cloud[0], cloud[1])


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=20)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--quick", action="store_true", help="skip the sub-measurements and the CPU baseline")
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
  ap.add_argument("--build-only", action="store_true",
                  help="run only the octree construction of the scene (12 builds) and print its time: "
                       "the workload of the per-kernel rocprof summary of the build")
  ap.add_argument("--calib", action="store_true",
                  help="also run a plain device copy of 1 GiB three times (the known-size kernel "
                       "that scales the FETCH_SIZE / WRITE_SIZE counters of a --pmc run)")
  args = ap.parse_args()
  if args.gpus != 1:
    print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
          file=sys.stderr)
    sys.exit(2)

  import torch
  oc = importlib.import_module("o-cnn_amd")
  F = oc.nn
  oc.lib.call("ocnn_device_check", 0)
  torch.cuda.set_device(0)
  dev = torch.device("cuda", 0)

  def timed(fn, steps, warmup):
    """average milliseconds per call, HIP events on the current stream"""
    for _ in range(warmup):
      fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
      fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps

  def points_tensor(p, n, f):
    return F.points_new(torch.from_numpy(p), torch.from_numpy(n),
                        torch.from_numpy(f) if f is not None else None).to(dev)

  # ---- scene octree, depth 9 (built on the GPU) ------------------------------------------
  pts, nrm, rgb = oc.synthetic.room_cloud(250000, 3)
  scene_pts = points_tensor(pts, nrm, rgb)
  scene_pts._ocnn_points_info = scene_pts[:88].cpu().numpy().copy()
  octree = F.points2octree_batch([scene_pts], 9, 2)
  info = F.octree_info(octree)
  depth = 9
  H9, H8, Hne9, Hne8 = info.nnum(9), info.nnum(8), info.nnum_nempty(9), info.nnum_nempty(8)

  if args.build_only:
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(12):
      F.points2octree_batch([scene_pts], 9, 2)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / 12
    print(json.dumps({"metric": "points2octree + octree_batch, depth-9 scene", "ms": t * 1e3,
                      "Mpts_per_s": 0.25 / t, "octants_d9": H9}))
    return

  C = 64
  g = torch.Generator(device="cpu").manual_seed(2)
  x32 = torch.randn(1, C, H9, 1, generator=g).to(dev)
  w32 = (torch.randn(C, C * 27, generator=g) * 0.02).to(dev)

  def conv_step():
    return F.octree_conv(x32, w32, octree, depth, C, [3, 3, 3], 1, False)

  if args.calib:
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    for _ in range(3):
      dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

  # ---- timed region of the headline metric -------------------------------------------------
  for _ in range(args.warmup):
    conv_step()
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  t0 = time.perf_counter()
  e0.record()
  for _ in range(args.steps):
    conv_step()
  e1.record()
  torch.cuda.synchronize()
  wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
  ms = e0.elapsed_time(e1) / args.steps
  flops = 2.0 * H9 * 27 * C * C
  value = H9 / (ms * 1e-3)
  achieved_tflops = flops / (ms * 1e-3) / 1e12

  out = {
      "metric": "octree-conv octants/s (3x3x3 stride 1, Cin=Cout=64, depth 9)",
      "value": value,
      "unit": "octants/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": ms,
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "f32",
      "data": "synthetic",
      "config": {"workload": "cfg4 scene: 250000-point room, octree depth 9 full_depth 2, "
                             "conv 3x3x3 s1 64->64 over %d octants" % H9,
                 "octants_d9": H9, "octants_d8": H8, "nonempty_d9": Hne9, "points": 250000},
      "roofline": {"bound": "mfma", "achieved": achieved_tflops, "peak": PEAK_MFMA_TFLOPS["f32"],
                   "unit": "TFLOP/s", "frac": achieved_tflops / PEAK_MFMA_TFLOPS["f32"],
                   "traffic": recorded_traffic(("conv_s1_f32_lds_kernel", H9, C, C)),
                   "kernel": "conv_s1_f32_lds_kernel<2,27>",
                   "algorithmic_flops_per_launch": flops},
      "wall_ms_per_step": wall_ms,
  }

  extra = {}
  if not args.quick:
    reps, wu = max(3, args.steps // 4), 1
    headline_timed = timed

    def timed(fn, steps, warmup):
      """Rows of `extra`: kernels of tens of microseconds.  Warm up until the device has been
      busy for a few milliseconds (its clocks settle), then time enough calls for the region
      to last a few milliseconds; at least the given counts."""
      pilot = headline_timed(fn, 2, max(1, warmup))
      n_warm = max(warmup, min(200, int(5.0 / max(pilot, 1e-3))))
      n_rep = max(steps, min(400, int(10.0 / max(pilot, 1e-3))))
      return headline_timed(fn, n_rep, n_warm)

    def conv_case(name, oct_, d, x, w, ks, stride, nempty=False, deconv=False, n_out=C):
      fn = F.octree_deconv if deconv else F.octree_conv
      t = timed(lambda: fn(x, w, oct_, d, n_out, ks, stride, nempty), reps, wu)
      K = ks[0] * ks[1] * ks[2]
      cols = x.shape[2] if stride == 1 else (x.shape[2] // 8 if not deconv else x.shape[2])
      fl = 2.0 * cols * K * x.shape[1] * n_out
      dt = "bf16" if x.dtype == torch.bfloat16 else "f32"
      extra[name] = {"ms": t, "octants_per_s": x.shape[2] / (t * 1e-3),
                     "tflops": fl / (t * 1e-3) / 1e12,
                     "frac_mfma_peak": fl / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS[dt]}

    x16, w16 = x32.bfloat16(), w32.bfloat16()
    conv_case("conv333_s1_d9_bf16", octree, 9, x16, w16, [3, 3, 3], 1)
    # the same operator on row-major activations (input and output [H + 1][pitch] bf16): what a
    # member of a chain of convolutions costs once the chain keeps that layout between its members
    # (bit-identical results; the channel-major entry above copies its input row-major first)
    rows16 = F.to_rows(x16)
    rows_out = torch.empty(H9 + 1, F.rows_pitch(C), dtype=torch.bfloat16, device=dev)
    t = timed(lambda: F.octree_conv_rows(rows16, C, w16, octree, 9, C, out=rows_out), reps, wu)
    extra["conv333_s1_d9_bf16_rows"] = {
        "ms": t, "octants_per_s": H9 / (t * 1e-3), "tflops": flops / (t * 1e-3) / 1e12,
        "frac_mfma_peak": flops / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS["bf16"],
        "layout": "row-major in and out, no copy"}
    w2 = (torch.randn(C, C * 8, generator=g) * 0.02).to(dev)
    # 2x2x2 stride 2, row-major, with the pad (conv) / depad (deconv) of the reference's modules folded in
    t = timed(lambda: F.octree_conv_rows(rows16, C, w2.bfloat16(), octree, 9, C, kernel_size=(2, 2, 2), stride=2), reps, wu)
    by = (H9 * C + H8 * C) * 2 + H8 * 4
    extra["conv222_s2_d9_bf16_rows_padded"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS,
                                               "tflops": 2.0 * Hne8 * 8 * C * C / (t * 1e-3) / 1e12}
    rows8 = torch.randn(H8 + 1, C, generator=g).bfloat16().to(dev)
    t = timed(lambda: F.octree_conv_rows(rows8, C, w2.bfloat16(), octree, 8, C, deconv=True, kernel_size=(2, 2, 2),
                                         stride=2, out=rows_out), reps, wu)
    by = (Hne8 * C + H9 * C) * 2 + H8 * 4 + Hne8 * 4
    extra["deconv222_s2_d8to9_bf16_rows_depadded"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS,
                                                      "tflops": 2.0 * Hne8 * 8 * C * C / (t * 1e-3) / 1e12}
    del rows16, rows8, rows_out
    conv_case("conv222_s2_d9_f32", octree, 9, x32, w2, [2, 2, 2], 2)
    conv_case("conv222_s2_d9_bf16", octree, 9, x16, w2.bfloat16(), [2, 2, 2], 2)
    xne = torch.randn(1, C, Hne9, 1, generator=g).to(dev)
    conv_case("conv333_s1_d9_f32_nempty", octree, 9, xne, w32, [3, 3, 3], 1, nempty=True)
    conv_case("conv333_s1_d9_bf16_nempty", octree, 9, xne.bfloat16(), w16, [3, 3, 3], 1, nempty=True)
    # (over the non-empty nodes the table of source rows is kept with the octree, as a network's layers
    # of one depth share it; what the first call on an octree pays for making it is stated beside)
    def first_call(x, w):
      octree.__dict__.pop("_ocnn_sources", None)
      return F.octree_conv(x, w, octree, 9, C, [3, 3, 3], 1, True)
    for name, xx, ww in (("conv333_s1_d9_f32_nempty", xne, w32), ("conv333_s1_d9_bf16_nempty", xne.bfloat16(), w16)):
      t_first = timed(lambda: first_call(xx, ww), max(reps // 2, 3), 2)
      extra[name]["sources"] = "table of source rows kept with the octree (one per depth, kernel shape and direction)"
      extra[name]["ms_first_call_on_an_octree"] = t_first
    F.octree_conv(xne, w32, octree, 9, C, [3, 3, 3], 1, True)
    rows_ne = F.to_rows(xne.bfloat16())
    rows_ne_out = torch.empty(Hne9 + 1, F.rows_pitch(C), dtype=torch.bfloat16, device=dev)
    t = timed(lambda: F.octree_conv_rows(rows_ne, C, w16, octree, 9, C, out=rows_ne_out, nempty=True), reps, wu)
    fl = 2.0 * Hne9 * 27 * C * C
    extra["conv333_s1_d9_bf16_nempty_rows"] = {"ms": t, "octants_per_s": Hne9 / (t * 1e-3), "tflops": fl / (t * 1e-3) / 1e12,
                                               "frac_mfma_peak": fl / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS["bf16"],
                                               "layout": "row-major in and out, no copy; flops counted densely (27 taps a column)"}
    # the same as a layer of a network at inference sees it: the weights packed once, the table of
    # source rows of this level (octree, depth and kernel shape only) made once and kept
    t = timed(lambda: F.octree_conv_rows(rows_ne, C, w16, octree, 9, C, out=rows_ne_out, nempty=True,
                                         constant_weights=True), reps, wu)
    extra["conv333_s1_d9_bf16_nempty_rows_kept_tables"] = {
        "ms": t, "octants_per_s": Hne9 / (t * 1e-3), "tflops": fl / (t * 1e-3) / 1e12,
        "frac_mfma_peak": fl / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS["bf16"],
        "layout": "row-major in and out; packed weights and the level's source rows kept between calls; "
                  "flops counted densely (27 taps a column)"}
    del rows_ne, rows_ne_out
    x8 = torch.randn(1, C, Hne8, 1, generator=g).to(dev)
    conv_case("deconv222_s2_d8to9_f32", octree, 8, x8, w2, [2, 2, 2], 2, deconv=True)

    # bandwidth-bound kernels on the depth-9 scene (algorithmic bytes / time)
    s = 4
    t = timed(lambda: F.octree_max_pool(x32, octree, 9), reps, wu)
    by = C * H9 * s + C * (H9 // 8) * (s + 4)
    extra["max_pool_d9_f32"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}
    top, mask = F.octree_max_pool(x32, octree, 9)
    t = timed(lambda: F.octree_max_unpool(top, mask, octree, 9), reps, wu)
    extra["max_unpool_d9_f32"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}
    t = timed(lambda: F.octree_pad(top, octree, 8), reps, wu)
    by = C * (Hne8 + H8) * s + H8 * 4
    extra["pad_d8_f32"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}
    # neighbour table of depth 9 from depth 8 (the kernel octree_batch / octree_grow run)
    neigh8 = F.octree_property(octree, "neigh", 8).reshape(-1)
    child8 = F.octree_property(octree, "child", 8)
    neigh9 = torch.empty(H9 * 8, dtype=torch.int32, device=dev)
    import ctypes as Ct
    st = lambda: Ct.c_void_p(torch.cuda.current_stream().cuda_stream)
    t = timed(lambda: oc.lib.call("ocnn_calc_neigh_sparse", Ct.c_void_p(neigh9.data_ptr()),
                                  Ct.c_void_p(neigh8.data_ptr()), Ct.c_void_p(child8.data_ptr()),
                                  H8, st()), reps, wu)
    by = H9 * 8 * 4 + H8 * (4 + 8 * 4)
    extra["calc_neigh_d9"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}

    # octree construction: wall time including its one device-to-host copy
    def build_scene():
      return F.points2octree_batch([scene_pts], 9, 2)
    # (a call lasts 0.13 ms: a handful of calls would time the device's clocks coming up)
    n_build = max(reps, 50)
    for _ in range(10):
      build_scene()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_build):
      build_scene()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / n_build
    by = 250000 * (12 + 12 + 12) + sum(info.nnum(d) * (12 + 32) for d in range(10)) + H9 * 4 * 6 + 720
    extra["points2octree_scene_d9"] = {"ms": t * 1e3, "Mpts_per_s": 0.25 / t,
                                       "GBs": by / t / 1e9, "frac_hbm_peak": by / t / 1e9 / PEAK_HBM_GBS}

    # the same build at a size where launches no longer dominate: 8 scenes merged, 2 M points
    big = []
    for i in range(8):
      q = points_tensor(pts + np.float32(1e-4 * i), nrm, rgb)
      q._ocnn_points_info = q[:88].cpu().numpy().copy()
      big.append(q)
    for _ in range(4):
      ob = F.points2octree_batch(big, 9, 2)
    torch.cuda.synchronize()
    n_build = max(reps, 20)
    t0 = time.perf_counter()
    for _ in range(n_build):
      ob = F.points2octree_batch(big, 9, 2)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / n_build
    ib = F.octree_info(ob)
    nodes = sum(ib.nnum(d) for d in range(10))
    by = 2.0e6 * 48 + nodes * 44 + ib.nnum(9) * 4 * 6 + 720
    extra["points2octree_8scenes_d9"] = {"ms": t * 1e3, "Mpts_per_s": 2.0 / t, "nodes": nodes,
                                         "GBs": by / t / 1e9, "frac_hbm_peak": by / t / 1e9 / PEAK_HBM_GBS}
    del big, ob

    # point-cloud transforms in front of the build (normalise -> rotate/scale/jitter -> clip)
    def transform_scene():
      q = F.normalize_points(scene_pts, 1.05, [0.01, 0.0, -0.01])
      q = F.transform_points(q, [0.05, 0.1, -0.05], [1.1, 0.9, 1.0], [0.05, -0.05, 0.02], 0.0, "")
      return F.clip_points(q, [-1.0] * 3, [1.0] * 3)
    transform_scene()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
      transform_scene()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / reps
    pbytes = scene_pts.numel()
    extra["normalize_transform_clip_scene"] = {"ms": t * 1e3, "Mpts_per_s": 0.25 / t,
                                               "GBs": 6 * pbytes / t / 1e9}
    t0 = time.perf_counter()
    for _ in range(reps):
      F.bounding_sphere(scene_pts, "sphere")
    extra["bounding_sphere_scene"] = {"ms": (time.perf_counter() - t0) / reps * 1e3}

    # trilinear interpolation of 64 channels at 1 M points on the scanned surfaces (segmentation
    # head: the scene's own points, each four times with a jitter of a third of a cell, so that
    # nearly every corner exists), and octree_align of the depth-9 features onto the same octree
    base = torch.from_numpy(((pts + 1.0) * 256.0).astype(np.float32)).repeat(5, 1)[:1 << 20]
    base = (base + (torch.rand(base.shape, generator=g) - 0.5) * 0.66).clamp(0.51, 511.49)
    ipts = torch.cat([base, torch.zeros(1 << 20, 1)], dim=1).to(dev)
    t = timed(lambda: F.octree_interp_pts(x32, octree, 9, ipts, "linear"), reps, wu)
    extra["trilinear_1Mpts_c64_d9"] = {"ms": t, "Mpts_per_s": (1 << 20) / t / 1e3,
                                       "GBs": (1 << 20) * (64 * 4 * 9 + 16) / t / 1e6}
    _, iidx, iw = F.octree_interp_pts(x32, octree, 9, ipts, "linear")
    gpts = torch.randn(1, C, 1 << 20, 1, device=dev)
    t = timed(lambda: F.octree_interp_pts_grad(gpts, iidx, iw, H9, "linear"), reps, wu)
    extra["trilinear_grad_1Mpts_c64_d9"] = {"ms": t, "Mpts_per_s": (1 << 20) / t / 1e3}
    del gpts, iidx, iw
    t = timed(lambda: F.octree_align(x32, octree, octree, 9), reps, wu)
    by = 2 * C * H9 * 4 + H9 * 20
    extra["octree_align_d9_c64"] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}

    # depth-7 batch (configs[2]): 16 clouds of 50 000 points
    clouds = [oc.synthetic.shape_cloud(50000, 200 + i) for i in range(16)]
    cl = [points_tensor(*c) for c in clouds]
    for c in cl:
      c._ocnn_points_info = c[:88].cpu().numpy().copy()
    oct7 = F.points2octree_batch(cl, 7, 2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
      F.points2octree_batch(cl, 7, 2)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / reps
    extra["points2octree_batch16_d7"] = {"ms": t * 1e3, "Mpts_per_s": 0.8 / t}
    # the adaptive build of configs[4]'s input: all-depth signals, plane-fit errors, trimming,
    # the whole batch as one octree in merged layout (summation order of the reference kept: bit-exact)
    adp = dict(node_dis=True, split_label=True, adaptive=True, adp_depth=4, th_normal=0.1, th_distance=2.0)
    F.points2octree_batch(cl, 7, 2, **adp)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max(2, reps // 4)):
      F.points2octree_batch(cl, 7, 2, **adp)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / max(2, reps // 4)
    extra["points2octree_adaptive_batch16_d7"] = {"ms": t * 1e3, "Mpts_per_s": 0.8 / t}
    i7 = F.octree_info(oct7)
    H7 = i7.nnum(7)
    x7 = torch.randn(1, C, H7, 1, generator=g).to(dev)
    extra["octants_d7"] = H7
    conv_case("conv333_s1_d7_f32", oct7, 7, x7, w32, [3, 3, 3], 1)
    conv_case("conv333_s1_d7_bf16", oct7, 7, x7.bfloat16(), w16, [3, 3, 3], 1)
    conv_case("conv222_s2_d7_f32", oct7, 7, x7, w2, [2, 2, 2], 2)
    conv_case("conv222_s2_d7_bf16", oct7, 7, x7.bfloat16(), w2.bfloat16(), [2, 2, 2], 2)
    conv_case("deconv222_s2_d8to9_bf16", octree, 8, x8.bfloat16(), w2.bfloat16(), [2, 2, 2], 2, deconv=True)
    conv_case("deconv333_s1_d9_f32", octree, 9, x32, w32, [3, 3, 3], 1, deconv=True)
    # gradients of the headline conv: weight gradient (contraction over the octants) + data
    # gradient (the transposed operator); 2 x the forward flops in total
    gy = torch.randn(1, C, H9, 1, generator=g).to(dev)
    t = timed(lambda: F.octree_conv_grad(x32, w32, octree, gy, 9, C, [3, 3, 3], 1, False), max(4, reps // 2), 3)
    fl = 2 * 2.0 * H9 * 27 * C * C
    extra["conv333_s1_d9_f32_grad"] = {"ms": t, "octants_per_s": H9 / (t * 1e-3), "tflops": fl / (t * 1e-3) / 1e12,
                                       "frac_mfma_peak": fl / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS["f32"]}

    # the weight gradient alone, for the shapes a network over the non-empty nodes trains with
    # (3x3x3 over the non-empty nodes, 2x2x2 stride 2 down and its deconvolution up)
    def wgrad_case(name, fn, x, w_, gy_, depth, ks, stride, nempty, cols):
      t = timed(lambda: fn(x, w_, octree, gy_, depth, C, ks, stride, nempty, need_data=False), max(4, reps // 2), 3)
      fl = 2.0 * cols * ks[0] * ks[1] * ks[2] * C * C
      extra[name] = {"ms": t, "tflops": fl / (t * 1e-3) / 1e12, "frac_mfma_peak": fl / (t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS["f32"]}
    gne = torch.randn(1, C, Hne9, 1, generator=g).to(dev)
    wgrad_case("conv333_s1_d9_f32_nempty_wgrad", F.octree_conv_grad, xne, w32, gne, 9, [3, 3, 3], 1, True, Hne9)
    g8 = torch.randn(1, C, Hne8, 1, generator=g).to(dev)
    wgrad_case("conv222_s2_d9_f32_wgrad", F.octree_conv_grad, x32, w2, g8, 9, [2, 2, 2], 2, False, Hne8)
    wgrad_case("deconv222_s2_d8to9_f32_wgrad", F.octree_deconv_grad, x8, w2, gy, 8, [2, 2, 2], 2, False, Hne8)
    del gne, g8

    def hbm(name, t, by):
      extra[name] = {"ms": t, "GBs": by / t / 1e6, "frac_hbm_peak": by / t / 1e6 / PEAK_HBM_GBS}

    # remaining streaming ops of the path on the depth-9 scene
    pd8 = F.octree_pad(top, octree, 8)
    hbm("depad_d8_f32", timed(lambda: F.octree_depad(pd8, octree, 8), reps, wu), C * (Hne8 + H8) * s + H8 * 4)
    hbm("mask_pool_d9_f32", timed(lambda: F.octree_mask_pool(x32, mask, octree, 9), reps, wu),
        C * (H9 // 8) * (2 * s + 4))
    # the operation reads one of the eight children of every parent, i.e. 4 of every 32 bytes of
    # the input: every line of the input is fetched.  Bytes of the lines it touches, beside the
    # algorithmic ones (the counters agree: profiles/hbm_counters__bench_default_workloads.md)
    lines = C * H9 * s + C * (H9 // 8) * (s + 4)
    extra["mask_pool_d9_f32"].update({"GBs_of_touched_lines": lines / extra["mask_pool_d9_f32"]["ms"] / 1e6,
                                      "frac_hbm_peak_of_touched_lines": lines / extra["mask_pool_d9_f32"]["ms"] / 1e6 / PEAK_HBM_GBS})
    hbm("max_pool_d9_bf16", timed(lambda: F.octree_max_pool(x16, octree, 9), reps, wu),
        C * H9 * 2 + C * (H9 // 8) * (2 + 4))
    c8 = 8
    xc = x32[:, :c8].contiguous()
    col = F.octree2col(xc, octree, 9, [3, 3, 3], 1, False)
    by = c8 * H9 * s + H9 * 8 * 4 + c8 * 27 * H9 * s
    hbm("octree2col_333_d9_c8_f32", timed(lambda: F.octree2col(xc, octree, 9, [3, 3, 3], 1, False), reps, wu), by)
    hbm("col2octree_333_d9_c8_f32", timed(lambda: F.col2octree(col, octree, 9, [3, 3, 3], 1, False), reps, wu), by)
    del col
    # integer kernels
    key9 = F.octree_property(octree, "key", 9)
    hbm("xyz2key_d9", timed(lambda: F.octree_xyz2key(key9, 9), reps, wu), H9 * 16)
    q = key9[torch.randint(0, H9, (1 << 20,), generator=g).to(dev)]
    hbm("search_key_d9_1Mq", timed(lambda: F.octree_search_key(q, octree, 9, False, False), reps, wu),
        (1 << 20) * 12)
    # 1 M random queries in 1.5 M keys through the sample tables of ocnn_search_key_indexed: a line
    # of the fine table (L2) and a line of keys per query; the plain binary search took 0.086 ms and
    # fetched 435 bytes per query (profiles/hbm_counters__bench_default_workloads.md has the counters)
    lab = (child8 >= 0).to(torch.int32)
    P = lambda t_: Ct.c_void_p(t_.data_ptr())
    lab_out = torch.empty_like(lab)
    cnt = torch.zeros(1, dtype=torch.int32, device=dev)
    sb = oc.lib.get().ocnn_generate_label_scratch_bytes(H8)
    scratch = torch.empty(sb, dtype=torch.uint8, device=dev)
    hbm("generate_label_d8", timed(lambda: oc.lib.call("ocnn_generate_label", P(lab_out), P(cnt), P(lab), H8, 1,
                                                          P(scratch), Ct.c_size_t(sb), st()), reps, wu), H8 * 8)
    # decoder-side growth: octree_update(depth 8) + octree_grow(to depth 9) of the depth-8 prefix
    oct8 = F.octree_new(1, 4, False)
    for d in range(1, 3):
      oct8 = F.octree_grow(oct8, d, True)
    for d in range(2, 9):
      labd = (F.octree_property(octree, "child", d) >= 0).to(torch.int32)
      oct8 = F.octree_update(oct8, labd, d, 1)
      if d < 8:
        oct8 = F.octree_grow(oct8, d + 1, False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
      grown = F.octree_grow(F.octree_update(oct8, lab, 8, 1), 9, False)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / reps
    # (GBs: the bytes of the new level and what they are made from; moved: both operators return a
    # new blob as the reference's do, so the depth-8 blob is read twice and written once beside the
    # grown one)
    moved = 3 * oct8.numel() + grown.numel() + H8 * 4
    extra["octree_update_d8_plus_grow_d9"] = {
        "ms": t * 1e3, "new_nodes": F.octree_info(grown).nnum(9),
        "GBs": (H9 * (8 + 4 + 32) + H8 * (4 + 4 + 32 + 8)) / t / 1e9,
        "GBs_moved": moved / t / 1e9, "frac_hbm_peak_moved": moved / t / 1e9 / PEAK_HBM_GBS}
    # merge of 16 separately built, serialized octrees (octree_batch on device blobs)
    singles = [F.points2octree(c, 7, 2) for c in cl]
    for _ in range(2):   # untimed, like every other row: the first calls also grow torch's memory pool
      F.octree_batch(singles)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
      F.octree_batch(singles)
    torch.cuda.synchronize()
    extra["octree_batch_16_blobs_d7"] = {"ms": (time.perf_counter() - t0) / reps * 1e3,
                                         "nodes": int(sum(i7.nnum(d) for d in range(8)))}

    # operator sequences with folded BatchNorm (conv + bias + ReLU fused)
    def rand_params(spec):
      prm = {}
      for key, shape in spec.items():
        cout = shape[1] // 8 if key[0] == "up" else shape[0]
        fan = shape[0] if key[0] == "up" else shape[1]
        prm[key] = ((torch.randn(*shape, generator=g) / fan ** 0.5).to(dev),
                    (torch.randn(cout, generator=g) * 0.1).to(dev))
      return prm

    ch = {9: 32, 8: 64, 7: 128, 6: 256}
    spec = {("conv", 9): (32, 6 * 27)}
    for d in (9, 8, 7):
      spec[("down", d)] = (ch[d - 1], ch[d] * 8)
      spec[("conv", d - 1)] = (ch[d - 1], ch[d - 1] * 27)
    for d in (6, 7, 8):
      spec[("up", d)] = (ch[d], ch[d + 1] * 8)
      spec[("dec", d + 1)] = (ch[d + 1], 2 * ch[d + 1] * 27)
    up = rand_params(spec)
    feat9 = F.octree_property(octree, "feature", 9)
    t = timed(lambda: oc.stacks.unet_trunk(octree, 9, up, data=feat9), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_f32"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    up16 = {k: (w.bfloat16(), b) for k, (w, b) in up.items()}
    f16 = feat9.bfloat16()
    t = timed(lambda: oc.stacks.unet_trunk(octree, 9, up16, data=f16), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_bf16"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    # the same trunk with row-major activations between the operators (converted once at each end)
    t = timed(lambda: oc.stacks.unet_trunk_rows(octree, 9, up16, data=f16), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_bf16_rows"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    # the same trunk over the non-empty nodes only (the reference's ScanNet setting)
    fne = F.octree_depad(feat9, octree, 9)
    fne16 = fne.bfloat16()
    t = timed(lambda: oc.stacks.unet_trunk(octree, 9, up, data=fne, nempty=True), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_f32_nempty"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    t = timed(lambda: oc.stacks.unet_trunk(octree, 9, up16, data=fne16, nempty=True), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_bf16_nempty"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    t = timed(lambda: oc.stacks.unet_trunk_rows(octree, 9, up16, data=fne16, nempty=True), max(2, reps // 2), 1)
    extra["unet_trunk_scene_d9_bf16_nempty_rows"] = {"ms": t, "points_per_s": 250000 / (t * 1e-3)}
    clouds2 = [points_tensor(*oc.synthetic.shape_cloud(10000, 100 + i)) for i in range(32)]
    oct6 = F.points2octree_batch(clouds2, 6, 2)
    lch = {6: (3, 32), 5: (32, 64), 4: (64, 128), 3: (128, 256)}
    lp = {d: ((torch.randn(co, ci * 27, generator=g) / (ci * 27) ** 0.5).to(dev),
              (torch.randn(co, generator=g) * 0.1).to(dev)) for d, (ci, co) in lch.items()}
    t = timed(lambda: oc.stacks.lenet_trunk(oct6, 6, lp), reps, wu)
    extra["lenet_trunk_batch32_d6_f32"] = {"ms": t, "shapes_per_s": 32 / (t * 1e-3)}
    lp16 = {d: (w.bfloat16(), b) for d, (w, b) in lp.items()}
    feat6_16 = F.octree_property(oct6, "feature", 6).bfloat16()
    t = timed(lambda: oc.stacks.lenet_trunk(oct6, 6, lp16, data=feat6_16), reps, wu)
    extra["lenet_trunk_batch32_d6_bf16"] = {"ms": t, "shapes_per_s": 32 / (t * 1e-3)}
    t = timed(lambda: oc.stacks.lenet_trunk_rows(oct6, 6, lp16, data=feat6_16), reps, wu)
    extra["lenet_trunk_batch32_d6_bf16_rows"] = {"ms": t, "shapes_per_s": 32 / (t * 1e-3),
                                                 "layout": "row-major between conv and pool (pool + pad in one kernel)"}
    # the same trunk captured once in a HIP graph and replayed: what of the eager time is the host
    # getting from one launch to the next (little: the convolutions of the small levels take it)
    feat6 = F.octree_property(oct6, "feature", 6)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      for _ in range(2):
        oc.stacks.lenet_trunk(oct6, 6, lp, data=feat6)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      graph_out = oc.stacks.lenet_trunk(oct6, 6, lp, data=feat6)
    t = timed(graph.replay, reps, wu)
    torch.cuda.synchronize()
    same = bool(torch.equal(graph_out, oc.stacks.lenet_trunk(oct6, 6, lp, data=feat6)))
    extra["lenet_trunk_batch32_d6_f32_graph"] = {"ms": t, "shapes_per_s": 32 / (t * 1e-3), "equals_eager": same}
    del graph, graph_out
    # completion decoder loop (configs[4] shape, pytorch/ocnn/ounet.py:72-131): 16 octrees at depth 7
    # regrown from depth 2 with the split labels of the built batch; per depth a deconv up, the
    # encoder's feature moved onto the growing octree (octree_align) and added, a 3x3x3 conv, the
    # split head (1x1x1 -> 32 -> 2, argmax), octree_update and octree_grow; channels 256 -> 32
    dch = {2: 256, 3: 128, 4: 64, 5: 32, 6: 32, 7: 32}
    dspec = {}
    for d in range(3, 8):
      dspec[("up", d)] = (dch[d - 1], dch[d] * 8)
      dspec[("conv", d)] = (dch[d], dch[d] * 27)
    dp = rand_params(dspec)
    dlabels = {d: (F.octree_property(oct7, "child", d) >= 0).to(torch.int32) for d in range(2, 8)}
    code = torch.randn(1, 256, 16 * 64, 1, generator=g).to(dev)
    t = timed(lambda: oc.stacks.completion_decoder(code, dp, dlabels, 7, 2, batch_size=16), max(2, reps // 2), 1)
    extra["completion_decoder_batch16_d7_f32_plain"] = {"ms": t, "octants_d7": H7, "octrees_per_s": 16 / (t * 1e-3),
                                                        "ops": "deconv, conv, update, grow (no skips, no heads)"}
    heads = rand_params({("h1", d): (32, dch[d]) for d in range(2, 8)})
    heads2 = rand_params({("h2", d): (2, 32) for d in range(2, 8)})
    for d in range(2, 8):
      dp[("predict", d)] = (heads[("h1", d)], heads2[("h2", d)])
    i7 = F.octree_info(oct7)
    dskips = {d: torch.randn(1, dch[d], i7.nnum(d), 1, generator=g).to(dev) for d in range(3, 8)}
    t = timed(lambda: oc.stacks.completion_decoder(code, dp, dlabels, 7, 2, batch_size=16, skips=dskips, octree_in=oct7),
              max(2, reps // 2), 1)
    extra["completion_decoder_batch16_d7_f32"] = {"ms": t, "octants_d7": H7, "octrees_per_s": 16 / (t * 1e-3),
                                                  "ops": "deconv, octree_align skip, conv, split head + argmax, update, grow"}
  out["extra"] = extra

  # ---- CPU baseline (reported, not the target) -----------------------------------------------
  if not (args.quick or args.no_cpu):
    from oracle.checker import Checker, OctreeBlob
    orc = Checker("orc")
    # the reference's own CPU functions where oracle/_ref holds them compiled (octree2col_cpu, the
    # pooling and padding loops, the build); the GEMM is the oracle's textbook one either way: the
    # reference has no CPU GEMM of its own (its CPU path calls a BLAS, octree_conv.cpp:276-325)
    ref_ok = os.path.exists(os.path.join(ROOT, "oracle", "_ref", "libocnn_ref.so"))
    chk = Checker("ref") if ref_ok else orc
    kind = "reference" if ref_ok else "port"
    blob_host = octree.cpu().numpy()
    ob = OctreeBlob(blob_host)
    sample = 327680   # about 10 s of single-thread work
    neigh = ob.prop("neigh", 9).reshape(-1)
    xh = x32.cpu().numpy().reshape(C, H9)
    wh = w32.cpu().numpy()
    ni = chk.get_ni([3, 3, 3])
    col = np.empty((C * 27, sample), np.float32)
    import ctypes as Ct
    P = lambda a: a.ctypes.data_as(Ct.c_void_p)
    t0 = time.perf_counter()
    # first chunk of `sample` columns: octree2col_cpu chunk + single-thread SGEMM
    chk.fn("octree2col")(P(col), P(xh), C, H9, 27, 1, P(neigh), P(ni), sample, 0)
    y = orc.sgemm(wh, col)
    t = time.perf_counter() - t0
    out["cpu_baseline"] = {"value": sample / t, "unit": "octants/s", "cores": 1, "kind": kind,
                           "sample": "first %d of %d depth-9 octants: %s octree2col_cpu chunk + "
                                     "single-thread textbook SGEMM (64 x 1728 x %d; the reference has no CPU GEMM "
                                     "of its own), %.1f s"
                                     % (sample, H9, "the compiled reference's" if ref_ok else "the oracle's", sample, t)}
    # the host this ran on, and the same sample with the GEMM through torch.mm on all its threads
    # (the reference's CPU path calls a BLAS GEMM there, octree/octree/octree_conv.cpp:276-325)
    try:
      model = [l.split(":", 1)[1].strip() for l in open("/proc/cpuinfo") if l.startswith("model name")]
    except OSError:
      model = []
    out["cpu_baseline"]["host"] = {"nproc": os.cpu_count(), "cpu_model": model[0] if model else "unknown",
                                   "usable_cpus": len(os.sched_getaffinity(0))}
    wt, ct = torch.from_numpy(wh), torch.from_numpy(col)
    torch.mm(wt, ct)
    t0 = time.perf_counter()
    n_mm = 5
    for _ in range(n_mm):
      ymm = torch.mm(wt, ct)
    t_mm = (time.perf_counter() - t0) / n_mm
    t0 = time.perf_counter()
    chk.fn("octree2col")(P(col), P(xh), C, H9, 27, 1, P(neigh), P(ni), sample, 0)
    t_col = time.perf_counter() - t0
    out["cpu_baseline"]["blas_all_threads"] = {
        "value": sample / (t_col + t_mm), "unit": "octants/s", "threads": torch.get_num_threads(),
        "gemm_gflops": 2.0 * C * C * 27 * sample / t_mm / 1e9, "octree2col_seconds": t_col, "gemm_seconds": t_mm,
        "max_rel_diff_vs_port": float(np.abs(ymm.numpy() - y).max() / np.abs(y).max()),
        "sample": "the same %d columns: octree2col_cpu chunk on one core + torch.mm on all threads" % sample}
    # the sample also checks the GPU result
    yg = conv_step().cpu().numpy().reshape(C, H9)[:, :sample]
    out["cpu_baseline"]["gpu_vs_cpu_max_rel_err"] = float(np.abs(yg - y).max() / np.abs(y).max())
    pb = scene_pts.cpu().numpy()
    t0 = time.perf_counter()
    single = chk.points2octree(pb, 9, 2)
    merged = chk.octree_batch([single])
    t = time.perf_counter() - t0
    out["cpu_baseline"]["points2octree_plus_batch"] = {
        "Mpts_per_s": 0.25 / t, "seconds": t, "cores": 1, "kind": "reference" if ref_ok else "port",
        "bit_exact_vs_gpu": bool(np.array_equal(merged, blob_host))}
    # the other rows of the path on one host core, same scene (bounded: a few seconds in total)
    rows = {}

    def cpu_row(name, fn, units, unit):
      t0 = time.perf_counter()
      r = fn()
      dt = time.perf_counter() - t0
      rows[name] = {"seconds": dt, unit: units / dt, "cores": 1, "kind": kind if name not in port_only else "port"}
      return r

    port_only = ("octree_update_d8",)   # pytorch/cpp/octree_grow.cpp is part of the extension, not of the compiled library

    Cs = 16  # channels of the streaming samples
    xs = xh[:Cs]
    pooled, maskh = cpu_row("max_pool_d9", lambda: chk.max_pool(xs), H9, "octants_per_s")
    cpu_row("max_unpool_d9", lambda: chk.max_unpool(pooled, maskh), H9, "octants_per_s")
    cpu_row("mask_pool_d9", lambda: chk.mask_pool(xs, maskh), H9, "octants_per_s")
    child8 = ob.prop("child", 8)
    padded = cpu_row("pad_d8", lambda: chk.pad(pooled, child8), H8, "octants_per_s")
    cpu_row("depad_d8", lambda: chk.depad(padded, child8, pooled.shape[1]), H8, "octants_per_s")
    cpu_row("octree_batch_with_calc_neigh", lambda: chk.octree_batch([single]), sum(ob.nnum[:10]), "nodes_per_s")
    lab8 = (child8 >= 0).astype(np.int32)
    upd = cpu_row("octree_update_d8", lambda: orc.octree_update(merged, lab8, 8, 1), H8, "nodes_per_s")
    del upd
    pb5 = oc_points_blob(oc.synthetic.shape_cloud(50000, 200))
    cpu_row("points2octree_adaptive_one_cloud_d7", lambda: chk.points2octree(
        pb5, 7, 2, node_dis=True, split_label=True, adaptive=True, adp_depth=4, th_normal=0.1, th_distance=2.0),
        50000, "points_per_s")
    rows["points2octree_adaptive_one_cloud_d7"]["kind"] = "reference" if ref_ok else "port"
    out["cpu_baseline"]["rows"] = rows

  print(json.dumps(out))


if __name__ == "__main__":
  main()
