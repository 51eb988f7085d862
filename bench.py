#!/usr/bin/env python3
"""Benchmark of the BERT forward pass on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C1] [--no-cpu]

A step is one forward pass of the workload (default C1: BERT-base fp32, batch 128, seq_len 32,
the configuration the headline metric is quoted on) on inputs already resident in device memory.
Prints ONE JSON line:
  value / ms_per_step   sequences/s over the K timed device-resident steps (inputs already in HBM when the timed
                        region starts)
  reference_protocol    the same workload the way the reference's benchmark client measures it
                        (benchmark/benchmark_cu.cpp:68-78): host arrays in, POOLED_OUTPUT host array out, 10 warm-up
                        calls, then max(K, 50) timed calls, PCIe-inclusive; mean and p50 per call, sequences/s
  p50_ms_batch1_host_path   the same call with one sequence: the latency half of the headline metric
  roofline              the dominant fused kernel (bias+GELU), HIP events carried by its launches inside the timed steps
  kernels               every kernel kind of the forward pass: average launch time, GB/s, fraction of the HBM peak
                        (the dominant kernel's row is the `roofline` measurement: one timing per kernel)
  gemm                  the Dense GEMMs one by one and in total: FLOPs, average microseconds, TFLOP/s and the fraction
                        of the matrix-core peak of the arithmetic type (fp32 157.3 TFLOP/s, fp16 2.5 PFLOP/s)
  clean_roofline        `kernels` and `gemm` at C3 (BERT-base fp16, batch 64, seq_len 512), whose tensors do not fit the
                        256 MB Infinity Cache: the workload where a fraction of the HBM peak is an HBM statement
  cpu_baseline          the CPU oracle on this host's cores on a bounded sample of the same workload, with the
                        thread counts the libraries report and the time per part of a pass
"""
import argparse
import faulthandler
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0}  # dense matrix-core peaks of the part, by operand type
# How a launch's event pair reads against a profiler's kernel duration (measured on bias+GELU at C1: 17.2-17.4 us by
# the pair, 15.9-16.4 us by rocprofv3 in profiles/forward_C1_kernel_stats.md): fractions computed from event pairs are
# the lower of the two.
EVENT_PAIR_NOTE = ("HIP event pair carried by each launch (start/stop of the dispatch); reads 1-1.5 us above "
                   "rocprofv3's kernel duration for the same launch, so fractions from it are the conservative ones")

# Bytes per launch that crossed the L2 <-> memory boundary, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script scaled by a plain copy of known size (method and table: profiles/traffic_pmc.md).  Hardware counters
# need the profiler, so these are recorded values, not measured by a plain run: each is tied to the SHA-256 of the
# kernel source it was measured on and is reported only while that file is unchanged.
TRAFFIC_PROFILE = "profiles/traffic_pmc.md"
TRAFFIC_SOURCE = {  # kernel kind -> (source file under cubert_amd/csrc/kernels, first 16 hex digits of its SHA-256)
    "bias_gelu": ("elementwise.hip", "59dcc33f61344079"),
    "bias_tanh": ("elementwise.hip", "59dcc33f61344079"),
    "bias_res_ln": ("layernorm.hip", "63cfef94a6b85850"),
    "embed_ln": ("layernorm.hip", "63cfef94a6b85850"),
    "mask_scale_softmax": ("softmax.hip", "90a529eac55169fa"),
    "mean_pool": ("elementwise.hip", "59dcc33f61344079"),
    "classifier_head": ("elementwise.hip", "59dcc33f61344079"),
    "attention_fused": ("attention.hip", "4d44df3fda986cf4"),
}
MEASURED_TRAFFIC = {
    "C1": {
        "embed_ln": 25327834,
        "attention_fused": 50081947,
        "bias_res_ln": 37631060,
        "bias_gelu": 100340726,
        "classifier_head": 934419,
        "mask_scale_softmax": 12589780
    },
    "C2": {
        "embed_ln": 12897102,
        "attention_fused": 25138619,
        "bias_res_ln": 18850804,
        "bias_gelu": 50185082,
        "mean_pool": 6325077,
        "classifier_head": 147249,
        "mask_scale_softmax": 25117480
    },
    "C3": {
        "embed_ln": 99732176,
        "attention_fused": 128669549,
        "bias_res_ln": 150191566,
        "bias_gelu": 400908911,
        "classifier_head": 308694,
        "mask_scale_softmax": 801926098
    },
    "C4": {
        "embed_ln": 133757147,
        "attention_fused": 267267773,
        "bias_res_ln": 200203032,
        "bias_gelu": 534519157,
        "classifier_head": 1199518,
        "mask_scale_softmax": 267503966
    }
}


def recorded_traffic(workload, kind):
    """(bytes per launch or None, where the figure comes from / why it is withheld)."""
    value = MEASURED_TRAFFIC.get(workload, {}).get(kind)
    if value is None or kind not in TRAFFIC_SOURCE:
        return None, "no hardware-counter run recorded for this kernel and workload"
    name, digest = TRAFFIC_SOURCE[kind]
    path = os.path.join(ROOT, "cubert_amd", "csrc", "kernels", name)
    try:
        with open(path, "rb") as f:
            now = hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        return None, "kernel source %s not found" % name
    if now != digest:
        return None, "%s changed since the counter run recorded in %s (then %s, now %s)" % (name, TRAFFIC_PROFILE,
                                                                                           digest, now)
    return value, "recorded, not measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, %s; %s unchanged " \
                  "since (sha256 %s)" % (TRAFFIC_PROFILE, name, digest)


def two_term_dense():
    """CUBERT_FP32_DENSE=f16x3 in the environment: fp32 models run their Dense layers (requests of at least 384 tokens) on the
    fp16 matrix cores from two-term operands (opt-in; the default is the fp32 GEMM)."""
    return os.environ.get("CUBERT_FP32_DENSE") == "f16x3"


def algorithmic_bytes(cfg):
    """Minimum HBM traffic per launch of each fused kernel (bytes): every operand once."""
    m = cfg["model"]
    B, S = cfg["batch"], cfg["seq_length"]
    H, I, A = m["hidden"], m["intermediate"], m["heads"]
    e = 4 if cfg["dtype"] == "f32" else 2
    M = B * S
    if two_term_dense() and e == 4 and M >= 384:
        # bias+GELU reads fp32 and writes [hi | hi | lo] fp16 rows; the LayerNorm writes both forms
        extra = {"bias_gelu": M * I * (4 + 6) + I * 4, "bias_res_ln": 3 * M * H * 4 + 3 * H * 4 + 6 * M * H,
                 "dense_split": M * H * (4 + 6)}
    else:
        extra = {}
    return dict(_algorithmic_bytes(cfg), **extra)


def _algorithmic_bytes(cfg):
    m = cfg["model"]
    B, S = cfg["batch"], cfg["seq_length"]
    H, I, A = m["hidden"], m["intermediate"], m["heads"]
    e = 4 if cfg["dtype"] == "f32" else 2
    M = B * S
    return {
        "embed_ln": 2 * M * H * e + 5 * M + (S + 4) * H * e,
        "bias_res_ln": 3 * M * H * e + 3 * H * e,
        "bias_gelu": 2 * M * I * e + I * e,
        "mask_scale_softmax": 2 * B * A * S * S * e + B * S,
        "bias_tanh": 2 * B * H * e + H * e,
        "mean_pool": (M + B) * H * e,
        "row_softmax": 2 * B * cfg["labels"] * e,
        # pooler bias + tanh, classifier and softmax in one launch: pooled in and out, weights in, logits + probs out
        "classifier_head": (2 * B * H + H + cfg["labels"] * H + cfg["labels"] + 2 * B * cfg["labels"]) * e,
        # fused attention core (seq_len <= 128): Q, K, V read, context written, the scores never reach memory
        "attention_fused": 4 * M * H * e + B * S,
    }


def standalone_kernel(kind, cfg, mask, alg_bytes, reps=20):
    """One fused kernel (mask+scale+softmax or bias+GELU) outside the forward pass, at the workload's shape,
    through the C entry points only (no torch in this process: importing it after the library has initialised the
    GPU loads a second copy of the HIP runtime).  `reps` launches in a row on one stream between two events;
    buffers rotate so that no launch finds its input cached by the previous one."""
    import ctypes
    from cubert_amd._lib import lib
    L = lib()
    m = cfg["model"]
    B, S, A = cfg["batch"], cfg["seq_length"], m["heads"]
    half = cfg["dtype"] != "f32"
    dt = np.float16 if half else np.float32
    suffix = "_f16" if half else "_f32"
    n = B * A * S * S if kind == "mask_scale_softmax" else B * S * m["intermediate"]
    block = np.random.default_rng(0).normal(0, 1, 1 << 20).astype(dt)
    host = np.ascontiguousarray(np.resize(block, n))
    n_buf = max(2, min(8, int((1 << 30) // max(1, alg_bytes))))
    bufs = []
    for _ in range(n_buf):
        p = L.cubert_malloc(host.nbytes)
        if not p or L.cubert_memcpy(p, host.ctypes.data, host.nbytes, 1):
            raise RuntimeError("could not set up the buffers")
        bufs.append(p)
    side = np.ascontiguousarray(mask, dtype=np.int8) if kind == "mask_scale_softmax" else block[:m["intermediate"]].copy()
    dside = L.cubert_malloc(side.nbytes)
    L.cubert_memcpy(dside, side.ctypes.data, side.nbytes, 1)
    stream, start, stop = L.cubert_stream_create(), L.cubert_event_create(), L.cubert_event_create()
    fn = getattr(L, "cubert_" + kind + suffix)

    def launch(i):
        if kind == "mask_scale_softmax":
            rc = fn(bufs[i % n_buf], dside, 1.0, B, A, S, stream)
        else:
            rc = fn(bufs[i % n_buf], dside, B * S, m["intermediate"], stream)
        if rc:
            raise RuntimeError("cubert_%s failed with code %d" % (kind, rc))

    for i in range(3):
        launch(i)
    L.cubert_event_record(start, stream)
    for i in range(reps):
        launch(i)
    L.cubert_event_record(stop, stream)
    L.cubert_stream_synchronize(stream)
    ms = ctypes.c_float()
    L.cubert_event_elapsed_ms(start, stop, ctypes.byref(ms))
    for p in bufs + [dside]:
        L.cubert_free(p)
    L.cubert_event_destroy(start)
    L.cubert_event_destroy(stop)
    L.cubert_stream_destroy(stream)
    us = ms.value * 1e3 / reps
    return {"avg_us": round(us, 2), "launches": reps, "GB/s": round(alg_bytes / (us * 1e-6) / 1e9, 1),
            "frac_hbm_peak": round(alg_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "note": "standalone back-to-back launches: the forward pass of this workload does this work inside "
                    "another kernel (%s)" % ("attention_fused" if kind == "mask_scale_softmax" else "the few-token Dense")}


def dense_flops(cfg):
    """{Dense kind: (FLOPs per launch, launches per forward pass, out features, tokens, in features)}."""
    m = cfg["model"]
    B, S = cfg["batch"], cfg["seq_length"]
    H, I, L = m["hidden"], m["intermediate"], m["layers"]
    M = B * S
    shapes = {"dense_qkv": (3 * H, M, H, L), "dense_attention_output": (H, M, H, L),
              "dense_intermediate": (I, M, H, L), "dense_output": (H, M, I, L), "dense_pooler": (H, B, H, 1)}
    return {k: (2.0 * n * t * kk, count, n, t, kk) for k, (n, t, kk, count) in shapes.items()}


def gemm_table(bert, cfg, batch, passes, ms_per_step, kernels, kernel_passes):
    """The Dense GEMMs one by one, from `passes` extra forward passes in which only they are timed: FLOPs, average
    microseconds, TFLOP/s, fraction of the matrix-core peak of the operand type, and the total per forward pass.
    A library call may be several launches, so it sits between two marker events, and that interval also holds the
    gaps to the neighbouring kernels: these times are upper bounds (their sum over a pass plus the other kernels
    exceeds the step time).  `total.by_difference` is the lower bound: the step time minus the event-pair times of
    every other kernel of a pass (`kernels`, measured over `kernel_passes` passes).  The exact durations are the
    profiler's, profiles/forward_*_kernel_stats.md."""
    peak = MFMA_PEAK_TFLOPS[cfg["dtype"]]
    e = 4 if cfg["dtype"] == "f32" else 2
    flops = dense_flops(cfg)
    bert.profile(list(bert.DENSE_KINDS))
    for _ in range(passes):
        bert.compute_resident(batch)
    read = bert.profile_read()
    bert.profile([])
    rows, total_flop, total_ms = {}, 0.0, 0.0
    for k in bert.DENSE_KINDS:
        if k not in read:
            continue
        ms, n = read[k]
        us = ms * 1e3 / n
        fl, per_pass, out_f, tokens, in_f = flops[k]
        tf = fl / (us * 1e-6) / 1e12
        rows[k] = {"out_features": out_f, "tokens": tokens, "in_features": in_f, "GFLOP": round(fl / 1e9, 3),
                   "avg_us": round(us, 2), "launches": n, "TFLOP/s": round(tf, 2), "frac_mfma_peak": round(tf / peak, 4),
                   "weights_GB/s": round(out_f * in_f * e / (us * 1e-6) / 1e9, 1)}
        total_flop += fl * per_pass
        total_ms += ms / passes
    tf = total_flop / (total_ms * 1e-3) / 1e12 if total_ms > 0 else 0.0
    others_ms = sum(row["avg_us"] * 1e-3 * row["launches"] / kernel_passes for k, row in kernels.items()
                    if "note" not in row and k != "dense_gemm")
    rest_ms = ms_per_step - others_ms
    tf_rest = total_flop / (rest_ms * 1e-3) / 1e12 if rest_ms > 0 else 0.0
    return {"peak_TFLOP/s": peak, "operands": cfg["dtype"], "accumulate": "f32", "shapes": rows,
            "total": {"GFLOP_per_pass": round(total_flop / 1e9, 2), "ms_per_pass": round(total_ms, 4),
                      "TFLOP/s": round(tf, 2), "frac_mfma_peak": round(tf / peak, 4),
                      "by_difference": {"ms_per_pass": round(rest_ms, 4), "TFLOP/s": round(tf_rest, 2),
                                        "frac_mfma_peak": round(tf_rest / peak, 4),
                                        "share_of_step": round(rest_ms / ms_per_step, 4) if ms_per_step else None}},
            "timing": "per shape and `total`: marker events around each library call inside full forward passes "
                      "(includes the gaps to the neighbouring kernels: time is an upper bound, TFLOP/s a lower bound); "
                      "`by_difference`: step time minus the event-pair times of all other kernels of a pass (time is a "
                      "lower bound, TFLOP/s an upper bound)"}


def kernel_table(bert, cfg, mask, alg, batch, passes):
    """Every kernel kind of `passes` forward passes with an event pair around each launch:
    {kind: average microseconds, launches, and for the fused kernels GB/s and fraction of the HBM peak}."""
    table = {}
    bert.profile([k for k in bert.KINDS if k not in bert.DENSE_KINDS])
    for _ in range(passes):
        bert.compute_resident(batch)
    for k, (ms, n) in bert.profile_read().items():
        us = ms * 1e3 / n
        table[k] = {"avg_us": round(us, 2), "launches": n}
        if k in alg:
            table[k]["GB/s"] = round(alg[k] / (us * 1e-6) / 1e9, 1)
            table[k]["frac_hbm_peak"] = round(alg[k] / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
    bert.profile([])
    # the forward pass runs the attention core as one kernel where the shape allows and then never launches the
    # mask + scale + softmax kernel, and at <= 32 tokens bias + GELU runs inside the few-token Dense kernel: those are
    # timed by themselves at the workload's shape
    for kind in ("mask_scale_softmax", "bias_gelu"):
        if kind not in table:
            table[kind] = standalone_kernel(kind, cfg, mask, alg[kind])
    return table


def cpu_baseline(workload, cfg, w, ids, mask, seg):
    """The oracle (a port of the reference's CPU path) on this host's cores: a bounded sample of the workload at the
    default thread count and at 4 threads (the reference's CI setting, .travis.yml:25), each with the thread counts
    the libraries report for themselves and the seconds per part of a pass."""
    import ctypes
    import oracle
    m = cfg["model"]
    S = cfg["seq_length"]
    half = cfg["dtype"] == "f16"
    default_threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    oracle.lib()
    try:
        gomp = ctypes.CDLL("libgomp.so.1")
    except OSError:
        gomp = None
    wf = {k: oracle.round_to_half(v) for k, v in w.items()} if half else w
    vars_obj = oracle.Vars(wf)
    n = min(cfg["batch"], 128, max(1, 8192 // S))  # bounded sample: at most 128 sequences and 8192 tokens per pass

    def leg(threads, max_passes, budget_s):
        oracle.set_blas_threads(threads)
        if gomp is not None:
            gomp.omp_set_num_threads(threads)
        oracle.bert_forward(wf, ids[:n], mask[:n], seg[:n], m["layers"], m["heads"], vars_obj=vars_obj)  # warm-up
        oracle.profile_reset()
        times = []
        start = time.perf_counter()
        while len(times) < max_passes and time.perf_counter() - start < budget_s:
            t = time.perf_counter()
            oracle.bert_forward(wf, ids[:n], mask[:n], seg[:n], m["layers"], m["heads"], vars_obj=vars_obj)
            times.append(time.perf_counter() - t)
        parts = {k: round(v / len(times) * 1e3, 1) for k, v in oracle.profile_read().items()}
        return {"value": round(n / float(np.mean(times)), 2), "passes": len(times),
                "ms_per_pass": round(float(np.mean(times)) * 1e3, 1), "ms_per_pass_by_part": parts,
                "threads": oracle.threads_in_use()}

    # The box's CPU share may be smaller than the logical CPUs it shows, and then a full team of spinning OpenMP
    # threads is slower than a small one: the baseline is the best of the default team, half of it and 4 threads
    # (the reference's CI setting), and every leg is reported.
    counts = [default_threads] + [t for t in (default_threads // 2, 4) if 1 <= t < default_threads]
    counts = sorted(set(counts), reverse=True)
    legs = {t: leg(t, 3 if t == default_threads else 2, 12 if t == default_threads else 8) for t in counts}
    oracle.set_blas_threads(default_threads)
    if gomp is not None:
        gomp.omp_set_num_threads(default_threads)
    best = max(legs, key=lambda t: legs[t]["value"])
    main_leg = legs[best]
    four = legs.get(4)
    dense = main_leg["ms_per_pass_by_part"]["dense_gemm"]
    M, H, I = n * S, m["hidden"], m["intermediate"]
    dense_flop = 2.0 * M * (4 * H * H + 2 * H * I) * m["layers"]
    return {"value": main_leg["value"], "unit": "sequences/s", "cores": best, "kind": "port",
            "sample": "%d pass(es) of %d sequences of %s (seq_len %d), fp32, mean %.1f ms/pass" %
                      (main_leg["passes"], n, workload, S, main_leg["ms_per_pass"]),
            "blas": os.path.basename(oracle.blas_name()),
            "label": "restatement of the reference's CPU path on OpenBLAS (attention batches as an OpenMP loop around "
                     "single-threaded sgemm calls, the way cblas_sgemm_batch spreads a group)",
            "threads": main_leg["threads"], "ms_per_pass_by_part": main_leg["ms_per_pass_by_part"],
            "dense_gemm_GFLOPs": round(dense_flop / (dense * 1e-3) / 1e9, 1) if dense > 0 else None,
            "value_at_4_threads": four["value"] if four else None,
            "legs": {"%d threads" % t: legs[t] for t in counts}}


def main():
    faulthandler.enable()  # a crash inside the native library prints the Python stack
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C1")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--all-kernels", action="store_true",
                    help="kept for old command lines: the per-kernel table is always part of the line now")
    ap.add_argument("--no-clean-leg", action="store_true",
                    help="skip the extra leg that times every kernel at C3 (fp16, batch 64, seq_len 512), the workload "
                         "whose tensors do not fit the Infinity Cache (run by default when the workload is C1)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of the model: 10 launches of a plain row copy of known size (100 MB read, 100 MB "
                         "written), the yardstick for hardware traffic counters")
    ap.add_argument("--no-two-term", action="store_true",
                    help="skip the extra leg that repeats the steps with CUBERT_FP32_DENSE=f16x3 (fp32 workloads)")
    ap.add_argument("--device-only", action="store_true",
                    help="only the device-resident steps (no host-path / batch-1 latency loops): for profiler runs")
    ap.add_argument("--instances", type=int, default=0,
                    help="extra leg: this many model instances on the GPU, one caller thread each, every caller sending "
                         "the workload's batch through the host path (what CUBERT_MODELS_PER_GPU gives concurrent "
                         "callers of cuBERT_compute); reported as `concurrent_instances`")
    ap.add_argument("--fp32-dense", choices=["f32", "f16x3"], default=None,
                    help="f16x3: open the model with CUBERT_FP32_DENSE=f16x3 (the opt-in two-term fp16 Dense form of fp32 "
                         "models); default: whatever the environment says, normally the fp32 GEMM")
    args = ap.parse_args()
    if args.fp32_dense == "f16x3":
        os.environ["CUBERT_FP32_DENSE"] = "f16x3"
    elif args.fp32_dense == "f32":
        os.environ.pop("CUBERT_FP32_DENSE", None)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (replicas on several GPUs share nothing); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import cubert_amd
    from cubert_amd.testing import CONFIGS, config_inputs, config_weights

    if args.calibrate_copy:
        import torch
        from cubert_amd import kernels
        rows, width = 32768, 768
        table = torch.randn(rows, width, device="cuda")
        ids = torch.arange(rows, dtype=torch.int32, device="cuda")
        for _ in range(10):
            out = kernels.gather(ids, table)
        torch.cuda.synchronize()
        assert torch.equal(out, table)
        print(json.dumps({"copy_kernel": "gather_kernel<float, int, 4>", "bytes_read": rows * width * 4 + rows * 4,
                          "bytes_written": rows * width * 4, "launches": 10}))
        return

    cfg = CONFIGS[args.workload]
    m = cfg["model"]
    B, S = cfg["batch"], cfg["seq_length"]
    half = cfg["dtype"] == "f16"
    w = config_weights(args.workload, seed=0)
    ids, mask, seg = config_inputs(args.workload, seed=0)

    bert = cubert_amd.Bert(w, B, S, m["layers"], m["heads"], 1 if half else 0)
    bert.compute(ids, mask, seg)  # uploads the inputs; they stay resident
    bert.synchronize()
    for _ in range(args.warmup):
        bert.compute_resident(B)
    bert.synchronize()

    # ---- timed region: K device-resident forward passes; the dominant fused kernel is bracketed by events
    dominant = "bias_gelu"
    bert.profile([dominant])
    t0 = time.perf_counter()
    for _ in range(args.steps):
        bert.compute_resident(B)
    bert.synchronize()
    t1 = time.perf_counter()
    prof = bert.profile_read()
    bert.profile([])
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = B / (ms_per_step * 1e-3)

    alg = algorithmic_bytes(cfg)
    traffic, traffic_source = (None, "no counter run recorded for the two-term form") if two_term_dense() \
        else recorded_traffic(args.workload, dominant)
    if dominant in prof:
        total_ms, launches = prof[dominant]
        avg_us = total_ms * 1e3 / launches
    else:  # at <= 32 tokens bias+GELU runs inside the few-token Dense kernel: time it by itself
        alone = standalone_kernel(dominant, cfg, mask, alg[dominant])
        avg_us, launches = alone["avg_us"], alone["launches"]
    achieved = alg[dominant] / (avg_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "algorithmic_bytes_per_launch": alg[dominant], "avg_launch_us": round(avg_us, 2), "launches": launches,
                "timing": EVENT_PAIR_NOTE + "; launches inside the timed steps"}

    # ---- every kernel kind, in extra untimed passes (reported, not part of `value`)
    table_passes = max(5, args.steps // 5)
    kernels = kernel_table(bert, cfg, mask, alg, B, table_passes)
    gemm = gemm_table(bert, cfg, B, table_passes, ms_per_step, kernels, table_passes)
    if dominant in prof:
        # one timing per kernel: the dominant kernel's row is the measurement `roofline` reports
        kernels[dominant] = {"avg_us": roofline["avg_launch_us"], "launches": launches, "GB/s": roofline["achieved"],
                             "frac_hbm_peak": roofline["frac"], "source": "the timed steps (same figures as `roofline`)"}

    # ---- the public path: host arrays in, host array out (PCIe-inclusive), and p50 latency at batch 1
    host_path, p50_b1 = None, None
    if not args.device_only:
        out = np.empty((B, m["hidden"]), np.float16 if half else np.float32)
        o = cubert_amd.Output(out, cubert_amd.OutputType.POOLED_OUTPUT)
        lat = []
        calls = max(args.steps, 50)
        for i in range(10 + calls):  # 10 warm-up calls as the reference's benchmark client, then the timed ones
            t = time.perf_counter()
            bert.compute(ids, mask, seg)
            bert.output(B, o)
            if i >= 10:
                lat.append((time.perf_counter() - t) * 1e3)
        host_path = {"protocol": "benchmark/benchmark_cu.cpp:68-78 of the reference: host arrays in, POOLED_OUTPUT host "
                                 "array out per call (PCIe-inclusive), 10 warm-up calls, then the timed calls",
                     "warmup_calls": 10, "timed_calls": calls,
                     "mean_ms": round(float(np.mean(lat)), 3), "p50_ms": round(float(np.median(lat)), 3),
                     "sequences_per_s": round(B / (np.mean(lat) * 1e-3), 1), "output": "POOLED_OUTPUT"}
        lat1 = []
        for i in range(20 + 100):
            t = time.perf_counter()
            bert.compute(ids[:1], mask[:1], seg[:1])
            bert.output(1, o)
            if i >= 20:
                lat1.append((time.perf_counter() - t) * 1e3)
        p50_b1 = round(float(np.median(lat1)), 3)
    bert.close()

    # ---- every kernel at C3, where the tensors do not fit the Infinity Cache (same weights: both are BERT-base)
    clean = None
    if args.workload == "C1" and not args.device_only and not args.no_clean_leg and not two_term_dense():
        c3 = CONFIGS["C3"]
        ids3, mask3, seg3 = config_inputs("C3", seed=0)
        big = cubert_amd.Bert(w, c3["batch"], c3["seq_length"], m["layers"], m["heads"], 1)
        big.compute(ids3, mask3, seg3)
        big.synchronize()
        for _ in range(3):
            big.compute_resident(c3["batch"])
        big.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            big.compute_resident(c3["batch"])
        big.synchronize()
        ms3 = (time.perf_counter() - t0) * 1e3 / 10
        alg3 = algorithmic_bytes(c3)
        table3 = kernel_table(big, c3, mask3, alg3, c3["batch"], 5)
        gemm3 = gemm_table(big, c3, c3["batch"], 5, ms3, table3, 5)
        big.close()
        for k, row in table3.items():
            row["traffic"], _ = recorded_traffic("C3", k)
        clean = {"workload": "C3: BERT-base f16 batch %d seq_len %d, valid length min(512, 16 + Exp(96)), inputs "
                             "resident in HBM" % (c3["batch"], c3["seq_length"]),
                 "ms_per_step": round(ms3, 4), "sequences_per_s": round(c3["batch"] / (ms3 * 1e-3), 1), "steps": 10,
                 "kernels": table3, "gemm": gemm3, "kernel_timing": EVENT_PAIR_NOTE}

    # ---- the same steps with the opt-in two-term fp16 Dense form of fp32 models (reported beside `value`, never as it)
    two_term = None
    if not half and B * S >= 384 and not two_term_dense() and not args.device_only and not args.no_two_term:
        os.environ["CUBERT_FP32_DENSE"] = "f16x3"  # read when a model is opened
        try:
            other = cubert_amd.Bert(w, B, S, m["layers"], m["heads"], 0)
        finally:
            del os.environ["CUBERT_FP32_DENSE"]
        other.compute(ids, mask, seg)
        other.synchronize()
        for _ in range(args.warmup):
            other.compute_resident(B)
        other.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            other.compute_resident(B)
        other.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        other.close()
        two_term = {"value": round(B / (ms * 1e-3), 1), "unit": "sequences/s", "ms_per_step": round(ms, 4),
                    "dtype": "f32 storage and accumulation; Dense products as three f16 matrix-core products of two-term "
                             "operands (CUBERT_FP32_DENSE=f16x3, opt-in)"}

    # ---- several instances on the one GPU, one caller thread each (host arrays in, pooled output out)
    concurrent = None
    if args.instances > 0:
        import threading
        berts = [cubert_amd.Bert(w, B, S, m["layers"], m["heads"], 1 if half else 0) for _ in range(args.instances)]
        calls = max(50, args.steps)

        def caller(model, n, latencies):
            o = cubert_amd.Output(np.empty((B, m["hidden"]), np.float16 if half else np.float32),
                                  cubert_amd.OutputType.POOLED_OUTPUT)
            for _ in range(n):
                t = time.perf_counter()
                model.compute(ids, mask, seg)
                model.output(B, o)
                latencies.append((time.perf_counter() - t) * 1e3)

        for model in berts:
            caller(model, 10, [])
        lat = [[] for _ in berts]
        threads = [threading.Thread(target=caller, args=(model, calls, lat[i])) for i, model in enumerate(berts)]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        elapsed = time.perf_counter() - t0
        for model in berts:
            model.close()
        every = np.concatenate([np.array(x) for x in lat])
        concurrent = {"instances": args.instances, "callers": args.instances, "calls_per_caller": calls,
                      "requests_per_s": round(args.instances * calls / elapsed, 1),
                      "sequences_per_s": round(args.instances * calls * B / elapsed, 1),
                      "p50_ms": round(float(np.median(every)), 3), "p99_ms": round(float(np.percentile(every, 99)), 3)}

    # ---- CPU baseline: the oracle (a port of the reference's CPU path) on this host's cores
    cpu = None
    if not args.no_cpu and not args.device_only:
        cpu = cpu_baseline(args.workload, cfg, w, ids, mask, seg)

    line = {
        "metric": "sequences/s, BERT forward pass (%s)" % args.workload,
        "value": round(value, 1), "unit": "sequences/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": "%s: %s %s batch %d seq_len %d, random-init N(0,0.02) weights, inputs resident in HBM" %
                               (args.workload, "BERT-large" if m["hidden"] == 1024 else "BERT-base", cfg["dtype"], B, S),
                   "value_is": "forward passes on inputs already resident in HBM (what this bench's contract defines "
                               "`value` as; a PCIe-inclusive rate is never `value`). The same workload measured the way "
                               "the reference's benchmark client does it (host arrays in, host array out) is "
                               "`reference_protocol`, and `p50_ms_batch1_host_path` is that call with one sequence."},
        "reference_protocol": host_path, "p50_ms_batch1_host_path": p50_b1,
        "roofline": roofline, "cpu_baseline": cpu,
    }
    if two_term_dense() and not half:
        line["dtype"] = "f32 storage and accumulation; Dense products as three f16 matrix-core products of two-term operands"
    if two_term is not None:
        line["two_term_fp16_dense"] = two_term
    if concurrent is not None:
        line["concurrent_instances"] = concurrent
    for k, row in kernels.items():
        row["traffic"], _ = recorded_traffic(args.workload, k)
    line["kernels"] = kernels
    line["kernel_timing"] = EVENT_PAIR_NOTE
    line["gemm"] = gemm
    if clean is not None:
        line["clean_roofline"] = clean
    print(json.dumps(line))


if __name__ == "__main__":
    main()
