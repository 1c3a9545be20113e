#!/usr/bin/env python3
"""Benchmark of the routed-expert MXFP8 FFN forward (gate/up grouped GEMM -> clamped SwiGLU ->
MXFP8 requant -> down grouped GEMM -> bf16) on one MI355X.

One step = one forward over the whole batch: T=8192 tokens, d_model=d_ff=2880, 32 experts,
top-4 routing (32768 routed rows), inputs already resident in HBM.  Prints ONE JSON line:
metric = MXFP8 grouped-GEMM TFLOP/s on the algorithmic (unpadded) flop count
2*R*H*I*3 = 1.6307e12 per forward (weights in the layouts the kernel streams: K-tiled codes, slot-major scales), plus
  roofline      -- the forward's one kernel (both grouped GEMMs in one launch), its launch duration measured with HIP
                   events on its launch stream over the timed steps, against the 5.0 PFLOP/s dense FP8 MFMA peak; the
                   two GEMMs launched separately (the library's other mode) are timed beside it;
  cpu_baseline  -- the CPU oracle (torch fp32 dequant-then-matmul) timed on the host cores on
                   the whole batch of the same inputs, and on its first 1024 tokens;
  linked_over_one_unit -- paired ABBA/BAAB timing of the linked image against the one-unit
                   control (evaluator/harness/parity/example.py:104-166 in the reference);
  power         -- board power and shader clock the driver reports (hwmon power1_input,
                   pp_dpm_sclk) sampled while the timed steps run: this kernel runs at the
                   board's power cap, and the clock it is given there bounds what it can reach.

Before the warm-up steps the forward is looped, untimed, for --ramp-seconds: a GPU that has been
idle needs about a second of load to reach its sustained clock and power state, and steps timed
before that are neither the burst nor the sustained rate."""
from __future__ import annotations

import argparse
import glob
import json
import os
import re
import statistics
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

T, H, I, E, TOPK = 8192, 2880, 2880, 32, 4
FLOPS_GATE_UP = 2.0 * T * TOPK * H * I * 2
FLOPS_DOWN = 2.0 * T * TOPK * I * H
FLOPS_TOTAL = FLOPS_GATE_UP + FLOPS_DOWN
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
# HBM-side bytes of one launch of the forward's kernel: FETCH_SIZE + WRITE_SIZE of two rocprofv3 --pmc runs of this
# script, each scaled by what the same counter reads for a 1 GiB device copy (--copy-calibration).  The figures are
# kept in a JSON file next to the profile summary they come from; without the file `traffic` is null.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "pipelink_kernel_bench_shape_traffic.json")
TILE = 256  # the kernel's tile: 256 routed rows x 256 weight rows (gate/up: 128 gate + 128 up columns)


def traffic_bytes():
    try:
        with open(TRAFFIC_JSON) as f:
            return float(json.load(f)["traffic_bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None


def executed_flops(counts):
    """Flops the kernel's waves execute for these per-expert row counts.  A full tile: a wave multiplies its 128 x 128
    share over the whole contraction unless the share starts past the expert's last row or past the last output
    column (then it only loads); shares that are partly past the end are multiplied in full.  A tile of at most 64
    rows or at most 64 columns (per matrix) is in the small placement: four waves x 64 rows x the 32-row weight
    fragments they hold (few rows: 2 per wave; few columns: 2 per wave and matrix)."""
    total = 0.0
    for c in counts:
        for first in range(0, int(c), TILE):
            rows = int(c) - first
            row_waves = 1 if rows <= TILE // 2 else 2
            for cols, k, step, matrices in ((I, H, TILE // 2, 2), (H, I, TILE, 1)):  # gate/up (two matrices), down
                for col_begin in range(0, cols, step):
                    if rows <= 64:      # few rows: every wave 64 rows x 2 fragments of 32 weight rows
                        total += 4 * 64 * 64 * 2.0 * k
                    elif cols - col_begin <= 64:  # few columns: every wave 64 rows x 64 columns of each matrix
                        total += 4 * 64 * 64 * matrices * 2.0 * k
                    else:
                        col_waves = sum(col_begin + w * 64 < cols for w in (0, 1))
                        total += row_waves * col_waves * 128 * 128 * 2.0 * k  # (gate/up: 64 gate + 64 up columns per wave)
    return total


def make_inputs(dev, seed=0):
    """Seeded config-3 inputs: CPU generator, draw order logits, x, Wg, Wu, Wd (one expert at a
    time); quantised on the device (bit-exact with the host rule) into 128-byte-pitched rows."""
    import torch
    from pipelink_amd.host import mok_inputs
    from pipelink_amd.host.mok import (code_pitch, mxfp8_quantize_device, weight_codes_to_k64_tiled,
                                       weight_scales_to_slot_major)

    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    x = torch.randn(T, H, generator=g)
    counts, row_token = mok_inputs.route(logits, TOPK)
    x_q, x_sc = mxfp8_quantize_device(x.to(dev), code_pitch(H))

    def weights(n, k):
        qs, scs = [], []
        for _ in range(E):
            w = torch.randn(n, k, generator=g) * 0.02
            q, sc = mxfp8_quantize_device(w.to(dev), k)
            qs.append(q)
            scs.append(sc)
        q, sc = torch.stack(qs), torch.stack(scs)
        # (K-tiled codes, row-major scales, slot-major scales, row-major codes)
        return weight_codes_to_k64_tiled(q, k), sc, weight_scales_to_slot_major(sc, k), q

    wg = weights(I, H)
    wu = weights(I, H)
    wd = weights(H, I)
    dev_args = dict(tokens_per_expert=counts.to(dev), row_token=row_token.to(dev), x_q=x_q, x_sc=x_sc, w_gate_q=wg[0],
                    w_gate_sc=wg[2], w_up_q=wu[0], w_up_sc=wu[2], w_down_q=wd[0], w_down_sc=wd[2])
    # what the CPU oracle reads: row-major codes and scales
    row_major = dict(w_gate_sc=wg[1], w_up_sc=wu[1], w_down_sc=wd[1], w_gate_q=wg[3], w_up_q=wu[3], w_down_q=wd[3])
    return dev_args, row_major


class PowerSampler:
    """Reads board power (hwmon power1_input, microwatts) and the current shader clock level
    (pp_dpm_sclk, the line marked with *) every 10 ms on a thread; best effort: a box that
    does not expose them yields nulls."""

    def __init__(self):
        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.power = next((os.path.join(h, "power1_input") for h in hw if os.path.exists(os.path.join(h, "power1_input"))), None)
        self.cap = next((os.path.join(h, "power1_cap") for h in hw if os.path.exists(os.path.join(h, "power1_cap"))), None)
        sclk = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.sclk = sclk[0] if sclk else None
        self.watts, self.mhz = [], []
        self._stop = threading.Event()
        self._thread = None

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return f.read()
        except OSError:
            return None

    def _run(self):
        while not self._stop.is_set():
            w = self._read(self.power) if self.power else None
            if w and w.strip().isdigit():
                self.watts.append(int(w) / 1e6)
            c = self._read(self.sclk) if self.sclk else None
            m = re.search(r"(\d+)\s*Mhz\s*\*", c or "", re.IGNORECASE)
            if m:
                self.mhz.append(int(m.group(1)))
            self._stop.wait(0.01)

    def __enter__(self):
        self._thread = threading.Thread(target=self._run, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def report(self):
        cap = self._read(self.cap) if self.cap else None
        return {"cap_w": round(int(cap) / 1e6, 1) if cap and cap.strip().isdigit() else None,
                "draw_w": round(statistics.median(self.watts), 1) if self.watts else None,
                "sclk_mhz": round(statistics.median(self.mhz)) if self.mhz else None,
                "samples": len(self.watts),
                "source": "hwmon power1_input / power1_cap, pp_dpm_sclk, sampled every 10 ms while the forward runs back to back: "
                          "during the timed steps and, where those are too few for 10 samples, during untimed ones after them"}


def mfma_ceiling(be, torch, seconds=1.0):
    """What back-to-back v_mfma_scale_f32_32x32x64_f8f6f4 alone sustain on this board (one wave per
    SIMD, operands in registers, no LDS or memory traffic): with random e4m3 operands the board
    sits at its power limit and clocks down; with zero operands it runs at the full clock."""
    import ctypes

    path = os.path.join(ROOT, "pipelink_amd", "libplk_bench_probe.so")  # built by __graft_entry__.build()
    lib = ctypes.CDLL(path)
    lib.plk_probe_mfma_fp8.restype = ctypes.c_int
    lib.plk_probe_mfma_fp8.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64, ctypes.c_void_p]

    def check(status):
        if status != 0:
            raise RuntimeError(f"plk_probe_mfma_fp8 failed with status {status}")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.zeros(16, dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    iters, per_batch = 2000, 20
    flop_per_launch = cus * 4 * iters * 16 * 131072.0
    out = {}
    for name, zero in (("random_operands", 0), ("zero_operands", 1)):
        def batch():
            for _ in range(per_batch):
                check(lib.plk_probe_mfma_fp8(cus, iters, zero, sink.data_ptr(), stream))
        end = time.perf_counter() + seconds  # clock / power ramp
        while time.perf_counter() < end:
            batch()
            torch.cuda.synchronize()
        e0, e1 = be.event_create(), be.event_create()
        launches = 0
        with PowerSampler() as power:
            be.event_record(e0)
            end = time.perf_counter() + seconds
            while time.perf_counter() < end:
                batch()
                launches += per_batch
                torch.cuda.synchronize()
            be.event_record(e1)
            be.event_synchronize(e1)
        ms = be.event_elapsed_time(e0, e1)
        be.event_destroy(e0)
        be.event_destroy(e1)
        rep = power.report()
        out[name] = {"tflops": round(flop_per_launch * launches / (ms * 1e-3) / 1e12, 1), "draw_w": rep["draw_w"],
                     "sclk_mhz": rep["sclk_mhz"], "launches": launches}
    out["definition"] = (f"plk_probe_mfma_fp8: {cus} workgroups x 4 waves, {iters} x 16 MFMA 32x32x64 f8f6f4 per wave and "
                         f"launch, operands in registers; {seconds} s ramp then {seconds} s timed with HIP events")
    return out


def cpu_baseline(inp, row_major, slice_tokens=1024):
    """The oracle on the host cores: the whole batch of the same inputs, and its first `slice_tokens` tokens (each the
    median of 3 runs after a warm-up)."""
    import torch
    from oracle import moe_ffn
    from pipelink_amd.host import mok_inputs

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    host = {k: v.cpu() for k, v in {**inp, **row_major}.items()}

    def timed(tokens, reps):
        g = torch.Generator().manual_seed(0)
        logits = torch.randn(T, E, generator=g)[:tokens]
        counts, row_token = mok_inputs.route(logits, TOPK)
        args = dict(x_q=host["x_q"][:tokens, :H], x_sc=host["x_sc"][:tokens],
                    wg_q=host["w_gate_q"][:, :, :H], wg_sc=host["w_gate_sc"], wu_q=host["w_up_q"][:, :, :H],
                    wu_sc=host["w_up_sc"], wd_q=host["w_down_q"][:, :, :I], wd_sc=host["w_down_sc"], counts=counts,
                    row_token=row_token)
        times = []
        for rep in range(reps + 1):
            t0 = time.perf_counter()
            moe_ffn.moe_ffn_forward_torch(**args)
            if rep:
                times.append(time.perf_counter() - t0)
        return statistics.median(times)

    sec_slice = timed(slice_tokens, 3)
    sec_full = timed(T, 3)
    return {"value": round(FLOPS_TOTAL / sec_full / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"the whole batch ({T} tokens, {T * TOPK} routed rows; all {E} experts' weights dequantised inside the "
                      f"timed region): median of 3 runs after 1 warm-up, {sec_full * 1e3:.0f} ms per forward, torch {torch.__version__} fp32",
            "slice": {"value": round(FLOPS_TOTAL * slice_tokens / T / sec_slice / 1e12, 4), "tokens": slice_tokens,
                      "ms_per_forward": round(sec_slice * 1e3), "runs": "median of 3 after 1 warm-up"}}


def vendor_dense_fp8(inp, row_major, torch, ramp_seconds):
    """What the vendor library's dense FP8 GEMM (`torch._scaled_mm`, one scale per tensor, bf16 out) reaches on this
    board at the two GEMM shapes of the forward, on the forward's own e4m3 codes: the 32768 routed rows against
    ONE expert's weights (gate and up stacked; down), so no grouping, no block scales, no activation between the two,
    and 17 MB + 8 MB of weights instead of 531 MB + 265 MB.  Sustained the same way as the forward, with the board's
    power and clock beside each.  Best effort: null where the library has no such kernel."""
    fp8 = torch.float8_e4m3fn
    x = inp["x_q"][inp["row_token"].long()][:, :H].contiguous().view(fp8)
    one = torch.ones((), device=x.device)
    out = {"definition": "torch._scaled_mm(x8, w8.t(), scale_a=1, scale_b=1, out_dtype=bf16), dense, one expert's weights",
           "operands": "the forward's own e4m3 codes (gathered routed rows; expert 0)"}
    shapes = (("gate_up", torch.cat([row_major["w_gate_q"][0], row_major["w_up_q"][0]]).contiguous().view(fp8), FLOPS_GATE_UP),
              ("down", row_major["w_down_q"][0].contiguous().view(fp8), FLOPS_DOWN))
    try:
        for name, w, flop in shapes:
            def run(n):
                for _ in range(n):
                    torch._scaled_mm(x, w.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
            end = time.perf_counter() + ramp_seconds
            while time.perf_counter() < end:
                run(20)
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n = 200
            with PowerSampler() as power:
                e0.record()
                run(n)
                e1.record()
                torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / n
            rep = power.report()
            out[name] = {"m": int(x.shape[0]), "n": int(w.shape[0]), "k": int(w.shape[1]), "ms": round(ms, 4),
                         "tflops": round(flop / (ms * 1e-3) / 1e12, 1), "draw_w": rep["draw_w"], "sclk_mhz": rep["sclk_mhz"]}
        out["ms_both"] = round(out["gate_up"]["ms"] + out["down"]["ms"], 4)
    except Exception as ex:  # noqa: BLE001 -- a library without the kernel, not a failure of this bench
        out["error"] = repr(ex)[:200]
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--ramp-seconds", type=float, default=1.5,
                    help="loop the forward, untimed, for this long before the warm-up steps (clock and power ramp)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-pair", action="store_true", help="skip the linked vs one-unit paired timing")
    ap.add_argument("--no-mfma-ceiling", action="store_true",
                    help="skip the pure-MFMA run that measures what the matrix pipe sustains at the board's power limit")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="also time the vendor library's dense FP8 GEMM at the forward's two GEMM shapes (vendor_dense_fp8)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 1 GiB device copy, 10 times: the known-size kernel the FETCH_SIZE / "
                         "WRITE_SIZE counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the routed-expert FFN; --gpus must be 1",
              file=sys.stderr)
        return 2

    import torch
    if args.copy_calibration:
        src = torch.ones(1 << 30, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": 1 << 30, "copy_calibration_bytes_written": 1 << 30, "launches": 10}))
        return 0
    from pipelink_amd.host.backend import HipBackend
    from pipelink_amd.host.mok import MoKSession, code_pitch, scale_pitch
    from pipelink_amd.stages.mok import build as mok_build

    paths = mok_build.images()  # raises if the HIP images are missing: there is no fallback path
    dev = torch.device("cuda:0")
    inp, row_major = make_inputs(dev)
    rows = T * TOPK
    hq = torch.zeros((rows, code_pitch(I)), dtype=torch.uint8, device=dev)
    hsc = torch.zeros((rows, scale_pitch(I)), dtype=torch.uint8, device=dev)
    y = torch.full((rows, H), float("nan"), dtype=torch.bfloat16, device=dev)
    link_json = json.loads(paths["link_json"].read_text())
    linked = MoKSession(paths["linked"].read_bytes(), link_json)
    control = MoKSession(paths["one_unit"].read_bytes(), link_json)
    prob = linked.problem(hidden_q=hq, hidden_sc=hsc, y=y, **inp)
    stream = torch.cuda.current_stream().cuda_stream
    be = HipBackend(0, stream)

    ramp_end = time.perf_counter() + args.ramp_seconds
    while time.perf_counter() < ramp_end:
        for _ in range(50):
            linked.forward(prob)
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        linked.forward(prob)
    torch.cuda.synchronize()
    e0, e1 = be.event_create(), be.event_create()
    with PowerSampler() as power:
        t0 = time.perf_counter()
        be.event_record(e0)
        for _ in range(args.steps):
            linked.forward(prob)
        be.event_record(e1)
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        # the forward is one launch: the events bracket `steps` launches that run back to back on the launch stream
        ms_launch = be.event_elapsed_time(e0, e1) / args.steps
        while 0 < len(power.watts) < 10:  # too few timed steps for ten readings: go on, untimed
            for _ in range(20):
                linked.forward(prob)
            torch.cuda.synchronize()
    be.event_destroy(e0)
    be.event_destroy(e1)
    status = linked.status()
    if status != 0:
        print(f"bench.py: the forward raised status {status} (a tile gave up waiting for its rows)", file=sys.stderr)
        return 1

    def event_ms(sess, which, n):
        e0, e1 = be.event_create(), be.event_create()
        be.event_record(e0)
        for _ in range(n):
            sess.forward(prob, which=which)
        be.event_record(e1)
        be.event_synchronize(e1)
        ms = be.event_elapsed_time(e0, e1) / n
        be.event_destroy(e0)
        be.event_destroy(e1)
        return ms

    # the library's other mode, one launch per GEMM: the two passes in turn, each bracketed by its own pair of
    # events (a loop over one pass alone would keep that pass's weights in the last-level cache and change
    # the clock the other pass leaves it)
    n = min(max(args.steps, 10), 200)
    ev = [[be.event_create() for _ in range(3)] for _ in range(n)]
    for a, b, c in ev:
        be.event_record(a)
        linked.forward(prob, which=1)
        be.event_record(b)
        linked.forward(prob, which=2)
        be.event_record(c)
    be.event_synchronize(ev[-1][2])
    ms_gate_up = statistics.mean(be.event_elapsed_time(a, b) for a, b, c in ev)
    ms_down = statistics.mean(be.event_elapsed_time(b, c) for a, b, c in ev)
    for trio in ev:
        for e in trio:
            be.event_destroy(e)

    pair = None
    if not args.no_pair:
        # 8 blocks in the orders ABBA BAAB BAAB ABBA BAAB ABBA ABBA BAAB (A = linked, B = one-unit)
        orders = ["ABBA", "BAAB", "BAAB", "ABBA", "BAAB", "ABBA", "ABBA", "BAAB"]
        batch = max(5, int(16.0 / max(ms_per_step, 1e-3)))
        for s in (linked, control):
            for _ in range(8):
                s.forward(prob)
        ratios = []
        for order in orders:
            t = {"A": 0.0, "B": 0.0}
            for c in order:
                t[c] += event_ms(linked if c == "A" else control, 0, batch)
            ratios.append(t["B"] / t["A"])  # > 1: linked faster
        pair = {"speed_ratio": round(statistics.median(ratios), 5), "blocks": [round(r, 5) for r in ratios],
                "batch": batch, "definition": "one-unit time / linked time, median of 8 ABBA/BAAB blocks"}

    ceiling = None
    if not args.no_mfma_ceiling:
        ceiling = mfma_ceiling(be, torch)

    out = {
        "metric": "MXFP8 MoE grouped-GEMM TFLOP/s (% MFMA peak); linked/one-unit speed ratio",
        "value": round(FLOPS_TOTAL / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ramp_seconds": args.ramp_seconds,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3 (MXFP8, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "configs[2]: MXFP8 MoE expert FFN forward", "tokens": T, "d_model": H, "d_ff": I,
                   "experts": E, "top_k": TOPK, "routed_rows": rows, "image": "linked",
                   "pct_of_fp8_mfma_peak": round(FLOPS_TOTAL / (ms_per_step * 1e-3) / 1e12 / PEAK_FP8_TFLOPS * 100, 2),
                   "ms_per_token": round(ms_per_step / T, 7)},
        "roofline": {"bound": "mfma",
                     "kernel": "pipelink_kernel (one launch: gate/up grouped GEMM + SwiGLU + requant tiles, then down grouped "
                               "GEMM tiles that wait for their rows' readiness counters)",
                     "achieved": round(FLOPS_TOTAL / (ms_launch * 1e-3) / 1e12, 2), "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(FLOPS_TOTAL / (ms_launch * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4),
                     "traffic": traffic_bytes(), "launch_ms": round(ms_launch, 4),
                     "executed_over_algorithmic_flops": round(executed_flops(inp["tokens_per_expert"].tolist()) / FLOPS_TOTAL, 4),
                     "two_launches": {
                         "gate_up_pass": {"achieved": round(FLOPS_GATE_UP / (ms_gate_up * 1e-3) / 1e12, 2), "launch_ms": round(ms_gate_up, 4)},
                         "down_pass": {"achieved": round(FLOPS_DOWN / (ms_down * 1e-3) / 1e12, 2), "launch_ms": round(ms_down, 4)}}},
        "linked_over_one_unit": pair,
        "power": power.report(),
    }
    sclk = out["power"]["sclk_mhz"]
    if sclk:
        # the published peak is 256 CUs x 4 SIMDs x 2048 FP8 flop per clock at 2.4 GHz
        at_clock = PEAK_FP8_TFLOPS * sclk / 2400.0
        out["roofline"]["peak_at_reported_sclk"] = round(at_clock, 1)
        out["roofline"]["frac_at_reported_sclk"] = round(FLOPS_TOTAL / (ms_launch * 1e-3) / 1e12 / at_clock, 4)
    if ceiling:
        out["mfma_ceiling"] = ceiling
        rnd = ceiling["random_operands"]["tflops"]
        out["roofline"]["frac_of_measured_mfma_ceiling"] = round(FLOPS_TOTAL / (ms_launch * 1e-3) / 1e12 / rnd, 4)
    if args.vendor_gemm:
        out["vendor_dense_fp8"] = vendor_dense_fp8(inp, row_major, torch, args.ramp_seconds)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(inp, row_major)
    print(json.dumps(out))
    linked.close()
    control.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
