#!/usr/bin/env python3
"""Headline benchmark: deterministic bf16 GEMM at Qwen3-8B FFN shapes on one MI355X.

One "step" is one pass of the FFN hot path over one synthetic batch of T=4096
tokens: the gate_up GEMM X[4096,4096] x W[24576,4096]^T followed by the down GEMM
H[4096,12288] x W[4096,12288]^T, inputs resident in HBM. The JSON line also carries

* ``roofline``     - the dominant kernel (the 256x256-tile MFMA kernel on gate_up)
                     against the MI355X dense bf16 MFMA peak, timed with HIP events
                     on the launch stream; ``roofline.matrix_pipe_alone`` quotes, for orientation,
                     what the same MFMA sequence sustained out of registers with nothing else
                     running on machines of this pool (recorded constants, not measured here);
* ``cpu_baseline`` - the CPU oracle (``oracle/reference_math.det_gemm_ref_torch``) timed on
                     this box's host cores on the same step;
* ``shapes``       - every token count of the configuration (T = 1, 16, 64, 256, 1024, 4096)
                     with its own MFMA or HBM fraction; up to 1024 tokens also over copies of
                     the weight that rotate through 1.3 GB, so that it is read from HBM and
                     not from the 256 MB memory-side cache (``weights_from_hbm``);
* ``linear_logp``  - the fused linear-LogP at T=8192, V=151936, D=4096 in tokens/s, with its
                     backward and the from-logits stage;
* ``ffn``          - the gated FFN (fused gate/up + SwiGLU, then down) at T=4096.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-logp]
       python bench.py --only LEG [--rotate-weights]   (one leg, for profiling; see --help)
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT, ROOT / "rl-kernel_amd", ROOT / "tests"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

# MI355X published peaks used for every fraction below.
PEAK_BF16_TFLOPS = 2500.0  # dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0  # HBM3E

HIDDEN, INTER, VOCAB = 4096, 12288, 151936

# Steps launched before the caller's --warmup, always: after idle the part boosts, over-throttles around
# the sixth launch and settles after about thirty, so a short warm-up would time that transient.
CONDITIONING_STEPS = 40  # 80 kernel launches

# HBM bytes per launch of the dominant kernel come from a tracked record of two rocprofv3 --pmc runs
# (FETCH_SIZE, then WRITE_SIZE) of `bench.py --only gate_up`, each scaled by what the same counter reads on
# the plain copy kernel of `bench.py --only copy`; the record names the commit it was measured on.
TRAFFIC_RECORD = ROOT / "profiles" / "det_gemm_gate_up_T4096_traffic.txt"


def _measured_traffic() -> dict:
    """`key: value` lines of the traffic record -> {"bytes": float | None, "commit": str | None}."""
    out = {"bytes": None, "commit": None}
    try:
        for line in TRAFFIC_RECORD.read_text().splitlines():
            key, _, value = line.partition(":")
            if key.strip() == "traffic_bytes_per_launch":
                out["bytes"] = float(value)
            elif key.strip() == "measured_on_commit":
                out["commit"] = value.strip()
    except (OSError, ValueError):
        pass
    return out


# What the matrix pipe sustains at the power cap when nothing else runs: the MFMA sequence of the 256 x 256 tile
# kernel out of registers (no loads, no LDS), measured once with a stand-alone probe on machines of this pool
# (profiles/load_path_probe_mi355x.md, section 6). Constants, not measured by this run: the spread is the spread
# between machines.
MATRIX_PIPE_ALONE = {
    "random_operands_tflops": [1970.0, 2130.0],
    "zero_operands_tflops": [2440.0, 2450.0],
    "source": "profiles/load_path_probe_mi355x.md section 6",
}


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-logp", action="store_true", help="skip the linear-LogP leg")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-T table")
    ap.add_argument("--rotate-weights", action="store_true",
                    help="gate_up_tN / down_tN legs: launch over copies of the weight (~1.3 GB in rotation) so that it is read from HBM")
    ap.add_argument("--only", default="", help="run a single leg and print its JSON: gate_up|down|gate_up_tN|down_tN|logp|logp_decode|logp_mid|logp_logits|logp_bwd|logp_bwd_256|from_logits|from_logits_bwd|ffn|tree|tree_down|tree_decode|copy|power|host (used for profiling)")
    return ap.parse_args()


def _time_calls(fn, iters: int, warmup: int) -> float:
    """Average milliseconds per call, HIP events on the current (launch) stream."""
    import torch

    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def _launch_percentiles(fn, iters: int, warmup: int) -> dict:
    """Median and 95th percentile of single launches (one HIP event pair per launch), in ms."""
    import torch

    for _ in range(warmup):
        fn()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(stop) for start, stop in pairs)
    return {"median_ms": round(times[len(times) // 2], 4), "p95_ms": round(times[min(len(times) - 1, int(0.95 * len(times)))], 4)}


def _gemm_bytes(m, n, k):
    return 2.0 * (m * k + n * k + m * n)


def main() -> int:
    args = _parse()
    if args.gpus != 1:
        print(
            f"bench.py: --gpus {args.gpus} is not supported: this build runs on exactly one GPU "
            "(no collectives, no sharding); run with --gpus 1.",
            file=sys.stderr,
        )
        return 2

    import torch

    from rl_engine import _lib
    from rl_engine.backends.rocm.gemm import det_gemm as gemm
    from rl_engine.ops.logprob import deterministic_linear_logp

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    _lib.load()  # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2000)

    def randn(rows, cols, scale=1.0):
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=dev)
        step = 8192
        for r0 in range(0, rows, step):
            r1 = min(r0 + step, rows)
            out[r0:r1] = (torch.randn((r1 - r0, cols), generator=gen, device=dev, dtype=torch.float32) * scale).to(torch.bfloat16)
        return out

    T = 4096
    x = randn(T, HIDDEN)
    h = randn(T, INTER)
    w_gu = randn(2 * INTER, HIDDEN, 0.02)
    w_d = randn(HIDDEN, INTER, 0.02)
    out_gu = torch.empty((T, 2 * INTER), dtype=torch.bfloat16, device=dev)
    out_d = torch.empty((T, HIDDEN), dtype=torch.bfloat16, device=dev)

    def gate_up():
        gemm.mfma_gemm(x, w_gu.t(), out=out_gu)

    def down():
        gemm.mfma_gemm(h, w_d.t(), out=out_d)

    def step():
        gate_up()
        down()

    if args.only == "host":
        # Eager host cost per call of the Python entry points (facade -> ctypes -> launch) on tiny operands:
        # `steps` calls are queued without waiting for the GPU and the wall clock is divided by their number;
        # torch.matmul on the same operands is there for scale.
        from rl_engine import _C
        from rl_engine.ops.ffn import qwen3_ffn_packed_inference
        from rl_engine.ops.gemm import deterministic_gemm
        from rl_engine.ops.gemm.det_gemm import det_gemm_linear
        from rl_engine.ops.logprob import deterministic_linear_logp

        x1, w_s = randn(1, 512), randn(512, 512, 0.02)
        b_s = w_s.t().contiguous()
        out_s = torch.empty((1, 512), dtype=torch.bfloat16, device=dev)
        h4, w_v = randn(4, 512), randn(4096, 512, 0.02)
        t4 = torch.randint(0, 4096, (4,), device=dev)
        w_gu_s, w_d_s = randn(2 * 1024, 512, 0.02), randn(512, 1024, 0.02)
        calls = {
            "torch.matmul": lambda: torch.matmul(x1, b_s),
            "_C.gemm_strided(out=)": lambda: _C.gemm_strided(x1, b_s, out_s),
            "_C.det_gemm_fwd": lambda: _C.det_gemm_fwd(x1, b_s),
            "deterministic_gemm": lambda: deterministic_gemm(x1, b_s),
            "det_gemm_linear": lambda: det_gemm_linear(x1, w_s),
            "_C.fused_linear_logp": lambda: _C.fused_linear_logp(h4, w_v, t4),
            "deterministic_linear_logp": lambda: deterministic_linear_logp(h4, w_v, t4),
            "qwen3_ffn_packed_inference": lambda: qwen3_ffn_packed_inference(x1, w_gu_s, w_d_s),
        }
        n = max(args.steps, 1000)
        result = {}
        for name, fn in calls.items():
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            result[name] = round((time.perf_counter() - t0) / n * 1e6, 1)
            torch.cuda.synchronize()
        print(json.dumps({"leg": "host", "calls": n, "us_per_call": result}))
        return 0
    if args.only == "copy":
        # Calibration leg for the FETCH_SIZE / WRITE_SIZE counters: one plain device
        # copy kernel of known size (1 GiB read + 1 GiB written per launch).
        src = torch.empty((1 << 29,), dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        src.fill_(1.0)
        for _ in range(3):
            torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({"leg": "copy", "bytes_read": src.numel() * 2, "bytes_written": dst.numel() * 2, "launches": 3}))
        return 0
    if args.only == "logp":
        tl = 8192
        hid = randn(tl, HIDDEN)
        w_lm = randn(VOCAB, HIDDEN, 0.02)
        tgt = torch.randint(0, VOCAB, (tl,), generator=gen, device=dev)
        ms = _time_calls(lambda: deterministic_linear_logp(hid, w_lm, tgt), args.steps, args.warmup)
        print(json.dumps({"leg": "logp", "ms": ms, "tokens_per_s": tl / ms * 1e3, "launches": args.steps + args.warmup}))
        return 0
    if args.only in ("logp_decode", "logp_mid"):
        # the stream-group grid: 16 tokens (decode) or 512 tokens against the full vocabulary
        tl = 16 if args.only == "logp_decode" else 512
        hid = randn(tl, HIDDEN)
        w_lm = randn(VOCAB, HIDDEN, 0.02)
        tgt = torch.randint(0, VOCAB, (tl,), generator=gen, device=dev)
        ms = _time_calls(lambda: deterministic_linear_logp(hid, w_lm, tgt), args.steps, args.warmup)
        print(json.dumps({"leg": args.only, "tokens": tl, "ms": ms, "weight_gbps": 2.0 * VOCAB * HIDDEN / ms * 1e-6,
                          "launches": args.steps + args.warmup}))
        return 0
    if args.only.startswith(("down_t", "gate_up_t")):
        # a skinny-M leg at N tokens (gate_up_t1, down_t16 ...): 16-row kernel, streaming kernel or small tiles
        name, ts = args.only.rsplit("_t", 1)
        ts = int(ts)
        if not 1 <= ts <= T:
            raise SystemExit(f"--only {args.only}: token count must be in 1..{T}")
        if name == "down":
            a_s, w_s, o_s, k_s, n_s = h[:ts], w_d, out_d[:ts], INTER, HIDDEN
        else:
            a_s, w_s, o_s, k_s, n_s = x[:ts], w_gu, out_gu[:ts], HIDDEN, 2 * INTER
        if args.rotate_weights:
            # copies of the weight that rotate through ~1.3 GB, so that it comes from HBM and not from the
            # 256 MB memory-side cache
            copies = [w_s] + [w_s.clone() for _ in range(int(1.3e9 // (n_s * k_s * 2)))]

            def rotation():
                for w_c in copies:
                    gemm.mfma_gemm(a_s, w_c.t(), out=o_s)

            reps = max(1, args.steps // len(copies))
            ms = _time_calls(rotation, reps, max(1, args.warmup // len(copies))) / len(copies)
            launches = (reps + max(1, args.warmup // len(copies))) * len(copies)
        else:
            ms = _time_calls(lambda: gemm.mfma_gemm(a_s, w_s.t(), out=o_s), args.steps, args.warmup)
            launches = args.steps + args.warmup
        print(json.dumps({"leg": args.only, "tokens": ts, "rotating_weights": bool(args.rotate_weights), "ms": ms,
                          "gbps": _gemm_bytes(ts, n_s, k_s) / ms * 1e-6, "launches": launches}))
        return 0
    if args.only == "power":
        # Board power (hwmon, microwatts) while the gate_up GEMM loops on the benchmark's random
        # operands and on all-zero operands: the same instruction stream at two data-toggle rates.
        import glob

        def hwmon(name):
            vals = []
            for f in glob.glob(f"/sys/class/drm/card*/device/hwmon/hwmon*/{name}"):
                try:
                    vals.append(int(open(f).read()) / 1e6)
                except (OSError, ValueError):
                    pass
            return max(vals) if vals else None

        def looped(a_op, w_op, seconds=3.0):
            for _ in range(50):
                gemm.mfma_gemm(a_op, w_op.t(), out=out_gu)
            torch.cuda.synchronize()
            t0, n, watts = time.perf_counter(), 0, []
            while time.perf_counter() - t0 < seconds:
                for _ in range(200):
                    gemm.mfma_gemm(a_op, w_op.t(), out=out_gu)
                n += 200
                watts.append(hwmon("power1_average") or hwmon("power1_input"))  # sampled while the queue is busy
                torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            watts = sorted(w for w in watts if w is not None)
            return {"tflops": round(2.0 * T * 2 * INTER * HIDDEN * n / dt * 1e-12, 1),
                    "watts": watts[len(watts) // 2] if watts else None}

        idle = hwmon("power1_average") or hwmon("power1_input")
        res = {"leg": "power", "cap_watts": hwmon("power1_cap"), "idle_watts": idle,
               "random_operands": looped(x, w_gu), "zero_operands": looped(torch.zeros_like(x), torch.zeros_like(w_gu))}
        print(json.dumps(res))
        return 0
    if args.only == "tree_decode":
        # the k-tree contract at 1, 16 and 64 tokens: the node-per-wave kernels
        legs = []
        for ts in (1, 16, 64):
            for name, act, w, out in (("gate_up", x, w_gu, out_gu), ("down", h, w_d, out_d)):
                ms = _time_calls(lambda: gemm.tree_gemm(act[:ts], w.t(), out=out[:ts]), args.steps, args.warmup)
                legs.append({"op": name, "T": ts, "us": round(ms * 1e3, 1),
                             "weight_gbps": round(w.numel() * 2 / ms * 1e-6, 1)})
        print(json.dumps({"leg": "tree_decode", "legs": legs, "launches": 6 * (args.steps + args.warmup)}))
        return 0
    if args.only in ("tree", "tree_down"):
        if args.only == "tree":
            ms = _time_calls(lambda: gemm.tree_gemm(x, w_gu.t(), out=out_gu), args.steps, args.warmup)
            flops = 2.0 * T * 2 * INTER * HIDDEN
        else:
            ms = _time_calls(lambda: gemm.tree_gemm(h, w_d.t(), out=out_d), args.steps, args.warmup)
            flops = 2.0 * T * INTER * HIDDEN
        print(json.dumps({"leg": args.only, "ms": ms, "tflops": flops / ms * 1e-9,
                          "launches": args.steps + args.warmup}))
        return 0
    if args.only in ("logp_bwd", "logp_bwd_256", "logp_logits", "from_logits", "from_logits_bwd"):
        from rl_engine import _C

        tl = {"logp_bwd_256": 256, "logp_logits": 2048}.get(args.only, 8192)
        hid = randn(tl, HIDDEN)
        w_lm = randn(VOCAB, HIDDEN, 0.02)
        tgt = torch.randint(0, VOCAB, (tl,), generator=gen, device=dev)
        if args.only == "logp_logits":  # the forward that also stores the fp32 logits
            ms = _time_calls(lambda: deterministic_linear_logp(hid, w_lm, tgt, return_logits=True), args.steps, args.warmup)
        elif args.only.startswith("logp_bwd"):
            _, lse = _C.fused_linear_logp(hid, w_lm, tgt)
            g = torch.randn((tl,), generator=gen, device=dev)
            ms = _time_calls(lambda: _C.fused_linear_logp_bwd(hid, w_lm, tgt, lse, g, None), args.steps, args.warmup)
        elif args.only == "from_logits_bwd":
            logits = randn(tl, VOCAB, 4.0)
            lse = torch.full((tl,), 12.0, device=dev)
            g = torch.randn((tl,), generator=gen, device=dev)
            zero = torch.zeros((tl,), device=dev)
            ms = _time_calls(lambda: _C.hip_deterministic_logp_backward(logits, lse, g, zero, tgt, 0, VOCAB, False), args.steps, args.warmup)
        else:
            logits = randn(tl, VOCAB, 4.0)
            ms = _time_calls(lambda: _C.hip_deterministic_logp_from_logits(logits, tgt, 0, VOCAB, 64), args.steps, args.warmup)
        print(json.dumps({"leg": args.only, "ms": ms, "tokens_per_s": tl / ms * 1e3, "launches": args.steps + args.warmup}))
        return 0
    if args.only == "ffn":
        from rl_engine.ops.ffn import qwen3_ffn_packed_inference

        ms = _time_calls(lambda: qwen3_ffn_packed_inference(x, w_gu, w_d), args.steps, args.warmup)
        print(json.dumps({"leg": "ffn", "ms": ms, "launches": args.steps + args.warmup}))
        return 0
    if args.only in ("gate_up", "down"):
        fn = gate_up if args.only == "gate_up" else down
        ms = _time_calls(fn, args.steps, args.warmup)
        print(json.dumps({"leg": args.only, "ms": ms, "launches": args.steps + args.warmup}))
        return 0

    flops_gu = 2.0 * T * (2 * INTER) * HIDDEN
    flops_d = 2.0 * T * HIDDEN * INTER

    # ---- timed region: exactly `steps` steps, synchronised on both sides
    for _ in range(CONDITIONING_STEPS):  # fixed conditioning phase, then the caller's warm-up
        step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    tflops = (flops_gu + flops_d) / wall_ms * 1e-9

    # ---- dominant kernel, HIP events over the same launches
    ms_gu = _time_calls(gate_up, args.steps, 5)
    ms_d = _time_calls(down, args.steps, 5)
    achieved = flops_gu / ms_gu * 1e-9
    traffic = _measured_traffic()
    roofline = {
        "kernel": "det_gemm_kernel<256x256 tile, 8 waves> on gate_up [4096x4096]x[24576x4096]^T",
        "bound": "mfma",
        "achieved": round(achieved, 1),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
        "ms_per_launch": round(ms_gu, 4),
        "flops_per_launch": flops_gu,
        "traffic": traffic["bytes"],
        "traffic_measured_on_commit": traffic["commit"],
    }
    roofline.update(_launch_percentiles(gate_up, args.steps, 5))
    # orientation: the matrix pipe with nothing else running, same MFMA sequence, at the power cap (recorded range)
    lo, hi = MATRIX_PIPE_ALONE["random_operands_tflops"]
    roofline["matrix_pipe_alone"] = dict(
        MATRIX_PIPE_ALONE, frac_of_random_operands_rate=[round(achieved / hi, 4), round(achieved / lo, 4)])

    result = {
        "metric": "bf16 det-GEMM TFLOP/s at Qwen3-8B FFN shapes (gate_up + down, T=4096)",
        "value": round(tflops, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "conditioning_launches": 2 * CONDITIONING_STEPS,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "Qwen3-8B FFN det GEMMs: gate_up X[4096,4096]xW[24576,4096]^T then down H[4096,12288]xW[4096,12288]^T, "
            "bf16 in, fp32 MFMA accumulate in fixed K order, bf16 out, T=4096",
            "contract": gemm.det_gemm_backend_id(),
        },
        "frac_of_mfma_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "kernels": {
            "gate_up_ms": round(ms_gu, 4),
            "gate_up_tflops": round(flops_gu / ms_gu * 1e-9, 1),
            "down_ms": round(ms_d, 4),
            "down_tflops": round(flops_d / ms_d * 1e-9, 1),
        },
        "roofline": roofline,
    }

    # ---- orientation only: the vendor GEMM library on the same operands (not deterministic across
    # batch shapes, not part of the product)
    if not args.no_shapes:
        ms_lib = _time_calls(lambda: torch.nn.functional.linear(x, w_gu), args.steps, args.warmup)
        result["vendor_library_gemm"] = {
            "what": "torch.nn.functional.linear (hipBLASLt) on the gate_up operands, same data, same process",
            "ms": round(ms_lib, 4),
            "tflops": round(flops_gu / ms_lib * 1e-9, 1),
        }

    # ---- every token count of the configuration
    if not args.no_shapes:
        # A weight that is launched on again and again (the benchmark's habit) is served by the 256 MB
        # memory-side cache; a model's layers are not. Up to 1024 tokens (above that it makes no
        # difference) the launch therefore also runs over copies of the weight that rotate through
        # ~1.3 GB ("weights_from_hbm"): that is the figure `frac` is quoted on.
        shapes = []
        for name, act, w, n, k, out in (("gate_up", x, w_gu, 2 * INTER, HIDDEN, out_gu), ("down", h, w_d, HIDDEN, INTER, out_d)):
            copies = [w] + [w.clone() for _ in range(int(1.3e9 // (n * k * 2)))]
            for t in (1, 16, 64, 256, 1024, 4096):
                a_t, o_t = act[:t], out[:t]
                ms = _time_calls(lambda: gemm.mfma_gemm(a_t, w.t(), out=o_t), 30 if t <= 256 else 10, 10)
                fl = 2.0 * t * n * k
                by = _gemm_bytes(t, n, k)
                tf, gb = fl / ms * 1e-9, by / ms * 1e-6
                hbm_bound = (fl / by) < (PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBPS * 1e9))
                row = {
                    "op": name,
                    "T": t,
                    "ms": round(ms, 4),
                    "tflops": round(tf, 1),
                    "gbps": round(gb, 1),
                    "bound": "hbm" if hbm_bound else "mfma",
                    "frac": round(gb / PEAK_HBM_GBPS if hbm_bound else tf / PEAK_BF16_TFLOPS, 4),
                }
                if t <= 1024:
                    def rotation():
                        for w_c in copies:
                            gemm.mfma_gemm(a_t, w_c.t(), out=o_t)

                    ms_rot = _time_calls(rotation, 6, 2) / len(copies)
                    tf_rot, gb_rot = fl / ms_rot * 1e-9, by / ms_rot * 1e-6
                    row["weights_from_hbm"] = {
                        "ms": round(ms_rot, 4),
                        "tflops": round(tf_rot, 1),
                        "gbps": round(gb_rot, 1),
                        "frac": round(gb_rot / PEAK_HBM_GBPS if hbm_bound else tf_rot / PEAK_BF16_TFLOPS, 4),
                        "weight_copies": len(copies),
                    }
                    row["cache_resident_frac"] = row["frac"]
                    row["frac"] = row["weights_from_hbm"]["frac"]
                shapes.append(row)
            del copies
        result["shapes"] = shapes

    # ---- the eager host path at one token (no HIP graph): wall clock per call of det_gemm_linear from
    # Python against the kernel's own time, i.e. what a decode loop that does not capture graphs pays
    if not args.no_shapes:
        host = []
        for name, act, w in (("gate_up", x, w_gu), ("down", h, w_d)):
            a1 = act[:1]
            kernel_ms = _time_calls(lambda: gemm.det_gemm_linear(a1, w), 200, 50)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(200):
                gemm.det_gemm_linear(a1, w)
            issue_us = (time.perf_counter() - t0) / 200 * 1e6  # host time to issue a call (the queue absorbs the kernels)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(50):
                gemm.det_gemm_linear(a1, w)
                torch.cuda.synchronize()
            sync_us = (time.perf_counter() - t0) / 50 * 1e6  # one call and a wait for its result
            host.append({"op": name, "T": 1, "kernel_us_back_to_back": round(kernel_ms * 1e3, 1),
                         "host_issue_us_per_call": round(issue_us, 1), "call_and_wait_us": round(sync_us, 1)})
        result["eager_host_path"] = host

    # ---- attention projections at the packed token count (ragged packing does not change the launch)
    if not args.no_shapes:
        tp = 16384
        xa = randn(tp, HIDDEN)
        proj = []
        for name, n in (("qkv_proj", 6144), ("o_proj", 4096)):
            w_p = randn(n, HIDDEN, 0.02)
            o_p = torch.empty((tp, n), dtype=torch.bfloat16, device=dev)
            ms = _time_calls(lambda: gemm.mfma_gemm(xa, w_p.t(), out=o_p), 20, 20)
            fl = 2.0 * tp * n * HIDDEN
            proj.append({"op": name, "T": tp, "N": n, "K": HIDDEN, "ms": round(ms, 4), "tflops": round(fl / ms * 1e-9, 1),
                         "bound": "mfma", "frac": round(fl / ms * 1e-9 / PEAK_BF16_TFLOPS, 4)})
            del w_p, o_p
        result["attention_projections"] = proj
        del xa

    # ---- the k-tree contract (leaves on the fp32 matrix pipe, one reduction-length-one fp32 MFMA per k) on the same two GEMMs
    if not args.no_shapes:
        ms_tree = _time_calls(lambda: gemm.tree_gemm(x, w_gu.t(), out=out_gu), 3, 1)
        ms_tree_down = _time_calls(lambda: gemm.tree_gemm(h, w_d.t(), out=out_d), 3, 1)
        result["det_gemm_tree"] = {
            "workload": "gate_up X[4096,4096]xW[24576,4096]^T under the k-tree contract (fp32 FMA leaves of 32, bf16 midpoint tree)",
            "ms": round(ms_tree, 3),
            "tflops": round(flops_gu / ms_tree * 1e-9, 1),
            "bound": "fp32 mfma",
            "frac_of_fp32_mfma_peak": round(flops_gu / ms_tree * 1e-9 / 157.3, 4),
            "down": {"workload": "H[4096,12288]xW[4096,12288]^T, leaves of 24", "ms": round(ms_tree_down, 3),
                     "tflops": round(flops_d / ms_tree_down * 1e-9, 1),
                     "frac_of_fp32_mfma_peak": round(flops_d / ms_tree_down * 1e-9 / 157.3, 4)},
            "contract": _lib.load().rlk_det_gemm_tree_contract_id().decode(),
        }
        # the sequential fp32 chain (fp32-result GEMM for fp32 operands and under the k-tree backend): one
        # reduction-length-one fp32 MFMA per k
        from rl_engine import _C as _c_seq

        x_f32, w_f32 = x[:1024].float(), w_gu.float()
        ms_seq = _time_calls(lambda: _c_seq.det_gemm_fwd_fp32(x[:1024], w_gu.t()), 10, 4)
        ms_seq32 = _time_calls(lambda: _c_seq.det_gemm_fwd_fp32(x_f32, w_f32.t()), 10, 4)
        fl_seq = 2.0 * 1024 * 2 * INTER * HIDDEN
        result["det_gemm_seq"] = {
            "workload": "X[1024,4096]xW[24576,4096]^T, fp32 result, one fp32 fused multiply-add per k in ascending order",
            "ms": round(ms_seq, 3), "tflops": round(fl_seq / ms_seq * 1e-9, 1),
            "fp32_operands": {"ms": round(ms_seq32, 3), "tflops": round(fl_seq / ms_seq32 * 1e-9, 1),
                              "frac_of_fp32_mfma_peak": round(fl_seq / ms_seq32 * 1e-9 / 157.3, 4)},
            "bound": "fp32 mfma (157.3 TFLOP/s)",
            "frac_of_fp32_mfma_peak": round(fl_seq / ms_seq * 1e-9 / 157.3, 4),
            "contract": _lib.load().rlk_det_gemm_seq_contract_id().decode(),
        }
        del x_f32, w_f32
        # "us": the same weight relaunched (the 256 MB memory-side cache serves it); "us_weights_from_hbm": copies
        # of the weight rotating through ~1.3 GB, as in shapes[]
        decode = []
        for name, act, w, out in (("gate_up", x, w_gu, out_gu), ("down", h, w_d, out_d)):
            copies = [w] + [w.clone() for _ in range(int(1.3e9 // (w.numel() * 2)))]
            for ts in (1, 16, 64):
                a_t, o_t = act[:ts], out[:ts]
                ms_t = _time_calls(lambda: gemm.tree_gemm(a_t, w.t(), out=o_t), 20, 5)

                def rotation():
                    for w_c in copies:
                        gemm.tree_gemm(a_t, w_c.t(), out=o_t)

                ms_rot = _time_calls(rotation, 6, 2) / len(copies)
                decode.append({"op": name, "T": ts, "us": round(ms_t * 1e3, 1),
                               "weight_gbps": round(w.numel() * 2 / ms_t * 1e-6, 1),
                               "us_weights_from_hbm": round(ms_rot * 1e3, 1),
                               "weight_gbps_from_hbm": round(w.numel() * 2 / ms_rot * 1e-6, 1)})
            del copies
        decode.sort(key=lambda d: (d["T"], d["op"] != "gate_up"))
        result["det_gemm_tree"]["decode"] = decode

    # ---- fused linear-LogP at T=8192, V=151936
    if not args.no_logp:
        tl = 8192
        hid = randn(tl, HIDDEN)
        hid = (hid.float() * torch.rsqrt(hid.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
        w_lm = randn(VOCAB, HIDDEN, 0.02)
        tgt = torch.randint(0, VOCAB, (tl,), generator=gen, device=dev)
        from rl_engine import _C

        ms_lp = _time_calls(lambda: deterministic_linear_logp(hid, w_lm, tgt), 10, 4)
        fl_lp = 2.0 * tl * VOCAB * HIDDEN
        result["linear_logp"] = {
            "workload": "hidden[8192,4096] x lm_head[151936,4096]^T -> online LSE -> target gather, fp32 logp",
            "tokens_per_s": round(tl / ms_lp * 1e3, 1),
            "ms": round(ms_lp, 3),
            "tflops": round(fl_lp / ms_lp * 1e-9, 1),
            "frac_of_mfma_peak": round(fl_lp / ms_lp * 1e-9 / PEAK_BF16_TFLOPS, 4),
            "min_hbm_bytes": 2.0 * (VOCAB * HIDDEN + tl * HIDDEN) + 8.0 * tl,
        }
        # backward: logits recompute + grad_hidden + grad_weight = three GEMMs of the forward's size
        _, lse_lp = _C.fused_linear_logp(hid, w_lm, tgt)
        g_lp = torch.randn((tl,), generator=gen, device=dev)
        ms_bwd = _time_calls(lambda: _C.fused_linear_logp_bwd(hid, w_lm, tgt, lse_lp, g_lp, None), 5, 2)
        result["linear_logp"]["backward"] = {
            "workload": "d(logits) recompute (bf16, 2.49 GB) -> grad_hidden[8192,4096] and grad_weight[151936,4096]",
            "ms": round(ms_bwd, 3),
            "tokens_per_s": round(tl / ms_bwd * 1e3, 1),
            "tflops": round(3 * fl_lp / ms_bwd * 1e-9, 1),
            "frac_of_mfma_peak": round(3 * fl_lp / ms_bwd * 1e-9 / PEAK_BF16_TFLOPS, 4),
        }
        del lse_lp, g_lp
        # the same pass with the fp32 logits stored (return_logits=True) against the plain forward, at 2048 tokens
        hid_s, tgt_s = hid[:2048].contiguous(), tgt[:2048].contiguous()
        ms_plain = _time_calls(lambda: deterministic_linear_logp(hid_s, w_lm, tgt_s), 10, 4)
        ms_logits = _time_calls(lambda: deterministic_linear_logp(hid_s, w_lm, tgt_s, return_logits=True), 10, 4)
        result["linear_logp"]["return_logits"] = {
            "workload": "T=2048: LogP forward, and the same launch storing logits[2048,151936] as fp32 (1.24 GB written)",
            "ms_plain": round(ms_plain, 3), "ms_with_logits": round(ms_logits, 3), "ratio": round(ms_logits / ms_plain, 3),
        }
        # the backward below the token count where its GEMMs fill the chip: 256 tokens
        hid_b, tgt_b = hid[:256].contiguous(), tgt[:256].contiguous()
        _, lse_b = _C.fused_linear_logp(hid_b, w_lm, tgt_b)
        g_b = torch.randn((256,), generator=gen, device=dev)
        ms_bs = _time_calls(lambda: _C.fused_linear_logp_bwd(hid_b, w_lm, tgt_b, lse_b, g_b, None), 10, 4)
        result["linear_logp"]["backward_256_tokens"] = {
            "workload": "T=256: d(logits) recompute -> grad_hidden[256,4096] (reduction over 151936) and grad_weight[151936,4096]",
            "ms": round(ms_bs, 3),
            "min_hbm_bytes": 3 * 2.0 * VOCAB * HIDDEN,  # the weight read twice, its gradient written once
            "frac_of_hbm_peak": round(3 * 2.0 * VOCAB * HIDDEN / ms_bs * 1e-6 / PEAK_HBM_GBPS, 4),
        }
        # a token count that 64 does not divide: the weight gradient reduces over it (whole K tiles + a tail step)
        hid_r, tgt_r = hid[:8191].contiguous(), tgt[:8191].contiguous()
        _, lse_r = _C.fused_linear_logp(hid_r, w_lm, tgt_r)
        g_r = torch.randn((8191,), generator=gen, device=dev)
        ms_br = _time_calls(lambda: _C.fused_linear_logp_bwd(hid_r, w_lm, tgt_r, lse_r, g_r, None), 4, 2)
        result["linear_logp"]["backward_8191_tokens"] = {"ms": round(ms_br, 3), "ratio_to_8192_tokens": round(ms_br / ms_bwd, 3)}
        del hid_r, tgt_r, lse_r, g_r
        del hid_s, tgt_s, hid_b, tgt_b, lse_b, g_b
        # the stage that reuses materialised logits: one pass over [8192, 151936] bf16
        logits = randn(tl, VOCAB, 4.0)
        ms_fl = _time_calls(lambda: _C.hip_deterministic_logp_from_logits(logits, tgt, 0, VOCAB, 64), 10, 4)
        by_fl = 2.0 * tl * VOCAB
        result["linear_logp"]["from_logits"] = {
            "workload": "bf16 logits[8192,151936] -> 64 tile statistics -> merge -> target gather",
            "ms": round(ms_fl, 3),
            "tokens_per_s": round(tl / ms_fl * 1e3, 1),
            "bound": "hbm",
            "gbps": round(by_fl / ms_fl * 1e-6, 1),
            "frac_of_hbm_peak": round(by_fl / ms_fl * 1e-6 / PEAK_HBM_GBPS, 4),
        }
        # its backward: one read of the logits and one write of their gradient
        lse_fl = torch.full((tl,), 12.0, device=dev)
        g_fl = torch.randn((tl,), generator=gen, device=dev)
        z_fl = torch.zeros((tl,), device=dev)
        ms_fb = _time_calls(lambda: _C.hip_deterministic_logp_backward(logits, lse_fl, g_fl, z_fl, tgt, 0, VOCAB, False), 10, 4)
        result["linear_logp"]["from_logits_backward"] = {
            "workload": "bf16 logits[8192,151936] + lse -> bf16 d(logits) (coef * (onehot - p))",
            "ms": round(ms_fb, 3),
            "bound": "hbm",
            "gbps": round(2 * by_fl / ms_fb * 1e-6, 1),
            "frac_of_hbm_peak": round(2 * by_fl / ms_fb * 1e-6 / PEAK_HBM_GBPS, 4),
        }
        del logits, lse_fl, g_fl, z_fl
        # rollout scale: 64 rollouts x 1024 tokens through the fused LogP, then the GRPO ratio / k3-KL epilogue
        from rl_engine.ops.loss import grpo_ratio_kl_loss

        rollouts, per = 64, 1024
        tr = rollouts * per
        hid_r = randn(tr, HIDDEN)
        tgt_r = torch.randint(0, VOCAB, (tr,), generator=gen, device=dev)
        logp_r, _ = deterministic_linear_logp(hid_r, w_lm, tgt_r)
        old_r = (logp_r + 0.05 * torch.randn((tr,), generator=gen, device=dev)).view(rollouts, per)
        ref_r = (logp_r + 0.05 * torch.randn((tr,), generator=gen, device=dev)).view(rollouts, per)
        adv_r = torch.randn((rollouts,), generator=gen, device=dev)

        def rollout_step():
            lp, _ = deterministic_linear_logp(hid_r, w_lm, tgt_r)
            return grpo_ratio_kl_loss(lp.view(rollouts, per), old_r, ref_r, adv_r, clip_eps=0.2, beta=0.01)

        ms_r = _time_calls(rollout_step, 3, 2)
        ms_g = _time_calls(lambda: grpo_ratio_kl_loss(logp_r.view(rollouts, per), old_r, ref_r, adv_r, clip_eps=0.2, beta=0.01), 20, 5)
        result["linear_logp"]["rollout_grpo"] = {
            "workload": "64 rollouts x 1024 tokens: fused LogP (V=151936) -> ratio, k3-KL, clipped loss",
            "ms": round(ms_r, 3),
            "tokens_per_s": round(tr / ms_r * 1e3, 1),
            "tflops": round(2.0 * tr * VOCAB * HIDDEN / ms_r * 1e-9, 1),
            "frac_of_mfma_peak": round(2.0 * tr * VOCAB * HIDDEN / ms_r * 1e-9 / PEAK_BF16_TFLOPS, 4),
            "grpo_epilogue_ms": round(ms_g, 4),
        }
        del hid_r, tgt_r, logp_r, old_r, ref_r

    # ---- gated FFN at T=4096: fused gate/up + SwiGLU, then down
    if not args.no_shapes:
        from rl_engine.ops.ffn import qwen3_ffn_packed_inference

        ms_ffn = _time_calls(lambda: qwen3_ffn_packed_inference(x, w_gu, w_d), 20, 10)
        result["ffn"] = {
            "workload": "x[4096,4096] -> packed gate/up GEMM with SwiGLU epilogue -> down GEMM, bf16",
            "ms": round(ms_ffn, 4),
            "tflops": round((flops_gu + flops_d) / ms_ffn * 1e-9, 1),
            "frac_of_mfma_peak": round((flops_gu + flops_d) / ms_ffn * 1e-9 / PEAK_BF16_TFLOPS, 4),
            "tokens_per_s": round(T / ms_ffn * 1e3, 1),
        }

    # ---- CPU baseline: the oracle's torch forms (the reference's own CPU expressions) on the same step, on this
    # box's host cores
    if not args.no_cpu:
        import numpy as np

        from oracle import reference_math as oracle

        torch.set_num_threads(int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        threads = torch.get_num_threads()
        cpu_model = oracle.cpu_model_string()
        xc, hc, wgc, wdc = x.cpu(), h.cpu(), w_gu.cpu(), w_d.cpu()
        oracle.det_gemm_ref_torch(xc[:256], wgc)  # warm-up: thread pool, allocator
        times = []
        while len(times) < 3 or sum(times) < 10.0:  # about 10 s of host work, at least three runs
            t0 = time.perf_counter()
            oracle.det_gemm_ref_torch(xc, wgc)
            oracle.det_gemm_ref_torch(hc, wdc)
            times.append(time.perf_counter() - t0)
            if sum(times) > 30:
                break
        cpu_s = float(np.median(times))
        t0 = time.perf_counter()
        oracle.native_gemm_torch(xc, wgc)
        oracle.native_gemm_torch(hc, wdc)
        native_s = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": round((flops_gu + flops_d) / cpu_s * 1e-12, 4),
            "unit": "TFLOP/s",
            "cores": int(threads),
            "kind": "port",
            "cpu_model": cpu_model,
            "torch_num_threads": int(threads),
            "torch_version": torch.__version__,
            "sample": f"the full step (gate_up + down at T=4096, {(flops_gu + flops_d) / 1e9:.0f} GFLOP), "
            f"median of {len(times)} runs of oracle.det_gemm_ref_torch ((a.float() @ b.float()).to(bf16)), {cpu_s:.2f} s each",
            "native_bf16_matmul": {"value": round((flops_gu + flops_d) / native_s * 1e-12, 4), "unit": "TFLOP/s",
                                   "sample": f"one run of torch.matmul on the bf16 tensors (NativeGemmOp), {native_s:.2f} s"},
        }
        del xc, hc, wgc, wdc
        if not args.no_logp:
            ts = 8192  # the whole workload once: several seconds of host work
            t0 = time.perf_counter()
            oracle.linear_logp_chunked_torch(hid[:ts].cpu(), w_lm.cpu(), tgt[:ts].cpu(), chunk_elems=ts * 2048)
            cpu_lp = time.perf_counter() - t0
            result["linear_logp"]["cpu_baseline"] = {
                "value": round(ts / cpu_lp, 1),
                "unit": "tokens/s",
                "cores": int(threads),
                "kind": "port",
                "cpu_model": cpu_model,
                "torch_num_threads": int(threads),
                "sample": f"all {ts} tokens once, oracle.linear_logp_chunked_torch (2048-row vocabulary chunks), {cpu_lp:.2f} s",
            }

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
