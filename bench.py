#!/usr/bin/env python3
"""Benchmark of the CKKS hot path on one MI355X.

Headline (BASELINE.json configs[1]): batched RNS NTT/iNTT at N = 2^16, 24 primes < 2^36, a batch of 32 ciphertexts
(2 polynomials x 24 limbs each = 1536 limbs, 768 MiB of uniform u64 residues, seed 2), resident in HBM.
One step = inverse transform then forward transform of the whole batch (the order ntt_throughput.cu:51-60 uses)
= 2 * 1536 limb-transforms.  value = limb-transforms per second.

Also measured and reported in the same JSON line:
  roofline      - the slowest kernel launch of the step, HIP events on the launch stream; algorithmic bytes = 16*N per
                  limb-transform (all of it in one launch where the library takes the resident transform, half of it credited to
                  each launch of the two-launch form); beside the published peak the ceiling measured in the same run
  ppmm          - the ring-packed PPMM at the BERT-base shape (configs[3]), int8-MAC/s against the int8 MFMA peak
  keyswitch     - one textbook hybrid key switch at configs[2]
  cpu_baseline  - the CPU oracle (a port of the reference arithmetic, OpenMP) on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_I8_PEAK_TMACS = 2516.6          # 5.033 POP/s dense int8 = 2.5166e15 MAC/s
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_per_call.txt")


def kernel_sources_id():
    """Short hash of the HIP sources: the traffic figures below are only quoted for the kernels they were measured on."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "ckks_llm_amd", "csrc")
    for name in sorted(os.listdir(src)):
        if name.endswith((".hip", ".hpp")):
            with open(os.path.join(src, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:12]


def measured_traffic():
    """HBM bytes per call, from rocprofv3 counter runs (FETCH_SIZE, WRITE_SIZE, each scaled by what the same counter reads for a
    device-to-device copy of known size in the same run) summarised in profiles/hbm_traffic_per_call.txt.  The file names the
    kernel sources it was measured on; for other sources (or without the file) nothing is quoted."""
    out = {}
    try:
        with open(TRAFFIC_FILE) as f:
            lines = f.read().splitlines()
    except OSError:
        return out, "no traffic summary"
    measured_on = None
    for ln in lines:
        ln = ln.strip()
        if ln.startswith("kernel_sources_id"):
            measured_on = ln.split()[1]
        elif ln and not ln.startswith("#"):
            parts = ln.split()
            if len(parts) >= 2:
                try:
                    out[parts[0]] = float(parts[1])
                except ValueError:
                    pass
    if measured_on != kernel_sources_id():
        return {}, "traffic summary is for kernel sources %s, these are %s: not quoted" % (measured_on, kernel_sources_id())
    return out, "profiles/hbm_traffic_per_call.txt (kernel sources %s)" % measured_on


def uniform_limbs(seed, primes, polys, N):
    rng = np.random.default_rng(seed)
    out = np.empty((polys, len(primes), N), dtype=np.uint64)
    for j, q in enumerate(primes):
        out[:, j, :] = rng.integers(0, q, size=(polys, N), dtype=np.uint64)
    return out


def bench_ntt(args, P):
    from ckks_llm_amd import Context_23, DeviceBuffer
    logN, primes, cts = 16, P.CFG2_Q, args.batch
    N, L1, polys = 1 << logN, len(primes), 2 * cts
    limbs = polys * L1
    ctx = Context_23(logN, [], primes)
    if args.ntt_mode:
        ctx.set_ntt_mode(args.ntt_mode)                  # profiling aid: 2 = both passes chained in one launch, 3 = one workgroup per limb
        if args.ntt_mode == 2 and args.chain_skew:
            ctx.set_ntt_chain(args.chain_skew)
    # synthetic data: one ciphertext's worth of seeded residues, replicated over the batch (same distribution, bounded set-up time)
    one = uniform_limbs(2, primes, 2, N)
    buf = DeviceBuffer(8 * limbs * N)
    for c in range(cts):
        buf.L_.ckks_memcpy_h2d(buf.ptr + c * one.nbytes, one.ctypes.data, one.nbytes)
    ctx.sync()

    def step():
        ctx.FromNTTInplace(buf, 0, 0, polys, L1, L1)
        ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)

    # The timed steps carry a mark (an event record on the launch stream, nothing waits for it) in front of every transform, as long
    # as the marks last: the intervals between them, read after the region, are the transforms' durations inside the timed region.
    marked = min(args.steps, 2000)

    def marked_step(i):
        ctx.timer_mark(2 * i)
        ctx.FromNTTInplace(buf, 0, 0, polys, L1, L1)
        ctx.timer_mark(2 * i + 1)
        ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)

    for _ in range(args.warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        if i < marked:
            marked_step(i)
        else:
            step()
    ctx.timer_mark(2 * marked)          # behind the last marked step's forward transform when every step is marked
    ctx.sync()
    dt = time.perf_counter() - t0
    inv_in_region = sum(ctx.timer_between(2 * i, 2 * i + 1) for i in range(marked)) / marked
    n_fwd = marked if marked == args.steps else marked - 1          # the last mark sits behind the unmarked steps, if there are any
    fwd_in_region = sum(ctx.timer_between(2 * i + 1, 2 * i + 2) for i in range(n_fwd)) / max(1, n_fwd)
    # round trip must give the data back (bit-exact) - cheap end-to-end sanity on the timed buffer
    back = buf.download(np.uint64, one.size).reshape(one.shape)
    assert np.array_equal(back, one), "NTT round trip changed the data"
    ms_per_step = dt / args.steps * 1e3
    value = 2 * limbs * args.steps / dt

    # Per-kernel durations, HIP events on the launch stream.  Where the library takes the resident transform (one launch per
    # transform: N = 2^16, primes below 2^36, at least a limb per compute unit) the launch is the transform; otherwise a transform
    # is two launches and the events sit between them.
    reps = max(5, min(20, args.steps))
    per_round = ctx.info("ntt_resident_round")
    resident = args.ntt_mode in (0, 6) and per_round > 0 and limbs >= per_round and max(primes) < (1 << 36)
    one_launch = resident or args.ntt_mode in (2, 3, 4, 5)
    alg_bytes_transform = 16.0 * N * limbs
    traffic, traffic_note = measured_traffic()

    def timed(f, n):
        for _ in range(2):
            f(buf, 0, 0, polys, L1, L1)
        ctx.timer_start()
        for _ in range(n):
            f(buf, 0, 0, polys, L1, L1)
        return ctx.timer_stop() / n

    # the two-launch form, pass by pass (what the library falls back to, and the reference point of the one-launch forms)
    ctx.set_ntt_mode(0 if one_launch else args.ntt_mode)      # the timed entry point always takes two launches (5-byte form between them)
    f1 = f2 = i1 = i2 = 0.0
    for _ in range(reps):
        a, b = ctx.ntt_timed(buf, 0, 0, polys, L1, L1, True)
        i1 += a; i2 += b
        a, b = ctx.ntt_timed(buf, 0, 0, polys, L1, L1, False)
        f1 += a; f2 += b
    f1, f2, i1, i2 = [x / reps for x in (f1, f2, i1, i2)]
    ctx.set_ntt_mode(args.ntt_mode)
    passes = [("ntt_strided_pass(fwd)", f1), ("ntt_row_pass(fwd)", f2), ("ntt_row_pass(inv)", i1), ("ntt_strided_pass(inv)", i2)]
    pass_ms = {"fwd_strided": round(f1, 4), "fwd_row": round(f2, 4), "inv_row": round(i1, 4), "inv_strided": round(i2, 4)}
    if one_launch:
        # one launch per transform: the intervals between the marks of the timed region are the launches' durations
        fwd_ms, inv_ms = fwd_in_region, inv_in_region
        name = "ntt_resident_kernel" if resident else "one-launch transform (ntt_mode %d)" % args.ntt_mode
        dom_name, dom_ms = max([(name + "(fwd)", fwd_ms), (name + "(inv)", inv_ms)], key=lambda x: x[1])
        alg_bytes_launch = alg_bytes_transform
        key = "ntt_resident_fwd_1536_limbs" if dom_name.endswith("(fwd)") else "ntt_resident_inv_1536_limbs"
        kernel_ms = {"fwd": round(fwd_ms, 4), "inv": round(inv_ms, 4)}
    else:
        fwd_ms, inv_ms = f1 + f2, i1 + i2
        dom_name, dom_ms = max(passes, key=lambda x: x[1])          # the slowest of all four passes
        alg_bytes_launch = alg_bytes_transform / 2.0                # half a transform per launch
        key = {"ntt_strided_pass(fwd)": "ntt_strided_pass_fwd_1536_limbs", "ntt_row_pass(fwd)": "ntt_row_pass_fwd_1536_limbs",
               "ntt_row_pass(inv)": "ntt_row_pass_inv_1536_limbs", "ntt_strided_pass(inv)": "ntt_strided_pass_inv_1536_limbs"}[dom_name]
        kernel_ms = pass_ms
    achieved = alg_bytes_launch / (dom_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": dom_name, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic.get(key) if limbs == 1536 and resident == (args.ntt_mode in (0, 6)) else None,
                "traffic_source": traffic_note, "launches_per_transform": 1 if one_launch else 2, "kernel_ms": kernel_ms,
                "kernel_ms_is": "average over the launches of the timed region (marks on the launch stream between them)" if one_launch
                                else "average over %d transforms with events between the two launches, behind the timed region" % reps,
                "transform_ms_in_timed_region": {"fwd": round(fwd_in_region, 4), "inv": round(inv_in_region, 4)},

                "two_launch_form_pass_ms": pass_ms,
                "transform_algorithmic_GBps": {"fwd": round(alg_bytes_transform / (fwd_ms * 1e-3) / 1e9, 1),
                                               "inv": round(alg_bytes_transform / (inv_ms * 1e-3) / 1e9, 1)},
                "algorithmic_bytes_per_launch": alg_bytes_launch}
    # measured ceiling of the same run: a device-to-device copy of half the batch onto the other half (reads and writes %d MiB each)
    half = 4 * limbs * N
    for _ in range(2):
        buf.L_.ckks_memcpy_d2d(buf.ptr + half, buf.ptr, half)
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(5):
        buf.L_.ckks_memcpy_d2d(buf.ptr + half, buf.ptr, half)
    ctx.sync()
    copy_gbs = 2.0 * half * 5 / (time.perf_counter() - t0) / 1e9
    roofline["peak_measured"] = round(copy_gbs, 1)
    roofline["peak_measured_how"] = "device-to-device copy of %d MiB in the same run, bytes read + bytes written per second" % (half >> 20)
    roofline["frac_of_measured"] = round(achieved / copy_gbs, 4)
    # the copy overwrote half of the batch: put the seeded data back for what follows
    for c in range(cts):
        buf.L_.ckks_memcpy_h2d(buf.ptr + c * one.nbytes, one.ctypes.data, one.nbytes)
    ctx.sync()
    if args.batch_only:
        buf.free()
        return value, ms_per_step, roofline, None, limbs
    # one ciphertext (48 limbs, 24 MiB): the latency-oriented half of configs[1]
    one_ct = {}
    small = DeviceBuffer.from_numpy(one)
    for _ in range(5):
        ctx.ToNTTInplace(small, 0, 0, 2, L1, L1)
        ctx.FromNTTInplace(small, 0, 0, 2, L1, L1)
    ctx.timer_start()
    R = 50
    for _ in range(R):
        ctx.ToNTTInplace(small, 0, 0, 2, L1, L1)
    fw = ctx.timer_stop() / R
    ctx.timer_start()
    for _ in range(R):
        ctx.FromNTTInplace(small, 0, 0, 2, L1, L1)
    iv = ctx.timer_stop() / R
    one_ct = {"fwd_us": round(fw * 1e3, 2), "inv_us": round(iv * 1e3, 2),
              "fwd_limb_transforms_per_s": round(2 * L1 / (fw * 1e-3)), "inv_limb_transforms_per_s": round(2 * L1 / (iv * 1e-3))}
    # a ciphertext at level 15 (32 limbs): below 41 limbs the library takes the paired one-launch form; two launches beside it
    if not args.ntt_mode:
        lv = {}
        for label, mode in (("fwd_us", 0), ("two_launch_fwd_us", 1)):
            ctx.set_ntt_mode(mode)
            for _ in range(5):
                ctx.ToNTTInplace(small, 0, 0, 2, 16, L1)
            ctx.timer_start()
            for _ in range(R):
                ctx.ToNTTInplace(small, 0, 0, 2, 16, L1)
            lv[label] = round(ctx.timer_stop() / R * 1e3, 2)
        ctx.set_ntt_mode(0)
        one_ct["level15_32_limbs"] = lv
    buf.free(); small.free()
    return value, ms_per_step, roofline, one_ct, limbs


def bench_cpu_baseline(P, seconds_target=12.0):
    """Oracle (port of the reference arithmetic) on a bounded sample: forward+inverse of `limbs` limbs at N = 2^16."""
    from oracle import oracle_py as O
    primes = P.CFG2_Q
    ctx = O.OracleContext(16, [], primes)
    threads = O.lib().orc_max_threads()
    polys = 4
    data = uniform_limbs(2, primes, polys, 1 << 16)
    flat = data.reshape(-1)
    limbs = polys * len(primes)
    # one untimed pass to size the sample
    t0 = time.perf_counter()
    ctx.FromNTTInplace(flat, 0, 0, polys, len(primes), len(primes))
    ctx.ToNTTInplace(flat, 0, 0, polys, len(primes), len(primes))
    once = time.perf_counter() - t0
    reps = max(1, min(40, int(seconds_target / max(once, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(reps):
        ctx.FromNTTInplace(flat, 0, 0, polys, len(primes), len(primes))
        ctx.ToNTTInplace(flat, 0, 0, polys, len(primes), len(primes))
    dt = time.perf_counter() - t0
    assert np.array_equal(flat.reshape(data.shape), uniform_limbs(2, primes, polys, 1 << 16))
    return {"value": round(2 * limbs * reps / dt, 1), "unit": "limb-transforms/s", "cores": threads, "kind": "port",
            "sample": "%d x (iNTT+NTT) of %d limbs (N=2^16, %d primes, %d polys), OpenMP over limbs" % (reps, limbs, len(primes), polys)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: 30 warm-up steps (about 30 ms) carry the run past the clock ramp that follows an idle GPU (the first 15 ms or so
    # run about 8 % slower); 100 timed steps then take a tenth of a second
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--batch", type=int, default=32, help="ciphertexts per step (BASELINE configs[1]: 32)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--ntt-mode", type=int, default=0, help="profiling aid: launch form of the transforms (ckks_ctx_set_ntt_mode); with a "
                    "one-launch form the per-pass figures are half the transform's time")
    ap.add_argument("--chain-skew", type=int, default=0, help="profiling aid with --ntt-mode 2: limbs the first pass runs ahead")
    ap.add_argument("--skip-extra", action="store_true", help="skip the PPMM / key-switch side measurements")
    ap.add_argument("--batch-only", action="store_true",
                    help="profiling aid: only the batched NTT launches (no one-ciphertext, PPMM, key-switch or CPU legs); the "
                         "device-to-device copies of half the batch in it are the reference point of the traffic counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import ckks_llm_amd.params as P
    value, ms_per_step, roofline, one_ct, limbs = bench_ntt(args, P)
    line = {
        "metric": "NTT limb-transforms/s @N=2^16", "value": round(value, 1), "unit": "limb-transforms/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u64 residues (exact-integer f64 butterflies for q < 2^50, u64 butterflies above)", "data": "synthetic",
        "config": {"workload": "configs[1]: RNS NTT+iNTT, N=2^16, 24 primes <2^36, batch of %d ciphertexts (%d limbs, %d MiB) per step"
                               % (args.batch, limbs, limbs * 8 * 65536 >> 20), "limb_transforms_per_step": 2 * limbs},
        "roofline": roofline, "one_ciphertext": one_ct,
        "frac_of_hbm_roofline_whole_transform": round(value * 16 * 65536 / 1e9 / HBM_PEAK_GBS, 4),
    }
    if args.batch_only:
        del line["one_ciphertext"]
        args.skip_extra = args.skip_cpu = True
    if not args.skip_extra:
        try:
            import bench_extra
            line.update(bench_extra.run(P, measured_traffic(), roofline.get("peak_measured")))
        except ImportError:
            pass
    if not args.skip_cpu:
        line["cpu_baseline"] = bench_cpu_baseline(P)
        if not args.skip_extra:
            # the CPU oracle beside the other GPU figures of the line (bounded samples, a few seconds each)
            import bench_extra
            line["ppmm"]["cpu_baseline"] = bench_extra.cpu_ppmm(P)
            line["keyswitch"]["cpu_baseline"] = bench_extra.cpu_keyswitch(P)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
