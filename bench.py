#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of the bf16 causal prefill kernel over the headline workload
B=4, H=32, N=4096, D=128 (inputs resident in HBM before the timed region); the same run also
times the batched GQA decode workload (batch 64, 32 query / 8 kv heads, D=128, context lengths
uniform in [512, 8192], Lmax 8192) and reports it under "decode", and the f32 causal prefill of
B=1, H=8, N=2048, D=64 (the reference's own CPU-runnable case) under "f32_prefill", and the f32
backward on that shape under "f32_backward", the padded-batch prefill (B=16, H=16, D=64, lengths in [128, 1024])
under "padded_prefill", the long-context prefill (B=1, H=32, N=16384, D=128, Q scaled by 2) under
"long_prefill", a long prefill at the other head dim of the matrix-core kernels (B=4, H=32, N=4096, D=64) under
"d64_prefill", and under "other_shapes" the tile kernel at head dims 32, 96 and 256 (B=4, H=32, N=2048, causal) and
the bf16 masked self-attention of MultiHeadAttention (B=4, T=1024, H=16, hd=64, a sliding-window mask as an f32 bias)
and the sliding-window entry that needs no mask tensor (B=4, T=4096, H=16, hd=64, window 256).

Every leg first runs a settle phase: launches of the leg's own step until SETTLE_MS of device time have passed
(after an idle period the clocks first drop and then recover over some tens of milliseconds); the phase is
reported as settle_ms / settle_launches and is followed by the counted warm-up (--warmup) and the timed region
(--steps), which is the only part that enters value, ms_per_step and roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only prefill|decode|f32|bwd|padded|long|d64|shapes]

Prints ONE JSON line.  `value` is prefill TFLOP/s with causal-counted FLOPs
(4*B*H*D*N*(N+1)/2: skipped tiles are not credited); `roofline` prices it against the dense bf16
MFMA peak, `decode.roofline` against the HBM peak with algorithmic bytes (K+V read once per kv
head, Q in, O out).  Kernel durations are measured with HIP events on the stream the kernels
are launched on.  Every leg's parity check against the oracle prints `parity_max_abs` and
`parity_rel_fro` (the largest relative Frobenius error over blocks of 256 query rows of a (b,h)
slab; per (sequence, head) row for decode); bf16 legs must meet max-abs <= 2e-2 and relative
<= 1e-2, the f32 legs their max-abs bars.  `cpu_baseline` times the CPU oracle (a C restatement of the reference's CPU
path; the reference itself is Rust and cannot be built here) on a bounded sample, on this box's
host cores.
"""
import argparse
import ctypes as C
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
PEAK_F32_TFLOPS = 157.3     # MI355X dense f32 MFMA
SETTLE_MS = 100.0           # device time of the settle phase that precedes every leg's warm-up
PROFILES = os.path.join(ROOT, "profiles")


def profile_traffic(md_name, entry):
    """HBM bytes per launch of a kernel (or a step of several kernels) as measured with rocprofv3 --pmc and
    written down in profiles/<md_name>: the file carries a fenced block

        ```json traffic
        {"<entry>": {"fetch_size": F, "write_size": W}, ..., "scale": {"fetch_kib": 2.0, "write_kib": 1.0}}
        ```

    with the FETCH_SIZE / WRITE_SIZE readings per launch and the factors that a copy of known size gave for them.
    Counters cannot be read from inside this process: the figure is the committed measurement, and it is None
    when the file or the entry is not there."""
    import re
    try:
        text = open(os.path.join(PROFILES, md_name)).read()
    except OSError:
        return None
    m = re.search(r"```json traffic\n(.*?)```", text, re.S)
    if not m:
        return None
    try:
        block = json.loads(m.group(1))
        e, sc = block[entry], block["scale"]
        return (float(e["fetch_size"]) * float(sc["fetch_kib"]) + float(e["write_size"]) * float(sc["write_kib"])) * 1024
    except (ValueError, KeyError, TypeError):
        return None


class Hip:
    """The few HIP runtime calls the timing needs (stream + events), straight from libamdhip64."""

    def __init__(self):
        from rustorch_amd import _lib

        self.lib = _lib.hip_runtime()
        for name, args in (("hipStreamCreate", [C.POINTER(C.c_void_p)]), ("hipEventCreate", [C.POINTER(C.c_void_p)]),
                           ("hipEventRecord", [C.c_void_p, C.c_void_p]), ("hipEventSynchronize", [C.c_void_p]),
                           ("hipEventElapsedTime", [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]),
                           ("hipStreamSynchronize", [C.c_void_p]), ("hipDeviceSynchronize", [])):
            getattr(self.lib, name).argtypes = args

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with hipError {rc}")

    def stream(self):
        s = C.c_void_p()
        self.check(self.lib.hipStreamCreate(C.byref(s)), "hipStreamCreate")
        return s

    def event(self):
        e = C.c_void_p()
        self.check(self.lib.hipEventCreate(C.byref(e)), "hipEventCreate")
        return e

    def record(self, e, s):
        self.check(self.lib.hipEventRecord(e, s), "hipEventRecord")

    def elapsed_ms(self, e0, e1):
        self.check(self.lib.hipEventSynchronize(e1), "hipEventSynchronize")
        ms = C.c_float()
        self.check(self.lib.hipEventElapsedTime(C.byref(ms), e0, e1), "hipEventElapsedTime")
        return ms.value

    def sync(self):
        self.check(self.lib.hipDeviceSynchronize(), "hipDeviceSynchronize")


class Timing:
    """wall_ms: K steps by the wall clock, synchronised on both sides.  mean_ms: average duration of a step from ONE
    pair of HIP events on `stream` around the K steps (nothing is recorded between launches, so the stream runs
    them back to back as a serving loop would).  per: per-step durations of 100 further steps run after the timed
    region, each between its own pair of events (the spread; each reads a few microseconds longer than a
    back-to-back step).  settle_ms / settle_launches: the settle phase that ran before the warm-up."""

    def __init__(self, wall_ms, region_ms, steps, per, settle_ms, settle_launches):
        self.wall_ms, self.mean_ms, self.per = wall_ms, region_ms / steps, per
        self.settle_ms, self.settle_launches = settle_ms, settle_launches

    def settle(self):
        return {"settle_ms": self.settle_ms, "settle_launches": self.settle_launches}


def settle(hip, stream, launch, min_ms=SETTLE_MS):
    """Launches the step back to back until `min_ms` of device time have passed (event pairs around growing
    batches).  Returns (device ms, launches).  Not part of any reported rate."""
    done_ms, n, batch = 0.0, 0, 4
    e0, e1 = hip.event(), hip.event()
    while done_ms < min_ms and n < 100000:
        hip.record(e0, stream)
        for i in range(batch):
            launch(n + i)
        hip.record(e1, stream)
        ms = hip.elapsed_ms(e0, e1)
        done_ms += ms
        n += batch
        per = max(ms / batch, 1e-3)
        batch = int(min(max((min_ms - done_ms) / per, 1), 4096))
    return done_ms, n


def time_steps(hip, stream, launch, steps, warmup, spread_steps=100, settle_ms=SETTLE_MS):
    s_ms, s_n = settle(hip, stream, launch, settle_ms) if settle_ms > 0 else (0.0, 0)
    for i in range(warmup):
        launch(s_n + i)
    hip.sync()
    e0, e1 = hip.event(), hip.event()
    t0 = time.perf_counter()
    hip.record(e0, stream)
    for i in range(steps):
        launch(s_n + warmup + i)
    hip.record(e1, stream)
    hip.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    region_ms = hip.elapsed_ms(e0, e1)
    evs = [(hip.event(), hip.event()) for _ in range(spread_steps)]
    for j, (a, b) in enumerate(evs):
        hip.record(a, stream)
        launch(s_n + warmup + steps + j)
        hip.record(b, stream)
    hip.sync()
    per = np.array([hip.elapsed_ms(a, b) for a, b in evs]) if evs else np.zeros(0)
    return Timing(wall_ms, region_ms, steps, per, s_ms, s_n)


def spread(per):
    """Median, 99th percentile (the two figures the reference's own harness reports, bench-vs-pytorch/src/main.rs:28-42)
    and minimum of the per-step event durations taken after the timed region."""
    if per.size == 0:
        return {}
    return {"kernel_ms_median": float(np.median(per)), "kernel_ms_p99": float(np.percentile(per, 99)),
            "kernel_ms_min": float(per.min())}


def sustained_mfma():
    """Rate and shader clock of a pure bf16 MFMA loop on changing N(0,1)-like operands, launched back to back for
    about a second (a child process: rustorch_amd/lib/mfma_sustained, built with the library).  None when the
    program is missing or fails; the bench line is complete without it."""
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rustorch_amd", "lib", "mfma_sustained")
    if not os.path.exists(exe):
        return None
    try:
        r = subprocess.run([exe, "2", "12"], capture_output=True, text=True, timeout=60)
        last = r.stdout.strip().splitlines()[-1].split()
        if r.returncode != 0 or last[0] != "sustained":
            return None
        return {"tflops": float(last[1]), "shader_mhz": float(last[2]),
                "how": "v_mfma_f32_32x32x16_bf16 only, 8 waves/CU, operands changing per instruction, median of "
                       "launches 600-1199"}
    except (OSError, subprocess.SubprocessError, IndexError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # whatever --steps and --warmup are, every leg is preceded by its settle phase (see the module docstring)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the parity sample")
    ap.add_argument("--only", choices=["prefill", "decode", "f32", "bwd", "padded", "long", "d64", "shapes"], default=None)
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the run of rustorch_amd/lib/mfma_sustained (what a loop of nothing but bf16 MFMA "
                         "sustains on this GPU, reported beside the data-sheet peak)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also issue one 256 MiB device-to-device copy (a dispatch of known traffic, to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (attention shards over batch/heads "
              "with no exchange step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import rustorch_amd as ra
    from oracle import attn_oracle as oracle  # checker + cpu_baseline leg only

    ra.init(0)
    hip = Hip()
    stream = hip.stream()
    if args.calibrate_copy:
        n_copy = 256 << 20
        a, b_ = ra.HipStorage(n_copy), ra.HipStorage(n_copy)
        hip.lib.hipMemcpyDtoD.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        hip.check(hip.lib.hipMemcpyDtoD(b_.ptr, a.ptr, n_copy), "hipMemcpyDtoD")
        hip.sync()
        del a, b_
    K = ra.LlmKernels()
    rng = np.random.default_rng(1234)
    out = {}

    threads = min(oracle.max_threads(), 16)

    def causal_prefill(B, H, N, D, seed, q_scale, cpu_slabs, kernel_name, traffic):
        """bf16 causal prefill on [B,H,N,D]: timing, and (unless --no-cpu) parity and the CPU baseline on the first
        `cpu_slabs` (b,h) slabs."""
        rng_p = np.random.default_rng(seed)
        n_el = B * H * N * D
        qb = oracle.f32_to_bf16(rng_p.standard_normal(n_el, dtype=np.float32) * np.float32(q_scale))
        kb, vb = (oracle.f32_to_bf16(rng_p.standard_normal(n_el, dtype=np.float32)) for _ in range(2))
        dq, dk, dv = (ra.HipStorage.from_numpy(x) for x in (qb, kb, vb))
        dout = ra.HipStorage(n_el * 2)
        shape = ra.AttentionShape.new(B, H, N, D)
        causal = ra.Mask.causal()
        tm = time_steps(hip, stream, lambda i: ra.flash_forward_bf16_dev(shape, dq, dk, dv, dout, causal,
                                                                         stream=stream),
                        args.steps, args.warmup)
        flops_causal = 4.0 * B * H * D * (N * (N + 1) / 2.0)
        flops_full = 4.0 * B * H * D * float(N) * N
        ms_step = tm.wall_ms / args.steps
        ms_kernel = tm.mean_ms
        achieved = flops_causal / (ms_kernel * 1e-3) / 1e12
        leg = {"ms_per_step": ms_step, "kernel_ms_mean": ms_kernel, **spread(tm.per), **tm.settle(),
               "tflops": flops_causal / (ms_step * 1e-3) / 1e12,
               "tflops_unmasked_convention": flops_full / (ms_kernel * 1e-3) / 1e12,
               "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                            "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic, "kernel": kernel_name,
                            "kernel_ms_mean": ms_kernel, **spread(tm.per)}}
        if not args.no_cpu:
            # parity + CPU baseline on (b,h) slabs: the oracle computes every tile, like the reference
            slabs = list(range(min(cpu_slabs, B * H)))
            got = oracle.bf16_to_f32(dout.download(np.uint16)).reshape(B * H, N * D)
            qs, ks, vs = (np.stack([oracle.bf16_to_f32(x.reshape(B * H, -1)[s]) for s in slabs]) for x in (qb, kb, vb))
            t0 = time.perf_counter()
            want = oracle.flash_forward_masked(oracle.AttentionShape(1, len(slabs), N, D), qs, ks, vs, "causal",
                                               threads=threads).reshape(len(slabs), N * D)
            cpu_s = time.perf_counter() - t0
            err = float(np.abs(got[slabs] - want).max())
            rel = oracle.rel_fro_blocks(got[slabs], want, D, N)
            leg["parity_max_abs"] = err
            leg["parity_rel_fro"] = rel
            which = "all" if len(slabs) == B * H else "the first"
            leg["cpu_baseline"] = {"value": flops_causal * len(slabs) / (B * H) / cpu_s / 1e12, "unit": "TFLOP/s",
                                   "cores": min(threads, len(slabs)), "kind": "port",
                                   "sample": f"{which} {len(slabs)} of the {B * H} (b,h) slabs once, one task per slab "
                                             f"as rayon does, {cpu_s:.1f} s wall on {min(threads, len(slabs))} threads; "
                                             f"f32 on the bf16-rounded inputs; causal-counted FLOPs although every tile "
                                             f"is computed, as in the reference; the same slabs are the parity sample"}
            if not (err <= oracle.BF16_MAX_ABS and rel <= oracle.BF16_REL_FRO):
                print(f"PARITY FAILURE: prefill B={B} H={H} N={N} D={D} max-abs {err}, relative Frobenius error per "
                      f"256-row block {rel}", file=sys.stderr)
                sys.exit(1)
        return leg

    # ------------------------------------------------------------------ prefill (the step)
    B, H, N, D = 4, 32, 4096, 128
    prefill = None
    if args.only in (None, "prefill"):
        prefill = causal_prefill(B, H, N, D, 1234, 1.0, B * H, "flash_fwd_bf16_kernel<128, causal>",
                                 profile_traffic("flash_fwd_bf16_b4_h32_n4096_d128.md", "flash_fwd_bf16_kernel<128,causal>"))

    # ------------------------------------------------------------------ long-context prefill (Q scaled by 2)
    long_p = None
    if args.only in (None, "long"):
        Bl, Hl, Nl, Dl = 1, 32, 16384, 128
        # the CPU port needs ~5 s per slab per thread at this length: half of the 32 slabs, one per thread
        long_p = causal_prefill(Bl, Hl, Nl, Dl, 55, 2.0, 16, "flash_fwd_bf16_kernel<128, causal>",
                                profile_traffic("flash_fwd_bf16_b1_h32_n16384_d128.md", "flash_fwd_bf16_kernel<128,causal>"))
        long_p = {"metric": "prefill attn TFLOP/s", "value": long_p.pop("tflops"), "unit": "TFLOP/s", **long_p,
                  "config": {"workload": "bf16 long-context causal prefill, B=1 H=32 N=16384 D=128, N(0,1) inputs with Q "
                                         "scaled by 2.0 before rounding (seed 55), f32 accumulation",
                             "flop_convention": "4*B*H*D*N*(N+1)/2 (causal-counted)"}}

    # ------------------------------------------------------------------ long prefill at head dim 64
    d64_p = None
    if args.only in (None, "d64"):
        Bd, Hd, Nd, Dd = 4, 32, 4096, 64
        # (the library takes the tile kernel here; RT_ATTN_BF16_PREFILL=wide|persistent in the environment forces another,
        # which the leg then names)
        d64_kernel, d64_traffic = {
            "wide": ("flash_wide_bf16_kernel<causal>",
                     profile_traffic("flash_wide_bf16_b4_h32_n4096_d64.md", "flash_wide_bf16_kernel<causal>")),
            "persistent": ("flash_fwd_bf16_kernel<64, causal>", None),
        }.get(os.environ.get("RT_ATTN_BF16_PREFILL", ""),
              ("flash_tile_bf16_kernel<64, causal, direct>",
               profile_traffic("flash_tile_bf16_b4_h32_n4096_d64.md", "flash_tile_bf16_kernel<64,causal,direct>")))
        d64_p = causal_prefill(Bd, Hd, Nd, Dd, 64, 1.0, 32, d64_kernel, d64_traffic)
        d64_p = {"metric": "prefill attn TFLOP/s", "value": d64_p.pop("tflops"), "unit": "TFLOP/s", **d64_p,
                 "config": {"workload": "bf16 causal prefill at head dim 64, B=4 H=32 N=4096 D=64, N(0,1) inputs "
                                        "(seed 64), f32 accumulation",
                            "flop_convention": "4*B*H*D*N*(N+1)/2 (causal-counted)"}}

    # ------------------------------------------------------------------ shapes outside the five configurations the metric is quoted on: timed for the record
    shapes = None
    if args.only in (None, "shapes"):
        shapes = {}
        for Ds in (32, 96, 256):
            leg_s = causal_prefill(4, 32, 2048, Ds, 300 + Ds, 1.0, 8, f"flash_tile_bf16_kernel<{Ds}, causal>", None)
            leg_s["value"] = leg_s.pop("tflops")
            leg_s["unit"] = "TFLOP/s"
            shapes[f"causal_prefill_b4_h32_n2048_d{Ds}"] = leg_s
        # masked self-attention on bf16 [B,T,H*hd] activations with an additive f32 mask [T,T] (a sliding window of 256)
        Bm, Tm, Hm, Dm, win = 4, 1024, 16, 64, 256
        rng_m = np.random.default_rng(909)
        n_m = Bm * Tm * Hm * Dm
        qm, km, vm = (oracle.f32_to_bf16(rng_m.standard_normal(n_m, dtype=np.float32)) for _ in range(3))
        ii, jj = np.arange(Tm)[:, None], np.arange(Tm)[None, :]
        bias_m = np.where((jj <= ii) & (jj > ii - win), 0.0, -1.0e4).astype(np.float32)
        d_qm, d_km, d_vm, d_bm = (ra.HipStorage.from_numpy(x) for x in (qm, km, vm, bias_m.ravel()))
        d_om = ra.HipStorage(n_m * 2)
        tmm = time_steps(hip, stream, lambda i: ra.mha_forward_masked_bf16_dev(d_qm, d_km, d_vm, d_om, Bm, Tm, Tm, Hm, Dm,
                                                                               attn_mask=d_bm, mask_len=Tm * Tm,
                                                                               stream=stream), args.steps, args.warmup)
        flops_m = 4.0 * Bm * Hm * Dm * float(Tm) * Tm  # every (query, key) pair is scored: the mask is a bias
        ach_m = flops_m / (tmm.mean_ms * 1e-3) / 1e12
        leg_m = {"value": ach_m, "unit": "TFLOP/s", "us_per_call": tmm.mean_ms * 1e3, **spread(tmm.per), **tmm.settle(),
                 "roofline": {"bound": "mfma", "achieved": ach_m, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                              "frac": ach_m / PEAK_BF16_TFLOPS, "traffic": None,
                              "kernel": "flash_tile_bf16_kernel<64, none, bias>"},
                 "config": {"workload": "bf16 masked self-attention, B=4 T=1024 H=16 hd=64 on [B,T,H*hd] tensors, additive f32 "
                                        "mask [T,T] (causal sliding window of 256 keys, -1e4 elsewhere)",
                            "flop_convention": "4*B*H*T*T*hd (the mask is a bias: every pair is scored)"}}
        if not args.no_cpu:
            got_m = oracle.bf16_to_f32(d_om.download(np.uint16)).reshape(Bm, Tm, Hm * Dm)
            want_m = oracle.mha_forward_masked(oracle.bf16_to_f32(qm), oracle.bf16_to_f32(km), oracle.bf16_to_f32(vm), Bm, Tm,
                                               Tm, Hm, Dm, attn_mask=bias_m).reshape(Bm, Tm, Hm * Dm)
            leg_m["parity_max_abs"] = float(np.abs(got_m - want_m).max())
            leg_m["parity_rel_fro"] = float(np.linalg.norm(got_m - want_m) / np.linalg.norm(want_m))
            if not (leg_m["parity_max_abs"] <= oracle.BF16_MAX_ABS and leg_m["parity_rel_fro"] <= oracle.BF16_REL_FRO):
                print(f"PARITY FAILURE: masked MHA bf16 {leg_m['parity_max_abs']} {leg_m['parity_rel_fro']}", file=sys.stderr)
                sys.exit(1)
        shapes["mha_masked_bf16_b4_t1024_h16_hd64"] = leg_m
        del d_qm, d_km, d_vm, d_bm, d_om
        # the same kind of mask without the tensor: causal sliding window of 256 keys over T = 4096
        Bw, Tw, Hw, Dw, win_w = 4, 4096, 16, 64, 256
        rng_w = np.random.default_rng(910)
        n_w = Bw * Tw * Hw * Dw
        qw_, kw_, vw_ = (oracle.f32_to_bf16(rng_w.standard_normal(n_w, dtype=np.float32)) for _ in range(3))
        d_qw, d_kw, d_vw = (ra.HipStorage.from_numpy(x) for x in (qw_, kw_, vw_))
        d_ow = ra.HipStorage(n_w * 2)
        shape_w = ra.AttentionShape.new(Bw, Hw, Tw, Dw)
        tw = time_steps(hip, stream, lambda i: ra.flash_forward_window_bf16_dev(shape_w, d_qw, d_kw, d_vw, d_ow, win_w, bnhd=True,
                                                                                stream=stream), args.steps, args.warmup)
        pairs_w = float(sum(min(i + 1, win_w) for i in range(Tw)))
        ach_w = 4.0 * Bw * Hw * Dw * pairs_w / (tw.mean_ms * 1e-3) / 1e12
        leg_w = {"value": ach_w, "unit": "TFLOP/s", "us_per_call": tw.mean_ms * 1e3, **spread(tw.per), **tw.settle(),
                 "roofline": {"bound": "mfma", "achieved": ach_w, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                              "frac": ach_w / PEAK_BF16_TFLOPS, "traffic": None,
                              "kernel": "flash_tile_bf16_kernel<64, causal, window, direct>"},
                 "config": {"workload": "bf16 causal sliding-window self-attention, B=4 T=4096 H=16 hd=64 on [B,T,H*hd] tensors, "
                                        "window 256, rt_flash_forward_window_bnhd_bf16_dev (no mask tensor)",
                            "flop_convention": "4*B*H*hd*(visible pairs): sum over i of min(i + 1, window)"}}
        if not args.no_cpu:
            got_w = oracle.bf16_to_f32(d_ow.download(np.uint16)).reshape(Bw, Tw, Hw, Dw)
            hb, hh_ = 1, 5
            q1, k1, v1 = (oracle.bf16_to_f32(x).reshape(Bw, Tw, Hw, Dw)[hb, :, hh_] for x in (qw_, kw_, vw_))
            want_w = oracle.mha_forward_masked(q1, k1, v1, 1, Tw, Tw, 1, Dw,
                                               attn_mask=oracle.sliding_window_mask(Tw, win_w)).reshape(Tw, Dw)
            leg_w["parity_max_abs"] = float(np.abs(got_w[hb, :, hh_] - want_w).max())
            leg_w["parity_rel_fro"] = oracle.rel_fro_blocks(got_w[hb, :, hh_], want_w, Dw, Tw)
            leg_w["parity_sample"] = "one (batch, head) slab against the composed path with sliding_window_mask as its bias"
            if not (leg_w["parity_max_abs"] <= oracle.BF16_MAX_ABS and leg_w["parity_rel_fro"] <= oracle.BF16_REL_FRO):
                print(f"PARITY FAILURE: window {leg_w['parity_max_abs']} {leg_w['parity_rel_fro']}", file=sys.stderr)
                sys.exit(1)
        shapes["window_bf16_b4_t4096_h16_hd64_w256"] = leg_w
        del d_qw, d_kw, d_vw, d_ow

    # ------------------------------------------------------------------ padded-batch prefill (per-sequence lengths + causal)
    padded = None
    if args.only in (None, "padded"):
        Bp, Hp, Np, Dp = 16, 16, 1024, 64
        rng_v = np.random.default_rng(33)
        lens_p = rng_v.integers(128, 1025, size=Bp).astype(np.int32)
        n_el = Bp * Hp * Np * Dp
        qb, kb, vb = (oracle.f32_to_bf16(rng_v.standard_normal(n_el, dtype=np.float32)) for _ in range(3))
        dq, dk, dv = (ra.HipStorage.from_numpy(x) for x in (qb, kb, vb))
        dout = ra.HipStorage(n_el * 2)
        dlens = ra.HipStorage.from_numpy(lens_p)
        shape_p = ra.AttentionShape.new(Bp, Hp, Np, Dp)
        tm = time_steps(hip, stream, lambda i: ra.flash_forward_varlen_bf16_dev(shape_p, dq, dk, dv, dlens, dout, True,
                                                                                stream=stream),
                        args.steps, args.warmup)
        ll = lens_p.astype(np.float64)
        flops_p = float(4.0 * Hp * Dp * (ll * (ll + 1) / 2.0).sum())  # valid (query, key) pairs only
        achieved = flops_p / (tm.mean_ms * 1e-3) / 1e12
        padded = {"metric": "prefill attn TFLOP/s", "value": flops_p / (tm.wall_ms / args.steps * 1e-3) / 1e12,
                  "unit": "TFLOP/s", "ms_per_step": tm.wall_ms / args.steps, "kernel_ms_mean": tm.mean_ms,
                  **spread(tm.per), **tm.settle(),
                  "config": {"workload": "bf16 padded-batch prefill, B=16 H=16 D=64, max N=1024, valid lengths U[128,1024] "
                                         "(seed 33), key padding + causal, padded query rows written as zeros",
                             "seq_lens": [int(x) for x in lens_p],
                             "flop_convention": "4*H*D*sum_b len_b*(len_b+1)/2 (valid pairs only)"},
                  "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                               "frac": achieved / PEAK_BF16_TFLOPS,
                               "traffic": profile_traffic("flash_tile_bf16_varlen_b16_h16_n1024_d64.md",
                                                          "flash_tile_bf16_kernel<64,causal>"),
                               "kernel": "flash_tile_bf16_kernel<64, causal, direct> (per-sequence lengths)",
                               "kernel_ms_mean": tm.mean_ms}}
        if not args.no_cpu:
            # the oracle of a sequence is the reference's causal forward on the problem truncated to its length
            got = oracle.bf16_to_f32(dout.download(np.uint16)).reshape(Bp, Hp, Np, Dp)
            q4, k4, v4 = (oracle.bf16_to_f32(x).reshape(Bp, Hp, Np, Dp) for x in (qb, kb, vb))
            err, rel, cpu_s = 0.0, 0.0, 0.0
            zeros_ok = True
            for b in range(Bp):
                L = int(lens_p[b])
                qs, ks, vs = (np.ascontiguousarray(x[b, :, :L, :]).ravel() for x in (q4, k4, v4))
                t0 = time.perf_counter()
                want = oracle.flash_forward_masked(oracle.AttentionShape(1, Hp, L, Dp), qs, ks, vs, "causal",
                                                   threads=threads).reshape(Hp, L, Dp)
                cpu_s += time.perf_counter() - t0
                err = max(err, float(np.abs(got[b, :, :L, :] - want).max()))
                rel = max(rel, oracle.rel_fro_blocks(np.ascontiguousarray(got[b, :, :L, :]), want, Dp, L))
                pad = got[b, :, L:, :]
                zeros_ok &= bool((pad.view(np.uint32) == 0).all())  # exact +0.0
            padded["parity_max_abs"] = err
            padded["parity_rel_fro"] = rel
            padded["padded_rows_exact_zero"] = zeros_ok
            padded["cpu_baseline"] = {"value": flops_p / cpu_s / 1e12, "unit": "TFLOP/s", "cores": min(threads, Hp),
                                      "kind": "port",
                                      "sample": f"the whole workload once ({cpu_s:.2f} s): per sequence the reference's "
                                                f"causal forward on the problem truncated to its length, one task per "
                                                f"head; every tile computed, valid-pair FLOPs counted"}
            if not (err <= oracle.BF16_MAX_ABS and rel <= oracle.BF16_REL_FRO and zeros_ok):
                print(f"PARITY FAILURE: padded prefill max-abs {err}, relative Frobenius error per 256-row block {rel}, "
                      f"zero rows {zeros_ok}", file=sys.stderr)
                sys.exit(1)
        del dq, dk, dv, dout, dlens

    # ------------------------------------------------------------------ decode
    decode = None
    if args.only in (None, "decode"):
        Bd, Hq, Hkv, Dd, Lmax = 64, 32, 8, 128, 8192
        lens = np.random.default_rng(4).integers(512, 8193, size=Bd).astype(np.int32)
        n_cache = Bd * Hkv * Lmax * Dd
        kc = np.empty(n_cache, dtype=np.uint16)
        vc = np.empty(n_cache, dtype=np.uint16)
        step = n_cache // 16
        for i in range(16):
            kc[i * step:(i + 1) * step] = oracle.f32_to_bf16(rng.standard_normal(step, dtype=np.float32))
            vc[i * step:(i + 1) * step] = oracle.f32_to_bf16(rng.standard_normal(step, dtype=np.float32))
        qd = oracle.f32_to_bf16(rng.standard_normal(Bd * Hq * Dd, dtype=np.float32))
        # rotate over several copies of the cache so that a step never finds its keys in the 256 MB
        # last-level cache left there by the previous step
        n_sets = 3
        sets = [(ra.HipStorage.from_numpy(kc), ra.HipStorage.from_numpy(vc)) for _ in range(n_sets)]
        d_q = ra.HipStorage.from_numpy(qd)
        d_lens = ra.HipStorage.from_numpy(lens)
        d_o = ra.HipStorage(Bd * Hq * Dd * 2)
        ws_bytes = K.gqa_decode_workspace_bytes(Bd, Hq, Hkv, Dd, Lmax)
        ws = ra.HipStorage(max(ws_bytes, 256))

        def launch(i):
            k_, v_ = sets[i % n_sets]
            K.gqa_decode_batched_bf16(stream, d_q, k_, v_, d_o, d_lens, Bd, Hq, Hkv, Dd, Lmax, ws, ws.byte_len)

        tm = time_steps(hip, stream, launch, args.steps, args.warmup)
        alg_bytes = float(lens.astype(np.int64).sum()) * 2 * Hkv * Dd * 2 + Bd * Hq * Dd * 2 * 2
        ms_kernel = tm.mean_ms
        decode = {"metric": "decode attn HBM GB/s", "value": alg_bytes / (tm.wall_ms / args.steps * 1e-3) / 1e9,
                  "unit": "GB/s", "ms_per_step": tm.wall_ms / args.steps, "kernel_ms_mean": ms_kernel,
                  **spread(tm.per), **tm.settle(),
                  "algorithmic_bytes": alg_bytes,
                  "config": {"workload": "bf16 GQA decode, batch 64, 32 q / 8 kv heads, D=128, ctx U[512,8192] "
                                         "(seed 4), cache (B,Hkv,Lmax=8192,D)", "sum_len": int(lens.sum()),
                             "cache_sets_rotated": n_sets},
                  "roofline": {"bound": "hbm", "achieved": alg_bytes / (ms_kernel * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                               "unit": "GB/s", "frac": alg_bytes / (ms_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS,
                               "traffic": profile_traffic("decode_split_b64_hq32_hkv8_d128_ctx512-8192.md", "decode_step"),
                               "kernels": "decode_split + decode_merge (one event pair around the timed steps)"}}
        # the reference's own call: one sequence per launch (LlmKernels::gqa_decode_online_bf16), back to back on the
        # stream as a decode loop issues it, on sequence 0's cache
        single = {}
        d_o1 = ra.HipStorage(Hq * Dd * 2)
        for kv_len in (512, 2048, 8192):
            t1 = time_steps(hip, stream,
                            lambda i: K.gqa_decode_online_bf16(stream, d_q, sets[i % n_sets][0], sets[i % n_sets][1], d_o1,
                                                               Hq, Hkv, kv_len, Dd, Lmax),
                            args.steps, args.warmup, spread_steps=0)
            single[str(kv_len)] = {"us_per_call": t1.mean_ms * 1e3,
                                   "GB/s": (2 * Hkv * kv_len * Dd * 2 + 2 * Hq * Dd * 2) / (t1.mean_ms * 1e-3) / 1e9}
        decode["single_sequence"] = dict(single, note="rt_gqa_decode_online_bf16, 32 q / 8 kv heads, D=128: two launches "
                                                      "per call, issued back to back from the host")
        # several new positions of ONE sequence against its long cache, each causal to itself (the reference's
        # gqa_decode_batched_f32 call shape): the keys are cut into spans, a second kernel folds the partials.  Every
        # call reads another sequence's slab of the rotated caches (192 slabs of 34 MB), so none finds its keys in
        # the last-level cache.
        chunk = {}
        slab_bytes = Hkv * Lmax * Dd * 2
        for s_new in (4, 16):
            q_c = oracle.f32_to_bf16(np.random.default_rng(90 + s_new).standard_normal(s_new * Hq * Dd, dtype=np.float32))
            d_qc = ra.HipStorage.from_numpy(q_c)
            d_oc = ra.HipStorage(s_new * Hq * Dd * 2)

            def launch_chunk(i, d_qc=d_qc, d_oc=d_oc, s_new=s_new):
                k_, v_ = sets[(i // Bd) % n_sets]
                off = (i % Bd) * slab_bytes
                K.gqa_decode_chunk_bf16(stream, d_qc, k_.ptr + off, v_.ptr + off, d_oc, Lmax, 1, s_new, Hq, Hkv, Dd, Lmax)

            tc = time_steps(hip, stream, launch_chunk, args.steps, args.warmup)
            bytes_c = float(2 * Hkv * Lmax * Dd * 2 + 2 * s_new * Hq * Dd * 2)
            leg_c = {"us_per_call": tc.mean_ms * 1e3, **spread(tc.per), **tc.settle(), "algorithmic_bytes": bytes_c,
                     "roofline": {"bound": "hbm", "achieved": bytes_c / (tc.mean_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                                  "unit": "GB/s", "frac": bytes_c / (tc.mean_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                  "traffic": profile_traffic("chunk_decode_b1_hq32_hkv8_d128_ctx8192.md", f"chunk_{s_new}"),
                                  "kernels": "flash_tile_bf16_kernel<128, causal, packed, split, direct> + flash_split_merge_kernel "
                                             "(one event pair around the timed calls)"}}
            if not args.no_cpu:
                K.gqa_decode_chunk_bf16(stream, d_qc, sets[0][0], sets[0][1], d_oc, Lmax, 1, s_new, Hq, Hkv, Dd, Lmax)
                hip.sync()
                got_c = oracle.bf16_to_f32(d_oc.download(np.uint16))
                n_slab = Hkv * Lmax * Dd
                t0 = time.perf_counter()
                want_c = oracle.gqa_decode_chunk_bf16(q_c, kc[:n_slab], vc[:n_slab], [Lmax], 1, s_new, Hq, Hkv, Dd, Lmax,
                                                      threads=threads)
                cpu_c = time.perf_counter() - t0
                err_c = float(np.abs(got_c - want_c).max())
                rel_c = oracle.rel_fro_blocks(got_c, want_c, Dd, block_rows=1, min_elems=64)
                leg_c["parity_max_abs"], leg_c["parity_rel_fro"] = err_c, rel_c
                leg_c["cpu_baseline"] = {"value": bytes_c / cpu_c / 1e9, "unit": "GB/s", "cores": min(threads, Hq),
                                         "kind": "port",
                                         "sample": f"one call ({cpu_c * 1e3:.0f} ms): the shader's four phases per (position, "
                                                   f"head), one task per head; K and V are read once per query head and "
                                                   f"position there, once per kv head in the byte count"}
                if not (err_c <= oracle.BF16_MAX_ABS and rel_c <= oracle.BF16_REL_FRO):
                    print(f"PARITY FAILURE: chunk decode seq_new={s_new} max-abs {err_c}, relative {rel_c}", file=sys.stderr)
                    sys.exit(1)
            chunk[str(s_new)] = leg_c
        decode["chunk_decode"] = dict(chunk, config={"workload": "bf16 chunked causal decode of one sequence: batch 1, 32 q / 8 kv "
                                                                 "heads, D=128, seq_new new positions (4, 16) over a cache "
                                                                 "that holds 8192 keys with them (pos_base = 8192 - seq_new), "
                                                                 "rt_gqa_decode_chunk_bf16 with a host length"})
        # ---- the step ahead of decode attention (q/k RMSNorm + RoPE + cache append, one launch): a decode step of
        # the batch, and a prompt of the headline shape
        prep = {}
        rope_p = ra.RoPE(Dd, Lmax)
        rope_p.device_tables()
        d_g = ra.HipStorage.from_numpy(np.ones(Dd, dtype=np.float32) + 0.01 * np.arange(Dd, dtype=np.float32) / Dd)
        for name, (pb, pseq) in (("decode_step", (Bd, 1)), ("prompt", (4, 4096))):
            rng_r = np.random.default_rng(4242 + pseq)
            pq = oracle.f32_to_bf16(rng_r.standard_normal(pb * Hq * pseq * Dd, dtype=np.float32))
            pk, pv = (oracle.f32_to_bf16(rng_r.standard_normal(pb * Hkv * pseq * Dd, dtype=np.float32)) for _ in range(2))
            d_pq, d_pk, d_pv = (ra.HipStorage.from_numpy(x) for x in (pq, pk, pv))
            k_, v_ = sets[0]  # (pb sequences of the first cache set: positions 0 .. pseq - 1 are overwritten)
            launch_p = lambda i: K.qk_norm_rope_kv_append_bf16(stream, d_pq, d_pk, d_pv, k_, v_, 0, rope_p, pb, Hq, Hkv, Dd,
                                                               Lmax, q_gamma=d_g, k_gamma=d_g, seq=pseq)
            tp = time_steps(hip, stream, launch_p, args.steps, args.warmup)
            bytes_p = float(pb * pseq * Dd * 2 * (2 * Hq + 4 * Hkv))  # q in and out, k and v in, two cache rows out
            leg_p = {"us_per_call": tp.mean_ms * 1e3, **spread(tp.per), **tp.settle(), "algorithmic_bytes": bytes_p,
                     "roofline": {"bound": "hbm", "achieved": bytes_p / (tp.mean_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                                  "unit": "GB/s", "frac": bytes_p / (tp.mean_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                  "traffic": profile_traffic("prepare_hq32_hkv8_d128.md", name),
                                  "kernel": "prompt_prepare_kernel<64, 128>" if pseq >= 32 else "decode_prepare_kernel"}}
            if not args.no_cpu:
                # q is rewritten in place: a fresh copy of the inputs, one call, every bit against the oracle
                d_pq.upload(pq)
                launch_p(0)
                hip.sync()
                kc_w = np.zeros(pb * Hkv * pseq * Dd, dtype=np.uint16)  # the oracle's cache holds the new rows only
                vc_w = np.zeros_like(kc_w)
                oro_p = oracle.RoPE(Dd, Lmax)
                oro_p.cos, oro_p.sin = rope_p.cos.copy(), rope_p.sin.copy()
                g_host = d_g.download(np.float32)
                t0 = time.perf_counter()
                want_q = oracle.decode_prepare_bf16(pq, pk, pv, kc_w, vc_w, np.zeros(pb, dtype=np.int32), g_host, g_host, 1e-6,
                                                    oro_p, pb, Hq, Hkv, Dd, pseq, seq=pseq)
                cpu_p = time.perf_counter() - t0
                got_q = d_pq.download(np.uint16)
                got_kc = k_.download(np.uint16, pb * Hkv * Lmax * Dd).reshape(pb * Hkv, Lmax, Dd)[:, :pseq]
                got_vc = v_.download(np.uint16, pb * Hkv * Lmax * Dd).reshape(pb * Hkv, Lmax, Dd)[:, :pseq]
                same = (np.array_equal(got_q, want_q) and np.array_equal(got_kc, kc_w.reshape(pb * Hkv, pseq, Dd))
                        and np.array_equal(got_vc, vc_w.reshape(pb * Hkv, pseq, Dd)))
                leg_p["parity_bit_exact"] = bool(same)
                leg_p["cpu_baseline"] = {"value": bytes_p / cpu_p / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                         "sample": f"the whole call once ({cpu_p * 1e3:.0f} ms), single-threaded loops as in "
                                                   f"the reference's decode_step"}
                if not same:
                    print(f"PARITY FAILURE: prepare ({name}) differs from the oracle's bits", file=sys.stderr)
                    sys.exit(1)
            prep[name] = leg_p
            del d_pq, d_pk, d_pv
        decode["prepare"] = dict(prep, config={"workload": "rt_qk_norm_rope_kv_append_bf16, 32 q / 8 kv heads, D=128, both "
                                                           "gammas: decode_step = batch 64, one new token each; prompt = "
                                                           "batch 4, 4096 new tokens each at position 0"})
        if not args.no_cpu:
            got = oracle.bf16_to_f32(d_o.download(np.uint16))
            t0 = time.perf_counter()
            want = oracle.gqa_decode_batched_bf16(qd, kc, vc, lens, Bd, Hq, Hkv, Dd, Lmax, threads=threads)
            cpu_s = time.perf_counter() - t0
            err = float(np.abs(got - want).max())
            rel = oracle.rel_fro_blocks(got, want, Dd, block_rows=1, min_elems=64)  # per (sequence, head) row
            decode["parity_max_abs"] = err
            decode["parity_rel_fro"] = rel
            decode["cpu_baseline"] = {"value": alg_bytes / cpu_s / 1e9, "unit": "GB/s", "cores": threads,
                                      "kind": "port",
                                      "sample": f"the whole decode step once ({cpu_s:.1f} s): trim + decode_attn_row "
                                                f"per (sequence, kv head) task, f32 on bf16-rounded inputs; the "
                                                f"reference runs seq_q = 1 on a single thread"}
            if not (err <= oracle.BF16_MAX_ABS and rel <= oracle.BF16_REL_FRO):
                print(f"PARITY FAILURE: decode max-abs {err}, relative Frobenius error per row {rel}", file=sys.stderr)
                sys.exit(1)

    # ------------------------------------------------------------------ f32 prefill, the reference's own CPU-runnable case
    f32 = None
    if args.only in (None, "f32"):
        Bf, Hf, Nf, Df = 1, 8, 2048, 64
        rng_f = np.random.default_rng(77)
        qf, kf, vf = (rng_f.standard_normal(Bf * Hf * Nf * Df, dtype=np.float32) for _ in range(3))
        dqf, dkf, dvf = (ra.HipStorage.from_numpy(x) for x in (qf, kf, vf))
        dof = ra.HipStorage(Bf * Hf * Nf * Df * 4)
        shape_f = ra.AttentionShape.new(Bf, Hf, Nf, Df)
        causal_f = ra.Mask.causal()
        tm = time_steps(hip, stream, lambda i: ra.flash_forward_f32_dev(shape_f, dqf, dkf, dvf, dof, causal_f, stream=stream),
                        args.steps, args.warmup)
        flops_f = 4.0 * Bf * Hf * Df * (Nf * (Nf + 1) / 2.0)
        f32 = {"metric": "f32 prefill attn TFLOP/s", "value": flops_f / (tm.wall_ms / args.steps * 1e-3) / 1e12,
               "unit": "TFLOP/s", "ms_per_step": tm.wall_ms / args.steps, "kernel_ms_mean": tm.mean_ms, **spread(tm.per),
               **tm.settle(),
               "config": {"workload": "f32 causal flash-attention forward, B=1 H=8 N=2048 D=64, N(0,1) inputs (seed 77), "
                                      "tensors resident in HBM", "flop_convention": "4*B*H*D*N*(N+1)/2 (causal-counted)"},
               "roofline": {"bound": "mfma", "achieved": flops_f / (tm.mean_ms * 1e-3) / 1e12, "peak": PEAK_F32_TFLOPS,
                            "unit": "TFLOP/s", "frac": flops_f / (tm.mean_ms * 1e-3) / 1e12 / PEAK_F32_TFLOPS,
                            "traffic": profile_traffic("flash_fwd_f32_b1_h8_n2048_d64.md", "flash_fwd_f32_splitk_kernel<2,exact,causal>"), "kernel": "flash_fwd_f32_splitk_kernel<2, exact, causal>"}}
        if not args.no_cpu:
            got = dof.download(np.float32)
            oracle.flash_forward_masked(oracle.AttentionShape(Bf, Hf, Nf, Df), qf, kf, vf, "causal", threads=threads)  # warm
            reps = 5
            t0 = time.perf_counter()
            for _ in range(reps):
                want = oracle.flash_forward_masked(oracle.AttentionShape(Bf, Hf, Nf, Df), qf, kf, vf, "causal",
                                                   threads=threads)
            cpu_s = (time.perf_counter() - t0) / reps
            err = float(np.abs(got - want).max())
            f32["parity_max_abs"] = err
            f32["parity_rel_fro"] = oracle.rel_fro_blocks(got, want, Df, Nf)
            f32["cpu_baseline"] = {"value": flops_f / cpu_s / 1e12, "unit": "TFLOP/s", "cores": min(threads, Bf * Hf),
                                   "kind": "port",
                                   "sample": f"the whole workload, mean of {reps} runs ({cpu_s * 1e3:.0f} ms each): one task "
                                             f"per (b,h) slab as rayon does, so at most B*H = 8 threads work; every tile "
                                             f"computed, causal-counted FLOPs, as in the reference"}
            if not err <= 1e-5:
                print(f"PARITY FAILURE: f32 prefill max-abs {err}", file=sys.stderr)
                sys.exit(1)
        del dqf, dkf, dvf, dof

    # ------------------------------------------------------------------ f32 backward on the same shape (unmasked, as the reference's)
    bwd = None
    if args.only in (None, "bwd"):
        Bb, Hb, Nb, Db = 1, 8, 2048, 64
        rng_b = np.random.default_rng(78)
        n_b = Bb * Hb * Nb * Db
        host = [rng_b.uniform(-1.0, 1.0, n_b).astype(np.float32) for _ in range(4)]  # q, k, v, dO
        d_in = [ra.HipStorage.from_numpy(x) for x in host]
        d_g = [ra.HipStorage(n_b * 4) for _ in range(3)]
        shape_b = ra.AttentionShape.new(Bb, Hb, Nb, Db)
        ws_b = ra.flash_backward_workspace_bytes(shape_b)
        d_ws = ra.HipStorage(ws_b)
        tm = time_steps(hip, stream, lambda i: ra.flash_backward_f32_dev(shape_b, *d_in, *d_g, d_ws, ws_b, stream=stream),
                        args.steps, args.warmup)
        flops_b = 10.0 * Bb * Hb * Db * float(Nb) * Nb
        # the same gradients from a saved forward (O and m + ln l kept from the forward pass): no recomputation
        d_o, d_lse = ra.HipStorage(n_b * 4), ra.HipStorage(Bb * Hb * Nb * 4)
        ra.flash_forward_stats_f32_dev(shape_b, d_in[0], d_in[1], d_in[2], d_o, d_lse, stream=stream)
        tm_saved = time_steps(hip, stream,
                              lambda i: ra.flash_backward_saved_f32_dev(shape_b, d_in[0], d_in[1], d_in[2], d_o, d_lse,
                                                                        d_in[3], *d_g, d_ws, ws_b, stream=stream),
                              args.steps, args.warmup, spread_steps=0)
        bwd = {"metric": "f32 attention backward TFLOP/s", "value": flops_b / (tm.wall_ms / args.steps * 1e-3) / 1e12,
               "unit": "TFLOP/s", "ms_per_step": tm.wall_ms / args.steps, "kernel_ms_mean": tm.mean_ms, **spread(tm.per),
               **tm.settle(),
               "saved_forward": {"kernel_ms_mean": tm_saved.mean_ms, "tflops": flops_b / (tm_saved.mean_ms * 1e-3) / 1e12,
                                 "note": "rt_flash_backward_saved_f32_dev: O and the row statistic come from the forward "
                                         "pass instead of being recomputed (dQ, which also forms delta, then dK/dV)"},
               "config": {"workload": "f32 unmasked attention backward (dQ, dK, dV from Q, K, V, dO), B=1 H=8 N=2048 D=64, "
                                      "U(-1,1) inputs (seed 78), tensors resident in HBM",
                          "flop_convention": "10*B*H*N*N*D: the five N x N x D products of the backward; the step also "
                                             "re-runs the forward (2 products) and computes the scores twice (7 products "
                                             "in the two backward kernels), none of which is counted"},
               "roofline": {"bound": "mfma", "achieved": flops_b / (tm.mean_ms * 1e-3) / 1e12, "peak": PEAK_F32_TFLOPS,
                            "unit": "TFLOP/s", "frac": flops_b / (tm.mean_ms * 1e-3) / 1e12 / PEAK_F32_TFLOPS,
                            "traffic": profile_traffic("flash_bwd_f32_b1_h8_n2048_d64.md", "backward_step"),
                            "kernels": "flash_fwd_f32_splitk_kernel<2> + flash_bwd_f32_dq_kernel<2> (with the delta prologue) "
                                       "+ flash_bwd_f32_dkdv_kernel<2> (one event pair around the timed steps)"}}
        if not args.no_cpu:
            n_slab = Bb * Hb  # the reference's backward is a single-threaded loop; the whole workload is a second or two
            slab = Nb * Db
            t0 = time.perf_counter()
            want = oracle.flash_backward(oracle.AttentionShape(1, n_slab, Nb, Db), *[x[:n_slab * slab] for x in host])
            cpu_s = time.perf_counter() - t0
            got = [g.download(np.float32)[:n_slab * slab] for g in d_g]
            err = max(float(np.abs(a - b).max()) for a, b in zip(got, want))
            bwd["parity_max_abs"] = err
            bwd["parity_rel_fro"] = max(oracle.rel_fro_blocks(a, b, Db, Nb) for a, b in zip(got, want))
            bwd["cpu_baseline"] = {"value": flops_b * n_slab / (Bb * Hb) / cpu_s / 1e12, "unit": "TFLOP/s", "cores": 1,
                                   "kind": "port",
                                   "sample": f"{n_slab} of the {Bb * Hb} (b,h) slabs once ({cpu_s:.1f} s), the reference's "
                                             f"single-threaded loops with full N x N matrices; the same slabs are the "
                                             f"parity sample"}
            if not err <= 2e-5:
                print(f"PARITY FAILURE: f32 backward max-abs {err}", file=sys.stderr)
                sys.exit(1)
        del d_in, d_g, d_ws

    tail = dict(n_gpus=1, steps=args.steps, warmup=args.warmup, higher_is_better=True, data="synthetic",
                vs_baseline=None, scaling="weak")
    if prefill is None:  # --only <one of the other legs>: that leg is the line
        leg, dtype = next((x, t) for x, t in ((decode, "bf16"), (long_p, "bf16"), (padded, "bf16"), (d64_p, "bf16"),
                                              (shapes, "bf16"), (f32, "f32"), (bwd, "f32")) if x is not None)
        print(json.dumps(dict(leg, dtype=dtype, **tail)))
        return
    sustained = None if args.no_ceiling else sustained_mfma()
    out = {
        "metric": "prefill attn TFLOP/s (% bf16 MFMA peak); decode attn HBM GB/s (% peak)",
        "value": prefill["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": prefill["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "settle_ms": prefill["settle_ms"], "settle_launches": prefill["settle_launches"],
        "config": {"workload": "bf16 causal prefill attention, B=4 H=32 N=4096 D=128, N(0,1) inputs (seed 1234), "
                               "f32 accumulation", "flop_convention": "4*B*H*D*N*(N+1)/2 (causal-counted)",
                   "tflops_unmasked_convention_4BHN2D": prefill["tflops_unmasked_convention"],
                   "settle": f"every leg first launches its own step until {SETTLE_MS:.0f} ms of device time have "
                             f"passed (settle_ms, settle_launches), then runs the counted warm-up and the timed steps"},
        "roofline": prefill["roofline"],
    }
    if sustained is not None:
        # context for `frac`: under load the power limit, not the 2.4 GHz of the data sheet, sets the clock
        out["roofline"]["sustained_mfma"] = dict(sustained,
                                                 frac_of_sustained=prefill["roofline"]["achieved"] / sustained["tflops"])
    if "cpu_baseline" in prefill:
        out["cpu_baseline"] = prefill["cpu_baseline"]
        out["parity_max_abs"] = prefill["parity_max_abs"]
        out["parity_rel_fro"] = prefill["parity_rel_fro"]
    for key, leg in (("decode", decode), ("padded_prefill", padded), ("long_prefill", long_p), ("d64_prefill", d64_p),
                     ("other_shapes", shapes), ("f32_prefill", f32), ("f32_backward", bwd)):
        if leg is not None:
            out[key] = leg
    print(json.dumps(out))


if __name__ == "__main__":
    main()
