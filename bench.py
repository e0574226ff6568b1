#!/usr/bin/env python3
"""Benchmark of the ring-step attention hot path on one MI355X.  Prints ONE JSON line.

Headline workload = benchmark config 3: bf16, B=1, S=8192 in P=8 chunks of 1024, H=32, D=128,
causal; every rank's Q chunk against its prefix of KV chunks in ring order (8 diagonal + 28 full
block pairs), cast at the end.  One "step" is that whole 36-pair sweep; inputs are resident in
HBM before the timed region.  value = causal-adjusted TFLOP/s of the sweep (549.76 GFLOP / step).

The sweep runs through the C entry point spa_ring_fwd in three schedules, same (out, lse):
  all   ONE launch for the sweep: every rank's workgroups are in one grid; a workgroup keeps its
        query tile and accumulators in registers and walks its rank's KV chunks in ring order, so
        the merge of ring steps is the online softmax itself.  A one-GPU fusion (the eight ranks of
        a real ring are eight GPUs).  This is `value`.
  rank  one launch per rank: what one GPU of a ring runs when its KV chunks are resident.
  step  one launch per (rank, ring step), the running (out, lse) in HBM, the update_out_and_lse
        merge in the kernel's epilogue: what a rank runs while chunks arrive over the wire.
  rank_flags  (other_schedules, ring_step.flag_driven_tflops) the `rank` launches with a bounded wait for a
        per-chunk arrival flag before a chunk's first tile is loaded (spa_ring_fwd_flags): the other way to run while
        chunks arrive - one launch per rank, accumulators in registers across ring steps.
`other_schedules` holds rank and step; `ring_step` repeats the step figure as the per-ring-step
number; `roofline` carries both again as `rank_tflops` / `step_tflops`.  The line is kept below
7.5 KB (long texts live in this docstring and in ROW_NOTES, not in the line), with `rows` ahead of
`other_schedules`, `ring_step` and `protocol`, so that a reader who keeps only the end of the
output still has them; the host's core counts appear once, as `host`.

Timing protocol.  (1) settle: the same launch repeated in groups of 10 until the median of a group
is within 2 % of the median of the group before it (40 launches at least), or 0.3 s have passed (after an idle period the
first ~40 launches run 5-25 % slower while the power management answers the load step; reported
as `settle_launches`, `settle_ms`, `settle_ended_by` = "converged" or "cap", `cold_ms_per_step` =
mean of the first 5 launches).  (2) `--warmup` untimed steps.  (3) the timed
region: blocks of exactly `--steps` steps, each block bracketed by events on the launch stream and
a synchronize, repeated until >= 0.2 s are covered; `ms_per_step` is the MEDIAN block
(`timed_blocks`, `block_ms_min`, `block_ms_max` beside it).

`roofline` is for the dominant kernel, the block attention forward: algorithmic FLOPs per launch
/ its average launch duration, measured here with events over the timed region (in the `all`
schedule a step is one launch of that kernel and nothing else).  `rows` carries the other rows of
the path (configs 1, 2, 4, 5, merge), each with its own roofline and cpu_baseline.
`cpu_baseline` legs time the oracle's restatement of the reference's op sequence (SDPA for out +
a second q k^T / logsumexp for lse, sp_aurora/intel_flash_attn_optimized.py:156-193; sigmoid /
logsigmoid merge, sp_aurora/utils.py:103-104; reshape / transpose / contiguous re-layout,
sp_aurora/intel_ulysses_attn.py:95-138) on the host cores: 2 warm-up + 5 timed, median.

`--workload` prints a single row instead (profiling runs: one kernel family per trace).
Two helper modes for the HBM traffic figure (roofline.traffic):
  --traffic-leg          additionally runs a plain device copy of known size, so that a
                         `rocprofv3 --pmc FETCH_SIZE` (or WRITE_SIZE) run of this script holds
                         both the attention kernel and a calibration kernel
  --pmc-summary F W      reads the two counter_collection.csv files of such runs and writes
                         profiles/flash_fwd_traffic.json (no GPU needed)
  --pmc-summary-rows F W the same for the re-layout and merge kernels, from two runs of
                         `--workload hbm --traffic-leg`: writes profiles/hbm_rows_traffic.json
`--transient` prints, instead of the benchmark, the per-launch durations of the first 120 launches
after 3 s of idle together with the clock and board power read from sysfs (what the settle phase
is for).
"""
import argparse
import csv
import glob
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_FP8_BF16_MIX_PEAK_TFLOPS = 3333.3  # half the FLOPs at the fp8 rate (5000), half at the bf16 rate (2500)
HBM_PEAK_GBPS = 8000.0

B, S, H, D, P = 1, 8192, 32, 128, 8
SEED = 2
INPUT_SCALE = 0.5
COPY_BYTES = 1 << 30  # calibration copy of the traffic leg: reads and writes this many bytes
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "flash_fwd_traffic.json")
ROWS_TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_rows_traffic.json")  # the same for the HBM-bound rows
MIN_TIMED_S = 0.2
MAX_BLOCKS = 200


def sweep_flops():
    s = S // P
    full = 4.0 * B * H * s * s * D
    n_diag, n_full = P, P * (P - 1) // 2
    return n_full * full + n_diag * full / 2, n_diag + n_full, full


def algorithmic_bytes():
    """Bytes the sweep must move: per block pair its K and V chunk in (36 pairs: on a real ring
    they are 36 kernel inputs on 8 GPUs), per rank its Q chunk in, out and lse out."""
    chunk = B * (S // P) * H * D * 2
    n_pairs = P + P * (P - 1) // 2
    return n_pairs * 2 * chunk + P * chunk + P * chunk + B * H * S * 4


def rand_tensors(torch, shape, seed, n, scale=1.0, dtype=None, device=None):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n):
        t = torch.randn(shape, generator=g, dtype=torch.float32) * scale
        t = t.to(dtype or torch.bfloat16)
        out.append(t.to(device) if device is not None else t)
    return out


# ------------------------------------------------------------------------------------ GPU timing
def timed_block(torch, fn, iters):
    """ms per call over exactly `iters` calls, events on the current (= launch) stream."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def settle(torch, fn, max_s=0.3, need=10, tol=0.02, min_launches=40):
    """Repeats fn in groups of `need` launches until the median of a group is within `tol` of the
    median of the group before it (and at least min_launches have run: the slow stretch after an
    idle period lasts about 30), or max_s have passed.
    Returns (launches, ms spent, mean ms of the first 5 launches, "converged" | "cap")."""
    t0 = time.perf_counter()
    times = []
    prev = None
    while True:
        chunk = []
        for _ in range(need):
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            chunk.append((a, b))
        torch.cuda.synchronize()
        last = [a.elapsed_time(b) for a, b in chunk]
        times += last
        med = statistics.median(last)
        spent = time.perf_counter() - t0
        if prev is not None and len(times) >= min_launches and abs(med - prev) <= tol * prev:
            ended = "converged"
            break
        if spent >= max_s:
            ended = "cap"
            break
        prev = med
    return len(times), spent * 1e3, sum(times[:5]) / min(5, len(times)), ended


def measure(torch, fn, steps, warmup, min_s=MIN_TIMED_S, do_settle=True):
    """The protocol of the module docstring for one callable.  Returns a dict."""
    res = {}
    if do_settle:
        n, ms, cold, ended = settle(torch, fn)
        res.update(settle_launches=n, settle_ms=round(ms, 2), settle_ended_by=ended, cold_ms_per_step=round(cold, 4))
    for _ in range(warmup):
        fn()
    blocks = []
    covered = 0.0
    while covered < min_s and len(blocks) < MAX_BLOCKS:
        t = timed_block(torch, fn, steps)
        blocks.append(t)
        covered += t * steps * 1e-3
    res.update(ms_per_step=statistics.median(blocks), timed_blocks=len(blocks), block_ms_min=round(min(blocks), 4),
               block_ms_max=round(max(blocks), 4), timed_region_s=round(covered, 3))
    return res


# ------------------------------------------------------------------------------------ CPU baseline
def host_threads():
    """Threads for the CPU legs: every core this process may run on, bounded by the share the
    environment assigns through OMP_NUM_THREADS when it sets one."""
    logical = os.cpu_count() or 1
    try:
        affinity = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        affinity = logical
    physical = None
    try:
        cores = set()
        phys = core = None
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":")[1].strip()
            elif line.startswith("core id"):
                core = line.split(":")[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    cores.add((phys, core))
                phys = core = None
        physical = len(cores) or None
    except OSError:
        pass
    env = os.environ.get("OMP_NUM_THREADS")
    used = affinity
    if env and env.isdigit() and int(env) > 0:
        used = min(used, int(env))
    return used, {"logical": logical, "physical": physical, "affinity": affinity, "omp_num_threads_env": env}


def cpu_time(fn, warm=2, timed=5):
    for _ in range(warm):
        fn()
    ts = []
    for _ in range(timed):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts)


class CpuLegs:
    """The reference's op sequence per row on the host cores (oracle restatements, fp32 torch;
    bf16 inputs are up-cast to fp32: no fast bf16 GEMM is assumed on the host).  `sample` texts are
    short on purpose (the whole line must stay below 7.5 KB); what each leg runs:
      pairs   one diagonal and one full block pair [B,H,s,D] through torch CPU SDPA plus a second
              q k^T / logsumexp for the lse, median of 5 after 2 warm-up, extrapolated to the row's
              pair counts (d = diagonal, f = full)
      full    the row's whole workload, median of 5 (re-layout: of 3)
      backward  the same pairs through torch CPU autograd of softmax(q k^T) v (forward recompute
              included, as in the reference), median of 3, 5-GEMM FLOP count"""

    def __init__(self, torch):
        from oracle import attn_oracle as O
        self.torch, self.O = torch, O
        self.threads, self.host = host_threads()
        torch.set_num_threads(self.threads)
        self.host["torch_num_threads"] = torch.get_num_threads()
        self._pair_cache = {}

    def _entry(self, value, unit, sample, kind="port"):
        return {"value": float(f"{value:.4g}"), "unit": unit, "cores": self.threads, "kind": kind, "sample": sample}

    def pair_times(self, Bn, Hn, sn, Dn, seed):
        """seconds for one diagonal and one full block pair [Bn,Hn,sn,Dn] (SDPA + second QK^T/logsumexp)."""
        key = (Bn, Hn, sn, Dn)
        if key not in self._pair_cache:
            torch, O = self.torch, self.O
            q, k, v = rand_tensors(torch, (Bn, Hn, sn, Dn), seed, 3, INPUT_SCALE)
            f = lambda causal: O.attn_block_sdpa(q, k, v, None, causal, compute_dtype=torch.float32)
            self._pair_cache[key] = (cpu_time(lambda: f(True)), cpu_time(lambda: f(False)))
        return self._pair_cache[key]

    def ring_forward(self, Bn, Hn, sn, Dn, n_diag, n_full, seed):
        """Extrapolation from one measured diagonal and one measured full pair."""
        t_d, t_f = self.pair_times(Bn, Hn, sn, Dn, seed)
        full = 4.0 * Bn * Hn * sn * sn * Dn
        flops = n_full * full + n_diag * full / 2
        secs = n_diag * t_d + n_full * t_f
        return self._entry(flops / secs / 1e12, "TFLOP/s",
                           f"pairs [B{Bn},H{Hn},s{sn},D{Dn}]: 1 d {t_d * 1e3:.0f} ms + 1 f {t_f * 1e3:.0f} ms measured, x {n_diag} d + {n_full} f = {secs * 1e3:.0f} ms")

    def config1(self):
        torch, O = self.torch, self.O
        q, k, v = rand_tensors(torch, (1, 8, 512, 64), 0, 3, 1.0, torch.float32)
        t = cpu_time(lambda: O.attn_block_sdpa(q, k, v, 0.125, False, compute_dtype=torch.float32))
        return self._entry(4.0 * 8 * 512 * 512 * 64 / t / 1e12, "TFLOP/s", f"full: {t * 1e3:.2f} ms")

    def config2(self):
        """Rank 2 of the P=4 ring in full: 3 block pairs + 1 init, 2 merges (sigmoid / logsigmoid form)."""
        torch, O = self.torch, self.O
        Bn, Hn, sn, Dn = 2, 32, 1024, 64
        q, = rand_tensors(torch, (Bn, Hn, sn, Dn), 1, 1)
        ks = rand_tensors(torch, (Bn, Hn, sn, Dn), 11, 3)
        vs = rand_tensors(torch, (Bn, Hn, sn, Dn), 12, 3)

        def run():
            out = lse = None
            for t, c in enumerate((2, 1, 0)):
                bo, bl = O.attn_block_sdpa(q, ks[c], vs[c], None, t == 0, compute_dtype=torch.float32)
                if out is None:
                    out, lse = bo.float(), bl.unsqueeze(-1)
                else:
                    out, lse = O.merge(out, lse, bo, bl.unsqueeze(-1))
            return out.to(torch.bfloat16), lse

        t = cpu_time(run)
        flops = 2.5 * 4.0 * Bn * Hn * sn * sn * Dn
        return self._entry(flops / t / 1e12, "TFLOP/s", f"full (3 pairs + merges): {t * 1e3:.0f} ms")

    def relayout(self):
        torch, O = self.torch, self.O
        x, = rand_tensors(torch, (8, 1, 2048, 32, 128), 3, 1)
        xs = list(x)
        t_s2h = cpu_time(lambda: O.all_to_all_4d_s2h(xs), 1, 3)
        ys = O.all_to_all_4d_s2h(xs)
        t_h2s = cpu_time(lambda: O.all_to_all_4d_h2s(ys), 1, 3)
        nbytes = 2 * x.numel() * 2
        mk = lambda t: self._entry(nbytes / t / 1e9, "GB/s", f"full (reshape/transpose/contiguous chain): {t * 1e3:.0f} ms")
        return mk(t_s2h), mk(t_h2s)

    def merge(self):
        torch, O = self.torch, self.O
        g = torch.Generator().manual_seed(3)
        acc = torch.randn((1, 32, 1024, 128), generator=g)
        lse = torch.randn((1, 32, 1024, 1), generator=g)
        blk = torch.randn((1, 32, 1024, 128), generator=g).to(torch.bfloat16)
        bl = torch.randn((1, 32, 1024, 1), generator=g)
        t = cpu_time(lambda: O.merge(acc, lse, blk.float(), bl))
        return self._entry((acc.numel() * 10 + lse.numel() * 12) / t / 1e9, "GB/s", f"full (sigmoid/logsigmoid form): {t * 1e3:.1f} ms")

    def backward(self, n_diag, n_full):
        torch, O = self.torch, self.O
        q, k, v, do = rand_tensors(torch, (1, 2048, 16, 128), 4, 4)
        f = lambda causal: O.attn_backward_autograd(q, k, v, do, None, causal, compute_dtype=torch.float32)
        t_d = cpu_time(lambda: f(True), 1, 3)
        t_f = cpu_time(lambda: f(False), 1, 3)
        full = 2.5 * 4.0 * 16 * 2048 * 2048 * 128
        secs = n_diag * t_d + n_full * t_f
        return self._entry((n_full * full + n_diag * full / 2) / secs / 1e12, "TFLOP/s",
                           f"backward pairs [1,2048,16,128]: 1 d {t_d * 1e3:.0f} ms + 1 f {t_f * 1e3:.0f} ms measured, x {n_diag} d + {n_full} f = {secs:.1f} s")


# ------------------------------------------------------------------------------------ rows
# What each row of `rows` runs (the line itself carries a short `workload` only).
ROW_NOTES = {
    "config1_fp32_block_forward": "config 1: fp32 B=1 S=512 H=8 D=64 non-causal block forward, out + lse (flash_fwd32_splitk_kernel<64,8>)",
    "config2_ring_rank2_of_4": "config 2: bf16 B=2 S=4096 (P=4 chunks of 1024) H=32 D=64 causal, rank 2: diagonal chunk 2, then chunks 1, 0, "
                               "merged; value = one launch for the rank, step_tflops = one launch per ring step (3 launches)",
    "config3_zigzag_ring": "config 3 tensors with zigzag sharding (rank r holds half-chunks r and 15-r): every rank runs 1 diagonal "
                           "block [1024 x 1024], r blocks [1024 x 512] and 7-r blocks [512 x 1024]; same 549.76 GFLOP; value = one launch "
                           "per rank, step_tflops = one launch per (rank, step)",
    "config4_relayout_s2h": "config 4 re-layout: [P=8,B=1,s=2048,H=32,D=128] bf16 -> [8,1,16384,4,128], one tensor per launch, q / k / v in "
                            "turn (nothing cache-resident), recorded calls replayed (ops.prepared); host cost of the call included",
    "config4_relayout_h2s": "the inverse of config4_relayout_s2h",
    "config4_ulysses_forward": "config 4: 3 re-layouts in, full causal attention per head group [8,1,16384,4,128], 1 re-layout out, output "
                               "allocation included; views_tflops = the same result with head groups read and written in place (B = 1)",
    "block_forward_fp8": "causal block forward over the config-3 sequence [1,8192,32,128] as one call, q, K, V all e4m3 + fp32 scale per "
                         "(batch, head), out bf16: scores on the 8-bit matrix instruction (spa_flash_fwd_fp8qkv), P V on the 16-bit one; "
                         "peak = the mix of the two rates for equal FLOPs, 2 / (1/5000 + 1/2500); kv_only_tflops = bf16 q with e4m3 K / V "
                         "(spa_flash_fwd_fp8kv, both contractions 16-bit), bf16_tflops = the same call with bf16 q, K, V; "
                         "ring_rank_tflops / ring_step_tflops = the config-3 ring sweep (P = 8) on the e4m3 tensors, one launch per rank / "
                         "per (rank, step) (spa_ring_fwd_fp8qkv); ring_flags_tflops = one launch per rank that waits for each chunk's arrival "
                         "flag, all raised beforehand (spa_ring_fwd_flags_fp8qkv)",
    "merge_update_out_and_lse": "update_out_and_lse: merge of a bf16 block into the fp32 running (out, lse) of one config-3 rank "
                                "[1,1024,32,128], 8 operand sets in turn, recorded calls replayed; host cost of the call included",
    "config5_ring_forward": "config 5 forward: bf16 qkv [1,32768,3,16,128] (strided views) causal, ring of 16 chunks of 2048, 16 diagonal + "
                            "120 full pairs; value = schedule all, rank_tflops / step_tflops = 16 / 136 launches",
    "config5_ring_backward": "config 5 backward: dq/dk/dv by block-wise recompute with the global lse over the same 136 block pairs, one launch "
                             "per kernel, delta pre-pass and output allocation included, gradients written in bf16 (spa_flash_bwd_out); "
                             "5-GEMM FLOP count (the two kernels execute 7); step_tflops = one launch pair per block pair into fp32 "
                             "accumulators (spa_flash_bwd), zero-fill and final casts included",
}

# name -> (short workload text, unit, roofline bound, kernel, peak, extra config keys)
ROW_SPECS = {
    "config1_fp32_block_forward": ("config 1: fp32 [1,512,8,64] block forward", "TFLOP/s", "mfma", "flash_fwd32_splitk<64,8>", MFMA_F32_PEAK_TFLOPS, ()),
    "config2_ring_rank2_of_4": ("config 2: bf16 D=64, rank 2 of P=4, 1 launch", "TFLOP/s", "mfma", "flash_fwd16<bf16,64>", MFMA_BF16_PEAK_TFLOPS,
                                ("step_tflops",)),
    "config3_zigzag_ring": ("config 3, zigzag shards, 1 launch per rank", "TFLOP/s", "mfma", "flash_fwd16<bf16,128>", MFMA_BF16_PEAK_TFLOPS,
                            ("step_tflops", "all_tflops")),
    "config4_relayout_s2h": ("config 4 re-layout s2h, 268 MB per launch", "GB/s", "hbm", "relayout<16,s2h>", HBM_PEAK_GBPS, ()),
    "config4_relayout_h2s": ("config 4 re-layout h2s, 268 MB per launch", "GB/s", "hbm", "relayout<16,h2s>", HBM_PEAK_GBPS, ()),
    "config4_ulysses_forward": ("config 4: 3 re-layouts, attention, 1 re-layout", "TFLOP/s", "mfma", "relayout x4 + flash_fwd16<bf16,128>",
                                MFMA_BF16_PEAK_TFLOPS, ("views_tflops",)),
    "block_forward_fp8": ("causal block forward [1,8192,32,128], e4m3 q/K/V, 8-bit scores", "TFLOP/s", "mfma", "flash_fwd16<bf16,128,e4m3 q/K/V>",
                          MFMA_FP8_BF16_MIX_PEAK_TFLOPS, ("kv_only_tflops", "bf16_tflops", "ring_rank_tflops", "ring_step_tflops", "ring_flags_tflops")),
    "merge_update_out_and_lse": ("merge of a bf16 block [1,1024,32,128] into fp32 (out, lse), 42.3 MB", "GB/s", "hbm", "merge<bf16>",
                                 HBM_PEAK_GBPS, ()),
    "config5_ring_forward": ("config 5 forward, P=16, 1 launch", "TFLOP/s", "mfma", "flash_fwd16<bf16,128>", MFMA_BF16_PEAK_TFLOPS,
                             ("rank_tflops", "step_tflops")),
    "config5_ring_backward": ("config 5 backward, 1 launch per kernel, 5-GEMM count", "TFLOP/s", "mfma", "flash_bwd_dq + flash_bwd_dkdv",
                              MFMA_BF16_PEAK_TFLOPS, ("step_tflops",)),
}


# Rows that `--workload` can print and the default line leaves out (the line is short of room).
EXTRA_ROW_NOTES = {
    "decode_key_split": "a decode step against a long cache: bf16 q [1,1,32,128] (one new token) x K, V [1,32768,32,128], no mask; the keys "
                        "are cut into chunks that run side by side (spa_flash_fwd_splitkv, as many as the library suggests) on the kernel "
                        "that streams K and V past up to three query rows; value = K and V bytes per call time; plain_gbps = the same call "
                        "as one launch of 32 workgroups (spa_flash_fwd); mfma_gbps = the split call on the matrix-instruction kernels "
                        "(spa_tune few_rows = 1); e4m3_gbps / e4m3_mfma_gbps = the two on an e4m3 cache (half the bytes per key); "
                        "q128_tflops = the split call with 128 query rows",
}
EXTRA_ROW_SPECS = {
    "decode_key_split": ("decode: q [1,1,32,128] x K/V [1,32768,32,128] bf16, keys split", "GB/s", "hbm", "fewrows_fwd<bf16,128,1 row>",
                         HBM_PEAK_GBPS, ("plain_gbps", "mfma_gbps", "e4m3_gbps", "e4m3_mfma_gbps", "q128_tflops", "chunks")),
}


def make_row(name, ms_per_step, value, **extra):
    """One entry of `rows` (without cpu_baseline) from the table above."""
    workload, unit, bound, kernel, peak, keys = (ROW_SPECS.get(name) or EXTRA_ROW_SPECS[name])
    if set(extra) != set(keys):
        raise KeyError(f"{name}: expected extras {keys}, got {sorted(extra)}")
    cfg = {"workload": workload}
    cfg.update({k2: round(v2, 2) for k2, v2 in extra.items()})
    return {"row": name, "value": round(value, 2), "unit": unit, "ms_per_step": round(ms_per_step, 4), "config": cfg,
            "roofline": {"bound": bound, "achieved": round(value, 2), "peak": peak, "unit": unit,
                         "frac": round(value / peak, 4), "traffic": row_traffic(name)}}  # (the kernel's name stays in ROW_SPECS: the line is short of room)


def _lib_mod():
    from sp_aurora_amd import _lib
    return _lib


_ROW_TRAFFIC = None


def row_traffic(name):
    """HBM bytes per launch of a row's kernel as recorded by --pmc-summary-rows, or None."""
    global _ROW_TRAFFIC
    if _ROW_TRAFFIC is None:
        try:
            _ROW_TRAFFIC = json.load(open(ROWS_TRAFFIC_JSON))
        except (OSError, ValueError):
            _ROW_TRAFFIC = {}
    t = _ROW_TRAFFIC.get(name, {}).get("hbm_bytes_per_launch")
    return round(t) if t else None


def tfl(flops, m):
    return flops / (m["ms_per_step"] * 1e-3) / 1e12


def gpu_rows(torch, spa, ops, which, steps, warmup):
    """GPU legs of the side rows.  Returns {name: row-dict without cpu_baseline}."""
    dev = torch.device("cuda:0")
    rows = {}
    light = dict(min_s=0.05, do_settle=False)

    def finish(name, m, value, **extra):
        rows[name] = make_row(name, m["ms_per_step"], value, **extra)

    if "config1" in which:
        q, k, v = rand_tensors(torch, (1, 512, 8, 64), 0, 3, 1.0, torch.float32, dev)
        out = torch.empty_like(q)
        lse = torch.empty((1, 8, 512), dtype=torch.float32, device=dev)
        fn = lambda: ops.flash_fwd(q, k, v, 0.125, False, layout="bshd", out=out, lse=lse)
        m = measure(torch, fn, 20, 5, **light)
        tf = tfl(4.0 * 8 * 512 * 512 * 64, m)
        finish("config1_fp32_block_forward", m, tf)
    if "config2" in which:
        Bn, Sn, Hn, Dn, Pn, r = 2, 4096, 32, 64, 4, 2
        q, k, v = rand_tensors(torch, (Bn, Sn, Hn, Dn), 1, 3, 1.0, torch.bfloat16, dev)
        out = torch.empty_like(q)
        lse = torch.empty((Bn, Hn, Sn), dtype=torch.float32, device=dev)
        ws = ops.ring_fwd_workspace(q, Pn)
        flops = 2.5 * 4.0 * Bn * Hn * (Sn // Pn) ** 2 * Dn
        sched = {}
        for fuse in ("step", "rank"):
            fn = lambda fuse=fuse: ops.ring_fwd(q, k, v, Pn, None, True, rank=r, out=out, lse=lse, workspace=ws, fuse=fuse)
            sched[fuse] = measure(torch, fn, 20, 5, **light)
        m = sched["rank"]
        tf = tfl(flops, m)
        finish("config2_ring_rank2_of_4", m, tf, step_tflops=tfl(flops, sched["step"]))
    if "zigzag" in which and hasattr(spa.ring, "zigzag_order"):
        q, k, v = rand_tensors(torch, (B, S, H, D), SEED, 3, INPUT_SCALE, torch.bfloat16, dev)
        order = spa.ring.zigzag_order(S, P, dev)
        q, k, v = [t.index_select(1, order).contiguous() for t in (q, k, v)]
        total, _, _ = sweep_flops()
        sched = {}
        for fuse in ("step", "rank", "all"):
            f = spa.ring.make_ring_forward_step(q, k, v, D ** -0.5, True, P, fuse=fuse, sharding="zigzag")
            f()
            sched[fuse] = measure(torch, f, 20, 5, **light)
        m = sched["rank"]
        tf = tfl(total, m)
        finish("config3_zigzag_ring", m, tf, step_tflops=tfl(total, sched["step"]), all_tflops=tfl(total, sched["all"]))
        del q, k, v
    if "config4" in which:
        Pn, Bn, sn, Hn, Dn = 8, 1, 2048, 32, 128
        q, k, v = rand_tensors(torch, (Pn, Bn, sn, Hn, Dn), 3, 3, 1.0, torch.bfloat16, dev)
        # q, k, v take turns (and so do three destinations): 805 MB in flight, so that a launch finds
        # neither its source nor its destination in the 256 MB memory-side cache
        xs = [q, k, v]
        ys = [torch.empty((Pn, Bn, Pn * sn, Hn // Pn, Dn), dtype=q.dtype, device=dev) for _ in range(3)]
        backs = [torch.empty_like(q) for _ in range(3)]
        nbytes = 2 * q.numel() * 2
        turn = [0]

        # recorded once, replayed in the timed loop (ops.prepared: the library's path for tight loops)
        s2h_runs = [ops.prepared(ops.relayout_s2h, xs[i], Pn, out=ys[i])[0] for i in range(3)]
        h2s_runs = [ops.prepared(ops.relayout_h2s, ys[i], Pn, out=backs[i])[0] for i in range(3)]

        def s2h():
            i = turn[0] = (turn[0] + 1) % 3
            s2h_runs[i]()

        def h2s():
            i = turn[0] = (turn[0] + 1) % 3
            h2s_runs[i]()

        for name, fn in (("s2h", s2h), ("h2s", h2s)):
            m = measure(torch, fn, 21, 6, **light)
            gb = nbytes / (m["ms_per_step"] * 1e-3) / 1e9
            finish(f"config4_relayout_{name}", m, gb)
        y = ys[0]
        del ys, backs
        scale = Dn ** -0.5
        fn = lambda: spa.intel_ulysses_flash_attn_forward(None, q, k, v, scale, causal=True, relayout="kernels")
        fn()
        m = measure(torch, fn, 5, 2, **light)
        flops = 4.0 * Bn * Hn * (Pn * sn) ** 2 * Dn / 2
        tf = tfl(flops, m)
        # the same result with head groups read and written in place (B = 1: no re-layout pass at all)
        fv = lambda: spa.intel_ulysses_flash_attn_forward(None, q, k, v, scale, causal=True, relayout="views")
        fv()
        mv = measure(torch, fv, 5, 2, **light)
        finish("config4_ulysses_forward", m, tf, views_tflops=tfl(flops, mv))
        del q, k, v, y, xs
    if "fp8kv" in which:
        # the config-3 sequence as one causal block call, K / V in e4m3 with per-head scales, against
        # the same call with bf16 K / V (same kernel family, direct-to-LDS tiles)
        Bn, Sn, Hn, Dn = 1, 8192, 32, 128
        q, k, v = rand_tensors(torch, (Bn, Sn, Hn, Dn), SEED, 3, INPUT_SCALE, torch.bfloat16, dev)
        q8, qsc = ops.quantize_fp8_per_head(q)
        k8, ksc = ops.quantize_fp8_per_head(k)
        v8, vsc = ops.quantize_fp8_per_head(v)
        out = torch.empty_like(q)
        lse = torch.empty((Bn, Hn, Sn), dtype=torch.float32, device=dev)
        flops = 4.0 * Bn * Hn * Sn * Sn * Dn / 2
        f8 = lambda: ops.flash_fwd(q8, k8, v8, None, True, out=out, lse=lse, q_scale=qsc, k_scale=ksc, v_scale=vsc)
        f8kv = lambda: ops.flash_fwd(q, k8, v8, None, True, out=out, lse=lse, k_scale=ksc, v_scale=vsc)
        f16 = lambda: ops.flash_fwd(q, k, v, None, True, out=out, lse=lse)
        m16 = measure(torch, f16, 20, 5, **light)
        mkv = measure(torch, f8kv, 20, 5, **light)
        m = measure(torch, f8, 20, 5, **light)
        tf = tfl(flops, m)
        # the config-3 ring sweep itself with e4m3 q / K / V, one launch per rank and per (rank, step)
        ws = ops.ring_fwd_workspace(q8, P, out_dtype=torch.bfloat16)
        ring8 = {}
        for fuse in ("rank", "step"):
            fr = lambda fuse=fuse: ops.ring_fwd(q8, k8, v8, P, None, True, out=out, lse=lse, workspace=ws, fuse=fuse, q_scale=qsc,
                                                k_scale=ksc, v_scale=vsc)
            ring8[fuse] = tfl(flops, measure(torch, fr, 20, 5, **light))
        flags8 = ops.RingFlags(P, dev)
        flags8.set_all()
        ff = lambda: ops.ring_fwd_flags(q8, k8, v8, P, flags8, None, True, out=out, lse=lse, q_scale=qsc, k_scale=ksc, v_scale=vsc)
        ring8["flags"] = tfl(flops, measure(torch, ff, 20, 5, **light))
        if flags8.failed():
            raise RuntimeError("bench.py: a wave of the flag-driven e4m3 ring gave up waiting with every flag raised")
        finish("block_forward_fp8", m, tf, kv_only_tflops=tfl(flops, mkv), bf16_tflops=tfl(flops, m16),
               ring_rank_tflops=ring8["rank"], ring_step_tflops=ring8["step"], ring_flags_tflops=ring8["flags"])
        del q, k, v, q8, k8, v8
    if "merge" in which:
        Bn, sn, Hn, Dn = 1, 1024, 32, 128
        g = torch.Generator().manual_seed(3)
        NSET = 8  # 8 x 42 MB in turn: a launch finds none of its operands in the 256 MB memory-side cache
        sets = []
        for _ in range(NSET):
            acc = torch.randn((Bn, sn, Hn, Dn), generator=g, dtype=torch.float32).to(dev)
            lse = torch.randn((Bn, Hn, sn), generator=g, dtype=torch.float32).to(dev)
            blk = torch.randn((Bn, sn, Hn, Dn), generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
            blk_lse = torch.randn((Bn, Hn, sn), generator=g, dtype=torch.float32).to(dev)
            sets.append(ops.prepared(ops.merge, acc, lse, blk, blk_lse, layout="bshd")[0])
        turn = [0]

        def fn():
            i = turn[0] = (turn[0] + 1) % NSET
            sets[i]()

        m = measure(torch, fn, 24, 8, **light)
        nbytes = Bn * sn * Hn * Dn * 10 + Bn * Hn * sn * 12
        gb = nbytes / (m["ms_per_step"] * 1e-3) / 1e9
        finish("merge_update_out_and_lse", m, gb)
        del sets
    if "decode" in which:
        Bn, Hn, Skn, Dn = 1, 32, 32768, 128
        k, v = rand_tensors(torch, (Bn, Skn, Hn, Dn), 7, 2, 1.0, torch.bfloat16, dev)
        k8, ksc = ops.quantize_fp8_per_head(k.float())
        v8, vsc = ops.quantize_fp8_per_head(v.float())
        kv_bytes = 2.0 * Bn * Skn * Hn * Dn * 2
        res = {}
        for sq in (1, 128):
            (q,) = rand_tensors(torch, (Bn, sq, Hn, Dn), 8, 1, 1.0, torch.bfloat16, dev)
            out = torch.empty_like(q)
            lse = torch.empty((Bn, Hn, sq), dtype=torch.float32, device=dev)
            n = _lib_mod().load().spa_flash_fwd_splitkv_suggest(Bn, Hn, sq, Skn, Dn, 0, 1)
            ws = ops.flash_fwd_splitkv_workspace(q, max(n, 1))
            f_split = lambda: ops.flash_fwd(q, k, v, None, False, out=out, lse=lse, split_kv=n, workspace=ws)
            f_plain = lambda: ops.flash_fwd(q, k, v, None, False, out=out, lse=lse, split_kv=None)
            f_e4m3 = lambda: ops.flash_fwd(q, k8, v8, None, False, out=out, lse=lse, k_scale=ksc, v_scale=vsc, split_kv=n, workspace=ws)
            res[sq] = [n, measure(torch, f_split, 20, 5, **light), measure(torch, f_plain, 20, 5, **light), measure(torch, f_e4m3, 20, 5, **light)]
            if sq == 1:
                _lib_mod().tune("few_rows", 1)
                try:
                    res[sq] += [measure(torch, f_split, 20, 5, **light), measure(torch, f_e4m3, 20, 5, **light)]
                finally:
                    _lib_mod().tune("few_rows", 0)
        n1, m_split, m_plain, m_e4, m_mfma, m_e4_mfma = res[1]
        gbps = lambda nbytes, m: nbytes / (m["ms_per_step"] * 1e-3) / 1e9
        finish("decode_key_split", m_split, gbps(kv_bytes, m_split), plain_gbps=gbps(kv_bytes, m_plain), mfma_gbps=gbps(kv_bytes, m_mfma),
               e4m3_gbps=gbps(kv_bytes / 2, m_e4), e4m3_mfma_gbps=gbps(kv_bytes / 2, m_e4_mfma),
               q128_tflops=tfl(4.0 * Bn * Hn * 128 * Skn * Dn, res[128][1]), chunks=n1)
        del k, v, k8, v8
    if "config5" in which:
        Bn, Sn, Hn, Dn, Pn = 1, 32768, 16, 128, 16
        qkv, = rand_tensors(torch, (Bn, Sn, 3, Hn, Dn), 4, 1, 1.0, torch.bfloat16, dev)
        dout, = rand_tensors(torch, (Bn, Sn, Hn, Dn), 5, 1, 1.0, torch.bfloat16, dev)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        scale = Dn ** -0.5
        fstep = spa.ring.make_ring_forward_step(q, k, v, scale, True, Pn, fuse="all")
        out, lse = fstep()
        m = measure(torch, fstep, 3, 1, **light)
        fwd_flops = 4.0 * Bn * Hn * Sn * Sn * Dn / 2
        tf = tfl(fwd_flops, m)
        sched5 = {}
        for fuse in ("rank", "step"):
            f5 = spa.ring.make_ring_forward_step(q, k, v, scale, True, Pn, fuse=fuse)
            f5()
            sched5[fuse] = tfl(fwd_flops, measure(torch, f5, 3, 1, **light))
            del f5
        finish("config5_ring_forward", m, tf, rank_tflops=sched5["rank"], step_tflops=sched5["step"])
        fn = lambda: spa.ring.ring_flash_attn_backward(dout, q, k, v, out, lse, scale, True, Pn, fuse="all")
        fn()
        m = measure(torch, fn, 3, 1, **light)
        bwd_flops = 2.5 * fwd_flops
        tf = tfl(bwd_flops, m)
        fs = lambda: spa.ring.ring_flash_attn_backward(dout, q, k, v, out, lse, scale, True, Pn, fuse="step")
        fs()
        ms_ = measure(torch, fs, 2, 1, **light)
        finish("config5_ring_backward", m, tf, step_tflops=tfl(bwd_flops, ms_))
        del qkv, dout, out, lse
    torch.cuda.empty_cache()
    return rows


def attach_cpu(rows, cpu):
    """cpu_baseline per row (host legs run after every GPU leg, so they do not sit between launches)."""
    if "config1_fp32_block_forward" in rows:
        rows["config1_fp32_block_forward"]["cpu_baseline"] = cpu.config1()
    if "config2_ring_rank2_of_4" in rows:
        rows["config2_ring_rank2_of_4"]["cpu_baseline"] = cpu.config2()
    if "config3_zigzag_ring" in rows:
        # the same 36 block pairs' worth of work as config 3 (zigzag only reorders them)
        rows["config3_zigzag_ring"]["cpu_baseline"] = cpu.ring_forward(B, H, S // P, D, P, P * (P - 1) // 2, SEED)
    if "config4_relayout_s2h" in rows:
        a, b = cpu.relayout()
        rows["config4_relayout_s2h"]["cpu_baseline"] = a
        rows["config4_relayout_h2s"]["cpu_baseline"] = b
        # attention of one head group [1,4,16384,128] as 2048-row blocks (x 8 groups: same ratio); re-layouts not included
        rows["config4_ulysses_forward"]["cpu_baseline"] = cpu.ring_forward(1, 4, 2048, 128, 8, 28, 3)
    if "block_forward_fp8" in rows:
        # the same attention with dequantised q / K / V as 1024-row blocks (the reference has no 8-bit path)
        rows["block_forward_fp8"]["cpu_baseline"] = cpu.ring_forward(1, 32, 1024, 128, 8, 28, SEED)
    if "merge_update_out_and_lse" in rows:
        rows["merge_update_out_and_lse"]["cpu_baseline"] = cpu.merge()
    if "config5_ring_forward" in rows:
        rows["config5_ring_forward"]["cpu_baseline"] = cpu.ring_forward(1, 16, 2048, 128, 16, 120, 4)
        rows["config5_ring_backward"]["cpu_baseline"] = cpu.backward(16, 120)


# ------------------------------------------------------------------------------------ post-idle transient
def transient(torch, spa, idle_s=3.0, launches=120):
    """Per-launch durations of the config-3 `all` sweep after an idle period, with the shader
    clock and board power the driver reports (sysfs) sampled alongside.  One JSON line."""
    import threading

    def find(pattern):
        r = sorted(glob.glob(pattern))
        return r[0] if r else None

    f_sclk = find("/sys/class/drm/card*/device/pp_dpm_sclk")
    f_pow = find("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") or find("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average")

    def rd(path):
        try:
            return open(path).read()
        except OSError:
            return ""

    dev = torch.device("cuda:0")
    q, k, v = rand_tensors(torch, (B, S, H, D), SEED, 3, INPUT_SCALE, torch.bfloat16, dev)
    step = spa.ring.make_ring_forward_step(q, k, v, D ** -0.5, True, P, fuse="all")
    step()
    torch.cuda.synchronize()
    time.sleep(idle_s)
    samples, stop = [], []

    def sampler():
        while not stop:
            t = time.perf_counter()
            act = [l for l in rd(f_sclk).splitlines() if l.rstrip().endswith("*")] if f_sclk else []
            mhz = int("".join(ch for ch in act[0].split(":")[1] if ch.isdigit())) if act else None
            pw = rd(f_pow).strip() if f_pow else ""
            samples.append((t, mhz, int(pw) / 1e6 if pw.isdigit() else None))
            time.sleep(0.002)

    th = threading.Thread(target=sampler)
    th.start()
    time.sleep(0.03)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(launches):
        step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    time.sleep(0.03)
    stop.append(1)
    th.join()
    us = [round(ev[i].elapsed_time(ev[i + 1]) * 1e3, 1) for i in range(launches)]
    print(json.dumps({"workload": "config 3, schedule all: one launch per sweep", "idle_s": idle_s, "us_per_launch": us,
                      "samples_ms_mhz_watt": [(round((t - t0) * 1e3, 1), m, w) for t, m, w in samples]}))


# ------------------------------------------------------------------------------------ traffic helper
def calibration_copy(torch, dev):
    """A plain device copy of COPY_BYTES: what FETCH_SIZE / WRITE_SIZE read for it scales the kernels' readings."""
    src = torch.empty(COPY_BYTES, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def pmc_summary(fetch_dir, write_dir):
    """FETCH_SIZE / WRITE_SIZE (KiB per dispatch) of the attention kernel, each scaled by what the
    same counter reads for the calibration copy of COPY_BYTES."""
    def read(d, counter):
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit(f"no counter_collection.csv under {d}")
        attn, copy = [], []
        for f in files:
            for row in csv.DictReader(open(f)):
                if row.get("Counter_Name") != counter:
                    continue
                name, val = row["Kernel_Name"], float(row["Counter_Value"])
                if "flash_fwd16_kernel" in name:
                    attn.append(val)
                elif "copy" in name.lower() or "elementwise" in name.lower():
                    copy.append(val)
        if not attn or not copy:
            raise SystemExit(f"{counter}: attention or calibration kernel missing in {d}")
        copy_kib = max(copy)  # the 1 GiB copy dwarfs any other elementwise kernel of the run
        return sum(attn) / len(attn), copy_kib, len(attn)

    f_attn, f_copy, n = read(fetch_dir, "FETCH_SIZE")
    w_attn, w_copy, _ = read(write_dir, "WRITE_SIZE")
    f_factor = (COPY_BYTES / 1024.0) / f_copy   # true KiB per counted KiB
    w_factor = (COPY_BYTES / 1024.0) / w_copy
    fetch_b = f_attn * f_factor * 1024.0
    write_b = w_attn * w_factor * 1024.0
    res = {
        "kernel": "flash_fwd16_kernel<bf16,128,2>, config 3, schedule all (one launch per sweep)",
        "dispatches_averaged": n,
        "fetch_size_kib_per_dispatch": f_attn,
        "write_size_kib_per_dispatch": w_attn,
        "copy_fetch_size_kib": f_copy,
        "copy_write_size_kib": w_copy,
        "copy_bytes": COPY_BYTES,
        "fetch_factor": f_factor,
        "write_factor": w_factor,
        "hbm_fetch_bytes_per_launch": fetch_b,
        "hbm_write_bytes_per_launch": write_b,
        "hbm_bytes_per_launch": fetch_b + write_b,
        "algorithmic_bytes_per_launch": algorithmic_bytes(),
    }
    json.dump(res, open(TRAFFIC_JSON, "w"), indent=1)
    print(json.dumps(res, indent=1))


def pmc_summary_rows(fetch_dir, write_dir):
    """The same for the kernels of the HBM-bound rows (two runs of `--workload hbm --traffic-leg`): FETCH_SIZE and
    WRITE_SIZE per dispatch, each scaled by the calibration copy of the same run."""
    kernels = {"config4_relayout_s2h": ("relayout_kernel<16, true>", 268435456),
               "config4_relayout_h2s": ("relayout_kernel<16, false>", 268435456),
               "merge_update_out_and_lse": ("merge_kernelIDF16bLb0E", 42336256),  # (the profiler leaves bf16 names mangled)
               "decode_key_split": ("fewrows_fwd_kernelIDF16bLi128ELb0ELi1ELi4ELb1E", 2 * 32768 * 32 * 128 * 2)}  # K and V once

    def read(d, counter):
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit(f"no counter_collection.csv under {d}")
        per, copy = {n: [] for n in kernels}, []
        for f in files:
            for row in csv.DictReader(open(f)):
                if row.get("Counter_Name") != counter:
                    continue
                name, val = row["Kernel_Name"], float(row["Counter_Value"])
                for n, (pat, _) in kernels.items():
                    if pat in name:
                        per[n].append(val)
                if "copybuffer" in name.lower():
                    copy.append(val)
        if not copy or not all(per.values()):
            raise SystemExit(f"{counter}: a kernel or the calibration copy is missing in {d}")
        return per, max(copy)

    f_per, f_copy = read(fetch_dir, "FETCH_SIZE")
    w_per, w_copy = read(write_dir, "WRITE_SIZE")
    f_factor, w_factor = (COPY_BYTES / 1024.0) / f_copy, (COPY_BYTES / 1024.0) / w_copy
    res = {"copy_bytes": COPY_BYTES, "copy_fetch_size_kib": f_copy, "copy_write_size_kib": w_copy, "fetch_factor": f_factor, "write_factor": w_factor}
    for n, (_, alg) in kernels.items():
        fa, wa = statistics.median(f_per[n]), statistics.median(w_per[n])
        res[n] = {"dispatches": len(f_per[n]), "fetch_size_kib_per_dispatch": fa, "write_size_kib_per_dispatch": wa,
                  "hbm_fetch_bytes_per_launch": fa * f_factor * 1024.0, "hbm_write_bytes_per_launch": wa * w_factor * 1024.0,
                  "hbm_bytes_per_launch": (fa * f_factor + wa * w_factor) * 1024.0, "algorithmic_bytes_per_launch": alg}
    json.dump(res, open(ROWS_TRAFFIC_JSON, "w"), indent=1)
    print(json.dumps(res, indent=1))


# ------------------------------------------------------------------------------------ main
ROW_SETS = {"fp8kv": {"fp8kv"}, "relayout": {"config4"}, "ulysses": {"config4"}, "merge": {"merge"}, "backward": {"config5"},
            "config1": {"config1"}, "config2": {"config2"}, "zigzag": {"zigzag"}, "hbm": {"config4", "merge", "decode"}, "decode": {"decode"}}
ALL_ROWS = {"config1", "config2", "zigzag", "config4", "fp8kv", "merge", "config5"}
LINE_LIMIT = 7500  # bytes of the printed line: readers that keep only the end of the output keep 8 KB


def assemble_line(steps, warmup, head, m_head, other, rows, cpu_head, host, traffic, traffic_src):
    """The JSON line from the measurements (a pure function: tests build it from made-up numbers).
    Key order matters: `rows` come before `other_schedules`, `ring_step` and `protocol`."""
    total_flops, n_pairs, _ = sweep_flops()
    ms = m_head["ms_per_step"]
    tflops = total_flops / (ms * 1e-3) / 1e12
    launches = {"all": 1, "rank": P, "step": n_pairs}[head]
    roofline = {
        "bound": "mfma", "kernel": "flash_fwd16_kernel<bf16,128,2>", "achieved": round(tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
        "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic, "traffic_source": traffic_src,
        "avg_launch_us": round(ms * 1e3 / launches, 2), "flops_per_launch": total_flops / launches, "launches_per_step": launches,
        "algorithmic_bytes_per_launch": algorithmic_bytes() / launches,
    }
    for name in ("rank", "step"):
        if name in other:
            roofline[name + "_tflops"] = other[name]["tflops"]
            roofline[name + "_frac"] = round(other[name]["tflops"] / MFMA_BF16_PEAK_TFLOPS, 4)
    line = {
        "metric": "fwd attn TFLOP/s + % bf16 MFMA peak, ring-step causal S=8K H32 D128",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"config 3: simulated ring P=8, bf16 [1,8192,32,128] causal, 8 diagonal + 28 full block pairs, schedule '{head}'",
            "flops_per_step": total_flops,
            "block_pairs": n_pairs,
        },
        "pct_of_bf16_mfma_peak": round(100.0 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
        "roofline": roofline,
    }
    if cpu_head is not None:
        line["cpu_baseline"] = cpu_head
    if host is not None:
        line["host"] = host
    if rows:
        line["rows"] = list(rows.values())
    line["other_schedules"] = other
    if "step" in other:
        line["ring_step"] = {"what": "one launch per (rank, ring step), merge in the last step's epilogue",
                             "tflops": other["step"]["tflops"], "pct_of_bf16_mfma_peak": other["step"]["pct_of_bf16_mfma_peak"],
                             "avg_launch_us": other["step"]["avg_launch_us"]}
        if "rank_flags" in other:
            line["ring_step"]["flag_driven_tflops"] = other["rank_flags"]["tflops"]
    line["protocol"] = {k2: m_head[k2] for k2 in ("settle_launches", "settle_ms", "settle_ended_by", "cold_ms_per_step", "timed_blocks",
                                                  "block_ms_min", "block_ms_max", "timed_region_s") if k2 in m_head}
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline legs")
    ap.add_argument("--no-rows", action="store_true", help="headline only (profiling runs)")
    ap.add_argument("--only-all", action="store_true", help="skip the rank / step schedules (profiling runs)")
    ap.add_argument("--schedule", default="all", choices=["all", "rank", "step"],
                    help="which schedule --only-all runs (profiling runs); `value` is always the `all` schedule otherwise")
    ap.add_argument("--traffic-leg", action="store_true", help="also run the calibration copy (for --pmc runs)")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"))
    ap.add_argument("--pmc-summary-rows", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="the same for the re-layout and merge kernels (runs of --workload hbm --traffic-leg): writes profiles/hbm_rows_traffic.json")
    ap.add_argument("--transient", action="store_true",
                    help="instead of the benchmark: per-launch durations of the first 120 launches after 3 s of idle, with clock / power samples")
    ap.add_argument("--workload", default="config3", choices=["config3"] + sorted(ROW_SETS))
    args = ap.parse_args()
    if args.pmc_summary:
        pmc_summary(*args.pmc_summary)
        return
    if args.pmc_summary_rows:
        pmc_summary_rows(*args.pmc_summary_rows)
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU (the ring is simulated on it, no collectives); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import sp_aurora_amd as spa
    from sp_aurora_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.transient:
        transient(torch, spa)
        return
    if args.workload != "config3":
        rows = gpu_rows(torch, spa, ops, ROW_SETS[args.workload], args.steps, args.warmup)
        if args.traffic_leg:
            calibration_copy(torch, dev)
        if not args.no_cpu_baseline:
            attach_cpu(rows, CpuLegs(torch))
        print(json.dumps({"rows": list(rows.values())}))
        return

    q, k, v = rand_tensors(torch, (B, S, H, D), SEED, 3, INPUT_SCALE, torch.bfloat16, dev)
    scale = D ** -0.5
    total_flops, n_pairs, full_flops = sweep_flops()

    # preallocated buffers, no allocation per step
    steps = {m: spa.ring.make_ring_forward_step(q, k, v, scale, True, P, fuse=m) for m in ("all", "rank", "step")}
    head = args.schedule if args.only_all else "all"
    m_head = measure(torch, steps[head], args.steps, args.warmup)

    other = {}
    if not args.only_all:
        for name in ("rank", "step"):
            mm = measure(torch, steps[name], args.steps, args.warmup, min_s=0.1, do_settle=False)
            t = mm["ms_per_step"]
            launches = P if name == "rank" else n_pairs
            other[name] = {"ms_per_step": round(t, 4), "tflops": round(total_flops / (t * 1e-3) / 1e12, 2),
                           "pct_of_bf16_mfma_peak": round(100.0 * total_flops / (t * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
                           "launches_per_step": launches, "avg_launch_us": round(t * 1e3 / launches, 2)}

        # the schedule for chunks that arrive while a rank's one launch runs: the `rank` launches with a bounded wait for
        # each chunk's arrival flag (all raised beforehand here: everything is resident on one GPU)
        flags = ops.RingFlags(P, dev)
        flags.set_all()
        out_f = torch.empty_like(q)
        lse_f = torch.empty((B, H, S), dtype=torch.float32, device=dev)
        f_flags = lambda: ops.ring_fwd_flags(q, k, v, P, flags, scale, True, out=out_f, lse=lse_f)
        mm = measure(torch, f_flags, args.steps, args.warmup, min_s=0.1, do_settle=False)
        t = mm["ms_per_step"]
        other["rank_flags"] = {"ms_per_step": round(t, 4), "tflops": round(total_flops / (t * 1e-3) / 1e12, 2), "launches_per_step": P,
                               "faulted": flags.failed()}

    if args.traffic_leg:
        calibration_copy(torch, dev)

    traffic = traffic_src = None
    if os.path.exists(TRAFFIC_JSON):
        try:
            traffic = round(json.load(open(TRAFFIC_JSON)).get("hbm_bytes_per_launch"))
            traffic_src = "recorded: profiles/flash_fwd_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 1 GiB copy)"
        except (ValueError, OSError, TypeError):
            traffic = None

    rows = {}
    if not args.no_rows and not args.only_all:
        del steps
        rows = gpu_rows(torch, spa, ops, ALL_ROWS, args.steps, args.warmup)

    cpu_head = host = None
    if not args.no_cpu_baseline:
        cpu = CpuLegs(torch)
        cpu_head = cpu.ring_forward(B, H, S // P, D, P, P * (P - 1) // 2, SEED)
        attach_cpu(rows, cpu)
        host = cpu.host
    text = json.dumps(assemble_line(args.steps, args.warmup, head, m_head, other, rows, cpu_head, host, traffic, traffic_src))
    if len(text) > LINE_LIMIT:
        print(f"bench.py: the line is {len(text)} bytes, over {LINE_LIMIT}", file=sys.stderr)
    print(text)


if __name__ == "__main__":
    main()
