#!/usr/bin/env python3
"""Benchmark of the hot-op kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only headline|gemm|rows|reduce|attn|backward|gpt2|train|generate|copy|all]

Headline (the JSON line's ``value``): bf16 ``addmm`` with M=N=K=8192 and a [N] bias, fp32
accumulation — one *step* is one launch of that GEMM through the C ABI, inputs resident in HBM.
W untimed warm-up steps, then exactly K steps between two ``torch.cuda.synchronize()`` calls.
Defaults are the reference's own protocol (25 warm-ups, 100 timed launches, ``bench_gemm.py``):
the first ~25 ms after idle run about 6 % slower while the clocks settle, so 50 untimed launches
precede the W warm-up steps whatever W is (``config.preheat_launches``).

The same line carries
  * ``roofline``   — the GEMM kernel against the MI355X dense bf16 MFMA peak (2.5 PFLOP/s):
                     algorithmic FLOPs (2*M*N*K) / average launch duration from HIP events on
                     the launch stream;
  * ``cpu_baseline`` — the CPU oracle (a C restatement of the reference's CPU GEMM loop, OpenMP
                     over rows) timed on this host on a bounded slab of the same product;
  * ``sweep``      — every other row of the workload definition (remaining GEMM shapes, bmm,
                     softmax, LayerNorm, sum/mean/amax, argmax, the GPT-2-small bf16 forward at
                     B=32, T=1024 through ``mojo_backend``), each with absolute throughput, the
                     fraction of its roofline (HBM 8 TB/s or MFMA 2.5 PFLOP/s) and a CPU figure.
Memory-bound rows rotate through enough distinct buffers that the 256 MB Infinity Cache cannot
serve them.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "torch-max-backend_amd"))

PEAK_BF16_DENSE_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA
PEAK_FP32_MFMA_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E

COUNTERS_FILE = os.path.join(ROOT, "profiles", "gemm_ring_bf16_addmm_8192_counters.txt")


def gemm_counters(path: str = COUNTERS_FILE) -> dict:
    """What the committed rocprofv3 --pmc summary of the headline says, per launch:
    ``traffic``: bytes between L2 and the memory side = FETCH_SIZE and WRITE_SIZE of the GEMM
    kernel, each scaled by what the same counter reads for tmb_copy_bytes moving exactly 1 GiB each
    way (the calibration lines of the same file); ``active_cycles``: GRBM_GUI_ACTIVE / 8 XCDs.
    Missing file or line -> the key is absent."""
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return {}
    reads: dict = {}
    for ln in lines:
        if ln.startswith("#") or "(per dispatch" not in ln:
            continue
        head = ln.split("(per dispatch")[0].split()
        if len(head) < 3:
            continue
        kernel, counter, value = " ".join(head[:-2]), head[-2], float(head[-1])
        kind = "copy" if "copy_kernel" in kernel else ("gemm" if "gemm_ring_kernel" in kernel else None)
        if kind:
            reads[(kind, counter)] = value
    out: dict = {}
    need = [("gemm", "FETCH_SIZE"), ("gemm", "WRITE_SIZE"), ("copy", "FETCH_SIZE"), ("copy", "WRITE_SIZE")]
    if all(k in reads for k in need):
        gib_kib = float(1 << 20)
        kib = reads[("gemm", "FETCH_SIZE")] * (gib_kib / reads[("copy", "FETCH_SIZE")]) + \
            reads[("gemm", "WRITE_SIZE")] * (gib_kib / reads[("copy", "WRITE_SIZE")])
        out["traffic"] = round(kib * 1024.0)
    if ("gemm", "GRBM_GUI_ACTIVE") in reads:
        out["active_cycles"] = reads[("gemm", "GRBM_GUI_ACTIVE")] / 8.0
    return out


def _parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=100)
    p.add_argument("--warmup", type=int, default=25)
    p.add_argument("--only", default="all", choices=["all", "headline", "gemm", "rows", "reduce", "attn", "backward", "gpt2", "train", "generate", "copy"])
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    return p.parse_args()


def main() -> int:
    args = _parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every row of the "
              "workload is a single-device kernel); run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 2
    from torch_mojo_backend import eager_kernels as ek
    from torch_mojo_backend.eager_kernels import hip_ops

    ek.lib()  # fail loudly right here if the HIP library is missing
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(0)
    host_cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    omp = int(os.environ.get("OMP_NUM_THREADS", host_cores))
    cpu_threads = max(1, min(host_cores, omp))
    torch.set_num_threads(cpu_threads)

    def sync():
        torch.cuda.synchronize()

    def timed(fn, steps, warmup):
        """(wall ms per step between two syncs, HIP-event ms per launch) over exactly `steps`."""
        for _ in range(warmup):
            fn()
        sync()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        start.record()
        for _ in range(steps):
            fn()
        end.record()
        sync()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return wall, start.elapsed_time(end) / steps

    def settle(fn, seconds=0.03):
        """Untimed launches for `seconds` of wall time in front of a timed region: the first
        launches after a pause (input generation, a CPU leg) run at whatever clock the idle chip
        was left at, 10-15 % slower on the 100 us products, and the yardstick beside a row would
        otherwise be measured on a warmer chip than the row itself."""
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(8):
                fn()
            sync()

    def cpu_time(fn, iters=3, warmup=1):
        for _ in range(warmup):
            fn()
        ts = []
        for _ in range(iters):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    def gen(shape, seed, dtype, scale=1.0, shift=0.0):
        g = torch.Generator(device=dev).manual_seed(seed)
        x = torch.randn(shape, generator=g, device=dev, dtype=torch.float32)
        if scale != 1.0 or shift != 0.0:
            x = x * scale + shift
        return x.to(dtype)

    sweep = {}
    want = args.only

    if want == "copy":
        # Calibration workload for the HBM counters: tmb_copy_bytes moves exactly 1 GiB in and
        # 1 GiB out per launch, so FETCH_SIZE / WRITE_SIZE of this kernel give the counters'
        # scale. Not a bench line.
        nbytes = 1 << 30
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        wall_ms, ev_ms = timed(lambda: hip_ops.copy_bytes(dst, src), args.steps, args.warmup)
        assert torch.equal(dst, src)
        print(json.dumps({"workload": "tmb_copy_bytes 1 GiB", "bytes_read": nbytes,
                          "bytes_written": nbytes, "launch_ms": round(ev_ms, 4),
                          "GB/s": round(2 * nbytes / (ev_ms * 1e-3) / 1e9, 1)}))
        return 0

    # ------------------------------------------------------------------ GEMM (headline)
    M = N = K = 8192
    PREHEAT = 50

    def run_headline():
        a = gen((M, K), 0, torch.bfloat16)
        b = gen((K, N), 1, torch.bfloat16)
        bias = gen((N,), 2, torch.bfloat16)
        flops = 2.0 * M * N * K
        # The first ~25 ms after idle run about 6 % slower while the clocks settle: 50 untimed launches
        # come before the W warm-up steps whatever W is (reported as config.preheat_launches).
        for _ in range(PREHEAT):
            hip_ops.gemm(a, b, bias)
        wall_ms, ev_ms = timed(lambda: hip_ops.gemm(a, b, bias), args.steps, args.warmup)
        value = flops / (wall_ms * 1e-3) / 1e12
        achieved = flops / (ev_ms * 1e-3) / 1e12
        counters = gemm_counters()
        roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_DENSE_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_DENSE_TFLOPS, 4),
                    "traffic": counters.get("traffic"), "kernel": "gemm_ring_kernel<bf16,256x256x64,2x4 waves,2 A + 3 B buffers,N-major B>",
                    "launch_ms": round(ev_ms, 4), "algorithmic_flops": flops}
        if "active_cycles" in counters:
            # the same FLOPs against the cycles the chip was active for in the committed counter
            # run: 2.5 PFLOP/s is 2.5e15 / 2.4e9 FLOP per cycle at the 2.4 GHz the peak assumes
            roofline["frac_at_sustained_clock"] = round(
                flops / (counters["active_cycles"] * (PEAK_BF16_DENSE_TFLOPS * 1e12 / 2.4e9)), 4)

        cpu_baseline = None
        if not args.no_cpu:
            import oracle  # the checker, timed here as the reported CPU baseline only

            # bounded sample: the [0:4096, 0:2048] slab of the same product (1/8 of the FLOPs, about
            # 15 s on 16 host threads)
            sm, sn = 4096, 2048
            a_h, b_h, bias_h = a[:sm].cpu(), b[:, :sn].contiguous().cpu(), bias[:sn].cpu()
            t0 = time.perf_counter()
            ref = oracle.gemm(a_h, b_h, bias_h).float()  # one run: timed and kept as the check below
            t = time.perf_counter() - t0
            cpu_baseline = {"value": round(2.0 * sm * sn * K / t / 1e12, 5), "unit": "TFLOP/s",
                            "cores": cpu_threads, "kind": "port",
                            "sample": f"C[0:{sm},0:{sn}] slab of the same 8192^3 bf16 addmm (1/8 of "
                                      f"the work), oracle/tmb_oracle.c orc_gemm, OpenMP over rows, "
                                      f"{t:.2f} s"}
            # context: a tuned CPU BLAS on the same slab (PyTorch CPU, fp32 math on bf16-rounded data)
            a32, b32, bias32 = a_h.float(), b_h.float(), bias_h.float()
            t_blas = cpu_time(lambda: torch.addmm(bias32, a32, b32), iters=3, warmup=1)
            cpu_baseline["torch_cpu_fp32_tflops_same_slab"] = round(2.0 * sm * sn * K / t_blas / 1e12, 4)
            # check the GPU result on that slab against the oracle while we are here
            got = hip_ops.gemm(a, b, bias)[:sm, :sn].float().cpu()
            rel = ((got - ref).norm() / ref.norm()).item()
            cpu_baseline["gpu_vs_oracle_rel_frobenius"] = rel
            if not rel < 1e-2:
                print(f"bench: GEMM result deviates from the oracle (rel Frobenius {rel})", file=sys.stderr)
                raise SystemExit(1)
        del a, b, bias
        return value, wall_ms, ev_ms, achieved, roofline, cpu_baseline

    value = wall_ms = ev_ms = achieved = roofline = cpu_baseline = None
    if want in ("all", "headline", "gemm"):
        value, wall_ms, ev_ms, achieved, roofline, cpu_baseline = run_headline()

    def gemm_row(name, m, n, k, batch=None, trans_b=False, steps=50, dtype=torch.bfloat16):
        if batch:
            x = gen((batch, m, k), 3, dtype)
            w = gen((batch, k, n), 4, dtype)
            bs = None
        else:
            x = gen((m, k), 3, dtype)
            w = gen((n, k), 4, dtype).t() if trans_b else gen((k, n), 4, dtype)
            bs = gen((n,), 5, dtype)
        settle(lambda: hip_ops.gemm(x, w, bs))
        _, ms = timed(lambda: hip_ops.gemm(x, w, bs), steps, 10)
        # yardstick, not part of the product: PyTorch-ROCm's own library GEMM on the same tensors
        if batch:
            settle(lambda: torch.bmm(x, w))
            _, yard = timed(lambda: torch.bmm(x, w), max(steps // 2, 5), 5)
        else:
            settle(lambda: torch.addmm(bs, x, w))
            _, yard = timed(lambda: torch.addmm(bs, x, w), max(steps // 2, 5), 5)
        bt = batch or 1
        size = x.element_size()
        peak = PEAK_FP32_MFMA_TFLOPS if dtype == torch.float32 else PEAK_BF16_DENSE_TFLOPS
        fl = 2.0 * bt * m * n * k
        by = size * (bt * (m * k + k * n + m * n) + (0 if batch else n))
        tf, gbs = fl / ms / 1e9, by / ms / 1e6
        sweep[name] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 2),
                       "frac_mfma": round(tf / peak, 4),
                       "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4),
                       "pytorch_rocm_us": round(yard * 1e3, 2)}

    if want in ("all", "gemm"):
        sweep["addmm_bf16_8192x8192x8192"] = {"us": round(ev_ms * 1e3, 2), "TFLOP/s": round(achieved, 2),
                                              "frac_mfma": round(achieved / PEAK_BF16_DENSE_TFLOPS, 4)}
        gemm_row("addmm_bf16_8192x8192x8192_Bt", 8192, 8192, 8192, trans_b=True, steps=args.steps)
        for (m, n, k) in ((128, 768, 768), (1024, 3072, 768), (1024, 768, 3072), (4096, 4096, 4096)):
            gemm_row(f"addmm_bf16_{m}x{n}x{k}", m, n, k)
        gemm_row("bmm_bf16_48x1024x64x1024", 1024, 1024, 64, batch=48)
        # GPT-2 small's projections at 32768 tokens (weights stored [out, in]: K-major B)
        for (m, n, k) in ((32768, 2304, 768), (32768, 3072, 768), (32768, 768, 3072), (32768, 768, 768)):
            gemm_row(f"linear_bf16_{m}x{n}x{k}", m, n, k, trans_b=True, steps=30)
        # the vocabulary projection, alone and behind other work (four 8192^3 products evict its
        # weight from the Infinity Cache, as the rest of a model does): the difference of the
        # pair's time and the other work's
        for m in (16384, 32768):
            xv, wv = gen((m, 768), 6, torch.bfloat16), gen((50257, 768), 7, torch.bfloat16, scale=0.02)
            other = gen((8192, 8192), 8, torch.bfloat16)
            _, alone = timed(lambda: hip_ops.gemm(xv, wv.t()), 10, 5)

            def evict():
                for _ in range(4):
                    hip_ops.gemm(other, other)

            def pair():
                evict()
                return hip_ops.gemm(xv, wv.t())

            _, both = timed(pair, 6, 2)
            _, rest = timed(evict, 6, 2)
            fl = 2.0 * m * 50257 * 768
            sweep[f"linear_bf16_{m}x50257x768"] = {
                "us": round(alone * 1e3, 1), "TFLOP/s": round(fl / alone / 1e9, 1),
                "us_behind_other_work": round((both - rest) * 1e3, 1),
                "frac_mfma": round(fl / alone / 1e9 / PEAK_BF16_DENSE_TFLOPS, 4)}
            del xv, wv, other
        # fp32 storage: true fp32 products on the matrix cores (peak 157.3 TFLOP/s)
        gemm_row("addmm_fp32_4096x4096x4096", 4096, 4096, 4096, steps=20, dtype=torch.float32)
        gemm_row("addmm_fp32_128x3072x768", 128, 3072, 768, dtype=torch.float32)
        gemm_row("linear_fp32_128x50257x768", 128, 50257, 768, trans_b=True, dtype=torch.float32)

    # ------------------------------------------------------------------ memory-bound rows
    # Launched straight through the C ABI with preallocated outputs, so the timed region holds
    # kernel launches only (the PyTorch-side allocation of outputs costs more host time than
    # the smaller kernels run for).
    lib = ek.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def rotating(make, bytes_per_buffer):
        # fresh segments for every row's buffers: blocks carved out of segments that earlier rows
        # left behind measured up to 12 % slower on the same kernel (layer norm bf16 [16384, 4096]:
        # 47 us with --only rows, 53 us behind the GEMM and attention rows)
        torch.cuda.empty_cache()
        n = max(2, math.ceil(768e6 / max(bytes_per_buffer, 1)) + 1)
        n = min(n, 16)
        return [make(i) for i in range(n)]

    def hbm_row(name, nbuf, launch, bytes_algo, steps=40, cpu_fn=None):
        state = {"i": 0}

        def step():
            rc = launch(state["i"] % nbuf)
            if rc != 0:
                raise RuntimeError(f"{name}: launch failed with {ek.status_string(rc)}")
            state["i"] += 1

        settle(step)
        _, ms = timed(step, steps, 8)
        gbs = bytes_algo / ms / 1e6
        row = {"us": round(ms * 1e3, 2), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4),
               "bytes": bytes_algo, "buffers": nbuf}
        if cpu_fn is not None and not args.no_cpu:
            t = cpu_fn()
            row["cpu_GB/s"] = round(t[1] / t[0] / 1e9, 3)
            row["cpu_note"] = t[2]
        sweep[name] = row
        return (state["i"] - 1) % nbuf   # the buffer the last launch worked on

    def with_copy(name, nbuf, ptrs, nbytes):
        """Beside a row-wise kernel's row: tmb_copy_bytes over the same buffers (the same bytes
        read and written by a kernel that does nothing else), timed in the same run."""
        state = {"i": 0}

        def step():
            o, x = ptrs[state["i"] % nbuf]
            lib.tmb_copy_bytes(o, x, nbytes, stream)
            state["i"] += 1

        settle(step)
        _, ms = timed(step, 40, 8)
        sweep[name]["copy_us_same_bytes"] = round(ms * 1e3, 2)
        sweep[name]["vs_copy"] = round(ms * 1e3 / sweep[name]["us"], 3)

    def with_read(name, nbuf, in_ptrs, nbytes):
        """Beside a reduction's row: tmb_read_bytes over the same buffers (the same bytes read by
        a kernel that keeps nothing), timed in the same run."""
        state = {"i": 0}
        sink = torch.zeros(4, dtype=torch.int32, device=dev)

        def step():
            lib.tmb_read_bytes(in_ptrs[state["i"] % nbuf], nbytes, sink.data_ptr(), stream)
            state["i"] += 1

        settle(step)
        _, ms = timed(step, 40, 8)
        sweep[name]["read_us_same_bytes"] = round(ms * 1e3, 2)
        sweep[name]["vs_read"] = round(ms * 1e3 / sweep[name]["us"], 3)

    if want in ("all", "attn"):
        # attention of the GPT-2 workload (B=32, H=12, T=1024, head_dim 64, bf16), q/k/v as the
        # strided thirds of the packed projection, exactly as the compiled graph hands them over
        Bq, Hq, Tq = 32, 12, 1024
        qkv = gen((Bq, Tq, 3 * Hq * 64), 30, torch.bfloat16)
        q4, k4, v4 = (x.view(Bq, Tq, Hq, 64).transpose(1, 2) for x in qkv.split(Hq * 64, dim=2))
        _, ms = timed(lambda: hip_ops.attention(q4, k4, v4, 0.125, True), 30, 8)
        useful = 4.0 * Bq * Hq * Tq * Tq * 64 / 2   # causal: half of the score matrix
        algo_bytes = 4 * Bq * Hq * Tq * 64 * 2      # q, k, v in, out once
        sweep["attention_causal_bf16_32x12x1024x64"] = {
            "us": round(ms * 1e3, 2), "TFLOP/s": round(useful / ms / 1e9, 1),
            "frac_mfma": round(useful / ms / 1e9 / PEAK_BF16_DENSE_TFLOPS, 4),
            "GB/s": round(algo_bytes / ms / 1e6, 1), "flops": useful, "bytes": algo_bytes,
            "note": "useful FLOPs (masked half not counted); scores never reach memory"}
        # its backward: dq, dk, dv from q, k, v, out, dout and the forward's log-sum-exp, gradients
        # written as the thirds of one packed buffer. Useful FLOPs = 2.5 x the forward's (five
        # products against two); the kernels recompute scores and dP in both launches (seven).
        out_f, lse_f = hip_ops.attention(q4, k4, v4, 0.125, True, return_lse=True)
        dout = gen((Bq, Tq, Hq, 64), 34, torch.bfloat16).transpose(1, 2)
        _, ms = timed(lambda: hip_ops.attention_backward(dout, q4, k4, v4, out_f.transpose(1, 2), lse_f,
                                                         0.125, True, packed=True), 30, 8)
        sweep["attention_backward_causal_bf16_32x12x1024x64"] = {
            "us": round(ms * 1e3, 2), "TFLOP/s": round(2.5 * useful / ms / 1e9, 1),
            "frac_mfma": round(2.5 * useful / ms / 1e9 / PEAK_BF16_DENSE_TFLOPS, 4),
            "flops": 2.5 * useful,
            "note": "two launches (dq; dk and dv), no atomics; useful FLOPs = 5 products over the "
                    "unmasked half"}
        del out_f, lse_f, dout
        # a decode step of the eager generation benchmark (batch 512, 12 heads, 1 query, 208 keys):
        # K and V are read once; rotated over several caches so no cache level holds them
        Bd, Sd = 512, 208
        qd = gen((Bd, Hq, 1, 64), 32, torch.bfloat16)
        caches = rotating(lambda i: gen((2, Bd, Hq, Sd, 64), 33 + i, torch.bfloat16), 2 * Bd * Hq * Sd * 64 * 2)
        state = {"i": 0}

        def decode_step():
            kv = caches[state["i"] % len(caches)]
            state["i"] += 1
            hip_ops.attention_decode(qd, kv[0], kv[1], 0.125, False, None)

        _, ms = timed(decode_step, 60, 10)
        dec_bytes = 2 * Bd * Hq * Sd * 64 * 2 + 2 * Bd * Hq * 64 * 2
        sweep["attention_decode_bf16_512x12x1x208x64"] = {
            "us": round(ms * 1e3, 2), "GB/s": round(dec_bytes / ms / 1e6, 1),
            "frac_hbm": round(dec_bytes / ms / 1e6 / PEAK_HBM_GBS, 4), "bytes": dec_bytes,
            "note": "one wave per query row, K and V read once (includes the Python wrapper)"}
        del caches
        # the softmax of the same attention when it runs on its own: [B*H*T, T] scores in,
        # probabilities out; the masked half of every row is not read
        rows, cols = Bq * Hq * Tq, Tq
        xs = [gen((Bq * Hq, Tq, Tq), 31 + i, torch.bfloat16, scale=4.0) for i in range(2)]
        os_ = [torch.empty_like(x) for x in xs]
        code = hip_ops.code_of(torch.bfloat16)
        nbytes = rows * cols * 2
        hbm_row("softmax_scaled_causal_bf16_393216x1024", 2,
                lambda i: lib.tmb_softmax_rows_scaled(os_[i].data_ptr(), xs[i].data_ptr(), rows, cols,
                                                      code, 0.125, 1, Tq, stream),
                nbytes // 2 + nbytes, steps=30)
        sweep["softmax_scaled_causal_bf16_393216x1024"]["note"] = \
            "bytes = half of the input (causal) + the whole output"
        del xs, os_, qkv

    if want in ("all", "rows"):
        import oracle

        for dtype, dn in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            es = torch.finfo(dtype).bits // 8
            code = hip_ops.code_of(dtype)
            for (B, H, S) in ((8, 12, 1024), (4, 32, 4096)):
                rows, cols = B * H * S, S
                nbytes = rows * cols * es
                if nbytes > 3e9:
                    bufs = [gen((rows, cols), 10, dtype, scale=4.0)]  # 8.6 GB: no cache can hold it
                else:
                    bufs = rotating(lambda i: gen((rows, cols), 10 + i, dtype, scale=4.0), nbytes)
                outs = [torch.empty_like(b_) for b_ in bufs]
                ptrs = [(o.data_ptr(), b_.data_ptr()) for o, b_ in zip(outs, bufs)]

                def cpu_softmax(rows=rows, cols=cols, dtype=dtype, es=es):
                    sub = min(rows, 8192)
                    xh = (torch.randn(sub, cols) * 4).to(dtype)
                    t = cpu_time(lambda: oracle.softmax_rows(xh), iters=3, warmup=1)
                    return t, 2 * sub * cols * es, f"first {sub} rows, C oracle, {cpu_threads} threads"

                hbm_row(f"softmax_{dn}_{rows}x{cols}", len(bufs),
                        lambda i: lib.tmb_softmax_rows(ptrs[i][0], ptrs[i][1], rows, cols, code, code, 0, stream),
                        2 * nbytes, steps=20 if nbytes > 3e9 else 40, cpu_fn=cpu_softmax)
                # spot-check the raw launch against the tensor-level op
                assert torch.equal(outs[0], hip_ops.softmax(bufs[0], -1))
                with_copy(f"softmax_{dn}_{rows}x{cols}", len(bufs), ptrs, nbytes)
                del bufs, outs
            # log-softmax over GPT-2's vocabulary: the pitch is odd, no row but the first starts on
            # a 16-byte boundary
            rows, cols = 16384, 50257
            nbytes = rows * cols * es
            bufs = [gen((rows, cols), 20, dtype, scale=4.0)]
            outs = [torch.empty_like(bufs[0])]
            hbm_row(f"log_softmax_{dn}_{rows}x{cols}", 1,
                    lambda i: lib.tmb_softmax_rows(outs[0].data_ptr(), bufs[0].data_ptr(), rows, cols,
                                                   code, code, 1, stream), 2 * nbytes, steps=20)
            assert torch.equal(outs[0], hip_ops.softmax(bufs[0], -1, log=True))
            del bufs, outs
            for (rows, cols) in ((32768, 768), (16384, 4096)):
                nbytes = rows * cols * es
                g_ = gen((cols,), 1, dtype, scale=0.1, shift=1.0)
                b_ = gen((cols,), 2, dtype, scale=0.1)
                bufs = rotating(lambda i: gen((rows, cols), 20 + i, dtype), nbytes)
                outs = [torch.empty_like(x_) for x_ in bufs]
                mean = torch.empty(rows, dtype=torch.float32, device=dev)
                rstd = torch.empty(rows, dtype=torch.float32, device=dev)
                ptrs = [(o.data_ptr(), x_.data_ptr()) for o, x_ in zip(outs, bufs)]

                def cpu_ln(rows=rows, cols=cols, dtype=dtype, es=es):
                    sub = min(rows, 8192)
                    xh = torch.randn(sub, cols).to(dtype)
                    gh, bh = torch.ones(cols).to(dtype), torch.zeros(cols).to(dtype)
                    t = cpu_time(lambda: oracle.layer_norm_rows(xh, gh, bh, 1e-5), iters=3, warmup=1)
                    return t, 2 * sub * cols * es, f"first {sub} rows, C oracle, {cpu_threads} threads"

                hbm_row(f"layer_norm_{dn}_{rows}x{cols}", len(bufs),
                        lambda i: lib.tmb_layer_norm_rows(ptrs[i][0], mean.data_ptr(), rstd.data_ptr(),
                                                          ptrs[i][1], g_.data_ptr(), b_.data_ptr(),
                                                          rows, cols, 1e-5, code, code, stream),
                        2 * nbytes + 2 * cols * es + 2 * rows * 4, cpu_fn=cpu_ln)
                assert torch.equal(outs[0], hip_ops.layer_norm(bufs[0], [cols], g_, b_, 1e-5)[0])
                with_copy(f"layer_norm_{dn}_{rows}x{cols}", len(bufs), ptrs, nbytes)
                del bufs, outs

    if want in ("all", "reduce"):
        import oracle

        for dtype, dn in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            es = torch.finfo(dtype).bits // 8
            code = hip_ops.code_of(dtype)
            rows, cols = 65536, 4096
            nbytes = rows * cols * es
            bufs = rotating(lambda i: gen((rows, cols), 30 + i, dtype), nbytes)
            in_ptrs = [x_.data_ptr() for x_ in bufs]
            out_rows = torch.empty(rows, dtype=dtype, device=dev)
            out_all = torch.empty(1, dtype=dtype, device=dev)
            ws_bytes = lib.tmb_reduce_workspace_bytes(1, rows * cols, code)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
            for opname, op in (("sum", ek.SUM), ("mean", ek.MEAN), ("amax", ek.AMAX)):
                def cpu_red(op=op, dtype=dtype, es=es, cols=cols):
                    sub = 4096
                    xh = torch.randn(sub, cols).to(dtype)
                    t = cpu_time(lambda: oracle.reduce_rows(xh, op), iters=3, warmup=1)
                    return t, sub * cols * es, f"first {sub} rows, C oracle, {cpu_threads} threads"

                hbm_row(f"{opname}_{dn}_rows_{rows}x{cols}", len(bufs),
                        lambda i, op=op: lib.tmb_reduce_rows(out_rows.data_ptr(), in_ptrs[i], rows, cols, op,
                                                             code, None, 0, stream),
                        nbytes + rows * es, cpu_fn=cpu_red)
                last = hbm_row(f"{opname}_{dn}_all_{rows}x{cols}", len(bufs),
                               lambda i, op=op: lib.tmb_reduce_rows(out_all.data_ptr(), in_ptrs[i], 1, rows * cols,
                                                                    op, code, ws.data_ptr(), ws_bytes, stream),
                               nbytes + es)
            assert torch.equal(out_all.reshape(()), hip_ops.reduce(bufs[last], [0, 1], False, ek.AMAX))
            # the same matrices summed over their leading dimension (the bias gradient of a linear
            # layer): out[c] = sum_r x[r, c]
            out_cols = torch.empty(cols, dtype=dtype, device=dev)
            cws_bytes = lib.tmb_reduce_cols_workspace_bytes(rows, cols, code)
            cws = torch.empty(max(cws_bytes, 16), dtype=torch.uint8, device=dev)
            last = hbm_row(f"sum_{dn}_cols_{rows}x{cols}", len(bufs),
                           lambda i: lib.tmb_reduce_cols(out_cols.data_ptr(), in_ptrs[i], rows, cols, ek.SUM, code,
                                                         cws.data_ptr(), cws_bytes, stream),
                           nbytes + cols * es)
            assert torch.allclose(out_cols.float(), bufs[last].float().sum(0), rtol=2e-2, atol=2.0)
            del bufs
        rows, cols = 512, 50257
        bufs = rotating(lambda i: gen((rows, cols), 40 + i, torch.float32), rows * cols * 4)
        in_ptrs = [x_.data_ptr() for x_ in bufs]
        out_idx = torch.empty(rows, dtype=torch.int64, device=dev)
        ws_bytes = lib.tmb_argmax_workspace_bytes(rows, cols, ek.F32)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)

        def cpu_argmax():
            xh = torch.randn(rows, cols)
            t = cpu_time(lambda: oracle.argmax_rows(xh), iters=3, warmup=1)
            return t, rows * cols * 4, f"all {rows} rows, C oracle, {cpu_threads} threads"

        last = hbm_row(f"argmax_fp32_{rows}x{cols}", len(bufs),
                       lambda i: lib.tmb_argmax_rows(out_idx.data_ptr(), in_ptrs[i], rows, cols, ek.F32,
                                                     ws.data_ptr(), ws_bytes, stream),
                       rows * cols * 4 + rows * 8, steps=100, cpu_fn=cpu_argmax)
        assert torch.equal(out_idx, torch.argmax(bufs[last], dim=1))
        with_read(f"argmax_fp32_{rows}x{cols}", len(bufs), in_ptrs, rows * cols * 4)
        del bufs

    # ------------------------------------------------------------------ backward twins
    # Shapes of the GPT-2 training step at B=32, T=1024 (bf16) and the forward sweep's row shapes.
    # Algorithmic bytes: every input read once, every output written once (the layer-norm
    # backward reads dy and x a second time for the parameter gradients: counted once here).
    if want in ("all", "backward"):
        for dtype, dn in ((torch.bfloat16, "bf16"), (torch.float32, "fp32")):
            es = torch.finfo(dtype).bits // 8
            code = hip_ops.code_of(dtype)
            # gelu_backward over the MLP activation [32768, 3072]
            numel = 32768 * 3072
            nb = numel * es
            xs = rotating(lambda i: gen((numel,), 40 + i, dtype), 2 * nb)
            gs = [gen((numel,), 60 + i, dtype) for i in range(len(xs))]
            outs = [torch.empty_like(x_) for x_ in xs]
            hbm_row(f"gelu_backward_tanh_{dn}_32768x3072", len(xs),
                    lambda i: lib.tmb_gelu_backward(outs[i].data_ptr(), gs[i].data_ptr(), xs[i].data_ptr(),
                                                    numel, code, 1, stream), 3 * nb)
            del xs, gs, outs
            # softmax backward over attention probabilities [98304, 1024]
            rows, cols = 98304, 1024
            nb = rows * cols * es
            ys = rotating(lambda i: torch.softmax(gen((rows, cols), 70 + i, torch.float32), -1).to(dtype), 2 * nb)
            gs = [gen((rows, cols), 80 + i, dtype) for i in range(len(ys))]
            outs = [torch.empty_like(y_) for y_ in ys]
            hbm_row(f"softmax_backward_{dn}_{rows}x{cols}", len(ys),
                    lambda i: lib.tmb_softmax_backward_rows(outs[i].data_ptr(), gs[i].data_ptr(),
                                                            ys[i].data_ptr(), rows, cols, code, 0, stream),
                    3 * nb)
            del ys, gs, outs
            # log-softmax backward over GPT-2's vocabulary (odd pitch)
            rows, cols = 16384, 50257
            nb = rows * cols * es
            ys = [torch.log_softmax(gen((rows, cols), 75, torch.float32), -1).to(dtype)]
            gs = [gen((rows, cols), 85, dtype)]
            outs = [torch.empty_like(ys[0])]
            hbm_row(f"log_softmax_backward_{dn}_{rows}x{cols}", 1,
                    lambda i: lib.tmb_softmax_backward_rows(outs[0].data_ptr(), gs[0].data_ptr(),
                                                            ys[0].data_ptr(), rows, cols, code, 1, stream),
                    3 * nb, steps=20)
            # the same gradient when it comes from a cross-entropy loss: one pass over the saved
            # log-probabilities, rows of whole vectors out (pitch 50304)
            ldo = (cols + 63) // 64 * 64
            tgt = torch.randint(0, cols, (rows,), device=dev, generator=torch.Generator(device=dev).manual_seed(7))
            one, tw = torch.ones((), dtype=dtype, device=dev), torch.full((), float(rows), dtype=dtype, device=dev)
            padded = torch.empty((rows, ldo), dtype=dtype, device=dev)
            hbm_row(f"cross_entropy_backward_{dn}_{rows}x{cols}", 1,
                    lambda i: lib.tmb_nll_log_softmax_backward_rows(
                        padded.data_ptr(), ys[0].data_ptr(), tgt.data_ptr(), one.data_ptr(), tw.data_ptr(),
                        rows, cols, cols, ldo, 1, -100, code, stream),
                    2 * nb, steps=20)
            del ys, gs, outs, padded
            # layer norm backward (all three outputs)
            for (rows, cols) in ((32768, 768), (16384, 4096)):
                nb = rows * cols * es
                xs = rotating(lambda i: gen((rows, cols), 90 + i, dtype), 2 * nb)
                gs = [gen((rows, cols), 100 + i, dtype) for i in range(len(xs))]
                dxs = [torch.empty_like(x_) for x_ in xs]
                gamma = gen((cols,), 1, dtype, scale=0.1, shift=1.0)
                dgm, dbt = torch.empty_like(gamma), torch.empty_like(gamma)
                stats = [hip_ops.layer_norm(x_, [cols], gamma, None, 1e-5)[1:] for x_ in xs]
                ws_b = lib.tmb_layer_norm_backward_workspace_bytes(rows, cols, code)
                wsp = torch.empty(max(ws_b, 16), dtype=torch.uint8, device=dev)
                hbm_row(f"layer_norm_backward_{dn}_{rows}x{cols}", len(xs),
                        lambda i: lib.tmb_layer_norm_backward_rows(
                            dxs[i].data_ptr(), dgm.data_ptr(), dbt.data_ptr(), gs[i].data_ptr(),
                            xs[i].data_ptr(), stats[i][0].data_ptr(), stats[i][1].data_ptr(),
                            gamma.data_ptr(), rows, cols, code, wsp.data_ptr(), ws_b, stream),
                        3 * nb + 3 * cols * es + 2 * rows * 4)
                # the same pass where its grad_input re-joins a residual stream: the by-passing
                # gradient added on the way out, the column sums of the result handed out as well
                # (the add and the bias-gradient sum that would follow as passes of their own)
                ws_a = lib.tmb_layer_norm_backward_add_workspace_bytes(rows, cols, code)
                wsa = torch.empty(max(ws_a, 16), dtype=torch.uint8, device=dev)
                dsm = torch.empty_like(gamma)
                hbm_row(f"layer_norm_backward_add_{dn}_{rows}x{cols}", len(xs),
                        lambda i: lib.tmb_layer_norm_backward_add_rows(
                            dxs[i].data_ptr(), dgm.data_ptr(), dbt.data_ptr(), dsm.data_ptr(),
                            gs[i].data_ptr(), xs[i].data_ptr(), stats[i][0].data_ptr(),
                            stats[i][1].data_ptr(), gamma.data_ptr(), gs[(i + 1) % len(xs)].data_ptr(),
                            rows, cols, code, wsa.data_ptr(), ws_a, stream),
                        4 * nb + 4 * cols * es + 2 * rows * 4)
                del xs, gs, dxs, stats
        # the two GEMMs of linear_backward for the MLP up-projection: dgrad (NN) and wgrad (TN)
        rows_, in_f, out_f = 32768, 768, 3072
        dy = gen((rows_, out_f), 110, torch.bfloat16)
        xin = gen((rows_, in_f), 111, torch.bfloat16)
        wt = gen((out_f, in_f), 112, torch.bfloat16)
        for name, fn, fl in (
                ("linear_backward_dgrad_bf16_32768x768x3072", lambda: hip_ops.gemm(dy, wt), 2.0 * rows_ * in_f * out_f),
                ("linear_backward_wgrad_bf16_3072x768x32768", lambda: hip_ops.gemm(dy.t(), xin), 2.0 * rows_ * in_f * out_f)):
            # (long enough for the clock to settle: the first launches after the memory-bound
            # rows above run 20-30 % slower than the steady state)
            _, ms = timed(fn, 80, 40)
            sweep[name] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(fl / ms / 1e9, 2),
                           "frac_mfma": round(fl / ms / 1e9 / PEAK_BF16_DENSE_TFLOPS, 4)}
        del dy, xin, wt

    # ------------------------------------------------------------------ GPT-2 forward
    if want in ("all", "gpt2"):
        from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
        from torch_mojo_backend import mojo_backend
        from torch_mojo_backend.torch_compile_backend import compiler

        B, T = 32, 1024
        model = build_gpt2_small(seed=0).to(torch.bfloat16).to(dev)
        idx = seeded_tokens(B, T, seed=0).to(dev)
        compiled = torch.compile(model, backend=mojo_backend, fullgraph=True)
        t0 = time.perf_counter()
        with torch.no_grad():
            compiled(idx)
            sync()
            compile_s = time.perf_counter() - t0

            def fwd():
                out = compiled(idx)
                del out

            wall, ev = timed(fwd, 10, 3)
            compiler.COLLECT_OP_TIMINGS = True
            compiled(idx)
            sync()
            compiler.COLLECT_OP_TIMINGS = False
        breakdown = compiler.summarize_op_timings()
        gemm_flops = 12 * (2 * B * T * 7077888) + 12 * (2 * 2 * B * 12 * T * T * 64) + 2 * B * T * 768 * 50257
        row = {"tokens/s": round(B * T / (wall * 1e-3), 1), "ms_per_forward": round(wall, 3),
               "gemm_TFLOP/s_over_whole_forward": round(gemm_flops / (wall * 1e-3) / 1e12, 2),
               "compile_s": round(compile_s, 2), "batch": B, "seq": T, "dtype": "bf16",
               "per_op_ms": breakdown}
        if not args.no_cpu:
            cpu_model = build_gpt2_small(seed=0)
            cb, ct = 1, 128
            cidx = seeded_tokens(cb, ct, seed=0)
            with torch.no_grad():
                t = cpu_time(lambda: cpu_model(cidx), iters=3, warmup=1)
            row["cpu_tokens/s"] = round(cb * ct / t, 1)
            row["cpu_note"] = (f"PyTorch CPU eager fp32 of the same module at B={cb}, T={ct} "
                               f"(the workload's CPU configuration), {cpu_threads} threads")
        sweep[f"gpt2_small_fwd_bf16_B{B}_T{T}"] = row
        # the workload's small configuration (B=1, T=128) is bound by the host's step per node:
        # the same forward step by step and as replays of one recorded HIP graph
        # (TORCH_MOJO_BACKEND_HIP_GRAPH=1), beside PyTorch-ROCm eager
        torch._dynamo.reset()
        sb, st = 1, 128
        sidx = seeded_tokens(sb, st, seed=0).to(dev)
        small = torch.compile(model, backend=mojo_backend, fullgraph=True)
        small_row = {"batch": sb, "seq": st, "dtype": "bf16"}
        saved_flag = os.environ.get("TORCH_MOJO_BACKEND_HIP_GRAPH")
        try:
            with torch.no_grad():
                for flag, key in (("0", "ms_step_by_step"), ("1", "ms_hip_graph_replay")):
                    os.environ["TORCH_MOJO_BACKEND_HIP_GRAPH"] = flag
                    for _ in range(3):
                        small(sidx)
                    sync()
                    t0 = time.perf_counter()
                    for _ in range(30):
                        small(sidx)
                    sync()
                    small_row[key] = round((time.perf_counter() - t0) / 30 * 1e3, 3)
                for _ in range(3):
                    model(sidx)
                sync()
                t0 = time.perf_counter()
                for _ in range(30):
                    model(sidx)
                sync()
                small_row["pytorch_rocm_eager_ms"] = round((time.perf_counter() - t0) / 30 * 1e3, 3)
        finally:
            if saved_flag is None:
                os.environ.pop("TORCH_MOJO_BACKEND_HIP_GRAPH", None)
            else:
                os.environ["TORCH_MOJO_BACKEND_HIP_GRAPH"] = saved_flag
        sweep[f"gpt2_small_fwd_bf16_B{sb}_T{st}"] = small_row
        del model, compiled, small

    # ------------------------------------------------------------------ GPT-2 training step
    # Forward + backward of the same module through mojo_backend (bf16, B=16, T=1024, mean
    # cross-entropy over all positions; no optimizer step: the reference's training path ends at
    # the gradients). The backward graph runs the backward twins of the hot ops and the GEMMs of
    # linear_backward; PyTorch-ROCm's eager forward + backward of the same module is timed beside
    # it. (Runs before the eager device is registered: afterwards PyTorch's autograd engine no
    # longer takes plain HIP tensors in this process.)
    if want in ("all", "train"):
        import torch.nn.functional as F
        from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
        from torch_mojo_backend import mojo_backend

        B, T = 16, 1024
        torch._dynamo.reset()  # its own static graph, whatever batch sizes ran before
        model = build_gpt2_small(seed=0).to(torch.bfloat16).to(dev)
        idx, targets = seeded_tokens(B, T, seed=0).to(dev), seeded_tokens(B, T, seed=1).to(dev)

        def train_step(m):
            logits, _ = m(idx)
            loss = F.cross_entropy(logits.view(-1, logits.shape[-1]), targets.view(-1))
            loss.backward()
            for p_ in model.parameters():
                p_.grad = None
            return loss

        compiled = torch.compile(model, backend=mojo_backend)
        t0 = time.perf_counter()
        loss_c = train_step(compiled).item()
        compile_s = time.perf_counter() - t0
        wall, _ = timed(lambda: train_step(compiled), 5, 2)

        # the same step with the loss inside the compiled graph (log-softmax forward and backward
        # over the vocabulary then run on this library's kernels too)
        def loss_of(i_, t_):
            logits, _ = model(i_)
            return F.cross_entropy(logits.view(-1, logits.shape[-1]), t_.view(-1))

        def train_step_whole(fn):
            loss = fn(idx, targets)
            loss.backward()
            for p_ in model.parameters():
                p_.grad = None
            return loss

        compiled_loss = torch.compile(loss_of, backend=mojo_backend)
        loss_w = train_step_whole(compiled_loss).item()
        wall_w, _ = timed(lambda: train_step_whole(compiled_loss), 5, 2)
        loss_e = train_step(model).item()
        wall_e, _ = timed(lambda: train_step(model), 5, 2)
        # forward FLOPs of the projections and attention; backward = 2x
        fwd_flops = 12 * (2 * B * T * 7077888) + 12 * (2 * 2 * B * 12 * T * T * 64) + 2 * B * T * 768 * 50257
        sweep[f"gpt2_small_train_step_bf16_B{B}_T{T}"] = {
            "tokens/s": round(B * T / (wall * 1e-3), 1), "ms_per_step": round(wall, 3),
            "TFLOP/s_over_whole_step": round(3 * fwd_flops / (wall * 1e-3) / 1e12, 2),
            "ms_per_step_loss_in_graph": round(wall_w, 3), "loss_in_graph": round(loss_w, 4),
            "pytorch_rocm_eager_ms_per_step": round(wall_e, 3), "compile_s": round(compile_s, 2),
            "loss": round(loss_c, 4), "pytorch_rocm_eager_loss": round(loss_e, 4),
            "batch": B, "seq": T, "dtype": "bf16",
            "note": "forward + backward through mojo_backend, no optimizer step"}
        del model, compiled

    # ------------------------------------------------------------------ eager decode loop
    # The reference's own eager benchmark (bench_gpt2_batch.py / current_bench/: HF GPT-2
    # `generate`, greedy, batch 512, prompt 8, 200 new tokens, bf16), with random-init weights
    # of the same architecture (no checkpoint offline), on the `mojo` device. Host-bound: about
    # 480 aten calls per decoded token; PyTorch-ROCm's own eager run is timed beside it.
    if want in ("all", "generate"):
        try:
            from transformers import GPT2Config, GPT2LMHeadModel
        except Exception as exc:  # noqa: BLE001
            sweep["gpt2_hf_generate_bf16_B512_eager"] = {"skipped": f"transformers not importable: {exc}"}
        else:
            from torch_mojo_backend import register_mojo_devices

            register_mojo_devices()
            torch.manual_seed(0)
            B, P, NEW = 512, 8, 200
            hf = GPT2LMHeadModel(GPT2Config()).eval().to(torch.bfloat16)
            ids = torch.randint(0, 50257, (B, P))
            mask = torch.ones_like(ids)

            def gen_rate(device):
                mdl, i, a = hf.to(device), ids.to(device), mask.to(device)
                kw = dict(do_sample=False, pad_token_id=50256, attention_mask=a)
                with torch.no_grad():
                    mdl.generate(i, max_new_tokens=8, min_new_tokens=8, **kw)
                    sync()
                    t0 = time.perf_counter()
                    mdl.generate(i, max_new_tokens=NEW, min_new_tokens=NEW, **kw)
                    sync()
                return B * NEW / (time.perf_counter() - t0)

            rocm = gen_rate(dev)
            ours = gen_rate("mojo")

            def host_breakdown(steps=40):
                """Host microseconds per call inside the registered implementations, by op, over
                `steps` decoded tokens (the time between a call from __torch_dispatch__ and its
                return; PyTorch's own dispatch and the model's Python come on top)."""
                from torch_mojo_backend.mojo_device import torch_mojo_tensor as tmt

                calls, spent = {}, {}
                saved = dict(tmt.DIRECT_IMPLS)

                def timed_impl(name, fn):
                    def run(*a, **k):
                        t = time.perf_counter()
                        out = fn(*a, **k)
                        spent[name] = spent.get(name, 0.0) + time.perf_counter() - t
                        calls[name] = calls.get(name, 0) + 1
                        return out
                    return run

                mdl, i, a = hf.to("mojo"), ids.to("mojo"), mask.to("mojo")
                try:
                    for op, fn in saved.items():
                        tmt.DIRECT_IMPLS[op] = timed_impl(str(op), fn)
                    with torch.no_grad():
                        mdl.generate(i, max_new_tokens=steps, min_new_tokens=steps, do_sample=False,
                                     pad_token_id=50256, attention_mask=a)
                        sync()
                finally:
                    tmt.DIRECT_IMPLS.update(saved)
                top = sorted(spent, key=spent.get, reverse=True)[:10]
                return {"ops_per_step": round(sum(calls.values()) / steps, 1),
                        "impl_ms_per_step": round(sum(spent.values()) / steps * 1e3, 3),
                        "top": {n: {"calls_per_step": round(calls[n] / steps, 1),
                                    "us_per_call": round(spent[n] / calls[n] * 1e6, 2)} for n in top}}

            sweep["gpt2_hf_generate_bf16_B512_eager"] = {
                "tokens/s": round(ours, 1), "ms_per_decode_step": round(B / ours * 1e3, 3),
                "pytorch_rocm_eager_tokens/s": round(rocm, 1),
                "vs_pytorch_rocm_eager": round(ours / rocm, 4), "batch": B, "prompt": P,
                "new_tokens": NEW, "dtype": "bf16", "host": host_breakdown(),
                "note": "HF GPT2LMHeadModel.generate on the eager mojo device, random-init weights"}
            del hf

    line = {
        "metric": "GEMM TFLOP/s (bf16 addmm M=N=K=8192, fp32 accumulate)",
        "value": None if value is None else round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": None if wall_ms is None else round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "standalone op sweep: aten.addmm bf16, (M,N,K)=(8192,8192,8192), "
                               "bias [N], seeded N(0,1) inputs resident in HBM",
                   "device": props.name, "compute_units": props.multi_processor_count,
                   "host_threads": cpu_threads, "preheat_launches": PREHEAT},
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "sweep": sweep,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
