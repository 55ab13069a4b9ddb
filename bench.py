#!/usr/bin/env python3
"""Benchmark of the two hot paths on one MI355X, through the C ABI (include/ahpc_hip.h).

Headline (the JSON line's metric/value): FlashAttention forward, bf16, causal, B=4, N=4096, H=32,
d=128, layout [B,N,H,d] - one "step" is one forward over that batch.  The same line carries the
PagedAttention decode result (fp16, B=64, H=32, d=128, page 16, context lengths U[512,4096]) under
"decode".  Inputs are synthetic and already resident in HBM when the timed region starts.

  value            whole-job throughput: algorithmic FLOP (2*B*H*N^2*d for causal) / wall time of the
                   K timed steps, bracketed by a device synchronize on both sides
  settle_ms        untimed launches of the same workload for that long in front of the W warm-up steps: the board's
                   clocks come out of idle over tens of milliseconds, whatever W is (see settle())
  roofline         algorithmic FLOP (or bytes) per launch / mean kernel duration measured with HIP
                   events on the launch stream, against MI355X's dense bf16 MFMA peak (2.5 PFLOP/s)
                   or HBM peak (8 TB/s)
  cpu_baseline     the CPU oracle (oracle/, a restatement of the reference's algorithm) timed on this
                   box's host cores over a bounded sample of the same workload: on all cores (OpenMP over rows)
                   and, under "single_thread", on one core as the reference's own CPU path runs
  extras           the other configurations (long-context decode, ragged prefill, backward, grouped heads,
                   batched append), one row each, timed in the same run

`--workload calib` prints yardsticks of the box (device copy, streaming read, the vendor library's bf16 matrix product,
matrix instructions only); `--workload sensors` prints the shader clock and board power the driver reports while the
headline forward, that matrix product and a device copy each run back to back for a few seconds.

Inputs of the two headline workloads come from the oracle's seeded generator (splitmix64 + Box-Muller, seeds
0xA77E0002 / 0xA77E0003, tensor ids 1-5), rounded to the storage type on the host, so that the CPU legs and the
GPU see the same values; the extras draw theirs with torch.randn on the GPU.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16/fp16
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of exactly these workloads (each counter
# scaled by its reading for a 1 GiB device copy).  The figure is not re-measured by this script: it is read from the
# committed summary of those runs, together with the kernel it was taken for, and reported as null when that summary
# is missing or names another kernel.
PROFILE_FLASH = os.path.join(ROOT, "profiles", "flash_fwd_wide_bf16_d128_causal_B4_N4096_H32.txt")
PROFILE_DECODE = os.path.join(ROOT, "profiles", "paged_decode_f16_d128_B64_ctx512-4096.txt")


def traffic_from_profile(path, kernel_word):
    """(bytes per launch, provenance) from the lines `traffic_bytes_per_launch = N` and `measured = ...` of a profile
    summary whose `kernel = ...` line contains kernel_word; (None, reason) otherwise."""
    try:
        text = open(path).read()
    except OSError:
        return None, "no profile summary at " + os.path.relpath(path, ROOT)
    fields = {}
    for line in text.splitlines():
        if " = " in line and not line.startswith(" "):
            k, v = line.split(" = ", 1)
            fields[k.strip()] = v.strip()
    if kernel_word not in fields.get("kernel", ""):
        return None, "profile summary is for another kernel: " + fields.get("kernel", "?")
    try:
        return int(fields["traffic_bytes_per_launch"]), os.path.relpath(path, ROOT) + " (" + fields.get("measured", "undated") + ")"
    except (KeyError, ValueError):
        return None, "profile summary holds no traffic figure"


FLASH = dict(B=4, N=4096, H=32, d=128, causal=True, dtype="bf16", seed=0xA77E0002)
DECODE = dict(B=64, H=32, d=128, P=16, lo=512, hi=4096, dtype="fp16", seed=0xA77E0003)


def lengths_and_table(cfg):
    """Seeded context lengths (tensor id 4) and a block table that is a slice of a seeded permutation of the page
    ids (tensor id 5), both from the oracle's generator."""
    from oracle import oracle as O
    lens = O.fill_lengths(cfg["B"], cfg["seed"], 4, cfg["lo"], cfg["hi"])
    P = cfg["P"]
    pages_per = (lens + P - 1) // P
    n_pages = int(pages_per.sum()) + 64
    ids = O.permutation(n_pages, cfg["seed"], 5)
    table = np.full((cfg["B"], int(pages_per.max())), -1, np.int32)
    c = 0
    for b in range(cfg["B"]):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    return lens, table, n_pages


def decode_bytes(lens, cfg):
    """Algorithmic bytes of one decode step: K and V of every cached token once, q and o once, the
    block-table entries and lengths once."""
    H, d, P, B = cfg["H"], cfg["d"], cfg["P"], cfg["B"]
    esz = 2
    L = lens.astype(np.int64)
    return int((2 * L * H * d * esz).sum() + 2 * B * H * d * esz + 4 * ((L + P - 1) // P).sum() + 4 * B)


class Timer:
    """HIP events on the launch stream (torch's events only see torch's own current stream)."""

    def __init__(self, hip, stream, n):
        import ctypes as C
        self.hip, self.stream, self.C = hip, stream, C
        self.lib = hip.load()
        self.ev = []
        for _ in range(2 * n):
            e = C.c_void_p()
            assert self.lib.ahpc_hip_event_create(C.byref(e)) == 0
            self.ev.append(e)

    def record(self, i):
        assert self.lib.ahpc_hip_event_record(self.ev[i], self.stream) == 0

    def elapsed_ms(self, i, j):
        ms = self.C.c_float()
        assert self.lib.ahpc_hip_event_synchronize(self.ev[j]) == 0
        assert self.lib.ahpc_hip_event_elapsed_ms(self.ev[i], self.ev[j], self.C.byref(ms)) == 0
        return ms.value

    def close(self):
        for e in self.ev:
            self.lib.ahpc_hip_event_destroy(e)


SETTLE_MS = 60.0  # untimed launches in front of every workload's warm-up, see settle()


def settle(hip, stream, launch):
    """Untimed launches for SETTLE_MS of wall clock (at most 400), in front of the W warm-up steps.  The board comes out
    of idle at a low shader clock and its power management needs some tens of milliseconds of load to arrive where it
    stays: the first 25 launches of the headline forward after idle average 0.61 ms, the next 25 0.58 ms, those after
    the first 50 0.52 ms, as do those after 1000.  W is the caller's; this phase makes what follows independent of it."""
    lib = hip.load()
    t0 = time.perf_counter()
    n = 0
    while n < 400 and (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(10):
            launch()
        assert lib.ahpc_hip_stream_synchronize(stream) == 0
        n += 10
    return n


def timed_steps(hip, stream, launch, steps, warmup):
    """Settling launches (see settle), W untimed launches, then exactly K timed ones: wall clock around all K
    (synchronised on both sides) and an event pair around each launch."""
    import torch
    lib = hip.load()
    # The workloads' tensors are made on torch's stream and the launches go to a stream of their own, which does not wait
    # for it: without this, the first launches overlap the kernels that still fill the inputs, and an output tensor that
    # torch's allocator carved out of a block whose last reader is still pending is written under that reader's feet.
    torch.cuda.synchronize()
    settle(hip, stream, launch)
    for _ in range(warmup):
        launch()
    assert lib.ahpc_hip_stream_synchronize(stream) == 0
    torch.cuda.synchronize()
    t = Timer(hip, stream, steps)
    t0 = time.perf_counter()
    for i in range(steps):
        t.record(2 * i)
        launch()
        t.record(2 * i + 1)
    assert lib.ahpc_hip_stream_synchronize(stream) == 0
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = [t.elapsed_ms(2 * i, 2 * i + 1) for i in range(steps)]
    t.close()
    return wall, per


def seeded_tensor(shape, seed, tensor_id, torch_dtype, code, keep_host=False, sigma=1.0):
    """N(0, sigma) from the oracle's generator, rounded to the storage type on the host, on the GPU.  Generated in
    pieces of 32 Mi elements so that the host never holds more than one piece (unless keep_host)."""
    import torch
    from oracle import oracle as O
    n = int(np.prod(shape))
    dev = torch.empty(n, dtype=torch_dtype, device="cuda")
    host = np.empty(n, np.float32) if keep_host else None
    piece = 1 << 25
    buf = np.empty(min(piece, n), np.float32)
    for first in range(0, n, piece):
        m = min(piece, n - first)
        x = O.fill_normal_at(buf[:m], seed, tensor_id, sigma, first)
        x = O.round_to(x, code)
        dev[first:first + m] = torch.from_numpy(x).to(torch_dtype)
        if keep_host:
            host[first:first + m] = x
    return dev.view(*shape), (host.reshape(shape) if keep_host else None)


def bench_flash(hip, stream, steps, warmup, cpu):
    import torch
    from oracle import oracle as O
    c = FLASH
    B, N, H, d = c["B"], c["N"], c["H"], c["d"]
    (q, qh), (k, kh), (v, vh) = (seeded_tensor((B, N, H, d), c["seed"], t, torch.bfloat16, O.BF16, keep_host=cpu) for t in (1, 2, 3))
    o = torch.empty_like(q)
    torch.cuda.synchronize()
    scale = 1.0 / np.sqrt(d)
    strides = (N * H * d, H * d, d)

    def launch():
        hip.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, d, strides, scale, True, stream)

    wall, per = timed_steps(hip, stream, launch, steps, warmup)
    flops = 2.0 * B * H * N * N * d            # causal convention; exact count 4*B*H*d*N(N+1)/2 is 0.02% higher
    value = flops * steps / wall / 1e12
    kern_ms = float(np.mean(per))
    achieved = flops / (kern_ms * 1e-3) / 1e12
    # the kernel this shape takes by default (256 query rows per workgroup); the tuning value flash_rows = 128 asks for the other
    wide = hip.get_tuning("flash_rows") != 128
    kernel_name = "flash_fwd_wide_kernel" if wide else "flash_fwd_mfma_kernel"
    flash_traffic, flash_traffic_src = traffic_from_profile(PROFILE_FLASH, kernel_name)
    res = {
        "metric": "FlashAttn fwd TFLOP/s (bf16, N=4096, d=128)", "value": round(value, 2), "unit": "TFLOP/s",
        "ms_per_step": round(wall / steps * 1e3, 4),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_PEAK_TFLOPS, 4), "traffic": flash_traffic, "traffic_source": flash_traffic_src,
                     "kernel": kernel_name + "<bf16,128,causal>", "kernel_ms_mean": round(kern_ms, 4),
                     "kernel_ms_median": round(float(np.median(per)), 4), "kernel_ms_min": round(float(np.min(per)), 4), "flop_per_launch": flops},
        "config": {"workload": "flash_fwd bf16 causal B=4 N=4096 H=32 d=128 layout [B,N,H,d], fp32 accumulate, bf16 out"},
    }
    if cpu:
        # all cores: the whole step (the same rounded inputs the GPU got), OpenMP over rows
        nb, reps = 4, 3
        threads = O.cpu_threads()
        t0 = time.perf_counter()
        for _ in range(reps):
            ref = O.attention(qh, kh, vh, nb, N, H, d, scale, True, threads=threads)
        dt = (time.perf_counter() - t0) / reps
        err = float(np.abs(o[0:nb].float().cpu().numpy() - ref).max())
        res["cpu_baseline"] = {"value": round(2.0 * nb * H * N * N * d / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
                               "kind": "port", "sample": f"the whole step ({nb}x32 heads x 4096 rows), mean of {reps} passes of "
                               f"{dt:.1f} s wall on {threads} threads", "max_abs_err_gpu_vs_cpu": err}
        # one core, as the reference's CPU path runs (it has no threading): 1/128 of the step - one head of one batch
        # entry, all 4096 rows - and the reference's own CPU-sized configuration in full
        q1, k1, v1 = (np.ascontiguousarray(x[0:1, :, 0:1, :]) for x in (qh, kh, vh))
        t0 = time.perf_counter()
        O.attention(q1, k1, v1, 1, N, 1, d, scale, True, threads=1)
        dt1 = time.perf_counter() - t0
        Bc, Nc, Hc, dc = 2, 512, 8, 64
        qc, kc, vc = (O.fill_normal((Bc, Nc, Hc, dc), 0xA77E0001, t) for t in (1, 2, 3))
        t0 = time.perf_counter()
        O.attention(qc, kc, vc, Bc, Nc, Hc, dc, 1.0 / np.sqrt(dc), False, threads=1)
        dtc = time.perf_counter() - t0
        res["cpu_baseline"]["single_thread"] = {
            "value": round(2.0 * N * N * d / dt1 / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
            "sample": f"1/128 of the step (batch entry 0, head 0, 4096 rows), one pass of {dt1:.2f} s; the whole step "
                      f"extrapolates to {dt1 * B * H:.0f} s",
            "reference_cpu_config": {"workload": "flash_fwd fp32 non-causal B=2 N=512 H=8 d=64 (in full)", "seconds": round(dtc, 3),
                                     "value": round(4.0 * Bc * Hc * Nc * Nc * dc / dtc / 1e12, 6), "unit": "TFLOP/s"}}
    return res


def bench_decode(hip, stream, steps, warmup, cpu):
    import torch
    c = DECODE
    B, H, d, P = c["B"], c["H"], c["d"], c["P"]
    from oracle import oracle as O
    lens, table, n_pages = lengths_and_table(c)
    elems = n_pages * P * H * d
    kpool, _ = seeded_tensor((elems,), c["seed"], 2, torch.float16, O.F16)
    vpool, _ = seeded_tensor((elems,), c["seed"], 3, torch.float16, O.F16)
    q, _ = seeded_tensor((B, H, d), c["seed"], 1, torch.float16, O.F16)
    o = torch.empty_like(q)
    dt_, dl = torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda()
    max_len, max_pages = int(lens.max()), table.shape[1]
    ws_bytes = hip.paged_decode_workspace_bytes(B, H, d, max_len, P, 0)
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    scale = 1.0 / np.sqrt(d)

    def launch():
        hip.paged_decode(q.data_ptr(), o.data_ptr(), hip.F16, kpool.data_ptr(), vpool.data_ptr(), hip.F16, dt_.data_ptr(),
                         dl.data_ptr(), None, B, H, d, P, max_pages, max_len, scale, 0, ws.data_ptr(), ws_bytes, stream)

    wall, per = timed_steps(hip, stream, launch, steps, warmup)
    nbytes = decode_bytes(lens, c)
    value = nbytes * steps / wall / 1e9
    kern_ms = float(np.mean(per))
    achieved = nbytes / (kern_ms * 1e-3) / 1e9
    decode_traffic, decode_traffic_src = traffic_from_profile(PROFILE_DECODE, "paged_decode_kernel")
    res = {
        "metric": "paged decode HBM GB/s", "value": round(value, 1), "unit": "GB/s",
        "ms_per_step": round(wall / steps * 1e3, 4),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": decode_traffic, "traffic_source": decode_traffic_src,
                     "kernel": "paged_decode_kernel<f16,128> + paged_merge_kernel", "kernel_ms_mean": round(kern_ms, 4),
                     "kernel_ms_median": round(float(np.median(per)), 4), "kernel_ms_min": round(float(np.min(per)), 4), "bytes_per_launch": nbytes},
        "config": {"workload": f"paged_decode fp16 B=64 H=32 d=128 page=16 context U[512,4096] (sum {int(lens.sum())} tokens), "
                               f"shuffled block table, pool {n_pages} pages"},
    }
    if cpu:
        # bounded sample: the first 32 of the 64 sequences, their pages copied to the host; 200 passes
        nb = 32
        pages_per = (lens + P - 1) // P
        sub_tables, kparts, vparts, c0 = [], [], [], 0
        for b in range(nb):
            pg = torch.from_numpy(table[b, :pages_per[b]].astype(np.int64)).cuda()
            kparts.append(kpool.view(n_pages, -1)[pg].float().cpu().numpy().reshape(-1))
            vparts.append(vpool.view(n_pages, -1)[pg].float().cpu().numpy().reshape(-1))
            sub_tables.append(np.arange(c0, c0 + pages_per[b], dtype=np.int32))
            c0 += int(pages_per[b])
        st = np.full((nb, int(pages_per[:nb].max())), -1, np.int32)
        for b in range(nb):
            st[b, :pages_per[b]] = sub_tables[b]
        kh, vh = np.concatenate(kparts), np.concatenate(vparts)
        qh = q[:nb].float().cpu().numpy()
        threads = O.cpu_threads()
        reps = 200
        t0 = time.perf_counter()
        for _ in range(reps):
            ref = O.paged_decode(qh, kh, vh, st, lens[:nb], None, nb, H, d, P, scale, threads=threads)
        dt = (time.perf_counter() - t0) / reps
        sub = dict(c, B=nb)
        err = float(np.abs(o[:nb].float().cpu().numpy() - ref).max())
        res["cpu_baseline"] = {"value": round(decode_bytes(lens[:nb], sub) / dt / 1e9, 3), "unit": "GB/s", "cores": threads,
                               "kind": "port", "sample": f"first {nb} of 64 sequences ({int(lens[:nb].sum())} tokens), mean of "
                               f"{reps} passes of {dt:.2f} s on {threads} threads; bytes counted at the GPU's 2-byte storage size "
                               "(the CPU path streams fp32 copies, twice as many bytes)", "max_abs_err_gpu_vs_cpu": err}
        reps1 = 10
        t0 = time.perf_counter()
        for _ in range(reps1):
            O.paged_decode(qh, kh, vh, st, lens[:nb], None, nb, H, d, P, scale, threads=1)
        dt1 = (time.perf_counter() - t0) / reps1
        res["cpu_baseline"]["single_thread"] = {"value": round(decode_bytes(lens[:nb], sub) / dt1 / 1e9, 3), "unit": "GB/s", "cores": 1,
                                                "sample": f"the same {nb} sequences, mean of {reps1} passes of {dt1:.2f} s on one thread"}
    return res


def bench_extras(hip, stream, steps, warmup):
    """The other BASELINE configurations and the widened paths, one row each (not the headline)."""
    import torch
    rows = []
    g = torch.Generator(device="cuda").manual_seed(0xA77E0009)

    def randn(shape, dtype):
        return torch.randn(shape, generator=g, device="cuda", dtype=torch.float32).to(dtype)

    def run(name, launch, flops=None, nbytes=None, fp32=False):
        wall, per = timed_steps(hip, stream, launch, steps, warmup)
        ms = float(np.mean(per))
        row = {"workload": name, "kernel_ms_mean": round(ms, 4), "kernel_ms_median": round(float(np.median(per)), 4),
               "kernel_ms_min": round(float(np.min(per)), 4)}
        if flops:
            row["TFLOP/s"] = round(flops / (ms * 1e-3) / 1e12, 1)
            if fp32:  # fp32 matrix instructions: MI355X's published dense fp32 peak
                row["frac_of_157.3_TFLOP/s_fp32"] = round(flops / (ms * 1e-3) / 1e12 / 157.3, 4)
            else:
                row["frac_of_2.5_PFLOP/s"] = round(flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)
        if nbytes:
            row["GB/s"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
            row["frac_of_8_TB/s"] = round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        rows.append(row)

    # flash forward, same shape as the headline: non-causal, fp16, grouped K/V heads
    B, N, H, d = 4, 4096, 32, 128
    q = randn((B, N, H, d), torch.bfloat16); k = randn((B, N, H, d), torch.bfloat16); v = randn((B, N, H, d), torch.bfloat16)
    o = torch.empty_like(q)
    sc = 1.0 / np.sqrt(d)
    st = (N * H * d, H * d, d)
    run("flash_fwd bf16 non-causal B=4 N=4096 H=32 d=128",
        lambda: hip.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, d, st, sc, False, stream),
        flops=4.0 * B * H * N * N * d)
    qh, kh, vh = q.to(torch.float16), k.to(torch.float16), v.to(torch.float16)
    run("flash_fwd fp16 causal B=4 N=4096 H=32 d=128",
        lambda: hip.flash_fwd(qh.data_ptr(), kh.data_ptr(), vh.data_ptr(), o.data_ptr(), hip.F16, B, N, H, d, st, sc, True, stream),
        flops=2.0 * B * H * N * N * d)
    Hkv = 8
    kg, vg = randn((B, N, Hkv, d), torch.bfloat16), randn((B, N, Hkv, d), torch.bfloat16)
    run("flash_fwd bf16 causal B=4 N=4096 H=32 (8 K/V heads) d=128",
        lambda: hip.flash_fwd_gqa(q.data_ptr(), kg.data_ptr(), vg.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, Hkv, d, st,
                                  (N * Hkv * d, Hkv * d, d), sc, True, stream),
        flops=2.0 * B * H * N * N * d)

    # one long sequence (1 x 32768 tokens, 16 times the headline's work): a workgroup walks 8 times as many key tiles
    # per query tile, so what a query tile and a launch cost at their start and end weighs less
    Nl = 32768
    ql, kl, vl = (randn((1, Nl, H, d), torch.bfloat16) for _ in range(3))
    ol = torch.empty_like(ql)
    stl = (Nl * H * d, H * d, d)
    run("flash_fwd bf16 causal B=1 N=32768 H=32 d=128 (one long sequence)",
        lambda: hip.flash_fwd(ql.data_ptr(), kl.data_ptr(), vl.data_ptr(), ol.data_ptr(), hip.BF16, 1, Nl, H, d, stl, sc, True, stream),
        flops=2.0 * H * Nl * Nl * d)
    del ql, kl, vl, ol

    # head dimension 256 (half the heads, the same tensor sizes): the 16-bit kernel's instantiation with one workgroup per CU
    Hw, dw = 16, 256
    qw, kw, vw = (randn((B, N, Hw, dw), torch.bfloat16) for _ in range(3))
    ow = torch.empty_like(qw)
    stw = (N * Hw * dw, Hw * dw, dw)
    run("flash_fwd bf16 causal B=4 N=4096 H=16 d=256",
        lambda: hip.flash_fwd(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), ow.data_ptr(), hip.BF16, B, N, Hw, dw, stw, 1.0 / np.sqrt(dw), True,
                              stream),
        flops=2.0 * B * Hw * N * N * dw)
    del qw, kw, vw, ow

    # the headline shape in fp32, the reference's default data type: the fp32 matrix-core kernel
    qf, kf, vf = randn((B, N, H, d), torch.float32), randn((B, N, H, d), torch.float32), randn((B, N, H, d), torch.float32)
    of = torch.empty_like(qf)
    run("flash_fwd fp32 causal B=4 N=4096 H=32 d=128",
        lambda: hip.flash_fwd(qf.data_ptr(), kf.data_ptr(), vf.data_ptr(), of.data_ptr(), hip.F32, B, N, H, d, st, sc, True, stream),
        flops=2.0 * B * H * N * N * d, fp32=True)
    del qf, kf, vf, of

    # backward at the headline shape.  FLOP by the usual convention: 2.5 x the forward's (five products
    # against two); the three launches here execute nine, because the interface passes neither the forward
    # output nor its softmax statistics and they are recomputed, and the dK/dV walk recomputes the scores as dQ does.
    go = randn((B, N, H, d), torch.bfloat16)
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    wsb = hip.flash_bwd_workspace_bytes(B, N, H)
    wsf = torch.empty(wsb // 4, dtype=torch.float32, device="cuda")
    run("flash_bwd bf16 causal B=4 N=4096 H=32 d=128",
        lambda: hip.flash_bwd(go.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), gq.data_ptr(), gk.data_ptr(),
                              gv.data_ptr(), hip.BF16, B, N, H, H, d, st, st, sc, True, wsf.data_ptr(), wsb, stream),
        flops=2.5 * 2.0 * B * H * N * N * d)

    # the same backward after a forward that kept its row statistics (ahpc_hip_flash_fwd_keep / _bwd_kept: an extension of
    # the reference's interface): no statistics launch, seven products instead of nine
    rs = torch.empty(hip.flash_row_stats_bytes(B, N, H) // 4, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    kept = hip.flash_fwd_keep(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, H, d, st, st, sc, True,
                              rs.data_ptr(), stream)
    assert hip.load().ahpc_hip_stream_synchronize(stream) == 0 and kept
    run("flash_bwd bf16 causal B=4 N=4096 H=32 d=128 on the forward's kept row statistics and output",
        lambda: hip.flash_bwd_kept(go.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), rs.data_ptr(),
                                   gq.data_ptr(), gk.data_ptr(), gv.data_ptr(), hip.BF16, B, N, H, H, d, st, st, sc, True,
                                   wsf.data_ptr(), wsb, stream),
        flops=2.5 * 2.0 * B * H * N * N * d)
    run("flash_fwd bf16 causal B=4 N=4096 H=32 d=128 keeping its row statistics",
        lambda: hip.flash_fwd_keep(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, H, d, st, st, sc, True,
                                   rs.data_ptr(), stream),
        flops=2.0 * B * H * N * N * d)

    # backward with head dimension 256 (half the heads, the same tensor sizes): one workgroup per CU, dK and dV in two walks
    qw, kw, vw, gow = (randn((B, N, 16, 256), torch.bfloat16) for _ in range(4))
    gqw, gkw, gvw = torch.empty_like(qw), torch.empty_like(kw), torch.empty_like(vw)
    stw = (N * 16 * 256, 16 * 256, 256)
    wsw = torch.empty(hip.flash_bwd_workspace_bytes(B, N, 16) // 4, dtype=torch.float32, device="cuda")
    run("flash_bwd bf16 causal B=4 N=4096 H=16 d=256",
        lambda: hip.flash_bwd(gow.data_ptr(), qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), gqw.data_ptr(), gkw.data_ptr(),
                              gvw.data_ptr(), hip.BF16, B, N, 16, 16, 256, stw, stw, 1.0 / 16.0, True, wsw.data_ptr(),
                              wsw.numel() * 4, stream),
        flops=2.5 * 2.0 * B * 16 * N * N * 256)
    del qw, kw, vw, gow, gqw, gkw, gvw, wsw

    # the same backward in fp32 (fp32 matrix-core kernels; dK and dV always in two walks)
    qf, kf, vf, gof = (randn((B, N, H, d), torch.float32) for _ in range(4))
    gqf, gkf, gvf = torch.empty_like(qf), torch.empty_like(kf), torch.empty_like(vf)
    run("flash_bwd fp32 causal B=4 N=4096 H=32 d=128",
        lambda: hip.flash_bwd(gof.data_ptr(), qf.data_ptr(), kf.data_ptr(), vf.data_ptr(), gqf.data_ptr(), gkf.data_ptr(),
                              gvf.data_ptr(), hip.F32, B, N, H, H, d, st, st, sc, True, wsf.data_ptr(), wsb, stream),
        flops=2.5 * 2.0 * B * H * N * N * d, fp32=True)
    del qf, kf, vf, gof, gqf, gkf, gvf

    # the headline shape, non-causal, with a dense random mask [B,N,N] (half the keys removed; flops counted as unmasked)
    dmask = (torch.rand((B, N, N), generator=g, device="cuda") > 0.5).float()
    run("flash_fwd bf16 non-causal B=4 N=4096 H=32 d=128 with a dense fp32 mask [B,N,N]",
        lambda: hip.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, d, st, sc, False, stream,
                              dmask.data_ptr()),
        flops=4.0 * B * H * N * N * d)
    run("flash_bwd bf16 non-causal B=4 N=4096 H=32 d=128 with a dense fp32 mask [B,N,N]",
        lambda: hip.flash_bwd(go.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), gq.data_ptr(), gk.data_ptr(),
                              gv.data_ptr(), hip.BF16, B, N, H, H, d, st, st, sc, False, wsf.data_ptr(), wsb, stream,
                              dmask.data_ptr()),
        flops=2.5 * 4.0 * B * H * N * N * d)
    del dmask

    # ragged fp16 causal batch: 16 sequences, lengths U[128,8192], H=32, d=64 (sigma 0.5)
    from oracle import oracle as O
    lens = O.fill_lengths(16, 0xA77E0005, 4, 128, 8192)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, Hv, dv_ = int(cu[-1]), 32, 64
    qv = (randn((T, Hv, dv_), torch.float32) * 0.5).to(torch.float16)
    kv = (randn((T, Hv, dv_), torch.float32) * 0.5).to(torch.float16)
    vv = (randn((T, Hv, dv_), torch.float32) * 0.5).to(torch.float16)
    ov = torch.empty_like(qv)
    dcu = torch.from_numpy(cu).cuda()
    L = lens.astype(np.float64)
    run(f"flash_fwd_varlen fp16 causal 16 seqs U[128,8192] ({T} tokens) H=32 d=64 (BASELINE config 5)",
        lambda: hip.flash_fwd_varlen(qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), ov.data_ptr(), hip.F16, dcu.data_ptr(), 16,
                                     int(lens.max()), Hv, dv_, Hv * dv_, dv_, 1.0 / np.sqrt(dv_), True, stream),
        flops=float((4.0 * Hv * dv_ * L * (L + 1) / 2).sum()))

    # decode: long contexts (bf16, B=8, U[16384,32768]) and grouped heads (H=32 over 8 pool heads)
    def decode_case(name, cfg, Hq, Hp, dtype_code, tdtype):
        lens, table, n_pages = lengths_and_table(cfg)
        P = cfg["P"]
        elems = n_pages * P * Hp * cfg["d"]
        kp, vp = randn(elems, tdtype), randn(elems, tdtype)
        qd = randn((cfg["B"], Hq, cfg["d"]), tdtype)
        od = torch.empty_like(qd)
        dt_, dl = torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda()
        max_len = int(lens.max())
        wsb = hip.paged_decode_workspace_bytes(cfg["B"], Hq, cfg["d"], max_len, P, 0)
        ws = torch.empty(max(wsb, 4) // 4, dtype=torch.float32, device="cuda")
        scl = 1.0 / np.sqrt(cfg["d"])
        nb = decode_bytes(lens, dict(cfg, H=Hp)) + 2 * cfg["B"] * (Hq - Hp) * cfg["d"] * 2
        run(name + f" (sum {int(lens.sum())} tokens)",
            lambda: hip.paged_decode_gqa(qd.data_ptr(), od.data_ptr(), dtype_code, kp.data_ptr(), vp.data_ptr(), dtype_code,
                                         dt_.data_ptr(), dl.data_ptr(), None, cfg["B"], Hq, Hp, cfg["d"], P, table.shape[1],
                                         max_len, scl, 0, ws.data_ptr(), wsb, stream),
            nbytes=nb)

    decode_case("paged_decode bf16 B=8 H=32 d=128 page=16 context U[16384,32768] (BASELINE config 4)",
                dict(B=8, H=32, d=128, P=16, lo=16384, hi=32768, seed=0xA77E0004), 32, 32, hip.BF16, torch.bfloat16)
    decode_case("paged_decode fp16 B=64 H=32 over 8 pool heads d=128 page=16 context U[512,4096]",
                dict(DECODE), 32, 8, hip.F16, torch.float16)
    # the same at a quarter of the batch: a launch with fewer workgroups than CUs, which gets narrower workgroups
    decode_case("paged_decode fp16 B=16 H=32 over 8 pool heads d=128 page=16 context U[512,4096]",
                dict(DECODE, B=16), 32, 8, hip.F16, torch.float16)
    # multi-query decode (32 query heads over one pool head): the matrix-core kernel
    decode_case("paged_decode (matrix-core kernel) fp16 B=64 H=32 over 1 pool head d=128 page=16 context U[512,4096]",
                dict(DECODE), 32, 1, hip.F16, torch.float16)
    # the same with long contexts: 814 MB instead of 82 MB, enough for the stream to set the time
    decode_case("paged_decode (matrix-core kernel) fp16 B=64 H=32 over 1 pool head d=128 page=16 context U[16384,32768]",
                dict(DECODE, lo=16384, hi=32768), 32, 1, hip.F16, torch.float16)

    # prefill -> cache hand-off: K and V of the headline prefill into the pool, one launch
    P = 16
    pages_per = N // P
    table = torch.randperm(B * pages_per, generator=torch.Generator().manual_seed(5)).to(torch.int32).reshape(B, pages_per).cuda()
    kpool = torch.empty(B * pages_per * P * H * d, dtype=torch.bfloat16, device="cuda")
    vpool = torch.empty_like(kpool)
    rows_ = torch.arange(B, dtype=torch.int32, device="cuda")
    run("kv_scatter_batch bf16 B=4 N=4096 H=32 d=128 -> pool (page 16)",
        lambda: hip.kv_scatter_batch(k.data_ptr(), v.data_ptr(), hip.BF16, N * H * d, H * d, kpool.data_ptr(), vpool.data_ptr(),
                                     hip.BF16, table.data_ptr(), pages_per, rows_.data_ptr(), B, N, H, d, P, stream=stream),
        nbytes=4 * B * N * H * d * 2)

    # Context, not product: what the vendor library's plain bf16 matrix product sustains on this box.  The board holds
    # its power limit under matrix load and lowers the shader clock, so this, not the 2.4-GHz figure, is what a kernel
    # that is nothing but matrix instructions reaches here.  Timed with torch's events on torch's stream.
    M = 8192
    a, b_ = randn((M, M), torch.bfloat16), randn((M, M), torch.bfloat16)
    for _ in range(5):
        torch.matmul(a, b_)
    torch.cuda.synchronize()
    reps = max(10, steps)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        torch.matmul(a, b_)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    rows.append({"workload": "context: torch.matmul bf16 8192x8192x8192 (hipBLASLt), not part of the product",
                 "kernel_ms_mean": round(ms, 4), "TFLOP/s": round(2.0 * M ** 3 / (ms * 1e-3) / 1e12, 1),
                 "frac_of_2.5_PFLOP/s": round(2.0 * M ** 3 / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)})
    del a, b_

    # Context for the copy-shaped rows (scatter into the pool): torch's device-to-device copy of 1 GiB,
    # counted as bytes read plus bytes written, on the same box.
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    rows.append({"workload": "context: torch device-to-device copy of 1 GiB (read + write), not part of the product",
                 "kernel_ms_mean": round(ms, 4), "GB/s": round(2.0 * n / (ms * 1e-3) / 1e9, 1),
                 "frac_of_8_TB/s": round(2.0 * n / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    return rows


def run_calibration(steps):
    """A plain device-to-device copy of known size (1 GiB read + 1 GiB written per launch): what the
    FETCH_SIZE / WRITE_SIZE counters read for it is the scale for the same counters on our kernels."""
    import torch
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    print(json.dumps({"workload": "calibration copy", "bytes_read": n, "bytes_written": n, "launches": steps,
                      "ms_per_launch": round(dt * 1e3, 4), "GBps_read_plus_write": round(2 * n / dt / 1e9, 1)}))
    # Two yardsticks from the vendor libraries, for context next to the roofline fractions: what a plain
    # streaming read and a plain bf16 matrix product reach on this box (both well below the published peaks).
    del dst
    x = src.view(torch.float32)
    x.zero_()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        x.sum()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    print(json.dumps({"workload": "streaming read (torch sum over 1 GiB)", "ms_per_launch": round(dt * 1e3, 4),
                      "GBps_read": round(n / dt / 1e9, 1)}))
    m = 8192
    a = torch.randn((m, m), device="cuda", dtype=torch.float32).to(torch.bfloat16)
    b = torch.randn((m, m), device="cuda", dtype=torch.float32).to(torch.bfloat16)
    for _ in range(3):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    print(json.dumps({"workload": "bf16 matrix product 8192^3 (torch.matmul)", "ms_per_launch": round(dt * 1e3, 4),
                      "TFLOPs": round(2.0 * m ** 3 / dt / 1e12, 1)}))


def read_sensors():
    """Shader clock and board power as the amdgpu driver reports them (read-only sysfs files; absent ones are left out)."""
    import glob
    out = {}
    for dev in sorted(glob.glob("/sys/class/drm/card*/device")):
        card = dev.split("/")[4]
        try:
            cur = [l for l in open(dev + "/pp_dpm_sclk").read().split("\n") if l.endswith("*")]
            if cur:
                out[card + ".sclk_mhz"] = int("".join(c for c in cur[0].split(":")[1] if c.isdigit()))
        except (OSError, ValueError, IndexError):
            pass
        for hw in glob.glob(dev + "/hwmon/hwmon*"):
            for name in ("power1_input", "power1_average", "power1_cap"):
                try:
                    out[card + "." + name + "_w"] = int(open(os.path.join(hw, name)).read()) / 1e6
                except (OSError, ValueError):
                    pass
    return out


def run_sensors(seconds):
    """Clock and power while a workload runs back to back: the headline forward, the vendor library's bf16 matrix product,
    a device copy.  One thread launches, this one reads the sensors every 0.3 s (after a second of settling)."""
    import threading
    import torch
    from attention_amd import hip
    c = FLASH
    B, N, H, d = c["B"], c["N"], c["H"], c["d"]
    q = torch.randn((B, N, H, d), device="cuda", dtype=torch.float32).to(torch.bfloat16)
    k, v, o = torch.randn_like(q), torch.randn_like(q), torch.empty_like(q)
    a = torch.randn((8192, 8192), device="cuda", dtype=torch.float32).to(torch.bfloat16)
    b = torch.randn_like(a)
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    kz, az = torch.zeros_like(k), torch.zeros_like(a)
    st = (N * H * d, H * d, d)
    work = [
        ("flash_fwd bf16 causal B=4 N=4096 H=32 d=128",
         lambda: hip.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, d, st, 1.0 / np.sqrt(d), True, None)),
        ("torch.matmul bf16 8192^3", lambda: torch.matmul(a, b)),
        ("1 GiB device copy", lambda: dst.copy_(src)),
        # The same two matrix workloads on tensors of zeros: the same instructions, far fewer bits that change from one
        # operand to the next.  What they draw and how they clock shows how much of the N(0,1) figures is the power limit.
        ("flash_fwd bf16 causal B=4 N=4096 H=32 d=128, K and V all zeros",
         lambda: hip.flash_fwd(q.data_ptr(), kz.data_ptr(), kz.data_ptr(), o.data_ptr(), hip.BF16, B, N, H, d, st, 1.0 / np.sqrt(d), True, None)),
        ("torch.matmul bf16 8192^3, both factors all zeros", lambda: torch.matmul(az, az)),
    ]
    print(json.dumps({"workload": "idle", "sensors": read_sensors()}))
    for name, launch in work:
        done = threading.Event()
        res = {}

        def loop():
            launch()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            n = 0
            while time.perf_counter() - t0 < seconds:
                for _ in range(50):
                    launch()
                torch.cuda.synchronize()
                n += 50
            res["ms_per_launch"] = round((time.perf_counter() - t0) / n * 1e3, 4)
            done.set()
        th = threading.Thread(target=loop)
        th.start()
        time.sleep(1.0)
        samples = []
        while not done.is_set():
            samples.append(read_sensors())
            time.sleep(0.3)
        th.join()
        keys = sorted({kk for smp in samples for kk in smp})
        print(json.dumps({"workload": name, "ms_per_launch": res.get("ms_per_launch"), "samples": len(samples),
                          "sensors_min_max": {kk: [min(smp[kk] for smp in samples if kk in smp), max(smp[kk] for smp in samples if kk in smp)]
                                              for kk in keys}}))


def main():
    global SETTLE_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", choices=["all", "flash", "decode", "calib", "extras", "sensors"], default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline (profiling runs)")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed launches for this long in front of each workload's warm-up (0: none, for counter runs)")
    a = ap.parse_args()
    SETTLE_MS = a.settle_ms
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (both paths shard by head or sequence without communication); "
                 f"--gpus {a.gpus} is not supported")
    import torch
    from attention_amd import hip
    hip.load()
    if not torch.cuda.is_available() or hip.device_count() < 1:
        sys.exit("bench.py: no GPU visible")
    if a.workload == "calib":
        run_calibration(a.steps)
        return
    if a.workload == "sensors":
        run_sensors(5.0)
        return
    import ctypes as C
    s = C.c_void_p()
    assert hip.load().ahpc_hip_stream_create(C.byref(s)) == 0
    stream = s.value

    if a.workload == "extras":
        print(json.dumps({"extras": bench_extras(hip, stream, a.steps, a.warmup)}))
        hip.load().ahpc_hip_stream_destroy(stream)
        return
    out = {"n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "settle_ms": SETTLE_MS, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}
    flash = bench_flash(hip, stream, a.steps, a.warmup, not a.no_cpu) if a.workload in ("all", "flash") else None
    decode = bench_decode(hip, stream, a.steps, a.warmup, not a.no_cpu) if a.workload in ("all", "decode") else None
    head = flash or decode
    out.update({k: head[k] for k in ("metric", "value", "unit", "ms_per_step", "config", "roofline")})
    if "cpu_baseline" in head:
        out["cpu_baseline"] = head["cpu_baseline"]
    if flash is None:
        out["dtype"] = "f16"
    if flash and decode:
        out["decode"] = decode
        # the other configurations, in the same run and on the same box (inputs: torch.randn on the GPU)
        out["extras"] = bench_extras(hip, stream, min(a.steps, 20), min(a.warmup, 5))
    info = hip.device_info(0)
    out["device"] = {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units}
    hip.load().ahpc_hip_stream_destroy(stream)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
