"""Benchmark of the fp8 / int4 op family on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME...]] [--no-cpu]

A step is one call of the primary workload, benchmark configuration 3: fp8_gemm_v2 on
8192 x 4096 x 14336 (e4m3fn x e4m3fn -> bf16, per-tensor inverse scales, bf16
bias), with all operands resident in HBM.  The single JSON line printed at the
end carries that as ``value`` (TFLOP/s) with its MFMA roofline, and under
``ops`` the HBM-bound members of the family (amax, cast_to_fp8_v2,
cast_from_fp8, convert_from_uint4 / int4, the decode-shaped GEMMs) and the MLP
block, each with its own roofline entry.

Timing: W untimed warm-up calls, then K calls bracketed by HIP events on the
stream the kernels are launched on (torch's current stream), divided by K.
The streaming kernels rotate through enough distinct buffer sets to exceed the
256 MiB Infinity Cache, so reads come from HBM.

The CPU baseline is the PyTorch-CPU float8 emulation of the same semantics
(oracle/oracle.py torch_* functions) timed on this host's cores on a bounded
sample; it is reported next to the GPU figure and is not the target.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP8_PEAK_TFLOPS = 5000.0     # MI355X dense OCP fp8 MFMA, published
E4 = torch.float8_e4m3fn
SEED = 0xC001A1
MALL_BYTES = 256 << 20

# HBM bytes per launch (read + written) measured with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE in two runs of this script per workload, each counter scaled by what it reads for
# the 16 MiB fp8 copy kernel (fetch x1.9974, write x1.0000); the tables are under profiles/.  Counters
# cannot be read from inside the timed run, so these are constants from the committed runs.
MEASURED_TRAFFIC = {
    "amax": 33.54e6,
    "cast_to_fp8_v2": 50.35e6,
    "cast_to_fp8_v2+amax": 50.37e6,
    "cast_from_fp8": 50.38e6,
    "copy_fp8": 33.55e6,
    "cast_to_fp8_v2_large": 804.68e6,
    "convert_from_uint4": 43.36e6,
    "convert_from_int4": 43.10e6,
    "fp8_gemm_v2": 939.89e6,
    "fp8_gemm_v2_B_NK": 939.33e6,
    "fp8_gemm_v2_decode_M16": 236.92e6,
    "fp8_gemm_v2_decode_M64": 243.07e6,
    "fp8_gemm_v2_decode_M256": 266.45e6,
    "w4a8_gemm_M16": 130.86e6,      # the partial sums of the two K parts on top of the 124 MB of operands
    "w4a8_gemm_M32": 139.63e6,
    "w4a8_gemm_M64": 157.22e6,
    "w4a8_gemm_M256": 153.68e6,     # two row blocks of 128 on one XCD share a strip's weights in its L2
    "w4a16_gemm_M16": 131.96e6,     # split_rows_vec_kernel + w4a8_wide_kernel<two planes>
    "w4a16_gemm_M64": 161.49e6,
    "w4a16_gemm_M256": 178.91e6,
    "fp8_sdpa_B1_L8192": 124.63e6,
    "fp8_sdpa_B4_L4096": 235.55e6,
    "fp8_sdpa_B1_L8192_D256": 347.00e6,   # k and v are re-read by the query blocks of a head group beyond L2
    "fp8_sdpa_decode_B64_S4096": 537.37e6,
    "fp8_sdpa_decode_B8_S8192": 143.15e6,   # fp8_sdpa_decode_kernel 138.81 + 4.34 written and read back by the merge
    "softmax_fp8": 1609.32e6,
    "sum_fp8_rows": 67.32e6,
    "sum_fp8_columns": 73.44e6,   # sum_columns_kernel 69.20 + sum_finish_kernel 4.24
}


RAMP_SECONDS = 0.15

# --only tokens: a group name runs the whole group, group_case one workload of it (one profile row per workload)
GROUPS = ("gemm", "cast", "castlarge", "int4", "decode", "mlp", "reduce", "w4a8", "w4a16", "sdpa", "ceilings")
DEFAULT_GROUPS = tuple(g for g in GROUPS if g != "ceilings")   # the probes run on request only
WHICH = set()


def want(group, case=None):
    """True when --only names the group, or this case of it (e.g. w4a8_M256, sdpa_B1, sdpa_decode_B8, decode_M64)."""
    if group in WHICH:
        return True
    if case is None:
        return any(t.startswith(group + "_") for t in WHICH)
    return f"{group}_{case}" in WHICH


def time_gpu(fn, steps, warmup):
    """Average milliseconds per call of fn(i), HIP events on the current stream.

    The GPU leaves its idle power state only under sustained load: the first tens of
    milliseconds of back-to-back launches run at rising clocks (a 0.36 ms GEMM takes
    0.58 ms at first and settles after about 60 calls).  The op is therefore run untimed
    for RAMP_SECONDS before the `warmup` untimed and `steps` timed calls, with no host
    synchronisation between the three phases.
    """
    t0 = time.perf_counter()
    n = 0
    while True:
        for _ in range(10):
            fn(n)
            n += 1
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > RAMP_SECONDS:
            break
    for _ in range(max(10, n // 4)):  # refill the queue after the last synchronisation
        fn(n)
        n += 1
    for i in range(warmup):
        fn(n + i)
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn(n + warmup + i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def time_cpu(fn, min_seconds=3.0, max_runs=5):
    """Median seconds of fn() over up to max_runs runs (at least one)."""
    ts = []
    t_total = 0.0
    while len(ts) < max_runs and (not ts or t_total < min_seconds):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        ts.append(dt)
        t_total += dt
    ts.sort()
    return ts[len(ts) // 2]


def hbm_entry(name, workload, bytes_per_call, ms, steps, kernel, cpu=None, extra=None, ceiling=None):
    """ceiling: GB/s of a plain 16-byte copy moving the same number of bytes in the same run (what a streaming
    kernel of this size can reach on this machine; reported beside the published peak, never instead of it)."""
    gbs = bytes_per_call / (ms * 1e-3) / 1e9
    e = {"name": name, "workload": workload, "metric": "GB/s", "value": round(gbs, 1), "unit": "GB/s",
         "ms_per_call": round(ms, 5), "steps": steps,
         "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                      "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                      "algorithmic_bytes": bytes_per_call, "traffic": MEASURED_TRAFFIC.get(name)}}
    if ceiling is not None:
        e["roofline"]["ceiling_same_size"] = {"what": "plain copy of the same number of bytes (read + written), same run",
                                              "GB/s": round(ceiling, 1), "frac_of_peak": round(ceiling / HBM_PEAK_GBS, 4)}
    if cpu is not None:
        e["cpu_baseline"] = cpu
    if extra:
        e.update(extra)
    return e


def n_sets(bytes_per_set):
    return max(2, -(-int(1.5 * MALL_BYTES) // bytes_per_set))


def c1_input(gen, rows=4096, cols=4096):
    x = torch.randn(rows, cols, generator=gen) * 3
    n = x.numel()
    k = -(-n // 1000)
    pos = torch.randperm(n, generator=gen)[:k]
    sign = torch.randint(0, 2, (k,), generator=gen).float() * 2 - 1
    x.view(-1)[pos] = sign * 1e4
    return x.bfloat16()


def bench_cast(pkg, oracle, dev, steps, warmup, cpu, c1=True, large=True):
    """benchmark configuration 1: amax pass, cast_to_fp8_v2 (scale given), cast_from_fp8.

    These kernels run for about ten microseconds, less than the host needs to
    dispatch a torch op, so they are timed through the C ABI (ctypes, outputs
    allocated up front): the figure is the kernels' rate, not the dispatcher's.
    """
    import ctypes
    lib = pkg.capi()
    out = []
    gen = torch.Generator().manual_seed(SEED)
    x = c1_input(gen)
    n = x.numel()
    amax = x.abs().max().float()
    scale = (448.0 / amax).reshape(())
    sets = n_sets(3 * n)
    xs = [x.to(dev).clone() for _ in range(sets)]
    y8 = [torch.empty(x.shape, dtype=E4, device=dev) for _ in range(sets)]
    yb = [torch.empty(x.shape, dtype=torch.bfloat16, device=dev) for _ in range(sets)]
    am = torch.zeros((), device=dev)
    sd, sinv = scale.to(dev), scale.reciprocal().to(dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cores = torch.get_num_threads()

    def ok(status):
        if status != 0:
            raise RuntimeError(lib.mi355q_status_string(status).decode())

    if not c1:
        del xs, y8, yb
        return out + bench_cast_large(lib, pkg, gen, dev, sd, st, ok, steps)

    def copy_rate(total_bytes):
        # the library's 16-byte copy kernel moving total_bytes (half read, half written) between the same rotating buffers
        half = total_bytes // 2
        t = time_gpu(lambda i: ok(lib.mi355q_cast_to_fp8(xs[i % sets].data_ptr(), pkg.E4M3FN, yb[i % sets].data_ptr(), pkg.E4M3FN,
                                                         None, 0.0, pkg.SCALE_NONE, half, 1, 1, None, st)), steps, warmup)
        return total_bytes / (t * 1e-3) / 1e9

    ceil_48 = copy_rate(3 * n)     # the casts move 48 MiB
    ceil_32 = copy_rate(2 * n)     # the amax pass reads 32 MiB
    ms = time_gpu(lambda i: ok(lib.mi355q_amax(xs[i % sets].data_ptr(), pkg.BF16, n, am.data_ptr(), st)), steps, warmup)
    assert am.cpu() == amax
    c = None
    if cpu:
        t = time_cpu(lambda: x.abs().max().float())
        c = {"value": round(2 * n / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": "full 4096x4096 bf16 tensor, x.abs().max()"}
    out.append(hbm_entry("amax", "C1a amax of bf16 [4096,4096]", 2 * n, ms, steps, "fill_u32 + amax_vec<bf16>", c, ceiling=ceil_32))

    def cast_to(i, with_amax):
        j = i % sets
        ok(lib.mi355q_cast_to_fp8(xs[j].data_ptr(), pkg.BF16, y8[j].data_ptr(), pkg.E4M3FN, sd.data_ptr(), 0.0,
                                  pkg.SCALE_DEV, n, 1, 1, am.data_ptr() if with_amax else None, st))

    ms = time_gpu(lambda i: cast_to(i, False), steps, warmup)
    c = None
    if cpu:
        t = time_cpu(lambda: oracle.torch_cast_to_fp8(x, scale, E4))
        c = {"value": round(3 * n / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": "full 4096x4096 bf16 tensor, (x*s.to(bf16)).clamp(-448,448).to(float8_e4m3fn)"}
    out.append(hbm_entry("cast_to_fp8_v2", "C1b cast_to_fp8_v2 bf16 [4096,4096] -> e4m3fn, per-tensor scale",
                         3 * n, ms, steps, "cast_to_fp8_vec8<bf16,e4m3fn,scalar>", c, ceiling=ceil_48))

    ms = time_gpu(lambda i: cast_to(i, True), steps, warmup)
    out.append(hbm_entry("cast_to_fp8_v2+amax", "C1 cast_to_fp8_v2 with is_amax=True (one pass)", 3 * n + 4, ms, steps,
                         "fill_u32 + cast_to_fp8_vec8<bf16,e4m3fn,scalar,amax>", ceiling=ceil_48))

    ms = time_gpu(lambda i: ok(lib.mi355q_cast_from_fp8(y8[i % sets].data_ptr(), pkg.E4M3FN, yb[i % sets].data_ptr(),
                                                        pkg.BF16, sinv.data_ptr(), 0.0, pkg.SCALE_DEV, n, 1, 1, st)),
                  steps, warmup)
    c = None
    if cpu:
        y_cpu = y8[0].cpu()
        t = time_cpu(lambda: oracle.torch_cast_from_fp8(y_cpu, scale.reciprocal(), torch.bfloat16))
        c = {"value": round(3 * n / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": "full 4096x4096 e4m3fn tensor, x8.to(bf16) * s_inv.to(bf16)"}
    out.append(hbm_entry("cast_from_fp8", "C1c cast_from_fp8 e4m3fn [4096,4096] -> bf16", 3 * n, ms, steps,
                         "cast_from_fp8_vec<e4m3fn,bf16,scalar>", c, ceiling=ceil_48))
    # fp8 -> fp8 is a plain copy (the reference forwards an fp8 input unchanged): the copy
    # kernel of known size that hardware byte counters are calibrated against
    ms = time_gpu(lambda i: ok(lib.mi355q_cast_to_fp8(y8[i % sets].data_ptr(), pkg.E4M3FN, yb[i % sets].data_ptr(),
                                                      pkg.E4M3FN, None, 0.0, pkg.SCALE_NONE, n, 1, 1, None, st)),
                  steps, warmup)
    out.append(hbm_entry("copy_fp8", "cast_to_fp8_v2 of an fp8 tensor: copy of 16 MiB", 2 * n, ms, steps, "copy_vec16"))
    del xs, y8, yb

    if large:
        out += bench_cast_large(lib, pkg, gen, dev, sd, st, ok, steps)
    return out


def bench_cast_large(lib, pkg, gen, dev, sd, st, ok, steps):
    """The C1 cast on a tensor 16x larger (not one of the benchmark configurations): the C1 kernels are so
    short that launch ramp-up is a visible share of them; this shows the streaming rate without it."""
    big = torch.randn(16384, 16384, generator=gen).bfloat16().to(dev) * 3
    nb = big.numel()
    big8 = [torch.empty(big.shape, dtype=E4, device=dev) for _ in range(2)]
    ms = time_gpu(lambda i: ok(lib.mi355q_cast_to_fp8(big.data_ptr(), pkg.BF16, big8[i % 2].data_ptr(), pkg.E4M3FN,
                                                      sd.data_ptr(), 0.0, pkg.SCALE_DEV, nb, 1, 1, None, st)),
                  max(steps // 5, 5), 3)
    return [hbm_entry("cast_to_fp8_v2_large", "cast_to_fp8_v2 bf16 [16384,16384] -> e4m3fn (not one of the benchmark configurations)",
                      3 * nb, ms, max(steps // 5, 5), "cast_to_fp8_vec8<bf16,e4m3fn,scalar>")]


def bench_ceilings(pkg, dev, steps, warmup):
    """What this GPU sustains in this run with nothing in the way: back-to-back fp8 MFMAs on register operands
    (one and two waves per SIMD), and 16-byte read-only / copy streams at three sizes (rotating over enough
    buffers to exceed the Infinity Cache).  Reference points for the roofline fractions, not workloads."""
    import ctypes
    lib = pkg.capi()
    probe = pkg.probes()     # libmi355q_probe.so: measurement kernels, not part of the product library
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.zeros(16, device=dev)
    out = []
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for wps in (1, 2):
        per_wave = 4000
        ms = time_gpu(lambda i: probe.mi355q_probe_mfma(wps, per_wave, cus, sink.data_ptr(), st), max(steps, 20), warmup)
        flop = 131072.0 * per_wave * 4 * wps * cus
        out.append({"name": f"ceiling_mfma_fp8_{wps}_wave_per_simd", "workload": f"{per_wave} back-to-back v_mfma_f32_32x32x64_f8f6f4 per wave, "
                    f"{4 * wps} waves on each of {cus} CUs, register operands", "metric": "TFLOP/s",
                    "value": round(flop / (ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "ms_per_call": round(ms, 5), "steps": max(steps, 20),
                    "implied_clock_ghz": round(per_wave * 64 / (ms * 1e-3) / 1e9 * wps, 3)})
    # MFMAs and vector work side by side (what the attention kernel's softmax can hide under its MFMAs, and how)
    passes = 4000
    for name, wps, m0, m1, what in (
            ("mfma_one_wave", 1, 1, 1, "four MFMAs per pass, one wave per SIMD"),
            ("exp_one_wave", 1, 2, 2, "32 x (v_exp_f32, v_mul_f32) per pass, one wave per SIMD"),
            ("mfma_and_exp_in_one_wave", 1, 3, 3, "both dealt out in turns in one wave per SIMD"),
            ("mfma_two_waves", 2, 1, 1, "four MFMAs per pass and wave, two waves per SIMD"),
            ("exp_two_waves", 2, 2, 2, "32 x (v_exp_f32, v_mul_f32) per pass and wave, two waves per SIMD"),
            ("mfma_wave_beside_exp_wave", 2, 1, 2, "one wave per SIMD issues only the MFMAs, the other only the vector work"),
            ("mfma_and_exp_in_both_waves", 2, 3, 3, "both dealt out in turns in each of two waves per SIMD")):
        ms = time_gpu(lambda i: probe.mi355q_probe_coexec(wps, passes, m0, m1, cus, sink.data_ptr(), st), max(steps, 20), warmup)
        out.append({"name": "coexec_" + name, "workload": what + f" ({passes} passes, {cus} workgroups, register operands)",
                    "metric": "ns per pass", "value": round(ms * 1e6 / passes, 1), "unit": "ns", "ms_per_call": round(ms, 5),
                    "steps": max(steps, 20)})
    for mib in (32, 128, 2048):
        nbytes = mib << 20
        sets = 1 if nbytes >= (1 << 30) else n_sets(nbytes)
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev).view(E4) for _ in range(sets)]
        k = max(steps, 20) if mib < 2048 else 5
        ms = time_gpu(lambda i: probe.mi355q_probe_read(bufs[i % sets].data_ptr(), nbytes, 2 * cus, sink.data_ptr(), st), k, warmup)
        out.append(hbm_entry(f"ceiling_read_{mib}MiB", f"read-only stream over {mib} MiB, 16-byte loads, nothing stored", nbytes, ms, k, "probe_read_kernel"))
        half = nbytes // 2
        dst = [torch.empty(half, dtype=E4, device=dev) for _ in range(min(sets, 4))]
        ms = time_gpu(lambda i: lib.mi355q_cast_to_fp8(bufs[i % sets].data_ptr(), pkg.E4M3FN, dst[i % len(dst)].data_ptr(), pkg.E4M3FN, None, 0.0,
                                                       pkg.SCALE_NONE, half, 1, 1, None, st), k, warmup)
        out.append(hbm_entry(f"ceiling_copy_{mib}MiB", f"copy of {mib // 2} MiB ({mib} MiB read + written), the library's 16-byte copy kernel",
                             nbytes, ms, k, "copy_vec16"))
        del bufs, dst
    # the weights of the decode GEMMs ([8192, 28672] fp8 bytes) read in strips, as those kernels read them
    pitch, rows = 28672, 8192
    sets = n_sets(pitch * rows)
    bufs = [torch.randint(0, 255, (rows * pitch,), dtype=torch.uint8, device=dev) for _ in range(sets)]
    for strip, parts, nt in ((64, 1, 1), (128, 1, 0), (128, 1, 1), (256, 2, 1)):
        k = max(steps, 20)
        ms = time_gpu(lambda i: probe.mi355q_probe_strip_read(bufs[i % sets].data_ptr(), pitch, rows, strip, parts, nt, sink.data_ptr(), st), k, warmup)
        out.append(hbm_entry(f"ceiling_strip_read_{strip}B" + ("_nt" if nt else "") + (f"_K{parts}" if parts > 1 else ""),
                             f"[{rows}, {pitch}] bytes read in strips of {strip} bytes per row, {pitch // strip * parts} workgroups"
                             + (f", the rows in {parts} ranges" if parts > 1 else "") + (", nontemporal loads" if nt else ""),
                             pitch * rows, ms, k, "probe_strip_read_kernel"))
    del bufs
    # the amax pass of C1 in the form that needs no zeroing launch (partial maxima, a ticket, the last workgroup
    # reduces), beside the product's form (a one-thread fill and atomicMax), same buffers, same run
    gen = torch.Generator().manual_seed(SEED)
    x = c1_input(gen)
    n = x.numel()
    sets = n_sets(2 * n)
    xs = [x.to(dev).clone() for _ in range(sets)]
    am = torch.zeros((), dtype=torch.float32, device=dev)
    k = max(steps, 50)
    ms_ticket = time_gpu(lambda i: probe.mi355q_probe_amax_ticket(xs[i % sets].data_ptr(), n, am.data_ptr(), st), k, warmup)
    assert float(am.cpu()) == float(x.abs().max().float())
    ms_fill = time_gpu(lambda i: lib.mi355q_amax(xs[i % sets].data_ptr(), pkg.BF16, n, am.data_ptr(), st), k, warmup)
    out.append(hbm_entry("probe_amax_ticket_form", "amax of bf16 [4096,4096] with partial maxima and a ticket instead of the zeroing launch",
                         2 * n, ms_ticket, k, "probe_amax_ticket_kernel",
                         extra={"product_form_ms_same_run": round(ms_fill, 5)}))
    del xs
    # the column sum of [8192, 8192] e4m3fn as one kernel (the slices merged by the last arrival of each column block)
    # beside the product's two kernels, same buffers, same run
    m = 8192
    codes = torch.tensor([0x00, 0x38, 0x40, 0x44, 0x48], dtype=torch.uint8)   # e4m3fn 0, 1, 2, 3, 4: every sum is exact
    x8 = [codes[torch.randint(0, 5, (m, m), generator=gen)].to(dev) for _ in range(n_sets(m * m))]
    res = torch.empty(m, dtype=torch.float32, device=dev)
    ws_bytes = lib.mi355q_sum_fp8_workspace_bytes(1, m, m)
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    k = max(steps, 50)
    ms_ticket = time_gpu(lambda i: probe.mi355q_probe_sum_columns_ticket(x8[i % len(x8)].data_ptr(), m, m, res.data_ptr(), st), k, warmup)
    ms_two = time_gpu(lambda i: lib.mi355q_sum_fp8(x8[i % len(x8)].data_ptr(), pkg.E4M3FN, 1, m, m, res.data_ptr(), pkg.F32,
                                                   ws.data_ptr(), ws_bytes, st), k, warmup)
    probe.mi355q_probe_sum_columns_ticket(x8[0].data_ptr(), m, m, res.data_ptr(), st)
    got = res.clone()
    lib.mi355q_sum_fp8(x8[0].data_ptr(), pkg.E4M3FN, 1, m, m, res.data_ptr(), pkg.F32, ws.data_ptr(), ws_bytes, st)
    assert torch.equal(got, res) and torch.equal(res.cpu(), x8[0].cpu().view(E4).float().sum(0))
    out.append(hbm_entry("probe_sum_columns_ticket_form", "sum_fp8 e4m3fn [8192,8192] over dim 0 as one kernel with a ticket merge",
                         m * m + 4 * m, ms_ticket, k, "probe_sum_columns_ticket_kernel",
                         extra={"product_form_ms_same_run": round(ms_two, 5)}))
    del x8
    return out


def bench_int4(pkg, oracle, dev, steps, warmup, cpu):
    """benchmark configuration 2: K = N = 4096, group 128 (timed through the C ABI, see bench_cast)."""
    import ctypes
    lib = pkg.capi()
    out = []
    gen = torch.Generator().manual_seed(SEED)
    K = N = 4096
    q = torch.randint(0, 16, (K, N), generator=gen)
    packed = oracle.pack_nibbles(q)
    s = (torch.rand(K // 128, N, generator=gen) * 0.019 + 0.001).bfloat16()
    zp = oracle.pack_nibbles(torch.randint(0, 16, (K // 128, N), generator=gen))
    b_u = K * N // 2 + s.numel() * 2 + zp.numel() * 4 + K * N * 2
    b_i = K * N // 2 + s.numel() * 2 + K * N * 2
    sets = n_sets(K * N // 2 + K * N * 2)
    ps = [packed.to(dev).clone() for _ in range(sets)]
    outs = [torch.empty(K, N, dtype=torch.bfloat16, device=dev) for _ in range(sets)]
    sd, zd = s.to(dev), zp.to(dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cores = torch.get_num_threads()

    def run(i, signed):
        j = i % sets
        status = lib.mi355q_dequant_4bit(ps[j].data_ptr(), sd.data_ptr(), None if signed else zd.data_ptr(),
                                         pkg.ZP_NONE if signed else pkg.ZP_PACKED, int(signed), pkg.BF16, K, N // 8, 128,
                                         outs[j].data_ptr(), st)
        if status != 0:
            raise RuntimeError(lib.mi355q_status_string(status).decode())

    ms = time_gpu(lambda i: run(i, False), steps, warmup)
    c = None
    if cpu:
        t = time_cpu(lambda: oracle.torch_dequant_4bit(packed, s, zp, torch.bfloat16, False), max_runs=3)
        c = {"value": round(b_u / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": "full K=N=4096 problem, shift/mask unpack + (q - z) * s in torch"}
    out.append(hbm_entry("convert_from_uint4", "C2 convert_from_uint4 K=N=4096 group 128, packed zero-points -> bf16",
                         b_u, ms, steps, "dequant_4bit_kernel<unsigned,bf16,packed zp>", c))
    ms = time_gpu(lambda i: run(i, True), steps, warmup)
    out.append(hbm_entry("convert_from_int4", "C2 convert_from_int4 K=N=4096 group 128, no zero-point -> bf16",
                         b_i, ms, steps, "dequant_4bit_kernel<signed,bf16,no zp>"))
    return out


def bench_reductions(pkg, oracle, dev, steps, warmup, cpu):
    """softmax_fp8 and sum_fp8 (no published configuration names sizes for them): attention-sized
    probabilities, bf16 scores [4, 32, 2048, 2048] -> e4m3fn, and sums of an e4m3fn [8192, 8192] over either
    dimension to fp32.  Timed through the torch ops (each call runs for 0.05 - 0.3 ms)."""
    out = []
    ops = torch.ops.hpu
    gen = torch.Generator().manual_seed(SEED)
    cores = torch.get_num_threads()
    shape = (4, 32, 2048, 2048)
    n = 4 * 32 * 2048 * 2048
    base = (torch.randn(2048, 2048, generator=gen) * 2).bfloat16().to(dev)
    xs = [(base.roll(i, 0)[None, None] + torch.zeros(shape[:2] + (1, 1), dtype=torch.bfloat16, device=dev)).contiguous() for i in range(2)]
    ms = time_gpu(lambda i: ops.softmax_fp8(xs[i % 2], -1, 0.125, 256.0, None), steps, warmup)
    c = None
    if cpu:
        sample = xs[0][0, :2].cpu()
        t = time_cpu(lambda: oracle.torch_softmax_fp8(sample, -1, 0.125, 256.0), max_runs=3)
        c = {"value": round(3 * sample.numel() / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": "2 of the 128 [2048, 2048] score matrices, torch.softmax in fp32, bf16 rounding, scaled e4m3fn cast"}
    out.append(hbm_entry("softmax_fp8", "softmax_fp8 bf16 [4,32,2048,2048] -> e4m3fn, scalar scales", 3 * n, ms, steps,
                         "softmax_rows_kernel<bf16,e4m3fn,1 wave per row,4 vectors per lane,1 row per wave>", c))
    del xs
    m = 8192
    x8 = [torch.randint(-8, 9, (m, m), generator=gen).float().to(E4).to(dev) for _ in range(n_sets(m * m))]
    for dim, what, kernel in ((1, "rows", "sum_rows_kernel<e4m3fn,16>"), (0, "columns", "sum_columns_kernel<e4m3fn,16> + sum_finish_kernel")):
        ms = time_gpu(lambda i: ops.sum_fp8(x8[i % len(x8)], [dim], False, torch.float), max(steps, 50), max(warmup, 10))
        c = None
        if cpu and dim == 1:
            xc = x8[0].cpu()
            t = time_cpu(lambda: oracle.torch_sum_fp8(xc, [1], False, torch.float), max_runs=3)
            c = {"value": round(m * m / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                 "sample": "the full [8192, 8192] tensor, torch.sum in float64"}
        out.append(hbm_entry(f"sum_fp8_{what}", f"sum_fp8 e4m3fn [8192,8192] over dim {dim} -> fp32", m * m + 4 * m, ms,
                             max(steps, 50), kernel, c))
    return out


def quant_per_tensor(ops, x_dev):
    amax = torch.ops.mi355q.amax(x_dev)
    s = 448.0 / amax
    return ops.cast_to_fp8_v2(x_dev, s, False, False, E4)[0], (1.0 / s)


def bench_gemm_c3(ops, oracle, pkg, dev, steps, warmup, cpu):
    gen = torch.Generator().manual_seed(SEED)
    M, K, N = 8192, 4096, 14336
    a = torch.randn(M, K, generator=gen).bfloat16().to(dev)
    w = (torch.randn(K, N, generator=gen) * 0.02).bfloat16().to(dev)
    bias = (torch.randn(N, generator=gen) * 0.01).bfloat16().to(dev)
    a8, sa_inv = quant_per_tensor(ops, a)
    w8, sw_inv = quant_per_tensor(ops, w)
    del a, w
    flop = 2.0 * M * N * K
    ms = time_gpu(lambda i: ops.fp8_gemm_v2(a8, False, w8, False, None, torch.bfloat16, sa_inv, sw_inv, bias, False),
                  steps, warmup)
    tflops = flop / (ms * 1e-3) / 1e12
    # the vendor library's fp8 GEMM on the same problem, as a calibration point for what this
    # machine sustains (it wants B column-major, its preferred layout; no bias).  Timed directly after the
    # headline, under the same load history: the GEMM runs at the power limit, and a chip that has idled
    # through the CPU baseline first sustains a higher clock for the first launches.
    lib_tflops = None
    try:
        w8_cm = w8.t().contiguous().t()
        # the first call sets the library up (hundreds of milliseconds): outside time_gpu, whose clock ramp is time-bound
        torch._scaled_mm(a8, w8_cm, scale_a=sa_inv, scale_b=sw_inv, out_dtype=torch.bfloat16)
        torch.cuda.synchronize()
        lib_ms = time_gpu(lambda i: torch._scaled_mm(a8, w8_cm, scale_a=sa_inv, scale_b=sw_inv, out_dtype=torch.bfloat16),
                          steps, warmup)
        lib_tflops = round(flop / (lib_ms * 1e-3) / 1e12, 1)
    except Exception:  # noqa: BLE001 - the comparison is optional, the library may refuse the call
        pass
    variant = pkg.capi().mi355q_fp8_gemm_variant(0, K, 0, N, M, N, K).decode()
    # the same product with the weights stored [N, K] (trans_B=True), the layout the vendor library wants
    w8_nk = w8.t().contiguous()
    ms_nk = time_gpu(lambda i: ops.fp8_gemm_v2(a8, False, w8_nk, True, None, torch.bfloat16, sa_inv, sw_inv, bias, False),
                     steps, warmup)
    variant_nk = pkg.capi().mi355q_fp8_gemm_variant(0, K, 1, K, M, N, K).decode()
    del w8_nk
    cpu_entry = None
    if cpu:
        rows = M
        a_cpu, w_cpu, b_cpu = a8[:rows].cpu(), w8.cpu(), bias.cpu()
        sa_c, sw_c = sa_inv.cpu(), sw_inv.cpu()
        t = time_cpu(lambda: oracle.torch_fp8_gemm(a_cpu, False, w_cpu, False, torch.bfloat16, sa_c, sw_c, bias=b_cpu),
                     min_seconds=10.0, max_runs=5)
        cpu_entry = {"value": round(2.0 * rows * N * K / t / 1e12, 4), "unit": "TFLOP/s",
                     "cores": torch.get_num_threads(), "kind": "port",
                     "sample": f"the full problem ({rows} rows of A), median of up to 5 runs / 10 s: "
                               "((A8.float() @ B8.float()) * sA * sB + bias).bfloat16()"}
    return {"ms": ms, "tflops": tflops, "flop": flop, "variant": variant, "cpu": cpu_entry, "library": lib_tflops,
            "ms_nk": ms_nk, "tflops_nk": flop / (ms_nk * 1e-3) / 1e12, "variant_nk": variant_nk}


def bench_gemm_decode(ops, oracle, dev, steps, warmup):
    """benchmark configuration 4: per-token x per-channel scales, K = 8192, N = 28672."""
    out = []
    gen = torch.Generator().manual_seed(SEED)
    K, N = 8192, 28672
    w = (torch.randn(K, N, generator=gen) * 0.02).bfloat16().to(dev)
    amax_c = w.abs().amax(dim=0).float()
    s_col = 448.0 / amax_c
    w8 = ops.cast_to_fp8_v2(w, s_col, False, False, E4, [1, N])[0]
    sw_inv = (1.0 / s_col).contiguous()
    del w
    # two copies of the weights exceed the Infinity Cache: alternate between them
    w8s = [w8, w8.clone()]
    # the vendor library's row-wise scaled fp8 GEMM as a calibration point (it wants B column-major)
    try:
        w8_cm = [t.t().contiguous().t() for t in w8s]
    except Exception:  # noqa: BLE001 - optional
        w8_cm = None
    cols = torch.randperm(K, generator=gen)[:82]
    for M in (16, 64, 256):
        x = torch.randn(M, K, generator=gen)
        x[:, cols] *= 20
        if not want("decode", f"M{M}"):
            continue
        x = x.bfloat16().to(dev)
        x8, sx_inv = torch.ops.mi355q.quantize_rows(x, E4)   # per-token amax, scale = 448 / amax, cast
        ms = time_gpu(lambda i: ops.fp8_gemm_v2(x8, False, w8s[i % 2], False, None, torch.bfloat16, sx_inv, sw_inv,
                                                None, False, [1, N]), steps, warmup)
        nbytes = K * N + M * K + 2 * M * N + 4 * (M + N)
        flop = 2.0 * M * N * K
        lib_ms = None
        if w8_cm is not None:
            try:
                sa2, sb2 = sx_inv.reshape(M, 1).contiguous(), sw_inv.reshape(1, N).contiguous()
                torch._scaled_mm(x8, w8_cm[0], scale_a=sa2, scale_b=sb2, out_dtype=torch.bfloat16)   # library set-up, untimed
                torch.cuda.synchronize()
                lib_ms = round(time_gpu(lambda i: torch._scaled_mm(x8, w8_cm[i % 2], scale_a=sa2, scale_b=sb2,
                                                                   out_dtype=torch.bfloat16), steps, warmup), 5)
            except Exception:  # noqa: BLE001 - the library may refuse the call
                lib_ms = None
        out.append(hbm_entry(f"fp8_gemm_v2_decode_M{M}",
                             f"C4 fp8_gemm_v2 M={M} K=8192 N=28672 per-token x per-channel scales -> bf16",
                             nbytes, ms, steps, "fp8_gemm_skinny_kernel" if M <= 128 else "fp8_gemm_tile_kernel<256,128>",
                             extra={"tflops": round(flop / (ms * 1e-3) / 1e12, 2), "library_gemm_ms_same_shape": lib_ms}))
    return out


def bench_w4a8(oracle, dev, steps, warmup, cpu):
    """The decode-shaped GEMM of configuration 4 with int4 weights: uint4 nibbles [K, N / 8] int32, bf16 scales and
    packed zero points per group of 128 along K, per-token e4m3fn activations; the weights are expanded inside the
    GEMM.  HBM-bound: the algorithmic bytes are the packed weights, their scales and zero points, A and C."""
    out = []
    gen = torch.Generator().manual_seed(SEED)
    K, N, G = 8192, 28672, 128
    packs = []
    for _ in range(3):   # three weight sets (3 x 117 MiB) exceed the Infinity Cache
        packs.append(torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=gen, dtype=torch.int64).to(torch.int32).to(dev))
    scale = (torch.rand(K // G, N, generator=gen) * 0.019 + 0.001).bfloat16().to(dev)
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // G, N // 8), generator=gen, dtype=torch.int64).to(torch.int32).to(dev)
    cols = torch.randperm(K, generator=gen)[:82]
    for M in (16, 32, 64, 256):
        x = torch.randn(M, K, generator=gen)
        x[:, cols] *= 20
        if not want("w4a8", f"M{M}"):
            continue
        x8, sx_inv = torch.ops.mi355q.quantize_rows(x.bfloat16().to(dev), E4)
        ms = time_gpu(lambda i: torch.ops.mi355q.w4a8_gemm(x8, packs[i % 3], scale, zp, False, torch.bfloat16, sx_inv, None),
                      steps, warmup)
        nbytes = K * N // 2 + (K // G) * N * 2 + (K // G) * N // 2 + M * K + 2 * M * N + 4 * M
        c = None
        if cpu and M == 16:
            rows_n = 1024    # a bounded sample: 1024 of the 28672 output columns
            pk, sc_c, zp_c = packs[0][:, :rows_n // 8].cpu(), scale[:, :rows_n].cpu(), zp[:, :rows_n // 8].cpu()
            x8c, sxc = x8.cpu(), sx_inv.cpu()
            t = time_cpu(lambda: oracle.torch_w4a8_gemm(x8c, pk, sc_c, zp_c, False, torch.bfloat16, sxc), min_seconds=3.0)
            c = {"value": round((K * rows_n // 2) / t / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                 "sample": f"M=16, {rows_n} of the 28672 output columns: unpack, (q - z) * s in float64, matmul, per-row scale"}
        out.append(hbm_entry(f"w4a8_gemm_M{M}", f"w4a8_gemm M={M} K=8192 N=28672: uint4 weights (group 128, bf16 scales, packed "
                                                "zero points) x per-token e4m3fn activations -> bf16",
                             nbytes, ms, steps, "w4a8_wide_kernel", c,
                             extra={"tflops": round(2.0 * M * N * K / (ms * 1e-3) / 1e12, 2)}))
    return out


def bench_w4a16(oracle, dev, steps, warmup, cpu):
    """The same weights against bf16 activations (mi355q::w4a16_gemm): what a GPTQ model with bf16 activations runs in
    place of convert_from_uint4 -> bf16 [K, N] -> matmul.  Algorithmic bytes: packed weights, scales, zero points, A (bf16)
    and C; the reference's route would write and read 470 MB of bf16 weights on top."""
    out = []
    gen = torch.Generator().manual_seed(SEED)
    K, N, G = 8192, 28672, 128
    packs = [torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=gen, dtype=torch.int64).to(torch.int32).to(dev) for _ in range(3)]
    scale = (torch.rand(K // G, N, generator=gen) * 0.019 + 0.001).bfloat16().to(dev)
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // G, N // 8), generator=gen, dtype=torch.int64).to(torch.int32).to(dev)
    cols = torch.randperm(K, generator=gen)[:82]
    for M in (16, 64, 256):
        x = torch.randn(M, K, generator=gen)
        x[:, cols] *= 20
        if not want("w4a16", f"M{M}"):
            continue
        xb = x.bfloat16().to(dev)
        ms = time_gpu(lambda i: torch.ops.mi355q.w4a16_gemm(xb, packs[i % 3], scale, zp, False, torch.bfloat16, None), steps, warmup)
        nbytes = K * N // 2 + (K // G) * N * 2 + (K // G) * N // 2 + 2 * M * K + 2 * M * N
        c = None
        if cpu and M == 16:
            cols_n = 1024
            pk, sc_c, zp_c, xc = packs[0][:, :cols_n // 8].cpu(), scale[:, :cols_n].cpu(), zp[:, :cols_n // 8].cpu(), xb.cpu()
            t = time_cpu(lambda: oracle.torch_w4a16_gemm(xc, pk, sc_c, zp_c, False, torch.bfloat16), min_seconds=3.0)
            c = {"value": round((K * cols_n // 2) / t / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                 "sample": f"M=16, {cols_n} of the 28672 output columns: unpack, (q - z) * s in float64, matmul"}
        out.append(hbm_entry(f"w4a16_gemm_M{M}", f"w4a16_gemm M={M} K=8192 N=28672: uint4 weights (group 128, bf16 scales, packed zero points) "
                                                 "x bf16 activations -> bf16", nbytes, ms, steps, "split_rows_vec_kernel + w4a8_wide_kernel<two planes>", c,
                             extra={"tflops": round(2.0 * M * N * K / (ms * 1e-3) / 1e12, 2)}))
    return out


def bench_sdpa(oracle, dev, steps, warmup, cpu):
    """hpu::fp8_sdpa_recomp_fwd, Llama-3-8B attention shapes (32 query heads, 8 key/value heads, head dimension 128),
    causal, e4m3fn q / k / v, q_scale_s = 128, bf16 output.  MFMA-bound: 4 L S D flop per head, halved by the mask."""
    import math
    out = []
    gen = torch.Generator().manual_seed(SEED)
    H, HK = 32, 8
    for B, L, D in ((1, 8192, 128), (4, 4096, 128), (1, 8192, 256)):
        if not want("sdpa", f"B{B}" if D == 128 else f"D{D}"):
            continue
        sc = 1.0 / math.sqrt(D)
        q = torch.randn(B, HK, H // HK, L, D, generator=gen).to(E4).to(dev)     # the grouped-query view of [B, H, L, D]
        k = torch.randn(B, HK, 1, L, D, generator=gen).to(E4).to(dev)
        v = torch.randn(B, HK, 1, L, D, generator=gen).to(E4).to(dev)
        f = lambda i: torch.ops.hpu.fp8_sdpa_recomp_fwd.scalar(q, k, v, None, 0.0, sc, True, False, "None", 1.0, 1.0, 1.0, 128.0,
                                                               0.0, 1.0 / 128.0, False, False, None, "left")
        ms = time_gpu(f, steps, warmup)
        flop = 4.0 * B * H * L * L * D * 0.5
        tf = flop / (ms * 1e-3) / 1e12
        name = f"fp8_sdpa_B{B}_L{L}" + ("" if D == 128 else f"_D{D}")
        e = {"name": name, "workload": f"fp8_sdpa_recomp_fwd causal, batch {B}, 32 query / 8 kv heads, "
                                       f"q_len = kv_len = {L}, head_dim {D}, e4m3fn -> bf16",
             "metric": "TFLOP/s", "value": round(tf, 1), "unit": "TFLOP/s", "ms_per_call": round(ms, 4), "steps": steps,
             "roofline": {"bound": "mfma", "kernel": f"fp8_sdpa_fwd_kernel<{D // 64},{D // 32},e4m3fn>", "achieved": round(tf, 1),
                          "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / FP8_PEAK_TFLOPS, 4),
                          "algorithmic_flop": flop, "traffic": MEASURED_TRAFFIC.get(name)}}
        if cpu and B == 1 and D == 128:
            n = 1024    # a bounded sample: one head, the first 1024 queries and keys
            qc, kc, vc = q[0, 0, 0, :n].cpu(), k[0, 0, 0, :n].cpu(), v[0, 0, 0, :n].cpu()
            t = time_cpu(lambda: oracle.torch_fp8_sdpa(qc, kc, vc, is_causal=True, q_scale_s=128.0, d_scale_s=1 / 128.0), min_seconds=3.0)
            e["cpu_baseline"] = {"value": round(4.0 * n * n * D * 0.5 / t / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                                 "kind": "port", "sample": f"one head, {n} queries x {n} keys, the float64 oracle"}
        out.append(e)
    # decoding: one query per head against a long cache; bound by reading k and v once
    D = 128
    sc = 1.0 / math.sqrt(D)
    for B, S in ((64, 4096), (8, 8192)):
        if not want("sdpa", f"decode_B{B}"):
            continue
        q = torch.randn(B, HK, H // HK, 1, D, generator=gen).to(E4).to(dev)
        sets = n_sets(2 * B * HK * S * D)
        ks = [torch.randn(B, HK, 1, S, D, generator=gen).to(E4).to(dev) for _ in range(sets)]
        vs = [torch.randn(B, HK, 1, S, D, generator=gen).to(E4).to(dev) for _ in range(sets)]
        f = lambda i: torch.ops.hpu.fp8_sdpa_recomp_fwd.scalar(q, ks[i % sets], vs[i % sets], None, 0.0, sc, False, False, "None", 1.0, 1.0,
                                                               1.0, 128.0, 0.0, 1.0 / 128.0, False, False, None, "left")
        ms = time_gpu(f, max(steps, 50), warmup)
        nbytes = 2 * B * HK * S * D + B * H * D + 2 * B * H * D
        out.append(hbm_entry(f"fp8_sdpa_decode_B{B}_S{S}", f"fp8_sdpa_recomp_fwd, one query per head, batch {B}, 32 query / 8 kv heads, "
                                                           f"kv_len = {S}, head_dim 128, e4m3fn -> bf16", nbytes, ms, max(steps, 50),
                             "fp8_sdpa_decode_kernel<2,4,e4m3fn>"))
        del ks, vs
    return out


def bench_mlp(ops, dev, steps, warmup):
    """benchmark configuration 5: fp8 decoder MLP block, Llama-3-8B dims, 4096 tokens."""
    gen = torch.Generator().manual_seed(SEED)
    T, d, ff = 4096, 4096, 14336

    def qweight(k, n):
        w = (torch.randn(k, n, generator=gen) * 0.02).bfloat16().to(dev)
        s = 448.0 / w.abs().amax(dim=0).float()
        return ops.cast_to_fp8_v2(w, s, False, False, E4, [1, n])[0], (1.0 / s).contiguous()

    wg, sg = qweight(d, ff)
    wu, su = qweight(d, ff)
    wd, sdn = qweight(ff, d)
    # gate and up weights side by side ([d, 2 ff], the usual serving layout): one GEMM of twice
    # the width computes both projections (same arithmetic, same bits as two GEMMs)
    wgu = torch.cat([wg, wu], dim=1).contiguous()
    sgu = torch.cat([sg, su]).contiguous()
    x = torch.randn(T, d, generator=gen).bfloat16().to(dev)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(8)]

    def quant_rows(t):
        # one kernel: per-token amax, scale = 448 / amax, cast_to_fp8_v2 semantics, 1 / scale for the GEMM
        return torch.ops.mi355q.quantize_rows(t, E4)

    def block(record=False):
        if record: ev[0].record()
        x8, sx = quant_rows(x)
        if record: ev[1].record()
        gu = ops.fp8_gemm_v2(x8, False, wgu, False, None, torch.bfloat16, sx, sgu, None, False, [1, 2 * ff])
        if record: ev[2].record()
        # bf16 SiLU(gate) * up and the per-token re-quantisation in one kernel
        h8, sh = torch.ops.mi355q.silu_mul_quantize_rows(gu[:, :ff], gu[:, ff:], E4)
        if record: ev[3].record()
        y = ops.fp8_gemm_v2(h8, False, wd, False, None, torch.bfloat16, sh, sdn, None, False, [1, d])
        if record: ev[4].record()
        return y

    def block_separate_ops():
        # the same block with two GEMMs, aten's silu and mul, and quantize_rows
        x8, sx = quant_rows(x)
        g = ops.fp8_gemm_v2(x8, False, wg, False, None, torch.bfloat16, sx, sg, None, False, [1, ff])
        u = ops.fp8_gemm_v2(x8, False, wu, False, None, torch.bfloat16, sx, su, None, False, [1, ff])
        h8, sh = quant_rows(torch.nn.functional.silu(g) * u)
        return ops.fp8_gemm_v2(h8, False, wd, False, None, torch.bfloat16, sh, sdn, None, False, [1, d])

    ya, yb = block().float(), block_separate_ops().float()
    agree = ((ya - yb).abs().max() / yb.abs().max()).item()
    ms_sep = time_gpu(lambda i: block_separate_ops(), steps, warmup)
    ms = time_gpu(lambda i: block(), steps, warmup)
    block(record=True)
    torch.cuda.synchronize()
    parts = [ev[i].elapsed_time(ev[i + 1]) for i in range(4)]
    flop = 3 * 2.0 * T * d * ff
    return {"name": "mlp_block", "workload": "C5 fp8 MLP block T=4096 d=4096 ff=14336, per-token x per-channel; "
                                             "gate and up as one GEMM over [d, 2 ff] weights, SiLU*up fused with the re-quantisation",
            "metric": "tokens/s", "value": round(T / (ms * 1e-3), 1), "unit": "tokens/s",
            "ms_per_call": round(ms, 4), "steps": steps, "gemm_tflops": round(flop / (ms * 1e-3) / 1e12, 1),
            "breakdown_ms": {"quant_x": round(parts[0], 4), "gemm_gate_up": round(parts[1], 4),
                             "silu_mul_quant_h": round(parts[2], 4), "gemm_down": round(parts[3], 4)},
            "separate_ops": {"what": "two GEMMs, aten silu and mul, quantize_rows", "ms_per_call": round(ms_sep, 4),
                             "tokens_per_s": round(T / (ms_sep * 1e-3), 1),
                             "max_abs_difference_of_outputs_rel_to_max": agree}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", type=str, default="",
                    help="comma list of groups (gemm,cast,castlarge,int4,decode,mlp,reduce,w4a8,w4a16,sdpa,ceilings) or single workloads "
                         "(decode_M16|M64|M256, w4a8_M16|M32|M64|M256, w4a16_M16|M64|M256, sdpa_B1|B4|D256|decode_B64|decode_B8); "
                         "default: every group but ceilings (the measurement probes)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here uses a second GPU.",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU fallback.", file=sys.stderr)
        sys.exit(1)

    import __graft_entry__ as ge
    pkg = ge.load_package()
    from oracle import oracle
    ops = torch.ops.hpu
    dev = torch.device("cuda:0")
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    WHICH.update(args.only.split(",") if args.only else DEFAULT_GROUPS)
    for t in WHICH:
        if t.split("_")[0] not in GROUPS:
            ap.error(f"--only: unknown workload {t!r}")
    which = {g for g in GROUPS if want(g)}
    cpu = not args.no_cpu
    k_stream = max(args.steps, 50)      # the microsecond-scale kernels need more calls for a stable mean
    w_stream = max(args.warmup, 10)

    # Rows beyond the five benchmark configurations come first and C5, C4, C2, C1 last: a log that keeps
    # only the end of this long line keeps the configurations.
    ops_out = []
    if "ceilings" in which:
        ops_out += bench_ceilings(pkg, dev, args.steps, args.warmup)
    if "reduce" in which:
        ops_out += bench_reductions(pkg, oracle, dev, args.steps, args.warmup, cpu)
    if "sdpa" in which:
        ops_out += bench_sdpa(oracle, dev, args.steps, args.warmup, cpu)
    if "w4a16" in which:
        ops_out += bench_w4a16(oracle, dev, args.steps, args.warmup, cpu)
    if "w4a8" in which:
        ops_out += bench_w4a8(oracle, dev, args.steps, args.warmup, cpu)
    if "mlp" in which:
        ops_out.append(bench_mlp(ops, dev, max(args.steps // 2, 5), args.warmup))
    if "decode" in which:
        ops_out += bench_gemm_decode(ops, oracle, dev, args.steps, args.warmup)
    if "int4" in which:
        ops_out += bench_int4(pkg, oracle, dev, k_stream, w_stream, cpu)
    if "cast" in which or "castlarge" in which:
        ops_out += bench_cast(pkg, oracle, dev, k_stream, w_stream, cpu, c1="cast" in which, large="castlarge" in which)

    line = {"metric": "cast/dequant GB/s (% HBM peak); fp8_gemm_v2 TFLOP/s (% fp8 MFMA peak)",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn x fp8_e4m3fn -> f32 accumulate -> bf16",
            "data": "synthetic",
            "preconditioning": f"every op runs untimed for {RAMP_SECONDS} s (clock ramp from idle) before its warmup and timed steps"}
    if "gemm" in which:
        g = bench_gemm_c3(ops, oracle, pkg, dev, args.steps, args.warmup, cpu)
        line.update({"value": round(g["tflops"], 1), "unit": "TFLOP/s", "ms_per_step": round(g["ms"], 4),
                     "config": {"workload": "C3 fp8_gemm_v2 M=8192 K=4096 N=14336 e4m3fn, per-tensor scales, bf16 bias",
                                "kernel_variant": g["variant"],
                                "library_gemm_tflops_same_shape": g["library"]},
                     "roofline": {"bound": "mfma", "kernel": "fp8_gemm_tile16_kernel", "achieved": round(g["tflops"], 1),
                                  "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(g["tflops"] / FP8_PEAK_TFLOPS, 4),
                                  "algorithmic_flop": g["flop"], "traffic": MEASURED_TRAFFIC.get("fp8_gemm_v2")}})
        if g["cpu"]:
            line["cpu_baseline"] = g["cpu"]
        ops_out.insert(0, {"name": "fp8_gemm_v2_B_NK", "workload": "C3 with the weights stored [N=14336, K=4096] (trans_B=True)",
                           "metric": "TFLOP/s", "value": round(g["tflops_nk"], 1), "unit": "TFLOP/s",
                           "ms_per_call": round(g["ms_nk"], 4), "steps": args.steps, "kernel_variant": g["variant_nk"],
                           "roofline": {"bound": "mfma", "kernel": "fp8_gemm_tile16_kernel", "achieved": round(g["tflops_nk"], 1),
                                        "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                                        "frac": round(g["tflops_nk"] / FP8_PEAK_TFLOPS, 4), "algorithmic_flop": g["flop"],
                                        "traffic": MEASURED_TRAFFIC.get("fp8_gemm_v2_B_NK")}})
    else:
        first = ops_out[0]
        line.update({"value": first["value"], "unit": first["unit"], "ms_per_step": first["ms_per_call"],
                     "config": {"workload": first["workload"]}, "roofline": first.get("roofline")})
        if "cpu_baseline" in first:
            line["cpu_baseline"] = first["cpu_baseline"]
    line["ops"] = ops_out
    # every entry once more in short form, last in the line: name -> [value, unit, fraction of the published peak]
    line["summary"] = {e["name"]: [e["value"], e["unit"], e.get("roofline", {}).get("frac")] for e in ops_out}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
