#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline workload (`value`): the Q4_0 decode GEMV, weight 9728 x 2560, one token, cache-cold:
every step quantises the activation and runs the GEMV against the next of >= 1 GB of distinct
resident weight copies, so no weight byte is served from the 256 MB Infinity Cache.  One step =
one pass of the path (activation quantiser + GEMV) over one synthetic activation.  Inputs are
resident in HBM before the timed region starts.

The run prints ONE short JSON line on stdout (under 4 KB): metric, value, config, the roofline of the
dominant kernel, the best int8 MFMA prefill GEMM with its roofline, the CPU baseline (the oracle's
restatement of the reference's CPU matmul, timed on this host) and a two-number summary of every other
workload.  The full record of every workload (Q8_0 / Q6_K GEMV, small batches, GEMMs, MoE, the decode
chain) goes to stderr as it is measured and into bench_workloads.json beside this script.

The records also carry what the machine allows at these sizes, measured in the same run by the
measurement-only kernels of strix.rs_amd/libstrix_bench.so (not part of the product library): the cost of
an empty launch, a kernel that only reads the weight bytes cache-cold (the floor of a GEMV of that size)
and the int8 GEMM's compute phase alone (MFMA + the two FMAs per output of exact per-block rescaling).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only name,...] [--no-cpu]

One workload never runs by default: `--only moe_prefill_timeline` reads the per-workgroup timeline of the grouped GEMM
launches from a development build of the library (python strix.rs_amd/build.py -DSMX_GEMM_TRACE).
"""
import ctypes
import argparse
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
# HBM bytes per launch of the headline kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by
# the same counter's reading for a 256 MiB copy (profiles/gemv_q4_0_9728x2560_hbm_traffic.md)
HEADLINE_TRAFFIC_BYTES = 14232463
# the same for the Q8_0 ffn_up GEMM launch (profiles/gemm_i8_q8_0_ffn_up_counters.md): L2 fills + writes
GEMM_TRAFFIC_BYTES = {"gemm_q8_0_ffn_up": 472727060}
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA
Q4_0, Q8_0, Q6_K = 2, 8, 14
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q6_K: 210}
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q6_K: 256}
KERNEL = {Q4_0: "gemv_q4_0", Q8_0: "gemv_q8_0", Q6_K: "gemv_q6_k"}
UPLOAD = {Q4_0: "upload_q4_0", Q8_0: "upload_q8_0", Q6_K: "upload_q6_k"}


def _load(name, path, search=None):
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=search)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


class Floors:
    """ctypes view of libstrix_bench.so (measurement-only kernels)."""

    def __init__(self):
        path = os.path.join(ROOT, "strix.rs_amd", "libstrix_bench.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is missing: build it with `python strix.rs_amd/build.py`")
        L = ctypes.CDLL(path)
        dp = ctypes.POINTER(ctypes.c_double)
        L.sbk_empty_launch.argtypes = [ctypes.c_uint, ctypes.c_uint, ctypes.c_int, dp]
        L.sbk_empty_launch_graph.argtypes = [ctypes.c_uint, ctypes.c_uint, ctypes.c_int, dp]
        L.sbk_skeleton_graph.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_int, dp]
        L.sbk_read_floor.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_uint, ctypes.c_uint, ctypes.c_int, ctypes.c_int, dp]
        L.sbk_copy.argtypes = [ctypes.c_size_t, ctypes.c_int, dp]
        L.sbk_mfma_valu.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, dp, dp, dp]
        self.L = L

    def empty_launch(self, grid, block, launches=2000):
        d = ctypes.c_double()
        assert self.L.sbk_empty_launch(grid, block, launches, ctypes.byref(d)) == 1
        return d.value

    def empty_launch_graph(self, grid, block, launches=400):
        """the same launches inside one replayed graph: the device-side cost of a dependent launch"""
        d = ctypes.c_double()
        assert self.L.sbk_empty_launch_graph(grid, block, launches, ctypes.byref(d)) == 1
        return d.value

    def skeleton_graph(self, K, rows, grid=256, launches=400):
        """a launch that only fetches the K-float activation its predecessor wrote and stores rows outputs per workgroup,
        inside one replayed graph: the part of a dependent GEMV launch that is not weight traffic"""
        d = ctypes.c_double()
        assert self.L.sbk_skeleton_graph(K, rows, grid, launches, ctypes.byref(d)) == 1
        return d.value

    def read_floor(self, nbytes, cold=True, launches=400):
        """us per launch of a kernel that only reads nbytes (256 x 1024 threads, four 16-byte loads in flight
        per thread), from rotating buffers of > 1 GB in total (cold) or from one buffer (hot)."""
        nbytes = nbytes // 16 * 16
        nbuf = max(2, int(1.2e9 // nbytes)) if cold else 1
        d = ctypes.c_double()
        assert self.L.sbk_read_floor(nbytes, nbuf, 256, 1024, 4, launches, ctypes.byref(d)) == 1
        return d.value

    def copy(self, nbytes, launches=20):
        d = ctypes.c_double()
        assert self.L.sbk_copy(nbytes, launches, ctypes.byref(d)) == 1
        return d.value

    def mfma_valu(self, mode, row_tiles, waves_per_simd, nblocks=4000, warm_launches=15):
        """15 untimed launches (30 ms) first: the rate the chip sustains, as for the GEMM workloads."""
        us, tops, cyc = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        assert self.L.sbk_mfma_valu(mode, row_tiles, waves_per_simd, nblocks, warm_launches, ctypes.byref(us), ctypes.byref(tops), ctypes.byref(cyc)) == 1
        return {"us": us.value, "TOPS": tops.value, "cycles_per_mfma_per_wave": cyc.value,
                "simd_cycles_per_mfma": cyc.value / waves_per_simd}


def machine_floors(log):
    """What the machine allows, measured with the measurement-only kernels in this run."""
    f = Floors()
    out = {"workload": "machine_floors",
           "method": "HIP events around back-to-back launches on one stream, like every other workload here"}
    out["empty_launch_us"] = {f"{g}x{b}": f.empty_launch(g, b) for g, b in ((1, 64), (256, 256), (256, 1024), (512, 256), (1024, 256))}
    out["empty_launch_in_a_graph_us"] = {f"{g}x{b}": f.empty_launch_graph(g, b) for g, b in ((1, 64), (256, 1024))}
    out["dependent_launch_skeleton_in_a_graph_us"] = {"2560_in_9728_out": f.skeleton_graph(2560, 38), "9728_in_9728_out": f.skeleton_graph(9728, 38)}
    sizes = {"14MB_q4_0_9728x2560": 14008320, "26MB_q8_0_2560x9728": 26460160, "48MB_q6_k_15360x3840": 48384000,
             "112MB_eight_q4_0_9728x2560": 8 * 14008320}
    # (the faster of two passes: the first measurement of a process may still run at rising clocks)
    out["read_only_cold_us"] = {k: min(f.read_floor(v, True, 400 if v < 1e8 else 100) for _ in range(2)) for k, v in sizes.items()}
    out["read_only_cold_GBps"] = {k: sizes[k] / out["read_only_cold_us"][k] / 1e3 for k in sizes}
    out["read_only_hot_us"] = {"14MB_q4_0_9728x2560": f.read_floor(14008320, False)}
    us = f.copy(256 << 20)
    out["copy_256MiB_GBps_read_plus_write"] = 2 * (256 << 20) / us / 1e3
    # the int8 GEMM's compute phase alone: 32 x 128 wave tiles, two waves per SIMD (what its registers allow)
    out["mfma_only"] = f.mfma_valu(0, 4, 2)
    out["fma_only"] = f.mfma_valu(1, 4, 2)
    out["mfma_plus_rescale_fma"] = f.mfma_valu(2, 4, 2)
    out["mfma_plus_rescale_fma_plus_lds_fragment_reads"] = f.mfma_valu(3, 4, 2)
    out["mfma_plus_rescale_fma_three_waves_per_simd"] = f.mfma_valu(2, 4, 3)
    # Q6_K: two K = 16 MFMAs per 32-block and row tile, each with its own weight scale: four vector operations per output
    out["mfma_plus_rescale_fma_q6_k"] = f.mfma_valu(6, 4, 2)
    out["note"] = ("mfma_only runs at the clock the chip sustains under matrix load; with the two FMAs per output that exact "
                   "per-block rescaling needs, the vector ALU bounds the rate: mfma_plus_rescale_fma is the ceiling of this arithmetic")
    log(json.dumps(out))
    return out


def gemv_bytes(ty, N, K, m=1):
    """Algorithmic bytes of one GEMV: weight blocks at on-disk density + int8 activations and their
    f32 scales (+ the packed sums Q4_0/Q6_K read) + fp32 outputs."""
    w = N * (K // BLOCK_ELEMS[ty]) * BLOCK_BYTES[ty]
    act = m * K * (1 + 4 / 32 + (4 / 32 if ty != Q8_0 else 0))
    return int(w + act + m * N * 4), w


class Bench:
    def __init__(self, steps, warmup):
        pkg_dir = os.path.join(ROOT, "strix.rs_amd")
        self.pkg = _load("strix_rs_amd", os.path.join(pkg_dir, "__init__.py"), [pkg_dir])
        self.synth = _load("strix_rs_amd_synth", os.path.join(pkg_dir, "synth.py"))
        self.acc = self.pkg.Mi355WeightAccel(0)
        self.steps, self.warmup = steps, warmup
        self.settle_ms = 30.0   # untimed replays of a workload's graph before its timed region (not the headline's)

    def log(self, *a):
        print(*a, file=sys.stderr, flush=True)

    def _first_touch(self, fn, n):
        """Part of a workload's set-up: one untimed step per rotating weight copy (n of them), so that no timed launch is
        the first access to freshly uploaded memory.  A decode loop reads every weight once per token; the first read
        after the upload costs 0.4-0.5 us more per 14 MB launch (address translation), which a run of 5 + 20 steps
        would otherwise measure instead of the kernel.  The rotation still exceeds the Infinity Cache: the data stay cold."""
        for i in range(n):
            fn(i)
        self.acc.sync()

    def _timed(self, fn, steps, warmup):
        """W untimed + exactly K timed steps, bracketed by stream syncs; HIP events on the stream."""
        acc = self.acc
        for i in range(warmup):
            fn(i)
        acc.sync()
        t0 = time.perf_counter()
        acc.timer_begin()
        for i in range(steps):
            fn(warmup + i)
        ms = acc.timer_end()
        acc.sync()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return ms, wall_ms

    def _timed_queued(self, fn, steps, warmup, settle_ms=None):
        """The K steps timed as ONE captured graph of the K calls, launched once between two events: the device runs them
        back to back however fast the host enqueued them.  This is the timed region of every decode workload.  A 5 us
        step is at the edge of what a Python caller submits per call (4.4-7.7 us per call across hosts; on a slow one a
        call-by-call region measures the host: 7.5 us per step where the kernel takes 4.9), so the call-by-call figure of
        the same K steps is reported beside it, as a field.  Returns (ms, wall_ms, info)."""
        acc = self.acc
        ms, wall_ms = self._timed(fn, steps, warmup)
        acc.graph_begin()
        for i in range(steps):
            fn(warmup + i)
        g = acc.graph_end()
        acc.graph_launch(g)          # untimed: the first launch of a graph also uploads it
        acc.sync()
        # settle_ms (workloads other than the headline): further untimed replays until the chip has run this load for that
        # long; under a bandwidth-heavy load it takes 20-30 ms to reach the clocks it then sustains (lm_head: 149 -> 141 us)
        settle_ms = self.settle_ms if settle_ms is None else settle_ms
        t_settle = time.perf_counter()
        for _ in range(40):
            if (time.perf_counter() - t_settle) * 1e3 >= settle_ms:
                break
            acc.graph_launch(g)
            acc.sync()
        t0 = time.perf_counter()
        acc.timer_begin()
        acc.graph_launch(g)
        gms = acc.timer_end()
        acc.sync()
        gwall = (time.perf_counter() - t0) * 1e3
        acc.graph_destroy(g)
        info = {"call_by_call_ms_per_step": ms / steps, "one_graph_ms_per_step": gms / steps,
                "timed_region": "one captured graph of the K steps"}
        return gms, gwall, info

    def _kernel_avg_us(self, fn, steps, warmup, prefix):
        """Second, identical pass with an event pair around every matmul kernel launch."""
        acc = self.acc
        acc.prof_reset()
        for i in range(warmup):
            fn(i)
        acc.sync()
        acc.prof_enable(True)
        for i in range(steps):
            fn(warmup + i)
        acc.sync()
        acc.prof_enable(False)
        ms, n = acc.prof_read(prefix)
        self.last_names = acc.prof_names()
        acc.prof_reset()
        return (ms / n * 1e3 if n else float("nan")), n

    # ------------------------------------------------------------------ GEMV
    def _trait_calls(self, keys, x, N, calls=200):
        """What a drop-in caller of the accelerator trait gets: host-pointer calls (activation in, result out, one stream
        synchronisation per call; PCIe-inclusive, never `value`), against the rotating weight copies.  us per call of
        smx_gemv (int8 activations), smx_gemv_f32 (the reference's per-weight gemv arithmetic) and smx_gemv_batch of 8."""
        acc = self.acc
        out = {}
        for label, fn in (("gemv", lambda i: acc.gemv(keys[i % len(keys)], x, N)),
                          ("gemv_f32", lambda i: acc.gemv_f32(keys[i % len(keys)], x, N))):
            for i in range(10):
                fn(i)
            t0 = time.perf_counter()
            for i in range(calls):
                fn(10 + i)
            out[label] = (time.perf_counter() - t0) / calls * 1e6
        nb = max(1, calls // 8)
        batch = lambda i: acc.gemv_batch([(keys[(8 * i + j) % len(keys)], x) for j in range(8)], [N] * 8)
        batch(0)
        t0 = time.perf_counter()
        for i in range(nb):
            batch(1 + i)
        out["gemv_batch_of_8"] = (time.perf_counter() - t0) / nb * 1e6
        out["note"] = "host-pointer trait calls, PCIe and one sync per call included"
        return out

    def gemv(self, name, ty, N, K, m, min_total_bytes, steps=None, warmup=None, f32=False, trait=False, settle_ms=None):
        """m rows against rotating weight copies.  m <= 4: the dot4 GEMV (quantiser fused for m = 1); 5..64 rows of a
        Q8_0 / Q4_0 weight: the small-batch kernel on the matrix cores; f32: the fp32-activation GEMV (no quantiser)."""
        acc, sy = self.acc, self.synth
        steps, warmup = steps or self.steps, warmup if warmup is not None else self.warmup
        algo, wbytes = gemv_bytes(ty, N, K, m)
        ncopies = max(2, -(-min_total_bytes // wbytes))
        self.log(f"[{name}] {ncopies} weight copies x {wbytes / 1e6:.1f} MB")
        nsrc = min(ncopies, 3)
        src = [sy.make_weight(ty, N, K, seed=1000 + i) for i in range(nsrc)]
        keys = []
        acc.sync()
        t_up = time.perf_counter()
        for i in range(ncopies):
            key = f"{name}.w{i}"
            assert getattr(acc, UPLOAD[ty])(key, src[i % nsrc], K, N)   # raw GGUF blocks from pageable memory, repacked on the device
            keys.append(key)
        acc.sync()
        upload_gbps = ncopies * src[0].nbytes / (time.perf_counter() - t_up) / 1e9
        del src
        x = sy.make_acts(m, K, seed=7)
        xd = acc.dev_alloc(x.nbytes)
        yd = acc.dev_alloc(m * N * 4)
        acc.h2d(xd, x)

        def step(i):
            if f32:
                acc.gemv_f32_dev(keys[i % ncopies], xd, yd)
            elif m > 32:    # a short prefill chunk: the GEMM entry point (33..64 rows: the small-batch kernel with two token tiles)
                acc.gemm_dev(keys[i % ncopies], xd, m, yd)
            else:
                acc.gemv_dev(keys[i % ncopies], xd, m, yd)

        self._first_touch(step, ncopies)
        kname = ("gemv_f32_" + KERNEL[ty][5:]) if f32 else (KERNEL[ty] if m <= 4 or ty == Q6_K else "skinny_" + KERNEL[ty][5:])
        # (the headline is run with settle_ms = 0: exactly W warm-up steps and one untimed replay in front of its timed region)
        ms, wall_ms, queued = self._timed_queued(step, steps, warmup, settle_ms=settle_ms)
        kus, nk = self._kernel_avg_us(step, steps, warmup, kname)
        trait_us = self._trait_calls(keys, x[0], N) if trait and m == 1 else None
        for k in keys:
            acc.evict(k)
        acc.dev_free(xd)
        acc.dev_free(yd)
        gbs = algo * steps / (ms * 1e-3) / 1e9
        # With one activation row the quantiser is fused: a step is exactly one launch of the GEMV
        # kernel, so the timed region's events give that kernel's average launch duration directly
        # (an event pair per launch adds about 2 us of its own and is reported separately).
        single = m == 1 or f32 or len(set(self.last_names)) == 1   # (2..4 rows may be quantised inside the GEMV: one launch)
        launch_us = ms / steps * 1e3 if single else kus
        kgbs = algo / (launch_us * 1e-6) / 1e9
        return {
            "workload": name, "shape": {"N": N, "K": K, "M": m}, "weight_copies": ncopies,
            "algorithmic_bytes": algo, "weight_bytes": wbytes, "steps": steps, "ms_per_step": ms / steps,
            "wall_ms_per_step": wall_ms / steps, "GBps": gbs, "weight_only_GBps": wbytes * steps / (ms * 1e-3) / 1e9,
            "frac_hbm_peak": gbs / HBM_PEAK_GBS,
            "kernel": kname, "kernel_avg_us": launch_us, "kernel_avg_us_event_pair": kus, "kernel_launches": nk,
            "kernel_GBps": kgbs, "kernel_frac_hbm_peak": kgbs / HBM_PEAK_GBS,
            "kernel_timing": ("events around the timed region's back-to-back launches / launches" if single
                              else "event pair around each launch"),
            "upload_GBps": upload_gbps,   # set-up: host call to synchronised device, raw block bytes per second
            **queued, **({"trait_call_us": trait_us} if trait_us else {}),
        }

    # ------------------------------------------------------------------ grouped GEMV (one launch, G weights)
    def gemv_group(self, name, ty, N, K, G, min_total_bytes, steps=None, warmup=None, act=0):
        """G single-token GEMVs of the same shape in one launch (the gate+up pair of a decode step for
        G = 2), rotating through >= 1 GB of weight copies; a step is one launch.  act = 1: the rmsnorm
        of the activation runs inside the same launch (norm + quantiser + G GEMVs)."""
        acc, sy = self.acc, self.synth
        steps, warmup = steps or self.steps, warmup if warmup is not None else self.warmup
        algo1, wbytes = gemv_bytes(ty, N, K, 1)
        ncopies = max(2 * G, -(-min_total_bytes // wbytes))
        ncopies = -(-ncopies // G) * G
        src = [sy.make_weight(ty, N, K, seed=1000 + i) for i in range(2)]
        keys = []
        for i in range(ncopies):
            key = f"{name}.w{i}"
            assert getattr(acc, UPLOAD[ty])(key, src[i % 2], K, N)
            keys.append(key)
        del src
        x = sy.make_acts(1, K, seed=7)
        xd = acc.dev_alloc(x.nbytes)
        acc.h2d(xd, x)
        yds = [acc.dev_alloc(N * 4) for _ in range(G)]
        ngroups = ncopies // G
        wd = 0
        if act:
            wd = acc.dev_alloc(K * 4)
            acc.h2d(wd, np.ones(K, np.float32) + 0.01 * x[0])

        def step(i):
            g0 = (i % ngroups) * G
            if act:
                acc.gemv_fused_dev(keys[g0:g0 + G], act, xd, wd, yds, 1e-6)
            else:
                acc.gemv_batch_dev(keys[g0:g0 + G], [xd] * G, yds)

        self._first_touch(step, ngroups)
        ms, wall_ms, queued = self._timed_queued(step, steps, warmup)
        for k in keys:
            acc.evict(k)
        acc.dev_free(xd)
        if wd:
            acc.dev_free(wd)
        for p in yds:
            acc.dev_free(p)
        algo = algo1 * G
        gbs = algo * steps / (ms * 1e-3) / 1e9
        return {"workload": name, "shape": {"N": N, "K": K, "M": 1, "weights_per_launch": G}, "weight_copies": ncopies,
                "algorithmic_bytes": algo, "steps": steps, "ms_per_step": ms / steps, "GBps": gbs,
                "frac_hbm_peak": gbs / HBM_PEAK_GBS, "kernel": KERNEL[ty], "kernel_avg_us": ms / steps * 1e3,
                "kernel_GBps": gbs, "kernel_frac_hbm_peak": gbs / HBM_PEAK_GBS, **queued}

    # ------------------------------------------------------------------ dense FFN decode step (2 calls, 2 launches)
    def ffn_block(self, name, ty, H, F, min_total_bytes, steps=None, warmup=None):
        """One token through a dense FFN in two launches: rmsnorm + quantiser + gate and up GEMVs with the SwiGLU
        product in the kernel's tail (smx_ffn_gate_up_dev), then quantiser + down GEMV on it; rotating through >= 1 GB
        of (gate, up, down) sets.  `three_launch_ms_per_step`: the same step as gate/up pair, SwiGLU quantiser, down."""
        acc, sy = self.acc, self.synth
        steps, warmup = steps or self.steps, warmup if warmup is not None else self.warmup
        a1, w1 = gemv_bytes(ty, F, H, 1)
        a2, w2 = gemv_bytes(ty, H, F, 1)
        nsets = max(2, -(-min_total_bytes // (2 * w1 + w2)))
        srcs = [(sy.make_weight(ty, F, H, seed=1500 + i), sy.make_weight(ty, H, F, seed=1600 + i)) for i in range(2)]
        for i in range(nsets):
            up_fn = getattr(acc, UPLOAD[ty])
            assert up_fn(f"{name}.g{i}", srcs[i % 2][0], H, F) and up_fn(f"{name}.u{i}", srcs[(i + 1) % 2][0], H, F)
            assert up_fn(f"{name}.d{i}", srcs[i % 2][1], F, H)
        del srcs
        x = sy.make_acts(1, H, seed=7)
        xd, wd, gd, ud, yd = (acc.dev_alloc(n * 4) for n in (H, H, F, F, H))
        acc.h2d(xd, x)
        acc.h2d(wd, np.ones(H, np.float32))

        def step3(i):
            j = i % nsets
            acc.gemv_fused_dev([f"{name}.g{j}", f"{name}.u{j}"], 1, xd, wd, [gd, ud], 1e-6)
            acc.gemv_fused_dev([f"{name}.d{j}"], 2, gd, ud, [yd])

        def step(i):
            j = i % nsets
            acc.ffn_gate_up_dev(f"{name}.g{j}", f"{name}.u{j}", 2, xd, gd, norm=True, norm_w_dev=wd, eps=1e-6)
            acc.gemv_dev(f"{name}.d{j}", gd, 1, yd)

        self._first_touch(step, nsets)
        ms3, _, _ = self._timed_queued(step3, steps, warmup)
        ms, wall_ms, queued = self._timed_queued(step, steps, warmup)
        for i in range(nsets):
            for t in "gud":
                acc.evict(f"{name}.{t}{i}")
        for p in (xd, wd, gd, ud, yd):
            acc.dev_free(p)
        algo = 2 * a1 + a2
        gbs = algo * steps / (ms * 1e-3) / 1e9
        return {"workload": name, "shape": {"hidden": H, "ffn": F, "M": 1, "calls_per_step": 2, "launches_per_step": 2}, "weight_sets": nsets,
                "algorithmic_bytes": algo, "steps": steps, "ms_per_step": ms / steps, "GBps": gbs,
                "frac_hbm_peak": gbs / HBM_PEAK_GBS, "three_launch_ms_per_step": ms3 / steps, **queued}

    # ------------------------------------------------------------------ dense FFN prefill block (3 GEMMs)
    def ffn_prefill_block(self, name, ty, H, F, M, steps=None, warmup=None):
        """M tokens through a dense FFN: rmsnorm + quantiser + gate GEMM, the same for up, then
        SwiGLU + quantiser + down GEMM (each producer runs inside its quantiser launch)."""
        acc, sy = self.acc, self.synth
        steps, warmup = steps or max(20, self.steps // 20), warmup if warmup is not None else 20   # sustained clocks: see gemm()
        up_fn = getattr(acc, UPLOAD[ty])
        assert up_fn(name + ".g", sy.make_weight(ty, F, H, seed=1700), H, F)
        assert up_fn(name + ".u", sy.make_weight(ty, F, H, seed=1701), H, F)
        assert up_fn(name + ".d", sy.make_weight(ty, H, F, seed=1702), F, H)
        x = sy.make_acts(M, H, seed=7)
        xd, wd, gd, ud, yd = (acc.dev_alloc(n * 4) for n in (M * H, H, M * F, M * F, M * H))
        acc.h2d(xd, x)
        acc.h2d(wd, np.ones(H, np.float32))

        def step(i):
            acc.gemm_fused_dev(name + ".g", 1, xd, wd, M, gd, 1e-6)
            acc.gemm_fused_dev(name + ".u", 1, xd, wd, M, ud, 1e-6)
            acc.gemm_fused_dev(name + ".d", 2, gd, ud, M, yd)

        ms, wall_ms = self._timed(step, steps, warmup)
        for t in "gud":
            acc.evict(f"{name}.{t}")
        for p in (xd, wd, gd, ud, yd):
            acc.dev_free(p)
        ops = 3 * 2 * M * F * H
        tops = ops * steps / (ms * 1e-3) / 1e12
        return {"workload": name, "shape": {"hidden": H, "ffn": F, "M": M, "gemms_per_step": 3}, "ops": ops, "steps": steps,
                "ms_per_step": ms / steps, "TOPS": tops, "frac_int8_peak": tops / INT8_PEAK_TOPS}

    # ------------------------------------------------------------------ copy (counter calibration)
    def copy_calib(self, nbytes=256 << 20, steps=20):
        """A plain copy of known size: what FETCH_SIZE / WRITE_SIZE read for it scales the counters."""
        acc = self.acc
        src, dst = acc.dev_alloc(nbytes), acc.dev_alloc(nbytes)
        acc.h2d(src, np.zeros(1 << 20, np.uint8))

        def step(i):
            acc.dev_copy(dst, src, nbytes)

        ms, _ = self._timed(step, steps, 2)
        acc.dev_free(src)
        acc.dev_free(dst)
        return {"workload": "copy_calib", "bytes_read": nbytes, "bytes_written": nbytes, "steps": steps,
                "ms_per_step": ms / steps, "GBps_read_plus_write": 2 * nbytes * steps / (ms * 1e-3) / 1e9}

    # ------------------------------------------------------------------ GEMM
    def gemm(self, name, ty, M, N, K, steps=None, warmup=None):
        acc, sy = self.acc, self.synth
        # Under matrix load the chip takes some 20 ms to settle at the clock it sustains (the first launches after idle
        # run 15 % slower, the next ones briefly faster): 50 untimed launches first, whatever --steps says; a prefill is
        # hundreds of such launches back to back.
        steps, warmup = steps or max(50, self.steps // 8), warmup if warmup is not None else 50
        raw = sy.make_weight(ty, N, K, seed=2000 + ty)
        assert getattr(acc, UPLOAD[ty])(name, raw, K, N)
        del raw
        xs = sy.make_acts(M, K, seed=8)
        xd = acc.dev_alloc(xs.nbytes)
        yd = acc.dev_alloc(M * N * 4)
        acc.h2d(xd, xs)

        def step(i):
            acc.gemm_dev(name, xd, M, yd)

        ms, wall_ms = self._timed(step, steps, warmup)
        kname = {Q4_0: "gemm_i8_q4_0", Q8_0: "gemm_i8_q8_0", Q6_K: "gemm_i8_q6_k"}[ty]
        kus, nk = self._kernel_avg_us(step, steps, warmup, kname)
        names = self.last_names
        acc.evict(name)
        acc.dev_free(xd)
        acc.dev_free(yd)
        ops = 2 * M * N * K
        tops = ops * steps / (ms * 1e-3) / 1e12
        ktops = ops / (kus * 1e-6) / 1e12
        return {
            "workload": name, "shape": {"M": M, "N": N, "K": K}, "ops": ops, "steps": steps,
            "ms_per_step": ms / steps, "wall_ms_per_step": wall_ms / steps, "TOPS": tops,
            "frac_int8_peak": tops / INT8_PEAK_TOPS, "kernel": kname, "kernel_avg_us": kus, "kernel_launches": nk,
            "kernel_TOPS": ktops, "kernel_frac_int8_peak": ktops / INT8_PEAK_TOPS,
            "split_k": "splitk_reduce" in names,
        }

    # ------------------------------------------------------------------ decode chain as one graph
    def decode_chain_graph(self, name, layers=4, hidden=2048, ffn=8192, ne=64, eff=768, k=8, nsets=4, steps=None, warmup=None):
        """`layers` decoder FFN halves per token, everything resident and routed on the device (strix.rs_amd/chain.py, the
        sequence tests/test_gpu_chain.py checks against the oracle): per layer rmsnorm + gate/up GEMVs + SwiGLU product
        (one launch), down GEMV, router logits GEMV, the k routed experts' FFN (two launches, the routing in the prologue of the first).  Attention
        is outside this path.  Q4_0 dense weights, Q8_0 experts and router.  Cache-cold: `nsets` complete weight sets
        (every layer's dense weights and expert tensors) are resident and ONE captured graph runs one token through each
        set in turn, so a token's weights were last read nsets - 1 tokens (> 1 GB of other weights) ago."""
        acc, sy = self.acc, self.synth
        chain_mod = _load("strix_rs_amd_chain", os.path.join(ROOT, "strix.rs_amd", "chain.py"))
        steps, warmup = steps or self.steps, warmup if warmup is not None else self.warmup
        base = 50
        nl = layers * nsets
        dense = [(sy.make_weight(Q4_0, ffn, hidden, seed=4000 + i), sy.make_weight(Q4_0, hidden, ffn, seed=4200 + i)) for i in range(2)]
        router = sy.make_weight(Q8_0, ne, hidden, seed=4300)
        gate, up, down = sy.make_moe_q8(ne, hidden, eff, seed=4400)
        for l in range(nl):
            assert acc.upload_q4_0(f"{name}.g{l}", dense[l % 2][0], hidden, ffn)
            assert acc.upload_q4_0(f"{name}.u{l}", dense[(l + 1) % 2][0], hidden, ffn)
            assert acc.upload_q4_0(f"{name}.d{l}", dense[l % 2][1], ffn, hidden)
            assert acc.upload_q8_0(f"{name}.r{l}", router, hidden, ne)
            assert acc.upload_moe_q8(base + l, gate, up, down, hidden, eff, ne)
        del dense, gate, up, down
        x = sy.make_acts(1, hidden, seed=11)
        xd, nw = acc.dev_alloc(hidden * 4), acc.dev_alloc(hidden * 4)
        acc.h2d(xd, x)
        acc.h2d(nw, np.ones(hidden, np.float32))
        keys = lambda l: tuple(f"{name}.{t}{l}" for t in "gudr")

        def measure(sets, route="in_launch"):
            ch = chain_mod.FfnMoeChain(acc, layers, hidden, ffn, ne, k, keys, lambda l: base + l, nw, route=route)

            def tokens():   # one token through each weight set
                for s_ in range(sets):
                    ch.enqueue(xd, layer_offset=s_ * layers)

            tokens()        # also the first read of every set's weights
            acc.sync()
            acc.graph_begin()
            tokens()
            g = acc.graph_end()
            reps = max(1, steps // sets)
            eager_ms, _ = self._timed(lambda i: tokens(), reps, max(1, warmup // sets))
            graph_ms, _ = self._timed(lambda i: acc.graph_launch(g), reps, max(1, warmup // sets))
            acc.graph_destroy(g)
            n_launch = ch.launches_per_token()
            ch.close()
            return graph_ms / (reps * sets) * 1e3, eager_ms / (reps * sets) * 1e3, n_launch

        cold_us, cold_eager_us, n_launch = measure(nsets)
        routed_by_a_launch_us, _, _ = measure(nsets, route="launches")
        hot_us, _, _ = measure(1)
        for l in range(nl):
            for t in "gudr":
                acc.evict(f"{name}.{t}{l}")
        acc.dev_free(xd)
        acc.dev_free(nw)
        wbytes = layers * (3 * gemv_bytes(Q4_0, ffn, hidden)[1] + gemv_bytes(Q8_0, ne, hidden)[1] + k * 3 * eff * (hidden // 32) * 34)
        gbs = wbytes / (cold_us * 1e-6) / 1e9
        return {"workload": name, "shape": {"layers": layers, "hidden": hidden, "ffn": ffn, "experts": ne, "eff": eff, "top_k": k,
                                            "launches_per_token": n_launch, "weight_sets_rotated": nsets},
                "weight_bytes_per_token": wbytes, "bytes_between_two_reads_of_a_weight": wbytes * (nsets - 1),
                "steps": max(1, steps // nsets) * nsets, "graph_us_per_token": cold_us, "eager_us_per_token": cold_eager_us,
                "routing_as_a_launch_of_its_own_us_per_token": routed_by_a_launch_us, "one_weight_set_us_per_token": hot_us,
                "GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS,
                "note": "graph_us_per_token is cache-cold (weight sets rotate); one_weight_set_us_per_token re-reads one 274 MB "
                        "set, partly from the 256 MB Infinity Cache"}

    def moe_prefill_timeline(self, name, ne, hidden, eff, k, m):
        """Start and end of every workgroup of the two grouped GEMM launches of one MoE prefill layer call (Q8_0 experts, the
        routing of moe_prefill_m512).  Runs only when named with --only, and needs a development build of the library with the
        kernel's timeline compiled in:  python strix.rs_amd/build.py -DSMX_GEMM_TRACE  (rebuild without the flag afterwards)."""
        import collections
        import ctypes
        acc, sy = self.acc, self.synth
        try:
            hook = acc._L.smx_debug_gemm_trace
        except AttributeError:
            return {"workload": name, "skipped": "the library was built without -DSMX_GEMM_TRACE"}
        hook.argtypes = [ctypes.c_void_p]
        gate, up, down = sy.make_moe_q8(ne, hidden, eff, seed=3000)
        assert acc.upload_moe_q8(0, gate, up, down, hidden, eff, ne)
        ids, w = sy.zipf_routing(m, ne, k, seed=5)
        plan, slot_tok, wslot = sy.group_by_expert(ids, w, ne)
        xs = sy.make_acts(m, hidden, seed=9)
        xd, yd, tb = acc.dev_alloc(xs.nbytes), acc.dev_alloc(xs.nbytes), acc.dev_alloc(8192 * 32)
        acc.h2d(xd, xs)
        for _ in range(100):   # the clock the chip sustains under this load
            acc.moe_layer_resident(0, xd, m, plan, slot_tok, wslot, yd)
        acc.h2d(tb, np.zeros(8192 * 4, np.uint64))
        assert hook(tb) == 0
        acc.moe_layer_resident(0, xd, m, plan, slot_tok, wslot, yd)
        acc.sync()
        t = acc.d2h(np.empty(8192 * 4, np.uint64), tb).reshape(8192, 4).copy()
        hook(None)
        out = {"workload": name, "shape": {"experts": ne, "hidden": hidden, "eff": eff, "top_k": k, "M": m}, "launches": {}}
        for lname, base in (("gate_up", 4096), ("down", 0)):
            r = t[base:base + 4096]
            r = r[r[:, 1] > 0]
            t0 = r[:, 0].min()
            st, en = (r[:, 0] - t0) / 100.0, (r[:, 1] - t0) / 100.0   # us on the 100 MHz clock
            live = (r[:, 2] & 0xffffffff).astype(int)
            hw, xcc = r[:, 3] & 0xffffffff, (r[:, 3] >> 32) & 0xf
            cu = ((hw >> 8) & 0xf) | (((hw >> 12) & 1) << 4) | (((hw >> 13) & 7) << 5) | (xcc << 8)
            rec = {"workgroups": int(len(r)), "makespan_us": float(en.max()), "compute_units": len(set(cu.tolist())), "classes": {}}
            for cname, sel in (("more_than_64_tokens", live > 64), ("33_to_64_tokens", (live > 32) & (live <= 64)), ("up_to_32_tokens", live <= 32)):
                if sel.any():
                    d = en[sel] - st[sel]
                    rec["classes"][cname] = {"tiles": int(sel.sum()), "duration_us_mean_min_max": [float(d.mean()), float(d.min()), float(d.max())],
                                             "start_us_mean_max": [float(st[sel].mean()), float(st[sel].max())], "last_end_us": float(en[sel].max())}
            last = collections.defaultdict(float)
            for i in range(len(r)):
                last[cu[i]] = max(last[cu[i]], en[i])
            ends = np.array(list(last.values()))
            rec["last_end_per_compute_unit_us_mean_min_max"] = [float(ends.mean()), float(ends.min()), float(ends.max())]
            rec["workgroups_running_at_us"] = {str(x): int(((st <= x) & (en > x)).sum()) for x in range(10, int(en.max()), 10)}
            rec["workgroups_not_started_at_us"] = {str(x): int((st > x).sum()) for x in range(10, int(en.max()), 10)}
            out["launches"][lname] = rec
        for p_ in (xd, yd, tb):
            acc.dev_free(p_)
        return out

    # ------------------------------------------------------------------ MoE
    def moe(self, name, ne, hidden, eff, k, m, layers, steps=None, warmup=None, ty=Q8_0):
        """Decode (m == 1): rotate over `layers` resident layers (320 MB each) so expert reads are
        cache-cold.  Prefill (m > 1): one layer, m tokens grouped by expert."""
        acc, sy = self.acc, self.synth
        steps, warmup = steps or self.steps, warmup if warmup is not None else self.warmup
        gate, up, down = (sy.make_moe_q6 if ty == Q6_K else sy.make_moe_q8)(ne, hidden, eff, seed=3000)
        for l in range(layers):
            assert (acc.upload_moe_q6 if ty == Q6_K else acc.upload_moe_q8)(l, gate, up, down, hidden, eff, ne)
        del gate, up, down
        out = {"workload": name, "shape": {"experts": ne, "hidden": hidden, "eff": eff, "top_k": k, "M": m}}
        if m == 1:
            ids, w = sy.zipf_routing(max(64, steps + warmup), ne, k, seed=5)
            x = sy.make_acts(1, hidden, seed=9)
            xd = acc.dev_alloc(x.nbytes)
            yd = acc.dev_alloc(hidden * 4)
            acc.h2d(xd, x)

            def step(i):
                acc.moe_ffn_dev(i % layers, ids[i % len(ids)], w[i % len(ids)], xd, yd)

            self._first_touch(step, len(ids))   # (nearly) every expert of every layer once
            ms, wall_ms, queued = self._timed_queued(step, steps, warmup)
            kus, nk = self._kernel_avg_us(step, steps, warmup, "moe_gemv")
            acc.dev_free(xd)
            acc.dev_free(yd)
            wbytes = k * 3 * eff * (hidden // 256 * 210 if ty == Q6_K else hidden // 32 * 34)
            gbs = wbytes * steps / (ms * 1e-3) / 1e9
            out.update({"expert_weight_bytes": wbytes, "layers_rotated": layers, "steps": steps,
                        "ms_per_step": ms / steps, "GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS,
                        "kernel": "moe_gemv_gate_up + moe_gemv_down", "kernel_avg_us_sum": kus * 2,
                        "kernel_GBps": wbytes / (kus * 2 * 1e-6) / 1e9, **queued})
        else:
            # Host-buffer calls (every call uploads its rows and tables and waits for the result), then the resident form
            # back to back: 100 untimed calls first so that the chip has settled at the clock it sustains (see gemm()),
            # then `steps` calls between two events, then as many with an event pair around every kernel.
            hsteps = max(5, steps // 20)
            steps = max(50, steps // 8)
            ids, w = sy.zipf_routing(m, ne, k, seed=5)
            plan, slot_tok, wslot = sy.group_by_expert(ids, w, ne)
            xs = sy.make_acts(m, hidden, seed=9)
            for _ in range(2):
                acc.moe_layer_q8_dev(0, xs, m, plan, slot_tok, wslot)
            t0 = time.perf_counter()
            for _ in range(hsteps):
                acc.moe_layer_q8_dev(0, xs, m, plan, slot_tok, wslot)
            wall_ms = (time.perf_counter() - t0) * 1e3 * steps / hsteps
            xd, yd = acc.dev_alloc(xs.nbytes), acc.dev_alloc(xs.nbytes)
            acc.h2d(xd, xs)
            for _ in range(100):
                acc.moe_layer_resident(0, xd, m, plan, slot_tok, wslot, yd)
            acc.sync()
            acc.timer_begin()
            for _ in range(steps):
                acc.moe_layer_resident(0, xd, m, plan, slot_tok, wslot, yd)
            res_ms = acc.timer_end()
            acc.prof_reset()
            acc.prof_enable(True)
            for _ in range(steps):
                acc.moe_layer_resident(0, xd, m, plan, slot_tok, wslot, yd)
            acc.sync()
            acc.prof_enable(False)
            g_ms, _ = acc.prof_read("moe_gemm")
            all_ms = sum(acc.prof_read(p)[0] for p in ("actquant", "moe_gemm", "silu_mul_quant", "moe_combine"))
            acc.prof_reset()
            acc.dev_free(xd)
            acc.dev_free(yd)
            ops = 2 * slot_tok.size * 3 * eff * hidden
            # This configuration is HBM-bound, not MFMA-bound: 38.65 GOP over the weights of every expert that got a token
            # (302 MB when all 64 did) is 128 op/B, far left of the 625 op/B ridge of 5 POP/s over 8 TB/s.
            active = sum(1 for e_, _, cnt in plan if cnt > 0)
            wbytes = active * 3 * eff * (hidden // 256 * 210 if ty == Q6_K else hidden // 32 * 34)
            out.update({"bound": "hbm", "active_experts": active, "expert_weight_bytes": wbytes,
                        "GBps": wbytes * steps / (all_ms * 1e-3) / 1e9,
                        "frac_hbm_peak": wbytes * steps / (all_ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
            out.update({"resident_ms_per_step": res_ms / steps, "resident_TOPS": ops * steps / (res_ms * 1e-3) / 1e12})
            out.update({"slots": int(slot_tok.size), "ops": ops, "steps": steps,
                        "device_ms_per_step": all_ms / steps, "host_call_ms_per_step": wall_ms / steps,
                        "TOPS": ops * steps / (all_ms * 1e-3) / 1e12,
                        "gemm_kernels_TOPS": ops * steps / (g_ms * 1e-3) / 1e12,
                        "frac_int8_peak": ops * steps / (all_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS})
        for l in range(layers):
            pass  # layers stay resident until the context closes (they are re-uploaded per workload)
        return out


def cpu_baseline(seconds=10.0, gemm_seconds=8.0):
    """The reference's CPU matmul (dequantise a row, f32 dot, rows split over the host's cores with rayon:
    crates/strix-backend-cpu/src/mellum.rs:219-237, gemma.rs:318) as restated by the oracle: the headline GEMV, and the
    batched form (mellum.rs:244-271: a row dequantised once, dotted with every token) on a row sample of the
    ffn_up GEMM.  Threads: every core this process may run on (the GPU box gives a one-GPU job 16 of its
    logical cores; both counts are reported)."""
    orc = _load("strix_oracle", os.path.join(ROOT, "oracle", "strix_oracle.py"))
    synth = sys.modules["strix_rs_amd_synth"]
    N, K = 9728, 2560
    logical = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = logical
    cores = max(1, min(usable, int(os.environ.get("OMP_NUM_THREADS", usable))))
    raws = [synth.make_weight(Q4_0, N, K, seed=1000 + i) for i in range(4)]
    x = synth.make_acts(1, K, seed=7)
    orc.matmul_f32(Q4_0, raws[0], K, N, x, 1, cores)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        orc.matmul_f32(Q4_0, raws[n % 4], K, N, x, 1, cores)
        n += 1
    dt = time.perf_counter() - t0
    algo, _ = gemv_bytes(Q4_0, N, K, 1)
    out = {"value": algo * n / dt / 1e9, "unit": "GB/s", "cores": cores, "host_logical_cores": logical, "kind": "port",
           "sample": f"{n} f32 GEMVs of the 9728x2560 Q4_0 weight over {dt:.1f} s, 4 rotating copies, "
                     f"row-parallel dequantise+dot on {cores} threads", "ms_per_gemv": dt / n * 1e3}
    # the prefill GEMM on the CPU: 2048 tokens x 3840, a sample of 256 of the 15360 Q8_0 weight rows per pass
    M, Kg, rows = 2048, 3840, 256
    rawg = synth.make_weight(Q8_0, rows, Kg, seed=2008)
    xs = synth.make_acts(M, Kg, seed=8)
    orc.matmul_f32(Q8_0, rawg, Kg, rows, xs, 1, cores)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < gemm_seconds:
        orc.matmul_f32(Q8_0, rawg, Kg, rows, xs, 1, cores)
        n += 1
    dt = time.perf_counter() - t0
    out["gemm"] = {"value": 2.0 * M * rows * Kg * n / dt / 1e9, "unit": "GOP/s", "cores": cores, "kind": "port",
                   "sample": f"{n} passes of 2048 tokens x 3840 against {rows} of the 15360 Q8_0 rows of ffn_up over {dt:.1f} s "
                             f"(a row dequantised once, f32 dot with every token), {cores} threads"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--only", default="", help="comma-separated workload names (default: all)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-floors", action="store_true", help="skip the measurement-only kernels (empty launch, read floor, MFMA+FMA ceiling)")
    ap.add_argument("--settle-ms", type=float, default=30.0, help="untimed graph replays of every workload but the headline until the chip has run it this long (0: one replay)")
    ap.add_argument("--no-trait", action="store_true", help="skip the host-pointer trait-call timing of the headline workload (keeps a kernel trace of the run to the timed launches)")
    ap.add_argument("--records", default=os.path.join(ROOT, "bench_workloads.json"), help="where the per-workload records are written")
    ap.add_argument("--no-headline", action="store_true", help="skip the headline GEMV when --only names other workloads")
    ap.add_argument("--tune", default="", help="launch-geometry overrides for sweeps, e.g. gemm_nw=4,gemm_splitk=2")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this path is built and measured on a single MI355X "
                 "(--gpus must be 1); over several GPUs the path would shard by output rows, one all-gather per group of GEMVs")
    only = set(filter(None, a.only.split(",")))
    want = lambda n: not only or n in only
    b = Bench(a.steps, a.warmup)
    b.settle_ms = a.settle_ms
    b.log("device:", b.acc.name())
    for kv in filter(None, a.tune.split(",")):
        knob, value = kv.split("=")
        b.acc.tune(knob, int(value))
    GB = 1 << 30
    work = {}
    floors = None
    if want("machine_floors") and not a.no_floors:   # first: it also brings the clocks up before the headline's few steps
        floors = machine_floors(b.log)
        work["machine_floors"] = floors
    if a.no_headline and only:
        head = None
    else:
        head = b.gemv("q4_0_gemv_9728x2560", Q4_0, 9728, 2560, 1, int(1.1 * GB), trait=not a.no_trait, settle_ms=0.0)
        work[head["workload"]] = head
        b.log(json.dumps(head))
    plans = [
        ("copy_calib", lambda: b.copy_calib()),
        ("q4_0_gemv_9728x2560_gate_up_pair", lambda: b.gemv_group("q4_0_gemv_9728x2560_gate_up_pair", Q4_0, 9728, 2560, 2, int(1.1 * GB))),
        ("q4_0_rmsnorm_gate_up_pair", lambda: b.gemv_group("q4_0_rmsnorm_gate_up_pair", Q4_0, 9728, 2560, 2, int(1.1 * GB), act=1)),
        ("q4_0_gemv_9728x2560_batch8", lambda: b.gemv_group("q4_0_gemv_9728x2560_batch8", Q4_0, 9728, 2560, 8, int(1.1 * GB))),
        ("q4_0_ffn_decode_block_2560x9728", lambda: b.ffn_block("q4_0_ffn_decode_block_2560x9728", Q4_0, 2560, 9728, int(1.1 * GB))),
        ("q8_0_gemv_2560x9728_m1", lambda: b.gemv("q8_0_gemv_2560x9728_m1", Q8_0, 2560, 9728, 1, int(1.1 * GB))),
        ("q8_0_gemv_2560x9728_m4", lambda: b.gemv("q8_0_gemv_2560x9728_m4", Q8_0, 2560, 9728, 4, int(1.1 * GB))),
        ("q8_0_gemv_2560x9728_m8", lambda: b.gemv("q8_0_gemv_2560x9728_m8", Q8_0, 2560, 9728, 8, int(1.1 * GB))),
        ("q8_0_small_batch_2560x9728_m16", lambda: b.gemv("q8_0_small_batch_2560x9728_m16", Q8_0, 2560, 9728, 16, int(1.1 * GB))),
        ("q8_0_small_batch_2560x9728_m32", lambda: b.gemv("q8_0_small_batch_2560x9728_m32", Q8_0, 2560, 9728, 32, int(1.1 * GB))),
        ("q8_0_small_batch_2560x9728_m64", lambda: b.gemv("q8_0_small_batch_2560x9728_m64", Q8_0, 2560, 9728, 64, int(1.1 * GB))),
        ("q4_0_gemv_f32_9728x2560", lambda: b.gemv("q4_0_gemv_f32_9728x2560", Q4_0, 9728, 2560, 1, int(1.1 * GB), f32=True)),
        ("q8_0_gemv_f32_2560x9728", lambda: b.gemv("q8_0_gemv_f32_2560x9728", Q8_0, 2560, 9728, 1, int(1.1 * GB), f32=True)),
        ("q6_k_gemv_f32_15360x3840", lambda: b.gemv("q6_k_gemv_f32_15360x3840", Q6_K, 15360, 3840, 1, int(1.1 * GB), f32=True)),
        ("q6_k_gemv_15360x3840", lambda: b.gemv("q6_k_gemv_15360x3840", Q6_K, 15360, 3840, 1, int(1.1 * GB))),
        ("q6_k_lm_head_262144x3840", lambda: b.gemv("q6_k_lm_head_262144x3840", Q6_K, 262144, 3840, 1, int(1.6 * GB),
                                                     steps=max(10, a.steps // 10), warmup=2)),
        ("gemm_q8_0_ffn_up", lambda: b.gemm("gemm_q8_0_ffn_up", Q8_0, 2048, 15360, 3840)),
        ("gemm_q4_0_ffn_up", lambda: b.gemm("gemm_q4_0_ffn_up", Q4_0, 2048, 15360, 3840)),
        ("gemm_q8_0_ffn_down", lambda: b.gemm("gemm_q8_0_ffn_down", Q8_0, 2048, 3840, 15360)),
        ("gemm_q4_0_ffn_down", lambda: b.gemm("gemm_q4_0_ffn_down", Q4_0, 2048, 3840, 15360)),
        ("q8_0_ffn_prefill_block_m2048", lambda: b.ffn_prefill_block("q8_0_ffn_prefill_block_m2048", Q8_0, 3840, 15360, 2048)),
        ("gemm_q6_k_ffn_up", lambda: b.gemm("gemm_q6_k_ffn_up", Q6_K, 2048, 15360, 3840)),
        ("gemm_q6_k_ffn_down", lambda: b.gemm("gemm_q6_k_ffn_down", Q6_K, 2048, 3840, 15360)),
        ("decode_chain_4layers_graph", lambda: b.decode_chain_graph("decode_chain_4layers_graph")),
        ("moe_decode", lambda: b.moe("moe_decode", 64, 2048, 768, 8, 1, layers=4)),
        ("moe_prefill_m512", lambda: b.moe("moe_prefill_m512", 64, 2048, 768, 8, 512, layers=1)),
        ("moe_decode_q6_k", lambda: b.moe("moe_decode_q6_k", 64, 2048, 768, 8, 1, layers=4, ty=Q6_K)),
        ("moe_prefill_m512_q6_k", lambda: b.moe("moe_prefill_m512_q6_k", 64, 2048, 768, 8, 512, layers=1, ty=Q6_K)),
    ]
    if "moe_prefill_timeline" in only:   # development builds only, never part of a default run
        plans.append(("moe_prefill_timeline", lambda: b.moe_prefill_timeline("moe_prefill_timeline", 64, 2048, 768, 8, 512)))
    for name, fn in plans:
        if want(name):
            r = fn()
            work[name] = r
            b.log(json.dumps(r))
    if floors:   # every GEMM against the measured ceiling of its own arithmetic (MFMA + the rescale operations its format needs)
        for n, w in work.items():
            if n.startswith("gemm_") and "kernel_TOPS" in w:
                ceil = floors["mfma_plus_rescale_fma_q6_k" if "q6_k" in n else "mfma_plus_rescale_fma"]["TOPS"]
                w["rescale_ceiling_TOPS"], w["kernel_over_ceiling"] = ceil, w["kernel_TOPS"] / ceil
                b.log(f"{n}: kernel {w['kernel_TOPS']:.0f} TOPS = {w['kernel_over_ceiling']:.2f} of its arithmetic's ceiling ({ceil:.0f} TOPS)")
    if head is None:  # sweep mode: per-workload records only, no headline line
        try:
            with open(a.records, "w") as f:
                json.dump({"workloads": work}, f, indent=1)
        except OSError as e:
            b.log(f"could not write {a.records}: {e}")
        print(json.dumps({"workloads": sorted(work)}), flush=True)
        return
    cpu = None if a.no_cpu else cpu_baseline()
    b.acc.close()
    wpath = a.records
    try:
        with open(wpath, "w") as f:
            json.dump({"workloads": work}, f, indent=1)
        b.log(f"per-workload records: {wpath}")
    except OSError as e:   # a read-only tree: the records are on stderr anyway
        b.log(f"could not write {wpath}: {e}")
    print(result_line(work, a.warmup, cpu), flush=True)


MAX_LINE_BYTES = 4096   # the final stdout line must fit the tail a harness keeps; per-workload records go to stderr and a file


def _r(v, digits=4):
    """Floats rounded to `digits` significant digits (the line is a summary; the records hold every digit)."""
    if isinstance(v, float):
        return float(f"{v:.{digits}g}")
    if isinstance(v, dict):
        return {k: _r(x, digits) for k, x in v.items()}
    return v


def _summary(w):
    """A workload's key figure for the result line: [us per step, fraction of its roofline's peak]."""
    us = None
    for k in ("ms_per_step", "device_ms_per_step"):
        if k in w:
            us = w[k] * 1e3
            break
    if us is None and "graph_us_per_token" in w:
        us = w["graph_us_per_token"]
    frac = w.get("frac_hbm_peak", w.get("frac_int8_peak"))
    return [_r(us), _r(frac)]


def result_line(work, warmup, cpu):
    """The ONE stdout line of the run, built from the per-workload records: metric, value, config, roofline of the dominant
    kernel, the best int8 GEMM with its roofline, the CPU baseline, and a two-number summary of every other workload.
    Always shorter than MAX_LINE_BYTES."""
    head = work["q4_0_gemv_9728x2560"]
    floors = work.get("machine_floors")
    gemms = [w for n, w in work.items() if n.startswith("gemm_")]
    best_gemm = max(gemms, key=lambda w: w["TOPS"]) if gemms else None
    config = {"workload": "Q4_0 decode GEMV, weight 9728x2560, 1 token, Q8 activations, cache-cold: "
                          f"{head['weight_copies']} rotating resident weight copies "
                          f"({head['weight_copies'] * head['weight_bytes'] / 1e9:.2f} GB), each read once before the warm-up; "
                          "step = one launch (activation quantiser fused into the GEMV)",
              "frac_hbm_peak": head["frac_hbm_peak"], "timed_region": head["timed_region"],
              "call_by_call_us": head["call_by_call_ms_per_step"] * 1e3, "one_graph_us": head["one_graph_ms_per_step"] * 1e3}
    if "trait_call_us" in head:
        config["trait_call_us"] = head["trait_call_us"]
    line = {
        "metric": "Q4_0 GEMV GB/s (% HBM peak); int8 prefill GEMM TOPS (% MFMA peak)",
        "value": head["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": head["steps"], "warmup": warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic", "config": config,
        "roofline": {"bound": "hbm", "achieved": head["kernel_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["kernel_frac_hbm_peak"], "traffic": HEADLINE_TRAFFIC_BYTES,
                     "traffic_source": "profiles/gemv_q4_0_9728x2560_hbm_traffic.md (constant, not measured by this run)",
                     "kernel": head["kernel"], "kernel_avg_us": head["kernel_avg_us"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "method": "HIP events on the launch stream around the timed region's K back-to-back launches"},
        "gemm": None if not best_gemm else {
            "workload": best_gemm["workload"], "value": best_gemm["TOPS"], "unit": "TOPS",
            "frac_int8_mfma_peak": best_gemm["frac_int8_peak"],
            "roofline": {"bound": "mfma", "achieved": best_gemm["kernel_TOPS"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": best_gemm["kernel_frac_int8_peak"], "traffic": GEMM_TRAFFIC_BYTES.get(best_gemm["workload"]),
                         "kernel": best_gemm["kernel"], "kernel_avg_us": best_gemm["kernel_avg_us"]}},
    }
    if floors:
        floor_us = floors["read_only_cold_us"]["14MB_q4_0_9728x2560"]
        line["roofline"]["read_only_floor_us"] = floor_us
        line["roofline"]["kernel_over_floor"] = head["kernel_avg_us"] / floor_us
        line["roofline"]["empty_launch_us"] = floors["empty_launch_us"]["256x1024"]
        if "empty_launch_in_a_graph_us" in floors:
            line["roofline"]["empty_launch_in_a_graph_us"] = floors["empty_launch_in_a_graph_us"]["256x1024"]
        if best_gemm:
            ceil = floors["mfma_plus_rescale_fma"]["TOPS"]
            line["gemm"]["roofline"]["rescale_ceiling_TOPS"] = ceil
            line["gemm"]["roofline"]["kernel_over_ceiling"] = best_gemm["kernel_TOPS"] / ceil
    if cpu is not None:
        line["cpu_baseline"] = cpu
    line = _r(line)
    # every other workload as [us per step, fraction of peak]; dropped from the end if the line would grow too long
    others = {n: _summary(w) for n, w in work.items() if n not in ("machine_floors", "copy_calib", head["workload"])}
    line["others_us_and_frac_of_peak"] = others
    text = json.dumps(line, separators=(",", ":"))
    while len(text) >= MAX_LINE_BYTES and others:
        others.popitem()
        text = json.dumps(line, separators=(",", ":"))
    assert len(text) < MAX_LINE_BYTES, len(text)
    return text


if __name__ == "__main__":
    main()
