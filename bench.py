#!/usr/bin/env python3
"""Benchmark of the quantized-weight linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One *step* is one pass of the decode hot path over the Qwen3-8B-shaped batched
decode configuration: int4 g32 weights with f16 scales, f16 activations, f32
accumulate, f16 out, for (K,N) in {(4096,4096), (4096,12288), (12288,4096)} and
M in {1,2,4,8,16} — 15 calls of the matmul seam (tlhip_matmul_quantized) through
the C ABI.  Every call reads a different weight buffer out of a pool larger than
the 256 MB last-level cache, so the rate is an HBM rate.  Inputs are resident in
HBM before the timed region.  The printed JSON line carries

  value        whole-step algorithmic bytes / time, GB/s
  roofline     the dominant kernel (largest share of the step), timed on its own
               with events on the launch stream, against the 8 TB/s HBM peak
  cpu_baseline the CPU restatement of the reference arithmetic (oracle/) timed
               on the host cores over the same step, single-threaded like the
               reference's CPU backend
  details      per-call times, the read-only probe at the same sizes, the
               0.6B decode sequence (us per decode token, plain and as a HIP
               graph), the LM head, the prefill GEMM (TFLOP/s) and config 1

Only one GPU is used; --gpus above 1 exits with a message.

The rocprofv3 summaries under profiles/ are made by this file as well (no GPU
needed for these three; each prints the table it writes):

    python bench.py --summarise-trace DIR OUT.txt "COMMAND" [run]
        DIR holds the *_kernel_trace.csv / *_kernel_stats.csv of
        `rocprofv3 --kernel-trace --stats --output-format csv -d DIR -- python3 bench.py ...`
    python bench.py --summarise-traffic FETCH.csv WRITE.csv PROBE.log OUT.txt OUT.json
        the counter_collection.csv files of two `rocprofv3 --pmc FETCH_SIZE` /
        `--pmc WRITE_SIZE` runs of `python3 bench.py --traffic-probe` and the
        stdout of one of them; OUT.json is what --traffic-file reads
    python bench.py --summarise-prefill-counters COUNTERS.csv PROBE.log OUT.txt "COMMAND"
        one `rocprofv3 --pmc ... -- python3 bench.py --prefill-probe` run
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
F16_MFMA_PEAK_TFLOPS = 2500.0
POOL_BYTES = 640e6  # per shape: well above the 256 MB last-level cache


def algorithmic_bytes(fmt: str, n: int, k: int, g: int, m: int, x_bytes: int, y_bytes: int) -> int:
    if fmt == "int4":
        return n * k // 2 + n * (k // g) * 2 + m * k * x_bytes + m * n * y_bytes
    if fmt == "int8-row":
        return n * k + n * 4 + m * k * x_bytes + m * n * y_bytes
    return n * k + n * (k // g) * 2 + m * k * x_bytes + m * n * y_bytes


class Bench:
    only_missing = False  # --autotune-missing: tune() skips problems that have an entry of their own

    def __init__(self):
        import torchlette_amd as T
        from torchlette_amd import _lib as L
        self.T, self.L = T, L
        self.be = T.getBackend(0)
        self.rng = np.random.default_rng(20251)
        self.ev0, self.ev1 = C.c_void_p(), C.c_void_p()
        L.call("tlhip_event_create", C.byref(self.ev0))
        L.call("tlhip_event_create", C.byref(self.ev1))
        self.sink = self.be._alloc([4], "u32")
        self.probe = None
        self.probe_stream = None

    # -------------------------------------------------------------- operands
    def weight_pool(self, fmt: str, n: int, k: int, g: int, element: str, pool_bytes: float = POOL_BYTES):
        """One synthetic packed weight generated on the host, replicated on the
        device into enough distinct buffers to exceed the last-level cache."""
        T, be, rng = self.T, self.be, self.rng
        per_word = 8 if fmt == "int4" else 4
        words = n * k // per_word
        nbuf = int(max(2, min(96, -(-pool_bytes // (words * 4)))))
        packed = rng.integers(0, 2 ** 32, words, dtype=np.uint64).astype(np.uint32)
        if fmt == "int8-row":
            # bytes uniform in [-127,127]: redraw the -128 pattern
            b = packed.view(np.uint8)
            b[b == 0x80] = 0x7F
            scales = rng.uniform(0.002, 0.01, n).astype(np.float32)
            name = "int8-row"
        elif fmt == "int4":
            scales = rng.uniform(0.01, 0.05, n * (k // g)).astype(np.float32).astype(np.float16).view(np.uint16)
            name = f"int4-{g}"
        else:
            scales = rng.uniform(0.01, 0.05, n * (k // g)).astype(np.float32).astype(np.float16).view(np.uint16)
            name = f"int8-{g}"
        first = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(name, element))
        pool = [first]
        for _ in range(nbuf - 1):
            pt = be._alloc([n, k // per_word], "u32")
            self.L.call("tlhip_memcpy_d2d", pt.ptr, first.ptr, pt.nbytes, None)
            st = be._alloc(first.scales.shape, first.scales.dtype)
            self.L.call("tlhip_memcpy_d2d", st.ptr, first.scales.ptr, st.nbytes, None)
            pool.append(T.HipTensor(be, [n, k], element, pt.ptr, pt.nbytes, False, [k, 1], first.format, st, pt))
        be.synchronize()
        return pool, (packed, scales)

    def activations(self, m: int, k: int, dtype: str = "f16", std: float = 1.0):
        x = (self.rng.standard_normal((m, k)) * std).astype(np.float32)
        host = x.astype(np.float16) if dtype == "f16" else x
        return self.be.ops.tensorFromArray(host, [m, k], dtype), host

    # ---------------------------------------------------------------- timing
    def time_region(self, enqueue, reps: int, stream=None) -> float:
        """Microseconds per repetition of `enqueue()` (which launches on `stream`;
        None = the library's stream), between two events recorded on that stream."""
        L = self.L
        L.call("tlhip_event_record", self.ev0, stream)
        for _ in range(reps):
            enqueue()
        L.call("tlhip_event_record", self.ev1, stream)
        L.call("tlhip_event_synchronize", self.ev1)
        us = C.c_double()
        L.call("tlhip_event_elapsed_us", self.ev0, self.ev1, C.byref(us))
        return us.value / reps

    warm_ms = 50.0

    def median_time(self, enqueue, reps: int, batches: int = 5, stream=None) -> float:
        # untimed batches first, `warm_ms` of GPU time: the section before may have left the
        # GPU idle while the host prepared data, and the launches after that run at a lower
        # clock for some milliseconds (the same kernel measured 8-12 % slower without)
        spent = 0.0
        while spent < self.warm_ms * 1e3:
            spent += self.time_region(enqueue, reps, stream) * reps
        return float(np.median([self.time_region(enqueue, reps, stream) for _ in range(batches)]))

    def make_call(self, pool, x, m: int, out, epilogue=None, out_dtype: str = "f16"):
        L, be = self.L, self.be
        qws = [be._qweight(w, False) for w in pool]
        xd = L.F16 if x.dtype == "f16" else L.F32
        yd = L.F16 if out_dtype == "f16" else L.F32
        ep = C.byref(epilogue) if epilogue is not None else None
        state = {"i": 0}
        fn = L.load().tlhip_matmul_quantized

        def call():
            qw = qws[state["i"] % len(qws)]
            state["i"] += 1
            rc = fn(C.byref(qw), x.ptr, xd, m, out.ptr, yd, 1.0, ep, None)
            if rc:
                L.check(rc)
        return call

    def probe_time(self, pool, nbytes: int) -> float:
        """The read-only streaming kernel of the benchmark's own library over `nbytes` of
        each pool buffer in turn, timed like the GEMV launches (on a stream of its own:
        the library's stream is not visible through the C ABI)."""
        if self.probe is None:
            path = os.path.join(ROOT, "torchlette_amd", "libtlhip_bench.so")
            if not os.path.exists(path):
                raise RuntimeError(f"{path} is missing: build it with make -C torchlette_amd/csrc")
            self.probe = C.CDLL(path).tlbench_hbm_read_probe
            self.probe.restype = C.c_int
            self.probe.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
            self.probe_stream = C.c_void_p()
            self.L.call("tlhip_stream_create", C.byref(self.probe_stream))
        state = {"i": 0}

        def call():
            w = pool[state["i"] % len(pool)]
            state["i"] += 1
            rc = self.probe(w.ptr, nbytes, self.sink.ptr, self.probe_stream)
            if rc:
                raise RuntimeError(f"tlbench_hbm_read_probe failed with code {rc}")
        self.be.synchronize()
        return self.median_time(call, 100, stream=self.probe_stream)

    def tune(self, pool, x, m: int, out, out_dtype: str = "f16", epilogue=None):
        """The library's tuner (tlhip_autotune_pool) over this pool: every candidate is
        timed in batches of back-to-back launches with the weights ROTATING through the
        pool, the three fastest once more, and the winner lands in the library's
        per-shape cache.  Returns its time per launch in microseconds."""
        L, be = self.L, self.be
        if self.only_missing:
            # --autotune-missing: problems that already have an entry of their own keep it
            w0 = pool[0]
            scheme, g = w0.format.packing.scheme, w0.format.packing.groupSize
            key = f"{m}_{w0.shape[0]}_{w0.shape[1]}_{scheme}_g{0 if scheme == 'int8-row' else g}_{x.dtype}_{out_dtype}"
            if key in json.loads(self.T.exportTuningCache())["entries"]:
                return 0.0
        qws = (L.QWeight * len(pool))(*[be._qweight(w, False) for w in pool])
        xd = L.F16 if x.dtype == "f16" else L.F32
        yd = L.F16 if out_dtype == "f16" else L.F32
        ep = C.byref(epilogue) if epilogue is not None else None
        opts = L.AutotuneOptions(0, 3, 3, 0, self.warm_ms, 0)
        best = C.c_double()
        L.call("tlhip_autotune_pool", qws, len(pool), x.ptr, xd, m, out.ptr, yd, ep, C.byref(opts), None, C.byref(best))
        return best.value


def kernel_name_of(cfg) -> str:
    return {0: "gemv_kernel (VALU dot2)", 1: "gemv_mfma_kernel (16x16x32 f16)", 2: "gemm_prefill_kernel (32x32x16 f16)",
            3: "gemm_direct_kernel (32x32x16 f16, weights dequantised in registers)",
            4: "gemv_xreg_kernel (16x16x32 f16, activations in registers)",
            5: "gemv_wave_kernel (16x16x32 f16, every wave its own K range)"}.get(cfg.variant, f"variant {cfg.variant}")


def cpu_step(cases, host_weights, host_x, threads: int, keep=None) -> float:
    """Seconds for one step on the CPU restatement: dequantise as the reference
    does, then the CPU-backend matmul (f64 accumulate in k order, f32 store).
    `keep`: a list that receives the 15 outputs, in the order of `cases`."""
    from oracle import quant_oracle as O
    t0 = time.perf_counter()
    deq = {}
    for (n, k) in {(c["n"], c["k"]) for c in cases}:
        packed, scales = host_weights[(n, k)]
        deq[(n, k)] = O.dequant_int4_grouped(packed, scales, n, k, 32)
    for c in cases:
        y = O.matmul_nt(host_x[(c["m"], c["k"])].astype(np.float32), deq[(c["n"], c["k"])], threads=threads)
        if keep is not None:
            keep.append(y)
    return time.perf_counter() - t0


# ---------------------------------------------------------------- profile summaries
def _short_kernel_name(n: str) -> str:
    import re
    m = re.match(r"_ZN5tlhip12_GLOBAL__N_111gemv_kernelILi(\d)E(DF16_|f)Li(\d)ELi(\d)ELi(\d)ELb(\d)E", n)
    if m:
        return (f"gemv_kernel<fmt={m.group(1)}, x={'f16' if m.group(2) == 'DF16_' else 'f32'}, rows={m.group(3)}, "
                f"R={m.group(4)}, U={m.group(5)}{', 4x4x4 mfma' if m.group(6) == '1' else ''}>")
    n = re.sub(r"tlhip::\(anonymous namespace\)::", "", n)
    n = re.sub(r"\(anonymous namespace\)::", "", n)
    n = re.sub(r"\(tlhip::.*", "", n)
    n = re.sub(r"void ", "", n)
    return n[:70]


def summarise_trace(d: str, out: str, cmd: str, want_run: bool) -> int:
    """rocprofv3 --kernel-trace --stats CSVs -> the short table kept under profiles/."""
    import collections
    import csv
    import glob
    import statistics

    def find(pat):
        r = glob.glob(os.path.join(d, "**", pat), recursive=True)
        return r[0] if r else None
    lines = [f"command: {cmd}", f"summary: python bench.py --summarise-trace <its output directory> <this file> \"<command>\"{' run' if want_run else ''}", ""]
    st = find("*kernel_stats.csv")
    if st:
        lines.append("rocprofv3 --stats (per kernel name, all shapes of that name pooled):")
        lines.append(f"{'kernel':70s} {'calls':>7s} {'total_us':>11s} {'avg_us':>9s} {'min_us':>8s} {'max_us':>9s} {'%':>6s}")
        for i, r in enumerate(csv.DictReader(open(st))):
            if i >= 14:
                break
            lines.append(f"{_short_kernel_name(r['Name']):70s} {int(r['Calls']):7d} {float(r['TotalDurationNs']) / 1e3:11.1f} "
                         f"{float(r['AverageNs']) / 1e3:9.2f} {float(r['MinNs']) / 1e3:8.2f} {float(r['MaxNs']) / 1e3:9.2f} "
                         f"{float(r['Percentage']):6.2f}")
    tr = find("*kernel_trace.csv")
    if tr:
        groups = collections.defaultdict(list)
        rows = list(csv.DictReader(open(tr)))
        for r in rows:
            key = (_short_kernel_name(r["Kernel_Name"]), int(r["Grid_Size_X"]) // max(1, int(r["Workgroup_Size_X"])),
                   int(r["Workgroup_Size_X"]), int(r["LDS_Block_Size"]))
            groups[key].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
        lines += ["", "kernel trace, dispatches grouped by (kernel, workgroups, threads, LDS bytes) = one shape each:",
                  f"{'kernel':70s} {'wgs':>6s} {'thr':>5s} {'lds':>7s} {'calls':>6s} {'avg_us':>9s} {'med_us':>9s} {'min_us':>8s}"]
        for (n, g, t, l), v in sorted(groups.items(), key=lambda kv: -sum(kv[1]))[:40]:
            lines.append(f"{n:70s} {g:6d} {t:5d} {l:7d} {len(v):6d} {sum(v) / len(v):9.2f} {statistics.median(v):9.2f} {min(v):8.2f}")
        if want_run:
            rows.sort(key=lambda r: int(r["Start_Timestamp"]))
            best, i = (0, 0, None), 0
            while i < len(rows):
                j = i
                while j < len(rows) and rows[j]["Kernel_Name"] == rows[i]["Kernel_Name"]:
                    j += 1
                if j - i > best[0]:
                    best = (j - i, i, rows[i]["Kernel_Name"])
                i = j
            n, i0, name = best
            v = [(int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3 for r in rows[i0:i0 + n]]
            lines += ["", "longest run of consecutive launches of one kernel (bench.py's dominant-kernel timing loop, one shape):",
                      f"{_short_kernel_name(name)}: {n} launches, avg {sum(v) / n:.2f} us, median {statistics.median(v):.2f} us, "
                      f"min {min(v):.2f} us"]
    open(out, "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))
    return 0


def _probe_record(path: str, key: str):
    for line in open(path):
        line = line.strip()
        if line.startswith("{") and key in line:
            return json.loads(line)[key]
    raise SystemExit(f"{path}: no {key} record")


def summarise_traffic(fetch_csv: str, write_csv: str, probe_file: str, out_txt: str, out_json: str) -> int:
    """FETCH_SIZE / WRITE_SIZE counter runs of --traffic-probe -> HBM bytes per launch of
    each call of the step, each counter scaled by what it reads for the 256 MiB
    device-to-device copies of the same run."""
    import csv
    probe = _probe_record(probe_file, "traffic_probe")
    cases, nl = probe["cases"], probe["launches"]
    res, lines = {}, [
        "commands: rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -o r -- python3 bench.py --traffic-probe",
        "          rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir> -o r -- python3 bench.py --traffic-probe",
        "summary:  python bench.py --summarise-traffic <fetch>/r_counter_collection.csv <write>/r_counter_collection.csv "
        "<stdout of one run> <this file> <the .json beside it>", ""]
    for path, counter in ((fetch_csv, "FETCH_SIZE"), (write_csv, "WRITE_SIZE")):
        rows = [r for r in csv.DictReader(open(path)) if r["Counter_Name"] == counter]
        rows.sort(key=lambda r: int(r["Start_Timestamp"]))
        gemv = [float(r["Counter_Value"]) for r in rows if "gemv" in r["Kernel_Name"]][-nl * len(cases):]
        copy = [float(r["Counter_Value"]) for r in rows if "copyBuffer" in r["Kernel_Name"]][-probe["copies"]:]
        c_avg = sum(copy) / len(copy)
        scale = (probe["copy_bytes"] / 1024.0) / c_avg  # known KiB per copy / counted KiB per copy
        lines.append(f"{counter}: copy kernel (256 MiB each way) avg {c_avg:.1f} KiB/dispatch -> scale {scale:.4f}")
        for i, c in enumerate(cases):
            v = gemv[i * nl:(i + 1) * nl]
            k_avg = sum(v) / len(v)
            res.setdefault(i, {})[counter] = (k_avg, scale, k_avg * scale * 1024)
            lines.append(f"  M={c['m']} N={c['n']} K={c['k']} {c['kernel']} config {c['config'][:6]}: avg {k_avg:.1f} KiB/dispatch "
                         f"over {len(v)} dispatches -> {k_avg * scale * 1024:.0f} bytes")
    out = {}
    for i, c in enumerate(cases):
        f, w = res[i]["FETCH_SIZE"], res[i]["WRITE_SIZE"]
        traffic = f[2] + w[2]
        lines.append(f"M={c['m']} N={c['n']} K={c['k']}: traffic (fetch + write, scaled) = {traffic:.0f} bytes per launch; "
                     f"algorithmic bytes = {c['algorithmic_bytes']}; ratio {traffic / c['algorithmic_bytes']:.3f}")
        out[f'{c["m"]}_{c["n"]}_{c["k"]}_int4-g32'] = {
            "config": c["config"], "kernel": c["kernel"], "traffic_bytes": round(traffic), "fetch_bytes": round(f[2]),
            "write_bytes": round(w[2]), "fetch_scale": round(f[1], 4), "write_scale": round(w[1], 4),
            "algorithmic_bytes": c["algorithmic_bytes"]}
    open(out_txt, "w").write("\n".join(lines) + "\n")
    json.dump(out, open(out_json, "w"), indent=1)
    print("\n".join(lines))
    return 0


def summarise_prefill_counters(csvf: str, logf: str, out: str, cmd: str) -> int:
    """One --pmc run of --prefill-probe -> matrix-pipe utilisation and VALU per MFMA."""
    import collections
    import csv
    probe = _probe_record(logf, "prefill_probe")
    rows = [r for r in csv.DictReader(open(csvf)) if "gemm_direct" in r["Kernel_Name"] or "gemm_prefill" in r["Kernel_Name"]]
    by_disp = collections.OrderedDict()
    for r in rows:
        by_disp.setdefault(int(r["Dispatch_Id"]), {"name": r["Kernel_Name"], "t0": int(r["Start_Timestamp"]),
                                                   "t1": int(r["End_Timestamp"])})[r["Counter_Name"]] = float(r["Counter_Value"])
    disp, nl = list(by_disp.values()), probe["launches"]
    lines = [f"command: {cmd}", "summary: python bench.py --summarise-prefill-counters <dir>/r_counter_collection.csv <stdout of the run> "
             "<this file> \"<command>\"", "",
             "one counter run; per case the mean over its 5 launches (durations under the profiler are 5-20 % longer than",
             "bench.py's own).  An MFMA 32x32x16 f16 occupies its SIMD's matrix pipe for 32 cycles, so",
             "SQ_VALU_MFMA_BUSY_CYCLES = 32 x MFMA count, and the pipe's utilisation at core clock f is",
             "busy / (1024 SIMDs x f x duration).  f: 2.4 GHz is the clock the 2.5 PFLOP/s peak is quoted at; rocm-smi",
             "--showclocks, sampled while the M = 8192 case ran in a loop for 4 s, read sclk = 1.80-1.81 GHz.", ""]
    for i, c in enumerate(probe["cases"]):
        ds = disp[i * nl:(i + 1) * nl]
        if len(ds) < nl:
            break

        def mean(k):
            return sum(d[k] for d in ds) / len(ds)
        dur_us = sum(d["t1"] - d["t0"] for d in ds) / len(ds) / 1e3
        mf, nm = mean("SQ_VALU_MFMA_BUSY_CYCLES"), c["flops"] / 32768
        name = ds[0]["name"].replace("void tlhip::(anonymous namespace)::", "").split("(")[0]
        lines += [f"M={c['m']} N={c['n']} K={c['k']} config {c['config'][:6]} {name}",
                  f"  duration under the profiler {dur_us:9.1f} us -> {c['flops'] / dur_us / 1e6:7.1f} TFLOP/s = "
                  f"{c['flops'] / dur_us / 1e6 / F16_MFMA_PEAK_TFLOPS:.3f} of {F16_MFMA_PEAK_TFLOPS:.0f}",
                  f"  SQ_VALU_MFMA_BUSY_CYCLES   {mf:12.0f}  = 32 x {mf / 32:.0f} (MFMAs the problem needs: {nm:.0f})",
                  f"  matrix pipe utilisation    {mf / (1024 * 2.4e3 * dur_us):.3f} at 2.4 GHz, {mf / (1024 * 1.8e3 * dur_us):.3f} at 1.8 GHz",
                  f"  SQ_INSTS_VALU {mean('SQ_INSTS_VALU'):.0f} (MFMA included) -> {(mean('SQ_INSTS_VALU') - nm) / nm:.2f} other VALU "
                  "instructions per MFMA",
                  f"  SQ_WAVE_CYCLES {mean('SQ_WAVE_CYCLES'):.0f}  SQ_WAIT_INST_ANY {mean('SQ_WAIT_INST_ANY'):.0f} "
                  f"({mean('SQ_WAIT_INST_ANY') / mean('SQ_WAVE_CYCLES'):.2f} of the wave cycles)  SQ_ACTIVE_INST_LDS "
                  f"{mean('SQ_ACTIVE_INST_LDS'):.0f}  SQ_BUSY_CYCLES {mean('SQ_BUSY_CYCLES'):.0f}  GRBM_GUI_ACTIVE "
                  f"{mean('GRBM_GUI_ACTIVE'):.0f}", ""]
    open(out, "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))
    return 0


def main() -> int:
    if len(sys.argv) > 1 and sys.argv[1] == "--summarise-trace":
        return summarise_trace(sys.argv[2], sys.argv[3], sys.argv[4], len(sys.argv) > 5 and sys.argv[5] == "run")
    if len(sys.argv) > 1 and sys.argv[1] == "--summarise-traffic":
        return summarise_traffic(*sys.argv[2:7])
    if len(sys.argv) > 1 and sys.argv[1] == "--summarise-prefill-counters":
        return summarise_prefill_counters(*sys.argv[2:6])
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--warm-ms", type=float, default=50.0,
                    help="GPU milliseconds of untimed launches before each timed section (small for profiler runs, "
                         "whose traces grow with every launch)")
    ap.add_argument("--no-details", action="store_true", help="skip the secondary measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-autotune", action="store_true", help="use the heuristic kernel choices")
    ap.add_argument("--dominant", default="",
                    help="M,N,K of the call to report in `roofline` instead of the slowest one measured in this run "
                         "(under a profiler the per-launch overhead shifts which call is slowest)")
    ap.add_argument("--no-graphs", action="store_true",
                    help="time the decode-token sections as stream launches only (no HIP graph capture / replay)")
    ap.add_argument("--autotune", action="store_true",
                    help="re-tune every case (weights rotating through HBM) even if a tuning cache file exists")
    ap.add_argument("--autotune-missing", action="store_true",
                    help="import the tuning cache file, tune only the cases it has no entry of their own for, and "
                         "write the file back")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for a counter run under rocprofv3 --pmc: 10 launches of each of the step's calls, then "
                         "three device-to-device copies of 256 MiB (the known size the counters are scaled by), and exit")
    ap.add_argument("--prefill-probe", action="store_true",
                    help="counter runs: only launch the prefill GEMM (M = 512, 2048, 8192; bias + silu), 5 launches each")
    ap.add_argument("--traffic-file", default=os.path.join(ROOT, "profiles", "decode_step_qwen3_8b_int4_hbm_traffic.json"),
                    help="measured HBM bytes per launch (from the counter runs), keyed by call; fills roofline.traffic")
    ap.add_argument("--tuning-cache", default=os.path.join(ROOT, "torchlette_amd", "tuning", "mi355x.json"),
                    help="JSON tuning cache to import before the run and to write after --autotune")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this path runs on one GPU; --gpus {args.gpus} is not supported "
              "(one MI355X is what this path is built and measured on; nothing here shards across devices)", file=sys.stderr)
        return 2

    B = Bench()
    B.warm_ms = args.warm_ms
    T, L, be = B.T, B.L, B.be
    info = be.deviceInfo()
    # Kernel choices: a committed tuning cache (importTuningCache) when there is one,
    # else a tuning pass; --autotune forces the pass and rewrites the file.
    tuning_source = "heuristic defaults"
    B.only_missing = False
    if args.autotune_missing and os.path.exists(args.tuning_cache):
        T.importTuningCache(open(args.tuning_cache).read())
        B.only_missing = True
        tuning_source = "tuned in this run"
    elif not args.no_autotune and not args.autotune and os.path.exists(args.tuning_cache):
        T.importTuningCache(open(args.tuning_cache).read())
        tuning_source = os.path.relpath(args.tuning_cache, ROOT)
        args.no_autotune = True  # nothing left to tune
    elif not args.no_autotune:
        tuning_source = "tuned in this run"

    # ------------------------------------------------------------ headline step
    shapes = [(4096, 4096), (12288, 4096), (4096, 12288)]  # (N, K)
    ms = [1, 2, 4, 8, 16]
    pools, host_weights, host_x, xs, outs = {}, {}, {}, {}, {}
    for (n, k) in shapes:
        pools[(n, k)], host_weights[(n, k)] = B.weight_pool("int4", n, k, 32, "f16")
    for k in {k for _, k in shapes}:
        for m in ms:
            xs[(m, k)], host_x[(m, k)] = B.activations(m, k)
    cases = []
    for (n, k) in shapes:
        for m in ms:
            outs[(m, n)] = outs.get((m, n)) or be._alloc([m, n], "f16")
            if not args.no_autotune:
                B.tune(pools[(n, k)], xs[(m, k)], m, outs[(m, n)])
            cfg = be.selectedConfig(pools[(n, k)][0], "f16", m, "f16")
            cases.append({"n": n, "k": k, "m": m, "bytes": algorithmic_bytes("int4", n, k, 32, m, 2, 2),
                          "call": B.make_call(pools[(n, k)], xs[(m, k)], m, outs[(m, n)]),
                          "config": list(cfg.as_tuple()), "kernel": kernel_name_of(cfg)})
    step_bytes = sum(c["bytes"] for c in cases)

    if args.traffic_probe:
        be.synchronize()
        for c in cases:  # fixed order, so that the FETCH and the WRITE run line up
            for _ in range(10):
                c["call"]()
            be.synchronize()
        slowest = cases
        nbytes = 256 << 20
        src, dst = be._alloc([nbytes // 4], "f32"), be._alloc([nbytes // 4], "f32")
        for _ in range(3):
            L.call("tlhip_memcpy_d2d", dst.ptr, src.ptr, nbytes, None)
        be.synchronize()
        print(json.dumps({"traffic_probe": {"cases": [
            {"m": c["m"], "n": c["n"], "k": c["k"], "kernel": c["kernel"], "config": c["config"],
             "algorithmic_bytes": c["bytes"]} for c in slowest], "launches": 10, "copy_bytes": nbytes, "copies": 3}}))
        return 0

    if args.prefill_probe:
        n, k = 12288, 4096
        w = pools[(n, k)][0]
        bias = be.ops.tensorFromArray((B.rng.standard_normal(n) * 0.1).astype(np.float16), [n], "f16")
        ep = be.makeEpilogue(bias, "silu")
        runs = []
        for m in (512, 2048, 8192):
            x, _ = B.activations(m, k, std=0.5)
            out = be._alloc([m, n], "f16")
            call = B.make_call([w], x, m, out, epilogue=ep)
            for _ in range(5):
                call()
            be.synchronize()
            runs.append({"m": m, "n": n, "k": k, "flops": 2.0 * m * n * k,
                         "config": list(be.selectedConfig(w, "f16", m, "f16").as_tuple())})
        print(json.dumps({"prefill_probe": {"cases": runs, "launches": 5}}))
        return 0

    def step():
        for c in cases:
            c["call"]()

    def timed_step():
        """One measurement of the step: `--warmup` untimed steps, then the median of
        five batches of exactly `--steps` steps between events on the launch stream."""
        for _ in range(args.warmup):
            step()
        be.synchronize()
        return float(np.median([B.time_region(step, args.steps) for _ in range(5)]))

    # `warm_ms` of untimed steps first, like every other section: after the host-side
    # set-up above the GPU starts from a low clock, and a 20-step batch is over in 3 ms
    spent = 0.0
    while spent < B.warm_ms * 1e3:
        spent += B.time_region(step, 10) * 10
    t0 = time.perf_counter()
    step_us = timed_step()
    be.synchronize()
    wall_s = time.perf_counter() - t0
    value = step_bytes / step_us / 1e3  # GB/s

    # the same step on the heuristic defaults (what a shape without a tuning entry and
    # without a tuned neighbour of its class gets): the gap to the tuned figure, recorded
    default_step = None
    if tuning_source != "heuristic defaults":
        saved = T.exportTuningCache()
        T.clearTuningCache()
        default_configs = [list(be.selectedConfig(pools[(c["n"], c["k"])][0], "f16", c["m"], "f16").as_tuple()) for c in cases]
        default_us = timed_step()
        T.importTuningCache(saved)
        default_step = {"us_per_step": round(default_us, 2), "gbps": round(step_bytes / default_us / 1e3, 1),
                        "calls_with_another_config": sum(1 for c, d in zip(cases, default_configs) if d != c["config"])}
        step()  # back on the tuned choices
        be.synchronize()

    # per-call times (each case on its own, back-to-back launches on the one stream)
    for c in cases:
        c["us"] = B.median_time(c["call"], 200)
        c["gbps"] = c["bytes"] / c["us"] / 1e3
    dominant = max(cases, key=lambda c: c["us"])
    if args.dominant:  # a profiler run: time the case the unprofiled run found dominant
        dm, dn, dk = (int(v) for v in args.dominant.split(","))
        dominant = next(c for c in cases if (c["m"], c["n"], c["k"]) == (dm, dn, dk))
    dom_us = B.median_time(dominant["call"], 500, batches=7)
    # HBM bytes per launch measured with FETCH_SIZE / WRITE_SIZE counter runs of --traffic-probe
    traffic = None
    if os.path.exists(args.traffic_file):
        rec = json.load(open(args.traffic_file)).get(f'{dominant["m"]}_{dominant["n"]}_{dominant["k"]}_int4-g32')
        if rec and rec.get("config") == dominant["config"]:
            traffic = rec["traffic_bytes"]
    roofline = {"bound": "hbm", "achieved": dominant["bytes"] / dom_us / 1e3, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": dominant["bytes"] / dom_us / 1e3 / HBM_PEAK_GBPS, "traffic": traffic,
                "kernel": dominant["kernel"], "launch_us": dom_us, "bytes_per_launch": dominant["bytes"],
                "shape": {"m": dominant["m"], "n": dominant["n"], "k": dominant["k"]}}

    result = {
        "metric": "quant-GEMV HBM GB/s (% peak) + \u00b5s/decode-token for linears; prefill TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_us / 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 x int4 -> f32 accumulate", "data": "synthetic",
        "config": {"workload": "configs[2]: Qwen3-8B-shaped batched decode, int4 g32 + f16 scales, M in {1,2,4,8,16}, "
                               "(K,N) in {(4096,4096),(4096,12288),(12288,4096)}; 15 calls per step, "
                               "weights rotated through >640 MB per shape",
                   "calls_per_step": len(cases), "bytes_per_step": step_bytes,
                   "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4), "kernel_choice": tuning_source,
                   "device": info["arch"], "compute_units": info["compute_units"]},
        "roofline": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in roofline.items()},
        "wall_s_timed_region": round(wall_s, 4),
        "timing": f"{B.warm_ms:g} ms of untimed steps, {args.warmup} warm-up steps, median of 5 batches of {args.steps} steps",
    }
    if default_step is not None:
        result["heuristic_defaults"] = default_step
    result["sum_of_per_call_us"] = round(sum(c["us"] for c in cases), 2)

    details = {}
    details["decode_calls"] = [
        {"m": c["m"], "n": c["n"], "k": c["k"], "us": round(c["us"], 2), "gbps": round(c["gbps"], 1),
         "frac_of_peak": round(c["gbps"] / HBM_PEAK_GBPS, 4), "kernel": c["kernel"], "config": c["config"]}
        for c in cases]

    if not args.no_details:
        # read-only probe at the three weight sizes: what one launch of that size can reach
        probe = {}
        for (n, k) in shapes:
            nbytes = n * k // 2
            us = B.probe_time(pools[(n, k)], nbytes)
            probe[f"{n}x{k}"] = {"bytes": nbytes, "us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1)}
        details["read_only_probe"] = probe

        # one Qwen3-8B-shaped decoder layer's Linears (q 4096, k 1024, v 1024, o 4096, gate 12288,
        # up 12288 from K = 4096; down 4096 from K = 12288): 7 launches, or 4 with the Linears
        # that share their activations (q/k/v, gate/up) grouped into one launch each
        # (packages/qwen3-browser/src/model.ts:341-361 issues them back to back)
        kv_pool, _ = B.weight_pool("int4", 1024, 4096, 32, "f16", pool_bytes=300e6)
        qkv_cat, _ = B.weight_pool("int4", 6144, 4096, 32, "f16")     # stand-ins of the groups' combined
        gu_cat, _ = B.weight_pool("int4", 24576, 4096, 32, "f16")     # rows, for the tuner only
        gfn = L.load().tlhip_gemv_grouped_rows
        layer_rows = []
        for m in (1, 8, 16):
            x4, x12 = xs[(m, 4096)], xs[(m, 12288)]
            y = {key: be._alloc([m, n], "f16") for key, n in
                 (("q", 4096), ("k", 1024), ("v", 1024), ("o", 4096), ("gate", 12288), ("up", 12288), ("down", 4096))}
            ycat = be._alloc([m, 24576], "f16")
            if not args.no_autotune:
                B.tune(kv_pool, x4, m, y["k"])
                B.tune(qkv_cat, x4, m, ycat)
                B.tune(gu_cat, x4, m, ycat)
            p44, p124, p412 = pools[(4096, 4096)], pools[(12288, 4096)], pools[(4096, 12288)]
            nlayers = 12  # distinct weight sets: 12 x 97 MB, far above the last-level cache

            def probs_of(items):
                arr = (L.GemvProblem * len(items))()
                for i, (w, x, out) in enumerate(items):
                    arr[i].w = be._qweight(w, False)
                    arr[i].x = x.ptr
                    arr[i].y = out.ptr
                    arr[i].epilogue = None
                return arr, len(items)
            sep, grp, gu_only = [], [], []
            for li in range(nlayers):
                wq, wo = p44[(2 * li) % len(p44)], p44[(2 * li + 1) % len(p44)]
                wk, wv = kv_pool[(2 * li) % len(kv_pool)], kv_pool[(2 * li + 1) % len(kv_pool)]
                wg, wu = p124[(2 * li) % len(p124)], p124[(2 * li + 1) % len(p124)]
                wd = p412[li % len(p412)]
                linears = [(wq, x4, y["q"]), (wk, x4, y["k"]), (wv, x4, y["v"]), (wo, x4, y["o"]), (wg, x4, y["gate"]),
                           (wu, x4, y["up"]), (wd, x12, y["down"])]
                sep.append([probs_of([t]) for t in linears])
                grp.append([probs_of(linears[0:3]), probs_of(linears[3:4]), probs_of(linears[4:6]), probs_of(linears[6:7])])
                gu_only.append(probs_of(linears[4:6]))
            state = {"i": 0}

            def runner(table):
                def call():
                    for arr, cnt in table[state["i"] % nlayers]:
                        rc = gfn(arr, cnt, L.F16, m, L.F16, 1.0, None)
                        if rc:
                            L.check(rc)
                    state["i"] += 1
                return call

            def gate_up():
                arr, cnt = gu_only[state["i"] % nlayers]
                state["i"] += 1
                rc = gfn(arr, cnt, L.F16, m, L.F16, 1.0, None)
                if rc:
                    L.check(rc)
            layer_bytes = sum(algorithmic_bytes("int4", n, k, 32, m, 2, 2) for (n, k) in
                              ((4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (12288, 4096), (12288, 4096), (4096, 12288)))
            gu_bytes = 2 * algorithmic_bytes("int4", 12288, 4096, 32, m, 2, 2) - m * 4096 * 2
            us_sep = B.median_time(runner(sep), 40)
            us_grp = B.median_time(runner(grp), 40)
            us_gu = B.median_time(gate_up, 100)
            # the MLP block (gate, up, act(gate) * up, down) three ways: one call into the
            # library (tlhip_mlp_decode: it issues gate/up grouped, the gated multiply and down),
            # the same three launches as three calls, and one sequence launch
            # (tlhip_gemv_sequence: a gated step and the down projection waiting for it)
            hbuf = be._alloc([m, 12288], "f16")
            mlp_q = [(be._qweight(p124[(2 * li) % len(p124)], False), be._qweight(p124[(2 * li + 1) % len(p124)], False),
                      be._qweight(p412[li % len(p412)], False)) for li in range(nlayers)]
            mlp_fn, gm_fn, seq_fn = L.load().tlhip_mlp_decode, L.load().tlhip_gated_mul, L.load().tlhip_gemv_sequence
            silu = be.makeEpilogue(None, "silu")
            seq_steps = []
            for qg, qu, qd in mlp_q:
                arr = (L.SequenceStep * 2)()
                arr[0].w, arr[0].w_up, arr[0].gated = qg, qu, 1
                arr[0].x, arr[0].y, arr[0].y_dtype, arr[0].epilogue = x4.ptr, hbuf.ptr, L.F16, C.pointer(silu)
                arr[1].w, arr[1].x, arr[1].y, arr[1].y_dtype, arr[1].wait = qd, hbuf.ptr, y["down"].ptr, L.F16, 1
                seq_steps.append(arr)

            def mlp_one_call():
                qg, qu, qd = mlp_q[state["i"] % nlayers]
                state["i"] += 1
                rc = mlp_fn(C.byref(qg), C.byref(qu), C.byref(qd), L.UNARY["silu"], x4.ptr, L.F16, m, hbuf.ptr, y["down"].ptr,
                            L.F16, None, None)
                if rc:
                    L.check(rc)

            def mlp_sequence_launch():
                arr = seq_steps[state["i"] % nlayers]
                state["i"] += 1
                rc = seq_fn(arr, 2, L.F16, m, 1.0, None)
                if rc:
                    L.check(rc)
            down_only = [probs_of([(p412[li % len(p412)], hbuf, y["down"])]) for li in range(nlayers)]

            def mlp_three_calls():
                i = state["i"] % nlayers
                state["i"] += 1
                arr, cnt = gu_only[i]
                rc = gfn(arr, cnt, L.F16, m, L.F16, 1.0, None)
                rc = rc or gm_fn(L.UNARY["silu"], y["gate"].ptr, y["up"].ptr, L.F16, hbuf.ptr, m * 12288, None)
                arr, cnt = down_only[i]
                rc = rc or gfn(arr, cnt, L.F16, m, L.F16, 1.0, None)
                if rc:
                    L.check(rc)
            mlp_bytes = gu_bytes + algorithmic_bytes("int4", 4096, 12288, 32, m, 2, 2)
            us_mlp1 = B.median_time(mlp_one_call, 40)
            us_mlp3 = B.median_time(mlp_three_calls, 40)
            us_mlps = B.median_time(mlp_sequence_launch, 40)
            err = C.c_int(0)
            L.call("tlhip_sequence_status", None, C.byref(err))
            hbuf.destroy()
            layer_rows.append({
                "m": m, "bytes": layer_bytes,
                "mlp_block": {"bytes": mlp_bytes, "us_one_call": round(us_mlp1, 2), "us_three_calls": round(us_mlp3, 2),
                              "us_one_sequence_launch": round(us_mlps, 2),
                              "gbps_one_call": round(mlp_bytes / us_mlp1 / 1e3, 1),
                              "gbps_one_sequence_launch": round(mlp_bytes / us_mlps / 1e3, 1),
                              "note": "tlhip_mlp_decode (gate/up grouped + gated multiply + down from one call) vs the "
                                      "same launches as three calls vs tlhip_gemv_sequence (one launch)"},
                "us_7_launches": round(us_sep, 2), "us_4_launches": round(us_grp, 2),
                "gbps_4_launches": round(layer_bytes / us_grp / 1e3, 1),
                "frac_of_peak_4_launches": round(layer_bytes / us_grp / 1e3 / HBM_PEAK_GBPS, 4),
                "gate_up_grouped_us": round(us_gu, 2), "gate_up_grouped_gbps": round(gu_bytes / us_gu / 1e3, 1),
                "gate_up_grouped_frac_of_peak": round(gu_bytes / us_gu / 1e3 / HBM_PEAK_GBPS, 4),
                "config_qkv": list(be.selectedConfig(qkv_cat[0], "f16", m, "f16").as_tuple()),
                "config_gate_up": list(be.selectedConfig(gu_cat[0], "f16", m, "f16").as_tuple())})
            for t in list(y.values()) + [ycat]:
                t.destroy()
        details["qwen3_8b_decode_layer"] = layer_rows
        for pool_ in (kv_pool, qkv_cat, gu_cat):
            for w in pool_[1:]:
                w._base.destroy()
                w.scales.destroy()

        # batched decode beyond 16 rows (batch 32 / 64 / 128 of a serving loop) at the same three
        # shapes: what the library selects (up to 64 rows per launch of the skinny matrix-core
        # kernel while that beats the tiles) beside ONE tiled launch (128 x 128 tiles)
        rows_section = []
        fnc = L.load().tlhip_matmul_quantized_config
        tile128 = L.KernelConfig.of(3, 128, 128, 128, 2, 2)
        for (n, k) in shapes:
            qws = [be._qweight(w, False) for w in pools[(n, k)]]
            for m in (32, 64, 128):
                x, _ = B.activations(m, k, std=0.5)
                out = be._alloc([m, n], "f16")
                if not args.no_autotune and m <= 64:
                    B.tune(pools[(n, k)], x, m, out)
                us = B.median_time(B.make_call(pools[(n, k)], x, m, out), 30)
                st = {"i": 0}

                def tiled_call():
                    qw = qws[st["i"] % len(qws)]
                    st["i"] += 1
                    rc = fnc(C.byref(qw), x.ptr, L.F16, m, out.ptr, L.F16, 1.0, None, C.byref(tile128), None)
                    if rc:
                        L.check(rc)
                us_tiled = B.median_time(tiled_call, 20)
                by = algorithmic_bytes("int4", n, k, 32, m, 2, 2)
                rows_section.append({"m": m, "n": n, "k": k, "us": round(us, 2), "gbps": round(by / us / 1e3, 1),
                                     "frac_of_peak": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                     "us_one_tiled_launch_128x128": round(us_tiled, 2),
                                     "config": list(be.selectedConfig(pools[(n, k)][0], "f16", m, "f16").as_tuple())})
                out.destroy()
                x.destroy()
        details["qwen3_8b_batched_decode_32_to_128_rows"] = rows_section

        # config 5: LM head 256000 x 2304 int8-row (f32 logits) and the MLP GEMVs
        lm_pool, _ = B.weight_pool("int8-row", 256000, 2304, 0, "f32", pool_bytes=1.25e9)
        lm = []
        for m in (1, 4, 8, 16):
            x, _ = B.activations(m, 2304)
            out = be._alloc([m, 256000], "f32")
            if not args.no_autotune:
                B.tune(lm_pool, x, m, out, out_dtype="f32")
            call = B.make_call(lm_pool, x, m, out, out_dtype="f32")
            us = B.median_time(call, 30)
            by = algorithmic_bytes("int8-row", 256000, 2304, 0, m, 2, 4)
            cfg = be.selectedConfig(lm_pool[0], "f16", m, "f32")
            lm.append({"m": m, "us": round(us, 2), "gbps": round(by / us / 1e3, 1),
                       "frac_of_peak": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "kernel": kernel_name_of(cfg),
                       "config": list(cfg.as_tuple())})
            out.destroy()
        details["lm_head_int8_row_256000x2304"] = lm
        # the same kind of matrix in the reference's own format: 151936 x 2048 (a Qwen3 LM head),
        # int8 with an f16 absmax per group of 64 (quantizeLinearWeight's default)
        g64_pool, _ = B.weight_pool("int8-grouped", 151936, 2048, 64, "f32", pool_bytes=1.0e9)
        lm64 = []
        for m in (1, 4, 8, 16):
            x, _ = B.activations(m, 2048)
            out = be._alloc([m, 151936], "f32")
            if not args.no_autotune:
                B.tune(g64_pool, x, m, out, out_dtype="f32")
            call = B.make_call(g64_pool, x, m, out, out_dtype="f32")
            us = B.median_time(call, 30)
            by = algorithmic_bytes("int8-grouped", 151936, 2048, 64, m, 2, 4)
            cfg = be.selectedConfig(g64_pool[0], "f16", m, "f32")
            lm64.append({"m": m, "us": round(us, 2), "gbps": round(by / us / 1e3, 1),
                         "frac_of_peak": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "kernel": kernel_name_of(cfg),
                         "config": list(cfg.as_tuple())})
            out.destroy()
        details["lm_head_int8_g64_151936x2048"] = lm64
        for w in g64_pool[1:]:
            w._base.destroy()
            w.scales.destroy()
        # the LM head's consumer: device top-k of the 256 000 logits (k = 64), 512 B read back
        logits = be._alloc([256000], "f32")
        tv, ti = be._alloc([64], "f32"), be._alloc([64], "i32")
        L.call("tlhip_topk", logits.ptr, 0, 256000, 64, tv.ptr, ti.ptr, L.I32, None)  # first use allocates workspace

        def topk_call():
            L.call("tlhip_topk", logits.ptr, 0, 256000, 64, tv.ptr, ti.ptr, L.I32, None)
        details["lm_head_topk64_of_256000"] = {"us": round(B.median_time(topk_call, 50), 2)}
        for t in (logits, tv, ti):
            t.destroy()
        us = B.probe_time(lm_pool, 256000 * 2304)
        details["read_only_probe"]["256000x2304"] = {"bytes": 256000 * 2304, "us": round(us, 2),
                                                     "gbps": round(256000 * 2304 / us / 1e3, 1)}
        for w in lm_pool[1:]:
            w._base.destroy()
            w.scales.destroy()
        mlp = []
        for (n, k) in ((9216, 2304), (2304, 9216)):
            pool, _ = B.weight_pool("int4", n, k, 32, "f16")
            for m in (1, 8):
                x, _ = B.activations(m, k)
                out = be._alloc([m, n], "f16")
                if not args.no_autotune:
                    B.tune(pool, x, m, out)
                us = B.median_time(B.make_call(pool, x, m, out), 200)
                by = algorithmic_bytes("int4", n, k, 32, m, 2, 2)
                mlp.append({"m": m, "n": n, "k": k, "us": round(us, 2), "gbps": round(by / us / 1e3, 1)})
            for w in pool[1:]:
                w._base.destroy()
                w.scales.destroy()
        details["gemma2_mlp_int4"] = mlp

        # config 2: Qwen3-0.6B decode linears, 28 layers x 7 GEMVs, M = 1
        layer = [(2048, 1024), (1024, 1024), (1024, 1024), (1024, 2048), (3072, 1024), (3072, 1024), (1024, 3072)]
        lpools = {}
        for (n, k) in set(layer):
            lpools[(n, k)], _ = B.weight_pool("int4", n, k, 32, "f16", pool_bytes=40e6)
        lx = {k: B.activations(1, k)[0] for k in {k for _, k in layer}}
        lout = {n: be._alloc([1, n], "f16") for n in {n for n, _ in layer}}
        if not args.no_autotune:
            for (n, k) in set(layer):
                B.tune(lpools[(n, k)], lx[k], 1, lout[n])
        calls = []
        for li in range(28):
            for (n, k) in layer:
                calls.append(B.make_call(lpools[(n, k)][li % len(lpools[(n, k)]):] + lpools[(n, k)][:li % len(lpools[(n, k)])],
                                         lx[k], 1, lout[n]))

        def token():
            for c in calls:
                c()
        token_bytes = 28 * sum(algorithmic_bytes("int4", n, k, 32, 1, 2, 2) for (n, k) in layer)
        us_stream = B.median_time(token, 5)
        L.call("tlhip_set_autotune_enabled", 0)

        def graph_time(enqueue):
            """Median time of replaying `enqueue`'s launches from one HIP graph (with
            --no-graphs: of the stream launches themselves)."""
            if args.no_graphs:
                return B.median_time(enqueue, 5)
            graph = C.c_void_p()
            enqueue()
            L.call("tlhip_graph_begin_capture", None)
            enqueue()
            L.call("tlhip_graph_end_capture", None, C.byref(graph))
            us = B.median_time(lambda: L.call("tlhip_graph_launch", graph, None), 5)
            L.call("tlhip_graph_destroy", graph)
            return us
        us_graph = graph_time(token)

        # the same 196 GEMVs with the Linears that share an activation row issued as
        # one launch each: (q, k, v), o, (gate, up), down = 4 launches per layer
        lout2 = {key: be._alloc([1, n], "f16") for key, n in
                 (("q", 2048), ("k", 1024), ("v", 1024), ("o", 1024), ("gate", 3072), ("up", 3072), ("down", 1024))}
        groups = [[("q", 2048, 1024), ("k", 1024, 1024), ("v", 1024, 1024)], [("o", 1024, 2048)],
                  [("gate", 3072, 1024), ("up", 3072, 1024)], [("down", 1024, 3072)]]
        gfn = L.load().tlhip_gemv_grouped
        gcalls = []
        for li in range(28):
            for gi, grp in enumerate(groups):
                probs = (L.GemvProblem * len(grp))()
                for i, (key, n, k) in enumerate(grp):
                    pool = lpools[(n, k)]
                    probs[i].w = be._qweight(pool[(li * 3 + i) % len(pool)], False)
                    probs[i].x = lx[k].ptr
                    probs[i].y = lout2[key].ptr
                    probs[i].epilogue = None
                gcalls.append((probs, len(grp)))

        def token_grouped():
            for probs, cnt in gcalls:
                rc = gfn(probs, cnt, L.F16, L.F16, 1.0, None)
                if rc:
                    L.check(rc)
        us_grouped = B.median_time(token_grouped, 5)
        us_grouped_graph = graph_time(token_grouped)
        # the same token with the producers of the Linears' inputs: RMSNorm in front of
        # (q, k, v) and of (gate, up), silu(gate) * up in front of down.  Apart: 7
        # launches per layer; fused into the GEMVs' activation staging: still 4.
        nw = be.ops.tensorFromArray(np.ones(1024, np.float32), [1024], "f32")
        xn = be._alloc([1, 1024], "f16")
        act = be._alloc([1, 3072], "f16")
        lib = L.load()
        pro_norm = L.Prologue(L.PRO_RMSNORM, 0, 1e-6, 0, nw.ptr)
        pro_gate = L.Prologue(L.PRO_GATED_MUL, L.UNARY["silu"], 0.0, 0, lout2["up"].ptr)

        def chk(rc):
            if rc:
                L.check(rc)

        def token_producers_apart():
            for i in range(0, len(gcalls), 4):
                (pq, nq), (po, no), (pg, ng), (pd, nd) = gcalls[i:i + 4]
                chk(lib.tlhip_rmsnorm(lx[1024].ptr, L.F16, nw.ptr, xn.ptr, L.F16, 1, 1024, 1e-6, None))
                chk(gfn(pq, nq, L.F16, L.F16, 1.0, None))
                chk(gfn(po, no, L.F16, L.F16, 1.0, None))
                chk(lib.tlhip_rmsnorm(lx[1024].ptr, L.F16, nw.ptr, xn.ptr, L.F16, 1, 1024, 1e-6, None))
                chk(gfn(pg, ng, L.F16, L.F16, 1.0, None))
                chk(lib.tlhip_gated_mul(L.UNARY["silu"], lout2["gate"].ptr, lout2["up"].ptr, L.F16, act.ptr, 3072, None))
                chk(gfn(pd, nd, L.F16, L.F16, 1.0, None))

        gpro = lib.tlhip_gemv_grouped_prologue
        down_x = []
        for i in range(3, len(gcalls), 4):
            # the down projection reads the gate row; `up` arrives through the prologue
            probs = (L.GemvProblem * 1)()
            probs[0] = gcalls[i][0][0]
            probs[0].x = lout2["gate"].ptr
            down_x.append(probs)

        def token_producers_fused():
            for j, i in enumerate(range(0, len(gcalls), 4)):
                (pq, nq), (po, no), (pg, ng), _ = gcalls[i:i + 4]
                chk(gpro(pq, nq, C.byref(pro_norm), L.F16, L.F16, 1.0, None))
                chk(gfn(po, no, L.F16, L.F16, 1.0, None))
                chk(gpro(pg, ng, C.byref(pro_norm), L.F16, L.F16, 1.0, None))
                chk(gpro(down_x[j], 1, C.byref(pro_gate), L.F16, L.F16, 1.0, None))

        producer_us = {"apart": graph_time(token_producers_apart), "fused": graph_time(token_producers_fused)}
        details["qwen3_0p6b_decode_token_with_producers"] = {
            "what": "28 layers: rmsnorm -> (q,k,v), o, rmsnorm -> (gate,up), silu(gate)*up -> down; "
                    + ("stream launches" if args.no_graphs else "HIP graph"),
            "launches_apart": 28 * 7, "us_per_token_apart": round(producer_us["apart"], 1),
            "launches_fused": 28 * 4, "us_per_token_fused": round(producer_us["fused"], 1)}

        details["qwen3_0p6b_decode_token"] = {
            "gemvs": len(calls), "bytes": token_bytes, "us_per_token_stream": round(us_stream, 1),
            "us_per_token_graph": round(us_graph, 1), "gbps_stream": round(token_bytes / us_stream / 1e3, 1),
            "gbps_graph": round(token_bytes / us_graph / 1e3, 1), "us_at_hbm_peak": round(token_bytes / 8e6, 1),
            "grouped_launches": len(gcalls), "us_per_token_grouped_stream": round(us_grouped, 1),
            "us_per_token_grouped_graph": round(us_grouped_graph, 1),
            "gbps_grouped_graph": round(token_bytes / us_grouped_graph / 1e3, 1)}

        # config 4: prefill GEMM, int4 g32, f16 bias then silu / gelu(tanh), f16 out
        n, k = 12288, 4096
        w = pools[(n, k)][0]
        bias = be.ops.tensorFromArray((B.rng.standard_normal(n) * 0.1).astype(np.float16), [n], "f16")
        pre = []
        for m in (512, 2048):
            x, _ = B.activations(m, k, std=0.5)
            out = be._alloc([m, n], "f16")
            if not args.no_autotune:
                B.tune([w], x, m, out, epilogue=be.makeEpilogue(bias, "silu"))
            for act in ("silu", "gelu"):
                ep = be.makeEpilogue(bias, act)
                us = B.median_time(B.make_call([w], x, m, out, epilogue=ep), 20)
                fl = 2.0 * m * n * k
                cfg = be.selectedConfig(w, "f16", m, "f16")
                pre.append({"m": m, "epilogue": f"bias+{act}", "us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                            "frac_of_f16_mfma_peak": round(fl / us / 1e6 / F16_MFMA_PEAK_TFLOPS, 4),
                            "config": list(cfg.as_tuple())})
            if m == 2048:
                # the chain a decoder block hands over: bias, activation, residual add ([M,N], f16)
                res = be._alloc([m, n], "f16")
                ep = be.makeEpilogue(bias, "silu", ("add", res))
                us = B.median_time(B.make_call([w], x, m, out, epilogue=ep), 20)
                pre.append({"m": m, "epilogue": "bias+silu+add[M,N]", "us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                            "frac_of_f16_mfma_peak": round(fl / us / 1e6 / F16_MFMA_PEAK_TFLOPS, 4),
                            "config": list(cfg.as_tuple())})
                res.destroy()
            out.destroy()
        details["prefill_gemm_int4_4096x12288"] = pre
        # the same GEMM on f32 activations with f32 output (the reference's default
        # dtype): one cast launch into the stream's workspace + the f16 problem's kernel
        pre32 = []
        for m in (512, 2048):
            x, _ = B.activations(m, k, dtype="f32", std=0.5)
            out = be._alloc([m, n], "f32")
            us = B.median_time(B.make_call([w], x, m, out, epilogue=be.makeEpilogue(bias, "silu"), out_dtype="f32"), 20)
            fl = 2.0 * m * n * k
            pre32.append({"m": m, "epilogue": "bias+silu", "us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                          "config": list(be.selectedConfig(w, "f32", m, "f32").as_tuple())})
            out.destroy()
        details["prefill_gemm_int4_4096x12288_f32_activations"] = pre32
        # the same GEMM on the reference's own format (int8, one f16 absmax per 64 weights),
        # heuristic defaults (no entry of the tuning file covers it)
        w8_pool, _ = B.weight_pool("int8-grouped", n, k, 64, "f16", pool_bytes=110e6)
        pre8 = []
        for m in (512, 2048):
            x, _ = B.activations(m, k, std=0.5)
            out = be._alloc([m, n], "f16")
            us = B.median_time(B.make_call(w8_pool, x, m, out, epilogue=be.makeEpilogue(bias, "silu")), 20)
            fl = 2.0 * m * n * k
            pre8.append({"m": m, "epilogue": "bias+silu", "us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                         "frac_of_f16_mfma_peak": round(fl / us / 1e6 / F16_MFMA_PEAK_TFLOPS, 4),
                         "config": list(be.selectedConfig(w8_pool[0], "f16", m, "f16").as_tuple())})
            out.destroy()
            x.destroy()
        details["prefill_gemm_int8_g64_4096x12288"] = pre8

        # config 1: int8-row 1024 x 1024, f32 activations and output, M = 1
        pool, _ = B.weight_pool("int8-row", 1024, 1024, 0, "f32", pool_bytes=64e6)
        x, _ = B.activations(1, 1024, dtype="f32")
        out = be._alloc([1, 1024], "f32")
        us = B.median_time(B.make_call(pool, x, 1, out, out_dtype="f32"), 500)
        details["int8_row_1024x1024_f32"] = {"us": round(us, 2), "note": "launch-bound: 1.06 MB per call"}

    if not args.no_cpu:
        # CPU baseline: the same step on the host, single-threaded like the reference's
        # CPU backend (bounded: one pass, about 10-20 s), then with all host cores.
        from oracle import quant_oracle as O
        sec1 = cpu_step(cases, host_weights, host_x, 1)
        cores = O.max_threads()
        cpu_out = []
        secn = cpu_step(cases, host_weights, host_x, cores, keep=cpu_out)
        # the step that was timed, checked: each of its 15 calls once more on the GPU (same
        # weights, activations and kernel configuration) against the host's result
        worst = 0.0
        for c, want in zip(cases, cpu_out):
            c["call"]()
            be.synchronize()
            got = outs[(c["m"], c["n"])].numpy().astype(np.float64)
            err = float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))
            worst = max(worst, err)
        if not worst <= 1e-3:
            print(f"bench: the timed step's outputs differ from the CPU restatement (rel-L2 {worst:.3g} > 1e-3)", file=sys.stderr)
            return 1
        result["cpu_baseline"] = {
            "value": round(step_bytes / sec1 / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "one full step (15 calls, dequantisation of the three weights included), C restatement of the "
                      "reference's CPU matmul: f64 accumulate in k order, f32 store",
            "seconds_per_step": round(sec1, 3),
            "gpu_outputs_checked": {"calls": len(cases), "max_rel_l2": float(f"{worst:.3g}"), "bar": 1e-3},
            "all_cores": {"value": round(step_bytes / secn / 1e9, 4), "cores": cores, "seconds_per_step": round(secn, 3)}}
    if tuning_source == "tuned in this run" and not args.no_details:
        os.makedirs(os.path.dirname(args.tuning_cache), exist_ok=True)
        text = T.exportTuningCache()
        with open(args.tuning_cache, "w") as f:
            f.write(text)
    result["details"] = details
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
