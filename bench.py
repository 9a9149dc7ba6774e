#!/usr/bin/env python3
"""Benchmark of the nvtext hot path on one MI355X.

A step is one wordpiece_tokenize call over the whole synthetic batch of configuration C2
(4M rows, lognormal mean 256 B, Zipf(1.1) words over a 30,522-entry vocabulary, 15 % OOV,
int32 offsets, max_words_per_row=128), inputs resident in HBM, output allocation included.
Prints one JSON line: input GB/s as `value`, plus Mrows/s, the roofline of the whole call,
the host-oracle baseline on a bounded sample, the minhash / minhash64 figures (configurations
C3 / C4 at a stated scale), the UTF-8 pipeline of C5 and the reference's own benchmark shapes.
Every leg carries the mean and the median step time and the device memory a call holds at its peak.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# Hardware counters cannot be read from inside this process.  The figures below were read off rocprofv3 --pmc runs
# of this same program; each names the file under profiles/ that holds the command and the raw readings, and is only
# reported for the workload it was measured on.
#
# HBM bytes per launch (fetched, written) of the tokenizer kernels on the full C2 workload: FETCH_SIZE / WRITE_SIZE
# scaled by a copy kernel of known size.
TRAFFIC_SOURCE = "profiles/hbm_traffic_pmc_all_workloads.md (library sources at commit 692bfef)"
MEASURED_TRAFFIC_C2 = {
    "range_first_row_kernel": (15968662, 248800),
    "wordpiece_word_kernel": (1742880831, 1556229099),
    "wordpiece_oov_kernel": (861252878, 857545519),
    "wordpiece_emit_kernel": (1393668802, 905164798),
}
# (the fetch counter prices a read that misses L2 at a whole 128-byte line whatever was asked for, and counts the misses
# that the Infinity Cache serves: most of what the tokenizer fetches on C5 is lines of its 8 MB table)
MEASURED_TRAFFIC_C5_TOKENIZE = {
    "range_first_row_kernel": (119625264, 995168),
    "wordpiece_word_kernel": (24310186114, 5163209271),
    "wordpiece_oov_kernel": (21481440462, 2092868777),
    "wordpiece_emit_kernel": (4729690208, 3361303065),
}
MEASURED_TRAFFIC_C5_NORMALIZE = {
    "normalize_count_kernel": (4575175068, 63532928),
    "normalize_tile_rows_kernel": (73449328, 7941632),
    "normalize_write_kernel": (5469615636, 4672395239),
}
# minhash: VALU wave-instructions executed per (window, parameter) of a wavefront (SQ_INSTS_VALU / (windows x P / 64)) and
# the share of SIMD cycles that issued one (SQ_INSTS_VALU x 4 / (1024 SIMDs x kernel cycles), capped at 1: adds and
# moves issue in fewer than 4 cycles).  The floor is the instruction sequence of the inner loop: uint32, one
# v_mad_u64_u32 per product and one v_min3_u32 per two (1.5); uint64, three v_mad_u64_u32 and a 32-bit add for (h * a + b)
# mod 2^64, a shift, a mask and one more v_mad_u64_u32 for the fold mod 2^61-1, one v_min_f64, one v_max3_u32 per two
# products (8.5).  Every window of the input counts as one, also those whose hash the wavefront met lately and does not
# fold again (windows of a row repeat, most in long rows: that is how C4 comes so near the floor).
VALU_SOURCE = "profiles/valu_issue_pmc_all_workloads.md (library sources at commit 692bfef)"
MINHASH_VALU = {
    "C3": {"floor": 1.5, "measured": 1.72, "issue": 0.97},
    "C4": {"floor": 8.5, "measured": 8.73, "issue": 0.88},
    "C5": {"floor": 8.5, "measured": 13.08, "issue": 1.05},
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def median(xs):
    s = sorted(xs)
    n = len(s)
    return s[n // 2] if n % 2 else 0.5 * (s[n // 2 - 1] + s[n // 2])


def input_bytes(col):
    """chars + (rows+1) offsets + validity mask (the input term of the algorithmic bytes)."""
    ow = col.offsets.dtype.itemsize
    return col.chars_bytes + (col.size + 1) * ow + ((col.size + 7) // 8 if col.mask is not None else 0)


def timed_steps(fn, steps, warmup, torch):
    """Seconds per step over exactly `steps` steps (wall clock between two synchronisations)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def median_step_ms(fn, reps, torch):
    """Median over `reps` single steps, each bracketed by events on the stream the library launches on."""
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return median(times)


def peak_device_bytes(fn, torch):
    """Device memory one call holds at its peak, results and temporaries together, beyond what was allocated before it
    (every allocation of the library goes through torch's allocator here)."""
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    out = fn()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - before
    del out
    return int(peak)


def host_threads(orc):
    """Threads for the host oracle and where the number comes from: every core this process may run on (affinity mask,
    cgroup quota), and no more than the CPU share the job was given when the environment states one."""
    n = orc.hardware_threads()
    src = "hardware_concurrency"
    try:
        aff = len(os.sched_getaffinity(0))
        if aff < n:
            n, src = aff, "sched_getaffinity"
    except AttributeError:
        pass
    try:
        quota, period = open("/sys/fs/cgroup/cpu.max").read().split()
        if quota != "max" and int(quota) // int(period) < n:
            n, src = max(1, int(quota) // int(period)), "cgroup cpu.max"
    except (OSError, ValueError):
        pass
    share = os.environ.get("OMP_NUM_THREADS", "")
    if share.isdigit() and 0 < int(share) < n:
        n, src = int(share), "OMP_NUM_THREADS (the job's CPU share)"
    return max(1, n), src


def cpu_leg(orc, value, seconds, sample):
    threads, src = host_threads(orc)
    return {"value": value, "unit": "GB/s", "cores": threads, "cores_from": src,
            "hardware_concurrency": orc.hardware_threads(), "kind": "port", "sample": f"{sample}, {seconds:.2f} s"}


def measure(fn, steps, warmup, capi, torch):
    """One leg: mean wall time per step over exactly `steps` steps, the median of at least ten single steps timed with
    events, the library's kernels, and the device memory a call holds at its peak."""
    sec = timed_steps(fn, steps, warmup, torch)
    med = median_step_ms(fn, max(10, steps), torch)
    kt = kernel_times(fn, 3, capi, torch)
    peak = peak_device_bytes(fn, torch)
    return sec, {"ms_per_step": round(sec * 1e3, 4), "median_ms": round(med, 4), "peak_device_bytes": peak,
                 "kernels_ms": {k: round(v, 4) for k, v in kt.items()}}, kt


def kernel_times(fn, reps, capi, torch):
    """Average duration of each library kernel, from HIP events recorded by the library on the
    stream it launches on."""
    capi.profile_enable(True)
    capi.profile_read()
    acc = {}
    for _ in range(reps):
        fn()
        torch.cuda.synchronize()
        for name, ms in capi.profile_read():
            acc.setdefault(name, []).append(ms)
    capi.profile_enable(False)
    return {k: sum(v) / len(v) for k, v in acc.items()}


def hbm_roofline(alg_bytes, sec, kt, traffic=None):
    """The roofline object of an HBM-bound call: `frac` prices the algorithmic bytes against the whole call (all of
    its kernels, its scans and its synchronisations); the longest kernel is named beside it."""
    dom = max(kt, key=kt.get)
    achieved = alg_bytes / sec / 1e9
    have = traffic is not None and all(sum(v) > 0 for v in traffic.values())
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": sum(sum(v) for v in traffic.values()) if have else None,
            "traffic_per_kernel": {k: sum(v) for k, v in traffic.items()} if have else None,
            "traffic_source": TRAFFIC_SOURCE if have else None,
            "algorithmic_bytes": alg_bytes, "kernel": dom, "kernel_ms": round(kt[dom], 4),
            "kernel_frac": round(alg_bytes / (kt[dom] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}


def valu_object(name):
    """minhash is bound by VALU issue: the share of the SIMDs' issue slots that the floor sequence of the inner loop
    would need, floor / measured instructions per permutation x measured issue rate.  It cannot exceed 1."""
    v = MINHASH_VALU[name]
    return {"bound": "valu issue", "floor_inst_per_perm": v["floor"], "measured_inst_per_perm": v["measured"],
            "valu_issue": v["issue"], "frac": round(v["floor"] / v["measured"] * min(1.0, v["issue"]), 3), "source": VALU_SOURCE}


# Peak of the VALUs: 1024 SIMDs x 2.4 GHz / 4 cycles per wave64 instruction = 614.4 G wave-instructions/s
# (profiles/valu_instruction_rates.md: multiply-adds issue in 4.7 cycles, which this figure does not discount).
VALU_WAVE_INST_PER_S = 1024 * 2.4e9 / 4


def valu_from_rate(perm_per_s, bits):
    """For a leg without a counter run of its own: the share of the VALUs' peak issue rate that the floor sequence of the
    inner loop alone accounts for at the measured permutation rate (64 permutations per wave-instruction)."""
    floor = 1.5 if bits == 32 else 8.5
    return {"bound": "valu issue", "floor_inst_per_perm": floor,
            "frac": round(perm_per_s / 64 * floor / VALU_WAVE_INST_PER_S, 3), "source": "measured rate x floor / peak issue rate"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--scale", type=float, default=1.0, help="row-count multiplier of the headline workload (1.0 = 4M rows)")
    ap.add_argument("--minhash-scale", type=float, default=1.0, help="row-count multiplier of the C3/C4/C5 legs (0 = skip)")
    ap.add_argument("--reference-shapes", type=int, default=1, help="run the reference's own benchmark shapes (0 = skip)")
    ap.add_argument("--legs", default="c2,c3,c4,ngrams,jaccard,c5,ref",
                    help="which workloads to run (profiling runs take them one group at a time); without c2 the line has no value")
    ap.add_argument("--cpu-sample-rows", type=int, default=4_000_000, help="rows of the workload given to the host oracle")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; the path shards by row ranges with no exchange step, "
              "run one process per GPU on disjoint row ranges instead (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from cudf_amd import _capi, datagen, nvtext
    from cudf_amd.arrow_host import HostStringsColumn
    _capi.load()
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    orc = None
    if not args.no_cpu:
        from oracle import pyoracle as orc
        threads, src = host_threads(orc)
        log(f"[bench] host oracle: {threads} threads ({src}); hardware_concurrency() = {orc.hardware_threads()}")
    side_steps = max(3, args.steps // 2)
    legs = set(args.legs.split(","))
    unknown = legs - {"c2", "c3", "c4", "ngrams", "jaccard", "c5", "ref"}
    if unknown:
        sys.exit(f"bench.py: unknown legs {sorted(unknown)}")
    if args.minhash_scale <= 0:
        legs -= {"c3", "c4", "ngrams", "jaccard", "c5"}
    if not args.reference_shapes:
        legs.discard("ref")

    # ------------------------------------------------------------------ headline: wordpiece_tokenize on C2
    line = None
    if "c2" in legs:
        t0 = time.time()
        wl = datagen.config2(args.scale)
        host = wl.rows
        log(f"[bench] C2 generated: rows={host.size} chars={host.chars_bytes / 1e9:.3f} GB in {time.time() - t0:.1f}s")
        dcol = nvtext.DeviceStringsColumn.from_host(host)
        dvoc = nvtext.WordPieceVocabulary(nvtext.DeviceStringsColumn.from_host(wl.vocab))
        mw = wl.params["max_words_per_row"]
        keep = {}

        def step():
            keep["o"] = nvtext.wordpiece_tokenize(dcol, dvoc, mw)
            return keep["o"]

        sec, head, kt = measure(step, args.steps, args.warmup, _capi, torch)
        tokens = keep["o"].child_size
        in_b = input_bytes(host)
        out_b = 4 * tokens + 4 * (host.size + 1) + ((host.size + 7) // 8 if host.mask is not None else 0)
        log(f"[bench] tokenize: {head}, tokens={tokens}")
        roofline = hbm_roofline(in_b + out_b, sec, kt, MEASURED_TRAFFIC_C2 if args.scale == 1.0 else None)
        roofline["all_kernels_ms"] = head["kernels_ms"]
        # what a call holds beyond its result at its peak, per input byte
        roofline["temporaries_bytes"] = head["peak_device_bytes"] - out_b
        roofline["temporaries_per_input_byte"] = round((head["peak_device_bytes"] - out_b) / in_b, 3)

        # ------------------------------------------------------------------ host oracle on a bounded sample (also the parity check)
        cpu = None
        parity = "skipped"
        if orc:
            n = min(args.cpu_sample_rows, host.size)
            sample = host.slice(0, n)
            ovoc = orc.Vocabulary(wl.vocab)
            t0 = time.perf_counter()
            exp = orc.wordpiece_tokenize(sample, ovoc, mw, nthreads=threads)
            cpu_s = time.perf_counter() - t0
            cpu = cpu_leg(orc, round(input_bytes(sample) / cpu_s / 1e9, 4), cpu_s,
                          f"first {n} rows of the same workload ({sample.chars_bytes / 1e6:.0f} MB)")
            cpu["mrows_per_s"] = round(n / cpu_s / 1e6, 3)
            got = nvtext.wordpiece_tokenize(dcol.slice(0, n, 0), dvoc, mw).to_host()
            parity = "PASS" if got.equals(exp) else "FAIL"
            log(f"[bench] oracle: {cpu_s:.2f}s on {threads} threads; parity {parity}")
            del exp, got
        del dcol, keep

        line = {
            "metric": "input GB/s + Mrows/s, wordpiece_tokenize & minhash, 1 MI355X, % of roofline",
            "value": round(in_b / sec / 1e9, 3), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(sec * 1e3, 4), "median_ms": head["median_ms"], "peak_device_bytes": head["peak_device_bytes"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "u8/int32", "data": "synthetic",
            "config": {"workload": f"C2 wordpiece_tokenize x{args.scale}", "rows": host.size, "chars_bytes": host.chars_bytes,
                       "vocab_entries": wl.vocab.size, "max_words_per_row": mw, "tokens_out": tokens, "offsets": "int32"},
            "mrows_per_s": round(host.size / sec / 1e6, 3),
            "roofline": roofline, "cpu_baseline": cpu, "parity_vs_oracle": parity,
        }

    # ------------------------------------------------------------------ minhash legs (C3 uint32, C4 uint64)
    extra = {}
    if legs & {"c3", "c4"}:
        for name, fn in (("C3", nvtext.minhash), ("C4", nvtext.minhash64)):
            if name.lower() not in legs:
                continue
            torch.cuda.empty_cache()
            t0 = time.time()
            w = datagen.CONFIGS[name](args.minhash_scale)
            p = w.params
            a, b = datagen.make_params(p["P"], p["hash_bits"], p["param_seed"])
            signed = np.int32 if p["hash_bits"] == 32 else np.int64
            da = torch.from_numpy(a.view(signed)).cuda()
            db = torch.from_numpy(b.view(signed)).cuda()
            log(f"[bench] {name} generated: rows={w.rows.size} chars={w.rows.chars_bytes / 1e9:.3f} GB in {time.time() - t0:.1f}s")
            dc = nvtext.DeviceStringsColumn.from_host(w.rows)
            keep = {}

            def mstep():
                keep["o"] = fn(dc, p["seed"], da, db, p["width"])
                return keep["o"]

            msec, leg, _ = measure(mstep, side_steps, 1, _capi, torch)
            ib = input_bytes(w.rows)
            valid = w.rows.size - w.rows.null_count
            windows = int(w.rows.chars_bytes - valid * (p["width"] - 1))  # ASCII rows longer than width
            leg.update({"workload": f"{name} x{args.minhash_scale}", "rows": w.rows.size, "chars_bytes": w.rows.chars_bytes,
                        "input_GBps": round(ib / msec / 1e9, 2), "mrows_per_s": round(w.rows.size / msec / 1e6, 3),
                        "gperm_per_s": round(windows * p["P"] / msec / 1e9, 1)})
            if args.minhash_scale == 1.0:
                leg["valu"] = valu_object(name)
            if orc:
                n = min(w.rows.size, 20000 if name == "C3" else 2000)
                smp = w.rows.slice(0, n)
                ofn = orc.minhash if name == "C3" else orc.minhash64
                t0 = time.perf_counter()
                exp = ofn(smp, p["seed"], a, b, p["width"], nthreads=threads)
                cs = time.perf_counter() - t0
                got = fn(dc.slice(0, n, smp.null_count), p["seed"], da, db, p["width"]).to_host()
                leg["cpu_baseline"] = cpu_leg(orc, round(input_bytes(smp) / cs / 1e9, 5), cs, f"first {n} rows ({smp.chars_bytes / 1e6:.1f} MB)")
                leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
            log(f"[bench] {name}: {leg}")
            extra["minhash" if name == "C3" else "minhash64"] = leg
            del dc, keep

    # ------------------------------------------------------------------ minhash_ngrams over the words of C3 (a quarter of its rows)
    if "ngrams" in legs:
        torch.cuda.empty_cache()
        t0 = time.time()
        w = datagen.config3(0.25 * args.minhash_scale)
        p = w.params
        lists = datagen.words_as_lists(w.rows)
        a, b = datagen.make_params(p["P"], 32, p["param_seed"])
        da = torch.from_numpy(a.view(np.int32)).cuda()
        db = torch.from_numpy(b.view(np.int32)).cuda()
        log(f"[bench] word lists of C3 x{0.25 * args.minhash_scale}: rows={lists.size} elements={lists.child.size} in {time.time() - t0:.1f}s")
        dl = nvtext.DeviceListStringsColumn.from_host(lists)
        keep = {}
        ngrams = 5

        def nstep():
            keep["o"] = nvtext.minhash_ngrams(dl, ngrams, p["seed"], da, db)
            return keep["o"]

        nsec, leg, _ = measure(nstep, side_steps, 1, _capi, torch)
        nb = lists.child.chars.size + (lists.child.size + 1) * lists.child.offsets.dtype.itemsize + (lists.size + 1) * 4
        leg.update({"workload": f"words of C3 x{0.25 * args.minhash_scale} as LIST<STRING>, ngrams={ngrams}, P={p['P']}", "rows": lists.size,
                    "elements": lists.child.size, "input_GBps": round(nb / nsec / 1e9, 2),
                    "mrows_per_s": round(lists.size / nsec / 1e6, 3), "gperm_per_s": round(lists.child.size * p["P"] / nsec / 1e9, 1)})
        if orc:
            n = min(lists.size, 20000)
            smp = lists.slice(0, n)
            t0 = time.perf_counter()
            exp = orc.minhash_ngrams(smp, ngrams, p["seed"], a, b, nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.minhash_ngrams(dl.slice(0, n, smp.null_count), ngrams, p["seed"], da, db).to_host()
            sample_bytes = int(lists.child.offsets[lists.offsets[n]])
            leg["cpu_baseline"] = cpu_leg(orc, round(sample_bytes / cs / 1e9, 5), cs, f"first {n} rows ({sample_bytes / 1e6:.1f} MB)")
            leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] minhash_ngrams: {leg}")
        extra["minhash_ngrams"] = leg
        del dl, keep

    # ------------------------------------------------------------------ jaccard_index of neighbouring rows of C3 (a quarter of its rows)
    if "jaccard" in legs:
        torch.cuda.empty_cache()
        w = datagen.config3(0.25 * args.minhash_scale)
        n = w.rows.size - 1
        dc = nvtext.DeviceStringsColumn.from_host(w.rows)
        d1, d2 = dc.slice(0, n, 0), dc.slice(1, n + 1, 0)
        keep = {}
        jwidth = 5

        def jstep():
            keep["o"] = nvtext.jaccard_index(d1, d2, jwidth)
            return keep["o"]

        jsec, leg, _ = measure(jstep, side_steps, 1, _capi, torch)
        jb = 2 * input_bytes(w.rows)
        leg.update({"workload": f"rows r and r+1 of C3 x{0.25 * args.minhash_scale}, width={jwidth}", "rows": n,
                    "input_GBps": round(jb / jsec / 1e9, 2), "mrows_per_s": round(n / jsec / 1e6, 3)})
        if orc:
            m = min(n, 20000)
            s1, s2 = w.rows.slice(0, m), w.rows.slice(1, m + 1)
            t0 = time.perf_counter()
            exp = orc.jaccard_index(s1, s2, jwidth, nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.jaccard_index(dc.slice(0, m, 0), dc.slice(1, m + 1, 0), jwidth).to_host()
            leg["cpu_baseline"] = cpu_leg(orc, round(2 * input_bytes(s1) / cs / 1e9, 5), cs, f"first {m} row pairs ({2 * s1.chars_bytes / 1e6:.1f} MB)")
            leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] jaccard_index: {leg}")
        extra["jaccard_index"] = leg
        del dc, d1, d2, keep

    # ------------------------------------------------------------------ C5: UTF-8 rows, int64 offsets, 250k vocabulary
    if "c5" in legs:
        torch.cuda.empty_cache()
        t0 = time.time()
        w = datagen.config5(args.minhash_scale)
        p = w.params
        log(f"[bench] C5 generated: rows={w.rows.size} chars={w.rows.chars_bytes / 1e9:.3f} GB in {time.time() - t0:.1f}s")
        dc = nvtext.DeviceStringsColumn.from_host(w.rows)
        dv5 = nvtext.WordPieceVocabulary(nvtext.DeviceStringsColumn.from_host(w.vocab))
        keep = {}

        def tstep():
            keep["o"] = nvtext.wordpiece_tokenize(dc, dv5, p["max_words_per_row"])
            return keep["o"]

        tsec, tleg, tk = measure(tstep, side_steps, 1, _capi, torch)
        ib = input_bytes(w.rows)
        ntok = keep["o"].child_size
        talg = ib + 4 * ntok + 4 * (w.rows.size + 1) + ((w.rows.size + 7) // 8 if w.rows.mask is not None else 0)
        tleg.update({"input_GBps": round(ib / tsec / 1e9, 2), "mrows_per_s": round(w.rows.size / tsec / 1e6, 3), "tokens_out": ntok,
                     "temporaries_bytes": tleg["peak_device_bytes"] - (talg - ib),
                     "temporaries_per_input_byte": round((tleg["peak_device_bytes"] - (talg - ib)) / ib, 3),
                     "roofline": hbm_roofline(talg, tsec, tk, MEASURED_TRAFFIC_C5_TOKENIZE if args.minhash_scale == 1.0 else None)})
        leg = {"workload": f"C5 x{args.minhash_scale}", "rows": w.rows.size, "chars_bytes": w.rows.chars_bytes, "offsets": "int64",
               "vocab_entries": w.vocab.size, "tokenize": tleg}
        keep.clear()
        # the same rows with the vocabulary of C2, which knows next to none of their words: four times the queued words per
        # byte that ordinary text has.  The call sizes its first attempt from a sample of the column; `word_pass_launches`
        # says whether that held (1) or the passes had to be repeated with larger temporaries (2).
        dv2 = nvtext.WordPieceVocabulary(nvtext.DeviceStringsColumn.from_host(datagen.config2(0.001).vocab))

        def fstep():
            keep["o"] = nvtext.wordpiece_tokenize(dc, dv2, p["max_words_per_row"])
            return keep["o"]

        fsec, fleg, _ = measure(fstep, max(2, side_steps // 2), 1, _capi, torch)
        _capi.profile_enable(True)
        _capi.profile_read()
        fstep()
        torch.cuda.synchronize()
        fleg.update({"workload": "C5 rows, the 30,522-entry vocabulary of C2", "input_GBps": round(ib / fsec / 1e9, 2), "tokens_out": keep["o"].child_size,
                     "word_pass_launches": sum(1 for name, _ in _capi.profile_read() if name == "wordpiece_word_kernel")})
        _capi.profile_enable(False)
        leg["tokenize_foreign_vocabulary"] = fleg
        keep.clear()
        del dv2
        # normalize_characters, the step that precedes the tokenizer in a BERT pipeline (lower-casing, five special tokens)
        special = nvtext.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist(["[CLS]", "[SEP]", "[PAD]", "[MASK]", "[UNK]"]))
        normalizer = nvtext.CharacterNormalizer(True, special)

        def zstep():
            keep["o"] = nvtext.normalize_characters(dc, normalizer)
            return keep["o"]

        zsec, zleg, zk = measure(zstep, side_steps, 1, _capi, torch)
        out_bytes = int(keep["o"].chars.numel())
        # algorithmic bytes of a call: chars + offsets in, chars + offsets (int64 from INT32_MAX bytes on) out
        zalg = ib + out_bytes + (8 if out_bytes >= 0x7FFFFFFF else 4) * (w.rows.size + 1)
        zleg.update({"input_GBps": round(ib / zsec / 1e9, 2), "mrows_per_s": round(w.rows.size / zsec / 1e6, 3), "chars_out": out_bytes,
                     "roofline": hbm_roofline(zalg, zsec, zk, MEASURED_TRAFFIC_C5_NORMALIZE if args.minhash_scale == 1.0 else None)})
        leg["normalize_characters"] = zleg
        if orc:
            from oracle import normalize_py
            normalize_py.rule_tables()  # built once, outside the timed part (the library's tables are built at create time)
            n = min(w.rows.size, 400000)
            smp = w.rows.slice(0, n)
            t0 = time.perf_counter()
            exp = normalize_py.normalize_characters_native(smp, True, [b"[CLS]", b"[SEP]", b"[PAD]", b"[MASK]", b"[UNK]"], nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.normalize_characters(dc.slice(0, n, smp.null_count), normalizer).to_host()
            zleg["cpu_baseline"] = cpu_leg(orc, round(input_bytes(smp) / cs / 1e9, 5), cs, f"first {n} rows ({smp.chars_bytes / 1e6:.0f} MB)")
            same = np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets)
            zleg["parity"] = "PASS" if same else "FAIL"
        keep.clear()
        a, b = datagen.make_params(p["P"], 64, p["param_seed"])
        da = torch.from_numpy(a.view(np.int64)).cuda()
        db = torch.from_numpy(b.view(np.int64)).cuda()

        def m5step():
            keep["o"] = nvtext.minhash64(dc, p["seed"], da, db, p["width"])
            return keep["o"]

        msec, mleg, _ = measure(m5step, side_steps, 1, _capi, torch)
        # windows of a row: its characters less width - 1, one for a shorter row that is not empty, none for a null row
        firsts = ((w.rows.chars & 0xC0) != 0x80)[: int(w.rows.offsets[-1])]
        begins = w.rows.offsets[:-1].astype(np.int64)
        inside = int(np.searchsorted(begins, firsts.size))  # (rows that begin at the end of the bytes are empty)
        row_chars = np.zeros(w.rows.size, np.int64)
        if inside:
            row_chars[:inside] = np.add.reduceat(firsts, begins[:inside], dtype=np.int64)
        row_chars[np.diff(w.rows.offsets) == 0] = 0
        if w.rows.mask is not None:
            from cudf_amd.arrow_host import unpack_validity
            row_chars[~unpack_validity(w.rows.mask, w.rows.size, w.rows.offset)] = 0
        windows = int(np.where(row_chars >= p["width"], row_chars - (p["width"] - 1), row_chars > 0).sum())
        del firsts, row_chars
        mleg.update({"input_GBps": round(ib / msec / 1e9, 2), "mrows_per_s": round(w.rows.size / msec / 1e6, 3),
                     "windows": windows, "parameters": p["P"], "gperm_per_s": round(windows * p["P"] / msec / 1e9, 1)})
        if args.minhash_scale == 1.0:
            mleg["valu"] = valu_object("C5")
        leg["minhash64"] = mleg
        if orc:
            n = min(w.rows.size, 400_000)
            smp = w.rows.slice(0, n)
            t0 = time.perf_counter()
            exp = orc.wordpiece_tokenize(smp, orc.Vocabulary(w.vocab), p["max_words_per_row"], nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.wordpiece_tokenize(dc.slice(0, n, smp.null_count), dv5, p["max_words_per_row"]).to_host()
            tleg["cpu_baseline"] = cpu_leg(orc, round(input_bytes(smp) / cs / 1e9, 4), cs, f"first {n} rows ({smp.chars_bytes / 1e6:.0f} MB)")
            tleg["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] C5: {leg}")
        extra["utf8_pipeline"] = leg
        del dc, dv5, keep

    # ------------------------------------------------------------------ the reference's own benchmark shapes
    if "ref" in legs:
        extra["reference_shapes"] = reference_shapes(args, orc, _capi, datagen, nvtext, HostStringsColumn, np, torch)

    if line is None:
        line = {"metric": "input GB/s + Mrows/s, wordpiece_tokenize & minhash, 1 MI355X, % of roofline", "value": None, "unit": "GB/s",
                "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "legs": sorted(legs)}
    line.update(extra)
    print(json.dumps(line), flush=True)


def reference_shapes(args, orc, _capi, datagen, nvtext, HostStringsColumn, np, torch):
    """The shapes of the reference's own benchmarks.  minhash over rows whose lengths are normal between 0 and
    row_width bytes: 60,000 x 28,000 with hash_width 12 / 24, 26 / 260 parameters and both hash widths, and the corners
    15,000 x 6,000 and 30,000 x 50,000 at hash_width 12 (cpp/benchmarks/text/minhash.cpp:16-62); wordpiece_tokenize
    over 32,768 / 262,144 / 2,097,152 copies of a 32-word row with a six-entry vocabulary, max_words 0 / 20 / 40
    (cpp/benchmarks/text/subword.cpp:18-52).  Random printable ASCII stands in for the reference's random strings;
    parity against the host oracle on the first rows of each shape."""
    legs = {"minhash": [], "wordpiece_tokenize": []}
    steps = max(3, args.steps // 2)
    threads = host_threads(orc)[0] if orc else 0

    for rows, row_width, widths, param_counts in ((60_000, 28_000, (12, 24), (26, 260)), (15_000, 6_000, (12,), (26, 260)),
                                                  (30_000, 50_000, (12,), (26, 260))):
        rng = np.random.default_rng(20231)
        lengths = np.clip(rng.normal(row_width / 2, row_width / 6, rows), 0, row_width).astype(np.int64)
        offsets = np.zeros(rows + 1, np.int32)
        np.cumsum(lengths, out=offsets[1:])
        chars = rng.integers(32, 127, int(offsets[-1]), dtype=np.uint8)
        col = HostStringsColumn(chars, offsets, None, rows, 0, 0)
        dc = nvtext.DeviceStringsColumn.from_host(col)
        ib = input_bytes(col)
        log(f"[bench] reference minhash shape: rows={rows} row_width={row_width} chars={col.chars_bytes / 1e9:.3f} GB")
        for bits, fn in ((32, nvtext.minhash), (64, nvtext.minhash64)):
            signed = np.int32 if bits == 32 else np.int64
            for nparams in param_counts:
                a, b = datagen.make_params(nparams, bits, 7)
                da = torch.from_numpy(a.view(signed)).cuda()
                db = torch.from_numpy(b.view(signed)).cuda()
                for width in widths:
                    keep = {}

                    def mstep():
                        keep["o"] = fn(dc, 0, da, db, width)
                        return keep["o"]

                    msec, leg, _ = measure(mstep, steps, 1, _capi, torch)
                    windows = int(np.maximum(lengths - (width - 1), (lengths > 0).astype(np.int64)).sum())
                    leg.update({"num_rows": rows, "row_width": row_width, "hash_width": width, "parameters": nparams, "hash_type": bits,
                                "input_GBps": round(ib / msec / 1e9, 2), "gperm_per_s": round(windows * nparams / msec / 1e9, 1),
                                "valu": valu_from_rate(windows * nparams / msec, bits)})
                    if orc:
                        n = (400 if bits == 32 else 100) * 28_000 // row_width
                        smp = col.slice(0, n)
                        exp = (orc.minhash if bits == 32 else orc.minhash64)(smp, 0, a, b, width, nthreads=threads)
                        got = fn(dc.slice(0, n, 0), 0, da, db, width).to_host()
                        leg["parity"] = ("PASS" if got.equals(exp) else "FAIL") + f" (first {n} rows)"
                    log(f"[bench] reference minhash: {leg}")
                    legs["minhash"].append(leg)
                    del keep
        del dc, col, chars

    text = b"This is a test " * 8
    vocab = HostStringsColumn.from_pylist(["", "[UNK]", "This", "is", "a", "test"])
    dv = nvtext.WordPieceVocabulary(nvtext.DeviceStringsColumn.from_host(vocab))
    for rows in (32_768, 262_144, 2_097_152):
        chars = np.frombuffer(text * rows, dtype=np.uint8)
        offsets = (np.arange(rows + 1, dtype=np.int64) * len(text)).astype(np.int32)
        col = HostStringsColumn(chars, offsets, None, rows, 0, 0)
        dc = nvtext.DeviceStringsColumn.from_host(col)
        ib = input_bytes(col)
        for max_words in (0, 20, 40):
            keep = {}

            def tstep():
                keep["o"] = nvtext.wordpiece_tokenize(dc, dv, max_words)
                return keep["o"]

            tsec, leg, tk = measure(tstep, steps if rows > 300_000 else 4 * steps, 1, _capi, torch)
            ntok = keep["o"].child_size
            leg.update({"num_rows": rows, "max_words": max_words, "chars_bytes": col.chars_bytes, "tokens_out": ntok,
                        "input_GBps": round(ib / tsec / 1e9, 2), "mrows_per_s": round(rows / tsec / 1e6, 2),
                        "launches": len(tk), "roofline": hbm_roofline(ib + 4 * ntok + 4 * (rows + 1), tsec, tk)})
            if orc:
                n = min(rows, 100_000)
                exp = orc.wordpiece_tokenize(col.slice(0, n), orc.Vocabulary(vocab), max_words, nthreads=threads)
                got = nvtext.wordpiece_tokenize(dc.slice(0, n, 0), dv, max_words).to_host()
                leg["parity"] = ("PASS" if got.equals(exp) else "FAIL") + f" (first {n} rows)"
            log(f"[bench] reference wordpiece_tokenize: {leg}")
            legs["wordpiece_tokenize"].append(leg)
            del keep
        del dc, col
    return legs


if __name__ == "__main__":
    main()
