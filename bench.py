#!/usr/bin/env python3
"""Benchmark of the nvtext hot path on one MI355X.

A step is one wordpiece_tokenize call over the whole synthetic batch of configuration C2
(4M rows, lognormal mean 256 B, Zipf(1.1) words over a 30,522-entry vocabulary, 15 % OOV,
int32 offsets, max_words_per_row=128), inputs resident in HBM, output allocation included.
Prints one JSON line: input GB/s as `value`, plus Mrows/s, the roofline of the dominant
kernel, the host-oracle baseline on a bounded sample, and the minhash / minhash64 figures
(configurations C3 / C4 at a stated scale).
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
VALU_PEAK_TOPS = 256 * 64 * 2.4e9 / 1e12  # 256 CUs x 64 lanes x 2.4 GHz: one 32-bit integer operation per lane and cycle

# HBM bytes per launch (fetched, written) of the tokenizer kernels on the full C2 workload, from two
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by a copy kernel of known size; the commands and
# raw readings are in profiles/hbm_traffic_pmc_all_workloads.md.  Counters cannot be read from inside this
# process, so the line reports these figures only for the workload they were measured on.
MEASURED_TRAFFIC_C2 = {
    "wordpiece_probe_kernel": (1766100000, 1970100000),
    "wordpiece_oov_kernel": (866200000, 1367300000),
    "wordpiece_emit_kernel": (2368800000, 862800000),
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
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--scale", type=float, default=1.0, help="row-count multiplier of the headline workload (1.0 = 4M rows)")
    ap.add_argument("--minhash-scale", type=float, default=1.0, help="row-count multiplier of the C3/C4/C5 legs (0 = skip)")
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

    # ------------------------------------------------------------------ headline: wordpiece_tokenize on C2
    t0 = time.time()
    wl = datagen.config2(args.scale)
    host = wl.rows
    log(f"[bench] C2 generated: rows={host.size} chars={host.chars_bytes / 1e9:.3f} GB in {time.time() - t0:.1f}s")
    dcol = nvtext.DeviceStringsColumn.from_host(host)
    dvoc = nvtext.WordPieceVocabulary(nvtext.DeviceStringsColumn.from_host(wl.vocab))
    mw = wl.params["max_words_per_row"]
    result = {}

    def step():
        result["out"] = nvtext.wordpiece_tokenize(dcol, dvoc, mw)

    sec = timed_steps(step, args.steps, args.warmup, torch)
    out = result["out"]
    tokens = out.child_size
    in_b = input_bytes(host)
    out_b = 4 * tokens + 4 * (host.size + 1) + ((host.size + 7) // 8 if host.mask is not None else 0)
    kt = kernel_times(step, 3, _capi, torch)
    log(f"[bench] tokenize: {sec * 1e3:.3f} ms/step, tokens={tokens}, kernels={ {k: round(v, 3) for k, v in kt.items()} }")
    dom = max(kt, key=kt.get)  # the kernel with the longest mean duration
    dom_ms = kt[dom]
    achieved = (in_b + out_b) / (dom_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": sum(MEASURED_TRAFFIC_C2[dom]) if args.scale == 1.0 and dom in MEASURED_TRAFFIC_C2 else None,
                "traffic_all_kernels": ({k: sum(v) for k, v in MEASURED_TRAFFIC_C2.items()} if args.scale == 1.0 else None),
                "algorithmic_bytes": in_b + out_b, "kernel_ms": round(dom_ms, 4),
                "all_kernels_ms": {k: round(v, 4) for k, v in kt.items()},
                "frac_whole_op": round((in_b + out_b) / sec / 1e9 / HBM_PEAK_GBS, 4)}

    # ------------------------------------------------------------------ host oracle on a bounded sample (also the parity check)
    cpu = None
    parity = "skipped"
    if not args.no_cpu:
        from oracle import pyoracle as orc
        n = min(args.cpu_sample_rows, host.size)
        sample = host.slice(0, n)
        ovoc = orc.Vocabulary(wl.vocab)
        threads = max(1, min(orc.hardware_threads(), 16))
        t0 = time.perf_counter()
        exp = orc.wordpiece_tokenize(sample, ovoc, mw, nthreads=threads)
        cpu_s = time.perf_counter() - t0
        cpu = {"value": round(input_bytes(sample) / cpu_s / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": f"first {n} rows of the same workload ({sample.chars_bytes / 1e6:.0f} MB), {cpu_s:.2f} s",
               "mrows_per_s": round(n / cpu_s / 1e6, 3)}
        got = nvtext.wordpiece_tokenize(dcol.slice(0, n, 0), dvoc, mw).to_host()
        parity = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] oracle: {cpu_s:.2f}s on {threads} threads; parity {parity}")
    del dcol, out, result

    # ------------------------------------------------------------------ minhash legs (C3 uint32, C4 uint64)
    extra = {}
    if args.minhash_scale > 0:
        for name, fn in (("C3", nvtext.minhash), ("C4", nvtext.minhash64)):
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

            msec = timed_steps(mstep, max(3, args.steps // 2), 1, torch)
            mk = kernel_times(mstep, 2, _capi, torch)
            ib = input_bytes(w.rows)
            valid = w.rows.size - w.rows.null_count
            windows = int(w.rows.chars_bytes - valid * (p["width"] - 1))  # ASCII rows longer than width
            leg = {"workload": f"{name} x{args.minhash_scale}", "rows": w.rows.size, "chars_bytes": w.rows.chars_bytes,
                   "ms_per_step": round(msec * 1e3, 3), "input_GBps": round(ib / msec / 1e9, 2),
                   "mrows_per_s": round(w.rows.size / msec / 1e6, 3),
                   "gperm_per_s": round(windows * p["P"] / msec / 1e9, 1),
                   "kernels_ms": {k: round(v, 3) for k, v in mk.items()}}
            # the bound of minhash is VALU issue: algorithmic lane-operations = windows x P x C_perm (2 for uint32:
            # multiply-add and min; 12 for uint64: three 32x32 multiply-adds, the fold mod 2^61-1, the 64-bit min)
            c_perm = 2 if p["hash_bits"] == 32 else 12
            ops = windows * p["P"] * c_perm
            leg["valu"] = {"algorithmic_ops": ops, "achieved": round(ops / msec / 1e12, 2), "peak": VALU_PEAK_TOPS,
                           "unit": "T lane-op/s", "frac": round(ops / msec / 1e12 / VALU_PEAK_TOPS, 3)}
            if not args.no_cpu:
                from oracle import pyoracle as orc
                n = min(w.rows.size, 20000 if name == "C3" else 2000)
                smp = w.rows.slice(0, n)
                ofn = orc.minhash if name == "C3" else orc.minhash64
                threads = max(1, min(orc.hardware_threads(), 16))
                t0 = time.perf_counter()
                exp = ofn(smp, p["seed"], a, b, p["width"], nthreads=threads)
                cs = time.perf_counter() - t0
                got = fn(dc.slice(0, n, smp.null_count), p["seed"], da, db, p["width"]).to_host()
                leg["cpu_baseline"] = {"value": round(input_bytes(smp) / cs / 1e9, 5), "unit": "GB/s", "cores": threads, "kind": "port",
                                       "sample": f"first {n} rows ({smp.chars_bytes / 1e6:.1f} MB), {cs:.2f} s"}
                leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
            log(f"[bench] {name}: {leg}")
            extra["minhash" if name == "C3" else "minhash64"] = leg
            del dc, keep

    # ------------------------------------------------------------------ minhash_ngrams over the words of C3 (a quarter of its rows)
    if args.minhash_scale > 0:
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

        nsec = timed_steps(nstep, max(3, args.steps // 2), 1, torch)
        nk = kernel_times(nstep, 2, _capi, torch)
        nb = lists.child.chars.size + (lists.child.size + 1) * lists.child.offsets.dtype.itemsize + (lists.size + 1) * 4
        leg = {"workload": f"words of C3 x{0.25 * args.minhash_scale} as LIST<STRING>, ngrams={ngrams}, P={p['P']}", "rows": lists.size,
               "elements": lists.child.size, "ms_per_step": round(nsec * 1e3, 3), "input_GBps": round(nb / nsec / 1e9, 2),
               "mrows_per_s": round(lists.size / nsec / 1e6, 3), "gperm_per_s": round(lists.child.size * p["P"] / nsec / 1e9, 1),
               "kernels_ms": {k: round(v, 3) for k, v in nk.items()}}
        if not args.no_cpu:
            from oracle import pyoracle as orc
            n = min(lists.size, 20000)
            smp = lists.slice(0, n)
            threads = max(1, min(orc.hardware_threads(), 16))
            t0 = time.perf_counter()
            exp = orc.minhash_ngrams(smp, ngrams, p["seed"], a, b, nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.minhash_ngrams(dl.slice(0, n, smp.null_count), ngrams, p["seed"], da, db).to_host()
            sample_bytes = int(lists.child.offsets[lists.offsets[n]])
            leg["cpu_baseline"] = {"value": round(sample_bytes / cs / 1e9, 5), "unit": "GB/s", "cores": threads, "kind": "port",
                                   "sample": f"first {n} rows ({sample_bytes / 1e6:.1f} MB), {cs:.2f} s"}
            leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] minhash_ngrams: {leg}")
        extra["minhash_ngrams"] = leg
        del dl, keep

    # ------------------------------------------------------------------ jaccard_index of neighbouring rows of C3 (a quarter of its rows)
    if args.minhash_scale > 0:
        torch.cuda.empty_cache()
        w = datagen.config3(0.25 * args.minhash_scale)
        n = w.rows.size - 1
        dc = nvtext.DeviceStringsColumn.from_host(w.rows)
        d1, d2 = dc.slice(0, n, 0), dc.slice(1, n + 1, 0)
        keep = {}
        jwidth = 5

        def jstep():
            keep["o"] = nvtext.jaccard_index(d1, d2, jwidth)

        jsec = timed_steps(jstep, max(3, args.steps // 2), 1, torch)
        jk = kernel_times(jstep, 2, _capi, torch)
        jb = 2 * input_bytes(w.rows)
        leg = {"workload": f"rows r and r+1 of C3 x{0.25 * args.minhash_scale}, width={jwidth}", "rows": n,
               "ms_per_step": round(jsec * 1e3, 3), "input_GBps": round(jb / jsec / 1e9, 2), "mrows_per_s": round(n / jsec / 1e6, 3),
               "kernels_ms": {k: round(v, 3) for k, v in jk.items()}}
        if not args.no_cpu:
            from oracle import pyoracle as orc
            m = min(n, 20000)
            s1, s2 = w.rows.slice(0, m), w.rows.slice(1, m + 1)
            threads = max(1, min(orc.hardware_threads(), 16))
            t0 = time.perf_counter()
            exp = orc.jaccard_index(s1, s2, jwidth, nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.jaccard_index(dc.slice(0, m, 0), dc.slice(1, m + 1, 0), jwidth).to_host()
            leg["cpu_baseline"] = {"value": round(2 * input_bytes(s1) / cs / 1e9, 5), "unit": "GB/s", "cores": threads, "kind": "port",
                                   "sample": f"first {m} row pairs ({2 * s1.chars_bytes / 1e6:.1f} MB), {cs:.2f} s"}
            leg["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] jaccard_index: {leg}")
        extra["jaccard_index"] = leg
        del dc, d1, d2, keep

    # ------------------------------------------------------------------ C5: UTF-8 rows, int64 offsets, 250k vocabulary
    if args.minhash_scale > 0:
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

        tsec = timed_steps(tstep, max(3, args.steps // 2), 1, torch)
        tk = kernel_times(tstep, 2, _capi, torch)
        ib = input_bytes(w.rows)
        leg = {"workload": f"C5 x{args.minhash_scale}", "rows": w.rows.size, "chars_bytes": w.rows.chars_bytes, "offsets": "int64",
               "vocab_entries": w.vocab.size,
               "tokenize": {"ms_per_step": round(tsec * 1e3, 3), "input_GBps": round(ib / tsec / 1e9, 2),
                            "mrows_per_s": round(w.rows.size / tsec / 1e6, 3), "tokens_out": keep["o"].child_size,
                            "kernels_ms": {k: round(v, 3) for k, v in tk.items()}}}
        keep.clear()
        # normalize_characters, the step that precedes the tokenizer in a BERT pipeline (lower-casing, five special tokens)
        special = nvtext.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist(["[CLS]", "[SEP]", "[PAD]", "[MASK]", "[UNK]"]))
        normalizer = nvtext.CharacterNormalizer(True, special)

        def zstep():
            keep["o"] = nvtext.normalize_characters(dc, normalizer)

        zsec = timed_steps(zstep, max(3, args.steps // 2), 1, torch)
        zk = kernel_times(zstep, 2, _capi, torch)
        out_bytes = int(keep["o"].chars.numel())
        # algorithmic bytes of a call: chars + offsets in, chars + offsets (int64 from INT32_MAX bytes on) out; priced against the longest kernel
        zalg = ib + out_bytes + (8 if out_bytes >= 0x7FFFFFFF else 4) * (w.rows.size + 1)
        zdom = max(zk, key=zk.get)
        leg["normalize_characters"] = {"ms_per_step": round(zsec * 1e3, 3), "input_GBps": round(ib / zsec / 1e9, 2),
                                       "mrows_per_s": round(w.rows.size / zsec / 1e6, 3), "chars_out": out_bytes,
                                       "kernels_ms": {k: round(v, 3) for k, v in zk.items()},
                                       "roofline": {"bound": "hbm", "kernel": zdom, "achieved": round(zalg / (zk[zdom] * 1e-3) / 1e9, 1),
                                                    "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                                    "frac": round(zalg / (zk[zdom] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                                    "algorithmic_bytes": zalg, "frac_whole_op": round(zalg / zsec / 1e9 / HBM_PEAK_GBS, 4),
                                                    "traffic": None}}
        if not args.no_cpu:
            from oracle import normalize_py
            from oracle import pyoracle as orc
            threads = max(1, min(orc.hardware_threads(), 16))
            normalize_py.rule_tables()  # built once, outside the timed part (the library's tables are built at create time)
            n = min(w.rows.size, 400000)
            smp = w.rows.slice(0, n)
            t0 = time.perf_counter()
            exp = normalize_py.normalize_characters_native(smp, True, [b"[CLS]", b"[SEP]", b"[PAD]", b"[MASK]", b"[UNK]"], nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.normalize_characters(dc.slice(0, n, smp.null_count), normalizer).to_host()
            leg["normalize_characters"]["cpu_baseline"] = {
                "value": round(input_bytes(smp) / cs / 1e9, 5), "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"first {n} rows ({smp.chars_bytes / 1e6:.0f} MB), {cs:.2f} s"}
            same = np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets)
            leg["normalize_characters"]["parity"] = "PASS" if same else "FAIL"
        keep.clear()
        a, b = datagen.make_params(p["P"], 64, p["param_seed"])
        da = torch.from_numpy(a.view(np.int64)).cuda()
        db = torch.from_numpy(b.view(np.int64)).cuda()

        def m5step():
            keep["o"] = nvtext.minhash64(dc, p["seed"], da, db, p["width"])

        msec = timed_steps(m5step, max(3, args.steps // 2), 1, torch)
        mk = kernel_times(m5step, 2, _capi, torch)
        leg["minhash64"] = {"ms_per_step": round(msec * 1e3, 3), "input_GBps": round(ib / msec / 1e9, 2),
                            "mrows_per_s": round(w.rows.size / msec / 1e6, 3), "kernels_ms": {k: round(v, 3) for k, v in mk.items()}}
        if not args.no_cpu:
            from oracle import pyoracle as orc
            n = min(w.rows.size, 400_000)
            smp = w.rows.slice(0, n)
            threads = max(1, min(orc.hardware_threads(), 16))
            t0 = time.perf_counter()
            exp = orc.wordpiece_tokenize(smp, orc.Vocabulary(w.vocab), p["max_words_per_row"], nthreads=threads)
            cs = time.perf_counter() - t0
            got = nvtext.wordpiece_tokenize(dc.slice(0, n, smp.null_count), dv5, p["max_words_per_row"]).to_host()
            leg["tokenize"]["cpu_baseline"] = {"value": round(input_bytes(smp) / cs / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
                                               "sample": f"first {n} rows ({smp.chars_bytes / 1e6:.0f} MB), {cs:.2f} s"}
            leg["tokenize"]["parity"] = "PASS" if got.equals(exp) else "FAIL"
        log(f"[bench] C5: {leg}")
        extra["utf8_pipeline"] = leg
        del dc, keep

    line = {
        "metric": "input GB/s + Mrows/s, wordpiece_tokenize & minhash, 1 MI355X, % of roofline",
        "value": round(in_b / sec / 1e9, 3), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8/int32", "data": "synthetic",
        "config": {"workload": f"C2 wordpiece_tokenize x{args.scale}", "rows": host.size, "chars_bytes": host.chars_bytes,
                   "vocab_entries": wl.vocab.size, "max_words_per_row": mw, "tokens_out": tokens, "offsets": "int32"},
        "mrows_per_s": round(host.size / sec / 1e6, 3),
        "roofline": roofline, "cpu_baseline": cpu, "parity_vs_oracle": parity,
    }
    line.update(extra)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
