#!/usr/bin/env python3
"""Benchmark of the per-partition suffix sort on one MI355X.

A step = one whole partition sort (all prefix-doubling generations, text resident in HBM at the
start, sa40 resident in HBM at the end) of a synthetic partition. Prints ONE JSON line:
suffixes sorted per second, the roofline of the dominant kernel (the radix pass) from HIP events
recorded on the sort's own stream, and the reference's CPU sort timed on this host beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--n N]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# algorithmic bytes of one radix pass per (key, index) pair: read + write of an 8-byte key and a 5-byte index
RADIX_PASS_BYTES_PER_PAIR = 2 * (8 + 5)


def algorithmic_bytes(n, active):
    """A = A_0 + sum A_g + A_out with 8-byte keys, 5-byte indices, 4-byte ranks and 8-bit digits:
    A_0 = 252 n + 9 m_1, A_g = 263 m_g + 9 m_{g+1}, A_out = 14 n; active[g] = m_g, active[0] = n."""
    m = list(active) + [0]
    per_gen = [252 * n + 9 * m[1]] + [263 * m[g] + 9 * m[g + 1] for g in range(1, len(active))]
    return per_gen, 14 * n


PROFILE_TAG = {2: "c2_256m", 3: "c3_1b", 4: "c4_2b", 5: "c5_512m"}


def measured_traffic(config):
    """HBM bytes moved, from the FETCH_SIZE / WRITE_SIZE counter runs of this same command on the same workload that are
    summarised in profiles/partition_sort_<workload>_pmc_traffic.txt (already scaled by what the counters read for the
    plain copy below; a sort of a given text moves the same bytes in every run). Lines read:
      fetch_bytes_per_pair = X / write_bytes_per_pair = Y     one radix pass, per (key, index) pair
      generation_traffic g=<g> read_GB=<r> write_GB=<w>       every generation
      sort_traffic read_GB=<r> write_GB=<w>                   the whole sort, output included
    Returns (source file, bytes per pair or None, {g: bytes}, job bytes or None); all None where no summary is committed."""
    name = f"partition_sort_{PROFILE_TAG.get(config, 'none')}_pmc_traffic.txt"
    path = os.path.join(ROOT, "profiles", name)
    per_pair, gens, job = {}, {}, None
    try:
        for line in open(path):
            f = line.split()
            for key in ("fetch_bytes_per_pair", "write_bytes_per_pair"):
                if line.startswith(key) and "=" in line:
                    per_pair[key] = float(line.split("=")[1].split()[0])
            if f and f[0] == "generation_traffic":
                kv = dict(x.split("=") for x in f[1:])
                gens[int(kv["g"])] = (float(kv["read_GB"]) + float(kv["write_GB"])) * 1e9
            if f and f[0] == "sort_traffic":
                kv = dict(x.split("=") for x in f[1:])
                job = (float(kv["read_GB"]) + float(kv["write_GB"])) * 1e9
    except OSError:
        return None, None, {}, None
    pp = per_pair["fetch_bytes_per_pair"] + per_pair["write_bytes_per_pair"] if len(per_pair) == 2 else None
    return "profiles/" + name, pp, gens, job


def cpu_baseline(config, sample_n):
    """The reference's CPU suffix sort (test/query.cpp:42-55, compiled from its sources into oracle/_ref) on a
    scaled-down partition of the same construction; falls back to the C restatement where _ref is absent."""
    import oracle_lib
    from cascade_amd import workloads
    T = workloads.generate(config, sample_n)
    ref = oracle_lib.ref()
    t0 = time.perf_counter()
    oracle_lib.build_sa40(T, lib=ref)
    dt = time.perf_counter() - t0
    return {
        "value": sample_n / dt,
        "unit": "suffixes/s",
        "cores": 1,
        "kind": "reference" if ref is not None else "port",
        "sample": f"config C{config} generated at n={sample_n} (same construction, scaled down), "
                  f"std::sort + cmp_suffixes, {dt:.1f} s; host has {os.cpu_count()} logical cores",
    }


def bench_partition_ids(args):
    """The step before the partition sort: partition id of every suffix of the workload's text against p - 1 pivots
    (packed map + partition sizes out). One step = one pass over the text resident in HBM."""
    import numpy as np
    import torch
    import oracle_lib
    from cascade_amd import _native, partition_ids, workloads
    dev = torch.device("cuda:0")
    n = args.n if args.n is not None else workloads.default_n(args.config)
    p, words = args.partitions, 2  # the reference's default pivot width: 2 words = 8 symbols (include/Packed_Prefix.hpp:30-34)
    T = workloads.generate(args.config, n)
    rng = np.random.default_rng(1)
    pivots = oracle_lib.sample_pivots(T[:1 << 22], p, words, rng)
    d_text = torch.from_numpy(T.view(np.int16)).to(dev)
    d_piv = torch.from_numpy(pivots.view(np.int64)).to(dev).reshape(-1, words)
    bits = int(_native.load().csa_partition_id_bits(p))
    for _ in range(args.warmup):
        partition_ids(d_text, d_piv, p, want_ids=False)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    t0 = time.perf_counter()
    ev[0].record()
    for _ in range(args.steps):
        _, packed, sizes = partition_ids(d_text, d_piv, p, want_ids=False)
    ev[1].record()
    torch.cuda.synchronize()
    ms = 1e3 * (time.perf_counter() - t0) / args.steps
    kernel_ms = ev[0].elapsed_time(ev[1]) / args.steps  # includes the zero fill of the outputs made by the wrapper
    alg_bytes = n * (2 + bits / 8.0)  # symbols in, packed entries out
    sample = min(n, 1 << 22)
    want_ids, _ = oracle_lib.partition_ids(T[:sample], pivots, p, words, text_len=sample)
    got = packed.cpu().numpy().view(np.uint64)
    ok = bool(np.array_equal(got[:oracle_lib.packed_words(sample - sample % 64, bits)],
                             oracle_lib.pack_partition_ids(want_ids[:sample - sample % 64], bits)[:oracle_lib.packed_words(sample - sample % 64, bits)]))
    ok = ok and int(sizes.sum().item()) == n
    t1 = time.perf_counter()
    cs = min(n, max(args.cpu_sample, 1) // 4) if args.cpu_sample else 0
    result = {
        "metric": "suffixes assigned to partitions/sec at 1 GPU", "value": n / (ms * 1e-3), "unit": "suffixes/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u64 keys", "data": "synthetic",
        "config": {"workload": workloads.NAMES[args.config], "n": n, "partitions": p, "pivot_words": words,
                   "checked_against_oracle": ok},
        "roofline": {"bound": "hbm", "kernel": "partition_ids_kernel<2>", "achieved": round(alg_bytes / (kernel_ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg_bytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "avg_launch_ms": round(kernel_ms, 4), "algorithmic_bytes_per_launch": round(alg_bytes)},
    }
    if cs:
        t1 = time.perf_counter()
        oracle_lib.partition_ids(T[:cs], pivots, p, words, text_len=cs)
        dt = time.perf_counter() - t1
        result["cpu_baseline"] = {"value": cs / dt, "unit": "suffixes/s", "cores": 1, "kind": "port",
                                  "sample": f"first {cs} symbols of the same text, C restatement of the reference's validator loop, {dt:.1f} s"}
    print(json.dumps(result), flush=True)
    if not ok:
        sys.exit(1)


def _row_result(metric, workload, n, ms, kernel, alg_bytes, extra, steps, warmup, ok):
    return {
        "metric": metric, "value": n / (ms * 1e-3), "unit": "suffixes/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u64 / u32 integers",
        "data": "synthetic", "config": dict({"workload": workload, "n": n, "checked_against_oracle": ok}, **extra),
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(alg_bytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "avg_launch_ms": round(ms, 4), "algorithmic_bytes_per_launch": round(alg_bytes)},
    }


def _timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    torch.cuda.synchronize()
    ev[0].record()
    for _ in range(steps):
        out = fn()
    ev[1].record()
    torch.cuda.synchronize()
    return ev[0].elapsed_time(ev[1]) / steps, out


def bench_next_rows(args):
    """The steps either side of the partition sort that exist for partitions exchanged with the host: slab staging
    (keys + routing tags from the text and the packed partition-id map), message count / offsets / emission, the join,
    and the rank-order scatter. One step = one launch sequence over a synthetic partition of n suffixes in HBM."""
    import ctypes as C
    import numpy as np
    import torch
    import oracle_lib
    import message_cases
    from cascade_amd import PartitionSorter, _native, partition_ids, stage_slab, workloads
    lib = _native.load()
    dev = torch.device("cuda:0")
    n = args.n if args.n is not None else 1 << 28
    p = args.partitions
    rng = np.random.default_rng(2)
    cs = 1 << 20  # the slice every row is checked on against the oracle
    if args.row == "stage_slab":
        T = workloads.generate(args.config, n)
        pivots = oracle_lib.sample_pivots(T[:1 << 22], p, 2, rng)
        d_text = torch.from_numpy(T.view(np.int16)).to(dev)
        ids, packed, _ = partition_ids(d_text, torch.from_numpy(pivots.view(np.int64)).to(dev).reshape(-1, 2), p)
        suf = torch.randperm(n, device=dev)  # a partition's suffixes arrive in no particular text order
        lanes = torch.stack([(suf >> (8 * b)) & 0xFF for b in range(5)], dim=1).to(torch.uint8).reshape(-1).contiguous()
        ms, (keys, beta) = _timed(torch, lambda: stage_slab(d_text, lanes, 1, packed, p, 4, True), args.steps, args.warmup)
        pid = ids[: n].cpu().numpy().view(np.uint16)
        h_suf = suf[:cs].cpu().numpy().astype(np.uint64)
        wk, wb = oracle_lib.stage_slab(T, h_suf, 1, pid, np.zeros(n, dtype=np.uint8), 4, True)
        ok = bool(np.array_equal(keys[:cs].cpu().numpy().view(np.uint64), wk) and np.array_equal(beta[:cs].cpu().numpy().view(np.uint32), wb))
        res = _row_result("suffixes staged/sec at 1 GPU", workloads.NAMES[args.config], n, ms, "stage_slab_kernel<1>",
                          n * (5 + 8 + 8 + 4), {"partitions": p, "key_words": 1, "generation": 0}, args.steps, args.warmup, ok)
    elif args.row == "messages":
        ctx = 1 << 12
        sa, keys, beta, active_sz = message_cases.cohort(n, p, ctx, True, seed=5)
        d_sa, d_keys = torch.from_numpy(sa.view(np.int64)).to(dev), torch.from_numpy(keys.view(np.int64)).to(dev)
        d_beta = torch.from_numpy(beta.view(np.int32)).to(dev)
        d_act = torch.tensor([active_sz], dtype=torch.int64, device=dev)
        d_off = torch.zeros(p + 1, dtype=torch.int32, device=dev)
        d_tgt = torch.empty(5 * 2 * n, dtype=torch.uint8, device=dev)
        d_rank = torch.empty(2 * n, dtype=torch.int32, device=dev)
        st = torch.cuda.current_stream(dev).cuda_stream

        def run():
            d_off.zero_()
            _native.check(lib.csa_count_messages_dev(d_sa.data_ptr(), d_keys.data_ptr(), d_beta.data_ptr(), n, ctx, 1, p, d_off.data_ptr(), st))
            _native.check(lib.csa_message_offsets_dev(d_off.data_ptr(), p + 1, st))
            _native.check(lib.csa_emit_messages_dev(d_sa.data_ptr(), d_keys.data_ptr(), d_beta.data_ptr(), n, ctx, 1, d_act.data_ptr(), p,
                                                    d_tgt.data_ptr(), d_rank.data_ptr(), d_off.data_ptr(), st))
        ms, _ = _timed(torch, run, args.steps, args.warmup)
        end = d_off.cpu().numpy().view(np.uint32)
        total = int(end[p - 1])
        want = oracle_lib.count_messages(sa, keys, beta, ctx, True, p)
        ok = bool(np.array_equal(np.diff(np.concatenate([[0], end[:p]])), want[:p]))
        res = _row_result("cohort members whose messages are emitted/sec at 1 GPU", "random cohort, 20% retired recipients, 30% pill receipts",
                          n, ms, "count_messages_kernel + emit_messages_kernel", 2 * n * 20 + total * 9,
                          {"partitions": p, "messages": total}, args.steps, args.warmup, ok)
    elif args.row == "join":
        suf = torch.sort(torch.randperm(1 << 31, device=dev)[:n]).values if n <= (1 << 27) else torch.arange(n, device=dev) * 3
        msg_c = n // 2
        pick = torch.randperm(n, device=dev)[:msg_c]
        tgt = suf[pick]
        lanes = torch.stack([(tgt >> (8 * b)) & 0xFF for b in range(5)], dim=1).to(torch.uint8).reshape(-1).contiguous()
        rank = torch.randint(0, 1 << 31, (msg_c,), dtype=torch.int32, device=dev)
        primary = torch.randint(0, 1 << 31, (n,), dtype=torch.int32, device=dev)
        keys = torch.full((n,), -1, dtype=torch.int64, device=dev)
        st = torch.cuda.current_stream(dev).cuda_stream
        ms, _ = _timed(torch, lambda: _native.check(lib.csa_join_messages_dev(lanes.data_ptr(), rank.data_ptr(), msg_c, suf.data_ptr(),
                                                                               primary.data_ptr(), keys.data_ptr(), n, st)), args.steps, args.warmup)
        want = (primary[pick].to(torch.int64) << 31) | rank.to(torch.int64)
        ok = bool(torch.equal(keys[pick], want))
        # the variant that sorts the inbox by target first (5 radix passes in a handle's scratch, then the same search)
        sorter = PartitionSorter(msg_c)
        keys.fill_(-1)
        ms_sorted, _ = _timed(torch, lambda: _native.check(lib.csa_join_messages_sorted_dev(
            sorter._h, lanes.data_ptr(), rank.data_ptr(), msg_c, suf.data_ptr(), primary.data_ptr(), keys.data_ptr(), n, st)), args.steps, args.warmup)
        ok = ok and bool(torch.equal(keys[pick], want))
        sorter.close()
        res = _row_result("messages joined/sec at 1 GPU", "messages for half of a suffix-ordered cohort", msg_c, ms_sorted,
                          "unpack + 5 radix passes + join_messages_kernel", msg_c * (9 + 8 + 4 + 8),
                          {"cohort": n, "ms_unsorted_inbox": round(ms, 3)}, args.steps, args.warmup, ok)
    elif args.row == "overlap":
        # Host buffers in and out, as the reference's pipeline hands partitions over: three dispatcher threads, each with its
        # own handle, stream and device buffers (STREAM_C = 3, include/GPU_SACA.hpp:90-91; the dispatcher loop of
        # src/GPU_SACA.cu:1539-1589), take independent texts from pinned host memory, sort them and bring the suffix arrays
        # back into pinned host memory. One thread's upload and download overlap the other threads' sorts.
        import threading
        parts = min(p, 12)
        n = args.n if args.n is not None else 1 << 26
        T = workloads.generate(args.config, parts * n)
        h_text = torch.from_numpy(T.view(np.int16)).reshape(parts, n).pin_memory()
        h_out = torch.empty((parts, 5 * n), dtype=torch.uint8).pin_memory()

        def run(dispatchers):
            errors, in_hbm_ms = [], [0.0] * dispatchers

            def dispatcher(t):
                try:
                    stream = torch.cuda.Stream(device=dev)
                    sorter = PartitionSorter(n)
                    d_text = torch.empty(n, dtype=torch.int16, device=dev)
                    d_out = torch.empty(5 * n + 128, dtype=torch.uint8, device=dev)
                    with torch.cuda.stream(stream):
                        for q in range(t, parts, dispatchers):
                            d_text.copy_(h_text[q], non_blocking=True)
                            st = sorter.sort_ptr(d_text.data_ptr(), n, d_out.data_ptr(), 0, stream.cuda_stream)
                            in_hbm_ms[t] += st["ms_total"]
                            h_out[q].copy_(d_out[:5 * n], non_blocking=True)
                        stream.synchronize()
                    sorter.close()
                except Exception as e:  # reported by the main thread
                    errors.append(e)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            threads = [threading.Thread(target=dispatcher, args=(t,)) for t in range(dispatchers)]
            for th in threads:
                th.start()
            for th in threads:
                th.join()
            torch.cuda.synchronize()
            if errors:
                raise errors[0]
            return (time.perf_counter() - t0) * 1e3, sum(in_hbm_ms)
        for _ in range(args.warmup):
            run(3)
        ms3 = min(run(3)[0] for _ in range(args.steps))
        ms1, in_hbm = run(1)
        sorter = PartitionSorter(n)
        ok = True
        for q in (0, parts // 2, parts - 1):
            ok = ok and sorter.verify(h_text[q].to(dev), h_out[q].to(dev))
        sorter.close()
        pcie_bytes = parts * n * 7
        res = _row_result("suffixes sorted/sec at 1 GPU, host buffers in and out", workloads.NAMES[args.config], parts * n, ms3,
                          "whole job: upload, partition sorts, download on three streams", pcie_bytes,
                          {"texts": parts, "n_each": n, "dispatchers": 3, "ms_one_dispatcher": round(ms1, 2),
                           "ms_in_hbm_sorts_only": round(in_hbm, 2), "pcie_GBps_both_ways": round(pcie_bytes / ms3 / 1e6, 1)},
                          args.steps, args.warmup, ok)
        res["roofline"]["bound"] = "pcie (not an HBM figure: 2 B up + 5 B down per suffix over the host link)"
        res["roofline"]["peak"] = None
        res["roofline"]["frac"] = None
    elif args.row == "pipeline":
        # The same job inside the library: csa_sort_partitions_u16 takes the list of pinned host texts and returns the suffix
        # arrays in pinned host memory; one handle, two device buffer sets, an upload and a download thread beside the
        # calling one (the reference's dispatcher overlap, src/GPU_SACA.cu:1539-1589, without Python in the loop).
        from cascade_amd import sort_partitions
        parts = min(p, 12)
        n = args.n if args.n is not None else 1 << 26
        T = workloads.generate(args.config, parts * n)
        h_text = torch.from_numpy(T.view(np.int16)).reshape(parts, n).pin_memory()
        h_out = torch.empty((parts, 5 * n), dtype=torch.uint8).pin_memory()
        ins = [h_text[q].numpy().view(np.uint16) for q in range(parts)]
        outs = [h_out[q].numpy() for q in range(parts)]

        def run():
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            _, stats = sort_partitions(ins, key_words=1, out=outs)
            return (time.perf_counter() - t0) * 1e3, sum(st["ms_total"] for st in stats)
        for _ in range(args.warmup):
            run()
        ms, in_hbm = min(run() for _ in range(args.steps))
        sorter = PartitionSorter(n)
        ok = True
        for q in (0, parts // 2, parts - 1):
            ok = ok and sorter.verify(h_text[q].to(dev), h_out[q].to(dev))
        sorter.close()
        pcie_bytes = parts * n * 7
        res = _row_result("suffixes sorted/sec at 1 GPU, host buffers in and out", workloads.NAMES[args.config], parts * n, ms,
                          "whole job inside csa_sort_partitions_u16: handle set-up, upload, partition sorts, download on three streams", pcie_bytes,
                          {"texts": parts, "n_each": n, "ms_in_hbm_sorts_only": round(in_hbm, 2),
                           "pcie_GBps_both_ways": round(pcie_bytes / ms / 1e6, 1)}, args.steps, args.warmup, ok)
        res["roofline"]["bound"] = "pcie (not an HBM figure: 2 B up + 5 B down per suffix over the host link)"
        res["roofline"]["peak"] = None
        res["roofline"]["frac"] = None
    elif args.row == "slab_pipeline":
        # The reference's own calling pattern, PCIe included: a text in 16 partitions, every partition a chain of pinned
        # host slabs of CHUNK_CAP = 2^21 suffixes (include/GPU_SACA.hpp:99), three dispatcher threads with a buffer set
        # and a stream each calling the three members concurrently (src/GPU_SACA.cu:1539-1589) through the C++ mirror
        # (tests/cpp/slab_pipeline.cpp, built by cascade_amd/build.py). The program times the dispatch phases (all
        # partitions of a generation through their step, uploads and downloads included; host staging between the phases
        # is not timed) and checks the finished suffix array against the resident sort; here the oracle's O(n) verifier
        # judges it too. Value: suffixes through generation 0 per second, link traffic included.
        import subprocess
        import tempfile
        exe = os.path.join(ROOT, "tests", "cpp", "slab_pipeline")
        n = args.n if args.n is not None else 1 << 26
        parts, threads = 16, 3
        T = workloads.generate(args.config, n)
        with tempfile.TemporaryDirectory(dir="/tmp") as tmp:
            text, out = os.path.join(tmp, "text.u16"), os.path.join(tmp, "sa40")
            T.tofile(text)
            infos = []
            for th in (threads, 1):
                run = subprocess.run([exe, "0", str(parts), str(args.key_words), str(1 << 21), "7", "1", out, str(th), text],
                                     capture_output=True, text=True)
                if run.returncode != 0 or not run.stdout.startswith("OK "):
                    print(run.stdout, run.stderr, file=sys.stderr)
                    sys.exit(1)
                infos.append(dict(kv.split("=") for kv in run.stdout.split() if "=" in kv and not kv.startswith("(")))
            ok = bool(oracle_lib.is_correct_sa40(np.fromfile(out, dtype=np.uint8), T))
        info, one = infos
        ms0, b0 = float(info["gen0_ms"]), int(info["gen0_link_bytes"])
        res = _row_result("suffixes through a generation-0 partition step/sec at 1 GPU, pinned host slabs in and out",
                          workloads.NAMES[args.config], n, ms0,
                          "sort_and_init_rank_and_filter on host slabs, three dispatcher threads (csa_sort_init_slabs)", b0,
                          {"partitions": parts, "chunk_cap": 1 << 21, "dispatchers": threads, "key_words": args.key_words,
                           "generations": int(info["generations"]), "largest_partition": int(info["max_part"]),
                           "device_bytes_three_buffer_sets": int(info["device_bytes"]),
                           "gen0_link_GBps": round(b0 / ms0 / 1e6, 1),
                           "all_generations_ms": round(float(info["dispatch_ms"]), 2),
                           "all_generations_link_GBps": round(int(info["link_bytes"]) / float(info["dispatch_ms"]) / 1e6, 1),
                           "scatter_ms": round(float(info["scatter_ms"]), 2),
                           "scatter_link_GBps": round(int(info["scatter_link_bytes"]) / float(info["scatter_ms"]) / 1e6, 1),
                           "gen0_ms_one_dispatcher": round(float(one["gen0_ms"]), 2),
                           "all_generations_ms_one_dispatcher": round(float(one["dispatch_ms"]), 2),
                           "scatter_ms_one_dispatcher": round(float(one["scatter_ms"]), 2)}, 1, 0, ok)
        res["roofline"]["bound"] = "pcie (not an HBM figure: bytes of the slabs' columns over the host link, both directions)"
        res["roofline"]["peak"] = None
        res["roofline"]["frac"] = None
    elif args.row in ("step_init", "step_rerank"):
        # one partition step under the exchange scheme: everything the reference does between the upload of a partition's
        # slabs and their download (src/GPU_SACA.cu:1112-1331 / 1715-1995). The synthetic partition: n suffixes of the
        # workload's text in random order, p partitions by sampled pivots.
        import ctypes as C
        StepResult = _native.CsaStepResult
        T = workloads.generate(args.config, n)
        pivots = oracle_lib.sample_pivots(T[:1 << 22], p, 2, rng)
        d_text = torch.from_numpy(T.view(np.int16)).to(dev)
        _, packed, _ = partition_ids(d_text, torch.from_numpy(pivots.view(np.int64)).to(dev).reshape(-1, 2), p, want_ids=False)
        suf = torch.randperm(n, device=dev)
        lanes = torch.stack([(suf >> (8 * b)) & 0xFF for b in range(5)], dim=1).to(torch.uint8).reshape(-1).contiguous()
        kw = args.key_words
        keys, beta = stage_slab(d_text, lanes, kw, packed, p, 4 * kw, True)
        sorter = PartitionSorter(n, key_words=kw, for_steps=True)  # the steps' own floor plan: csa_step_bytes_per_suffix
        rank_out = torch.empty(n, dtype=torch.int32, device=dev)
        suf_out = torch.empty(5 * n, dtype=torch.uint8, device=dev)
        mt, mr = torch.empty(5 * 2 * n, dtype=torch.uint8, device=dev), torch.empty(2 * n, dtype=torch.int32, device=dev)
        off = torch.zeros(p + 1, dtype=torch.int32, device=dev)
        res = StepResult()
        st = torch.cuda.current_stream(dev).cuda_stream
        init = lambda: _native.check(lib.csa_sort_init_dev(sorter._h, keys.data_ptr(), kw, lanes.data_ptr(), beta.data_ptr(), n, p,
                                                            rank_out.data_ptr(), suf_out.data_ptr(), mt.data_ptr(), mr.data_ptr(),
                                                            off.data_ptr(), st, C.byref(res)))
        if args.row == "step_init":
            ms, _ = _timed(torch, init, args.steps, args.warmup)
            # the whole text as one partition: its step-0 ranks are those of the resident sort's generation 0, so as many
            # suffixes survive as the partition sort reports active after generation 0
            check = PartitionSorter(n, key_words=kw)
            check.sort(d_text)
            resident = check.last_stats["active"][1] if check.last_stats["generations"] > 1 else 0
            # with several partitions the forward tag (the partition of the suffix one context further) refines the order
            ok = int(res.active) == resident if p == 1 else int(res.active) <= resident
            check.close()
            alg = n * (8 * kw + 5 + 4 + 2 * 2 * 24 + 8 * kw * 2 * 24 + 41 + 41 + 9)  # unpack, two tag passes, eight passes per key word, rank, split, narrow (src/GPU_SACA.cu:1157-1331)
            res_row = _row_result("suffixes through a generation-0 partition step/sec at 1 GPU", workloads.NAMES[args.config], n, ms,
                                  "csa_sort_init_dev (the reference: %d radix passes + glue)" % (2 + 8 * kw), alg,
                                  {"partitions": p, "key_words": kw, "active_after": int(res.active), "messages": int(res.messages)}, args.steps, args.warmup, ok)
        else:
            init()
            a = int(res.active)
            total = int(res.messages)
            # the next generation of the survivors, fed with their own outbox as the inbox of a one-partition run would be
            beta1 = torch.zeros(a, dtype=torch.int32, device=dev)
            rk_in, sf_in = rank_out[:a].clone(), suf_out[:5 * a].clone()
            in_t, in_r = mt[:5 * total].clone(), mr[:total].clone()
            rer = lambda: _native.check(lib.csa_sort_rerank_dev(sorter._h, rk_in.data_ptr(), sf_in.data_ptr(), beta1.data_ptr(), a,
                                                                 in_t.data_ptr(), in_r.data_ptr(), total, 8, p, rank_out.data_ptr(),
                                                                 suf_out.data_ptr(), mt.data_ptr(), mr.data_ptr(), off.data_ptr(), st,
                                                                 C.byref(res)))
            ms, _ = _timed(torch, rer, args.steps, args.warmup)
            ok = int(res.active) <= a
            alg = a * (5 * 2 * 24 + 29 + 8 * 2 * 24 + 90 + 9)  # the reference's plan: suffix-order sort, join, key sort, re-rank, narrow (src/GPU_SACA.cu:1769-1995)
            res_row = _row_result("active suffixes through a later partition step/sec at 1 GPU", workloads.NAMES[args.config], a, ms,
                                  "csa_sort_rerank_dev (the reference: 13 radix passes + join + glue; here 8 passes and a hash join)", alg,
                                  {"partitions": p, "inbox": total, "active_after": int(res.active)}, args.steps, args.warmup, ok)
        sorter.close()
        res = res_row
    else:  # scatter
        rank = torch.randperm(n, device=dev).to(torch.int32)
        lanes = torch.randint(0, 256, (5 * n,), dtype=torch.uint8, device=dev)
        out = torch.empty(5 * n + 128, dtype=torch.uint8, device=dev)
        h_rank = rank[:cs].cpu().numpy().view(np.uint32).astype(np.int64)

        def run(capacity):  # a handle smaller than the partition scatters directly, one that holds it buckets by windows first
            s = PartitionSorter(capacity)
            out.zero_()
            ms, _ = _timed(torch, lambda: s.scatter_to_rank_order(lanes, rank, out=out), args.steps, args.warmup)
            got = out[:5 * n].view(n, 5)[torch.from_numpy(h_rank).to(dev)].cpu().numpy()
            s.close()
            return ms, bool(np.array_equal(got, lanes[:5 * cs].view(cs, 5).cpu().numpy()))
        ms_direct, ok_direct = run(16)
        ms, ok = run(n)
        res = _row_result("suffixes scattered to rank order/sec at 1 GPU", "random permutation of ranks", n, ms,
                          "scatter_window_keys_kernel + one radix pass + scatter_window_lanes_kernel", n * 14,
                          {"ms_direct_scatter": round(ms_direct, 3)}, args.steps, args.warmup, ok and ok_direct)
    print(json.dumps(res), flush=True)
    if not res["config"]["checked_against_oracle"]:
        sys.exit(1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", type=int, default=3, help="workload 1..5 (3 = the 1B-token headline)")
    ap.add_argument("--n", type=int, default=None, help="override the partition size (scaled construction)")
    ap.add_argument("--key-words", type=int, default=1)
    ap.add_argument("--cpu-sample", type=int, default=None,
                    help="symbols of the CPU baseline sample (0 = skip); default: what the reference's comparison sort finishes "
                         "in 10 to 30 s on the workload (2^26 on the token corpora, less where long repeats make every comparison deep)")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--no-oracle-verify", action="store_true",
                    help="check the headline output with the device verifier only (the default also runs the CPU oracle's O(n) "
                         "verifier on it, about 23 bytes of host memory per suffix)")
    ap.add_argument("--generations", action="store_true", help="print the per-generation table to stderr")
    ap.add_argument("--row", default="sort", choices=["sort", "partition_ids", "stage_slab", "messages", "join", "scatter", "step_init", "step_rerank", "overlap", "pipeline", "slab_pipeline"],
                    help="which step to measure: the partition sort (the headline, default) or one of the steps around it")
    ap.add_argument("--shared-device", action="store_true",
                    help="measure the headline with the default tile order (safe next to other launches) only")
    ap.add_argument("--no-order-comparison", action="store_true",
                    help="do not also time the default tile order after the headline (counter runs want one sort per run)")
    ap.add_argument("--partitions", type=int, default=256, help="partitions of --row partition_ids")
    args = ap.parse_args()

    if args.cpu_sample is None:
        args.cpu_sample = {1: 1 << 20, 2: 1 << 26, 3: 1 << 26, 4: 1 << 23, 5: 1 << 18}.get(args.config, 1 << 20)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU: a partition is sorted inside one device's HBM and nothing here "
              "shards it; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from cascade_amd import PartitionSorter, _native, workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.row == "partition_ids":
        return bench_partition_ids(args)
    if args.row != "sort":
        return bench_next_rows(args)
    dev = torch.device("cuda:0")
    n = args.n if args.n is not None else workloads.default_n(args.config)

    t0 = time.perf_counter()
    T = workloads.generate(args.config, n)
    t_gen = time.perf_counter() - t0
    d_text = torch.from_numpy(T.view(np.int16)).to(dev)
    oracle_check = not (args.no_verify or args.no_oracle_verify)
    if not oracle_check:
        del T
    out = torch.empty(5 * n + 128, dtype=torch.uint8, device=dev)
    # bench.py is the only user of the GPU while it runs, which is what csa_set_device_exclusive asks the caller to
    # declare; the time of the default tile order (safe next to other launches) is measured beside it
    sorter = PartitionSorter(n, key_words=args.key_words, device_exclusive=not args.shared_device)
    print(f"[bench] C{args.config} n={n} generated in {t_gen:.1f}s; scratch {sorter.bytes_per_suffix() * n / 2**30:.1f} GiB",
          file=sys.stderr, flush=True)

    # One plain copy of known size (1 GiB read, 1 GiB written), outside the timed region: a counter run of this same
    # command scales FETCH_SIZE / WRITE_SIZE by what they read for it.
    cal = torch.empty(1 << 28, dtype=torch.int32, device=dev)
    cal.fill_(1)
    cal2 = torch.empty_like(cal)
    cal2.copy_(cal)
    torch.cuda.synchronize()
    del cal, cal2
    torch.cuda.empty_cache()

    for _ in range(args.warmup):
        sorter.sort(d_text, out=out)
    torch.cuda.synchronize()

    radix_ms = radix_pairs = radix_launches = 0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sorter.sort(d_text, out=out, flags=_native.CSA_FLAG_KERNEL_TIMING)
        st = sorter.last_stats
        radix_ms += st["radix_ms"]
        radix_pairs += st["radix_pairs"]
        radix_launches += st["radix_launches"]
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    st = sorter.last_stats
    verified = None
    verified_by = []
    if oracle_check:
        # the CPU oracle's O(n) verifier (the reference's rule, test/end-to-end.cpp:46-80) on the headline output:
        # outside the timed region, and the only use of the oracle besides the CPU baseline below
        import oracle_lib
        t1 = time.perf_counter()
        verified = bool(oracle_lib.is_correct_sa40(out[:5 * n].cpu().numpy(), T))
        print(f"[bench] oracle verifier: {verified} in {time.perf_counter() - t1:.1f} s", file=sys.stderr, flush=True)
        verified_by.append("oracle orc_is_correct_sa40_u16 (host, O(n): permutation + every adjacent pair in order)")
        del T
        if not verified:
            print("[bench] the oracle's verifier REJECTED the suffix array", file=sys.stderr)
    if not args.no_verify:
        ok_dev = sorter.verify(d_text, out)
        verified = ok_dev if verified is None else (verified and ok_dev)
        verified_by.append("csa_verify_sa40_dev (device, same rule)")
        if not ok_dev:
            print("[bench] the device verifier REJECTED the suffix array", file=sys.stderr)

    ms_by_arrival = ms_per_step
    if not args.shared_device and not args.no_order_comparison:
        sorter.set_device_exclusive(False)
        sorter.sort(d_text, out=out)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            sorter.sort(d_text, out=out)
        torch.cuda.synchronize()
        ms_by_arrival = 1e3 * (time.perf_counter() - t0) / args.steps
        sorter.set_device_exclusive(True)
        if verified and not sorter.verify(d_text, out):
            verified = False
            print("[bench] the device verifier REJECTED the suffix array of the default tile order", file=sys.stderr)

    per_gen, a_out = algorithmic_bytes(n, st["active"])
    a_total = sum(per_gen) + a_out
    full_workload = args.n is None and args.key_words == 1
    traffic_source, per_pair, moved_gen, moved_job = measured_traffic(args.config) if full_workload else (None, None, {}, None)
    # The per-generation bytes of the profile belong to this run only if the profile cut the sort into the same
    # generations; a share of the peak above 1 is no measurement either. In both cases the per-generation figures of
    # the profile are dropped (not printed), and the line says why.
    moved_gen_dropped = None
    ran = [g for g in range(st["generations"]) if not 1 <= g < st["first_sort_generations"]]  # (the others have no launches)
    if moved_gen and sorted(moved_gen) != ran:
        moved_gen_dropped = f"the profile holds generations {sorted(moved_gen)}, the run had {ran}"
    elif any(st["ms"][g] > 0 and moved_gen[g] / (st["ms"][g] * 1e-3) / 1e9 > HBM_PEAK_GBS for g in moved_gen):
        moved_gen_dropped = "a generation's bytes over this run's time exceed the HBM peak"
    if moved_gen_dropped:
        print(f"[bench] per-generation traffic of {traffic_source} not used: {moved_gen_dropped}", file=sys.stderr)
        moved_gen = {}
    gen_table = []
    for g in range(st["generations"]):
        gbs = per_gen[g] / (st["ms"][g] * 1e-3) / 1e9 if st["ms"][g] > 0 else 0.0
        # alg_over_peak: the yardstick's bytes (8 radix passes over every active suffix in every generation) over the time,
        # as a share of the HBM peak. It is NOT a roofline fraction: generations whose groups are sorted inside LDS move far
        # fewer bytes than the yardstick charges and come out above 1. frac_moved is the roofline fraction: bytes the
        # counters saw this generation move (from the committed profile of this workload) over this run's time.
        row = {"g": g, "active": st["active"][g], "groups": st["groups"][g], "big": st["big"][g], "presorted": st["presorted"][g], "passes": st["passes"][g],
               "rank_update": st["rank_update"][g], "small_only": st["small_only"][g], "dense": st["dense"][g], "ms": round(st["ms"][g], 3),
               "alg_GBps": round(gbs, 1), "alg_over_peak": round(gbs / HBM_PEAK_GBS, 4)}
        if 1 <= g < st["first_sort_generations"]:
            row["covered_by_first_sort"] = True  # its list is counted on the sorted keys; no time or passes of its own
        if g in moved_gen and st["ms"][g] > 0:
            mv = moved_gen[g] / (st["ms"][g] * 1e-3) / 1e9
            row["moved_GBps"] = round(mv, 1)
            row["frac_moved"] = round(mv / HBM_PEAK_GBS, 4)
        gen_table.append(row)
    if args.generations:
        for row in gen_table:
            print("[gen]", json.dumps(row), file=sys.stderr)
        print(f"[gen] output ms={st['ms_output']:.3f} device ms_total={st['ms_total']:.3f}", file=sys.stderr)

    # dominant kernel: the one-sweep radix pass, timed per launch with HIP events on the sort's stream
    avg_launch_ms = radix_ms / radix_launches if radix_launches else 0.0
    achieved = (RADIX_PASS_BYTES_PER_PAIR * radix_pairs / (radix_ms * 1e-3) / 1e9) if radix_ms > 0 else 0.0
    pairs_per_launch = radix_pairs / radix_launches if radix_launches else 0
    roofline = {
        "bound": "hbm", "kernel": "onesweep_kernel (one radix pass over (key, index) pairs)",
        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": round(per_pair * pairs_per_launch) if per_pair is not None else None,
        "traffic_source": traffic_source,
        "frac_moved": round(per_pair * radix_pairs / (radix_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if per_pair is not None and radix_ms > 0 else None,
        "algorithmic_bytes_per_launch": round(RADIX_PASS_BYTES_PER_PAIR * pairs_per_launch),
        "launches_per_step": radix_launches / args.steps, "avg_launch_ms": round(avg_launch_ms, 4),
        "pairs_per_launch": pairs_per_launch,
        "share_of_step": round(radix_ms / args.steps / ms_per_step, 3),
    }

    result = {
        "metric": "suffixes sorted/sec per partition at 1 GPU",
        "value": n / (ms_per_step * 1e-3),
        "unit": "suffixes/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64 keys / u32 ranks", "data": "synthetic",
        "config": {"workload": workloads.NAMES[args.config], "n": n, "key_words": args.key_words,
                   "generations": st["generations"], "key_symbols": st["key_symbols"],
                   "first_sort_generations": st["first_sort_generations"], "bit_exact_verified": verified, "verified_by": verified_by,
                   "tile_order": "by arrival" if args.shared_device else "XCD-chunked (device declared exclusive)",
                   "ms_per_step_tiles_by_arrival": round(ms_by_arrival, 3)},
        "roofline": roofline,
        "job_alg_over_peak": round(a_total / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "job_algorithmic_bytes_per_suffix": round(a_total / n, 1),
        "job_frac_moved": round(moved_job / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if moved_job else None,
        "job_moved_bytes_per_suffix": round(moved_job / n, 1) if moved_job else None,
        "generations": gen_table,
    }
    if st["first_sort_generations"] > 1:
        # the yardstick charges the reference's step list, generation by generation; the first sort took keys of
        # key_symbols packed symbols and stands for several of those generations at the price of one, so the ratio to the
        # peak says by how much that list is undercut, not how busy HBM was (that is job_frac_moved)
        result["job_alg_note"] = (f"the first sort (keys of {st['key_symbols']} packed symbols) stands for generations 0-"
                                  f"{st['first_sort_generations'] - 1} of the reference's list, whose bytes the yardstick still counts")
    if moved_gen_dropped:
        result["generation_traffic_dropped"] = moved_gen_dropped
    if args.cpu_sample > 0:
        result["cpu_baseline"] = cpu_baseline(args.config, min(args.cpu_sample, n))
    print(json.dumps(result), flush=True)
    sorter.close()
    if verified is False:
        sys.exit(1)


if __name__ == "__main__":
    main()
