#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of paged decode attention (split kernel + split reduce) over one batch of the
headline decode workload: batch 32, 32 query / 8 KV heads, head_dim 128, bf16, block size 16,
context lengths uniform in [512, 4096], block tables from a seeded permutation of a 16384-block
pool.  Inputs are resident in HBM before the timed region; three independent KV pools are rotated so
consecutive steps cannot be served from the 256 MB Infinity Cache.

Prints one JSON line: whole-job GB/s of algorithmic bytes over exactly --steps steps after --warmup
steps, the roofline of the dominant kernel and the CPU oracle timed on a bounded sample.  The same line
carries one object per further benchmark configuration ("prefill", "chunked_prefill", "fp8_decode",
"dense_f32"), "latent" (MLA attention over paged caches), "head_dim_64" (the matrix-core kernels at the
reference's other head dimensions, and the headline decode at eight and sixteen query heads per KV head), "mfma_ceiling" (what the matrix cores sustain on a register-only loop
of the prefill kernels' product, on zeros and on the benchmark's kind of data) and "hbm_ceiling" (what a kernel that
only reads gets out of HBM at the decode workloads' sizes).

How every kernel figure is taken, whatever --steps says: at least 300 ms of warm-up launches, then at
least 30 samples, each a pair of HIP events on the launch stream around a small group of back-to-back
launches; mean, median and the quartiles are reported (the reference times its kernels the same way:
singe-testing/src/bench.rs:11-13, singe/src/backend/cuda/kernel_tuning/measure/mod.rs:34-53).
`--only SECTION` runs one section alone and prints it, for rocprofv3 runs of its kernel.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
POOLS = 3
DECODE_BYTES = 305_940_888  # algorithmic bytes of the headline decode workload (its lengths sum to 74 560 keys)
WARMUP_SECONDS = 0.3
MIN_SAMPLES = 30

# HBM bytes per launch from rocprofv3 --pmc runs of `bench.py --only SECTION` (FETCH_SIZE, then WRITE_SIZE, each in
# a run of its own).  Both counters were calibrated in the same runs on torch's f32 -> bf16 copy of 2^28 elements
# (1 GiB read, 512 MiB written): FETCH_SIZE counts units of 2 KiB, WRITE_SIZE units of 1 KiB.  The figures belong
# to the kernel, workload and tuning named, are not re-measured by the run that prints them, and are listed with the
# profile summary they come from.
FETCH_UNIT_BYTES, WRITE_UNIT_BYTES = 2048, 1024
COUNTER_TRAFFIC = {
    "decode": {"kernel": "singe_paged_decode_bf16_d128_g1_b16", "FETCH_SIZE": 150137, "WRITE_SIZE": 4238,
               "source": "profiles/hbm_traffic_counters.md"},
    "prefill": {"kernel": "singe_fmha_prefill_pair_bf16_d128_causal", "FETCH_SIZE": 300835, "WRITE_SIZE": 131072,
                "source": "profiles/hbm_traffic_counters.md"},
    "chunked_prefill": {"kernel": "singe_paged_attention_pair_bf16_d128_i32", "FETCH_SIZE": 182670, "WRITE_SIZE": 66560,
                        "source": "profiles/hbm_traffic_counters.md"},
    "fp8_decode": {"kernel": "singe_paged_decode_f8kv_wide_d128_b16", "FETCH_SIZE": 2118890, "WRITE_SIZE": 8256,
                   "source": "profiles/hbm_traffic_counters.md"},
    "latent_decode": {"kernel": "singe_paged_mla_attention_bf16_l512_p64", "FETCH_SIZE": 608457, "WRITE_SIZE": 32896,
                      "source": "profiles/hbm_traffic_counters.md"},
    "latent_chunked_prefill": {"kernel": "singe_paged_mla_attention_bf16_l512_p64", "FETCH_SIZE": 867638,
                               "WRITE_SIZE": 526336, "source": "profiles/hbm_traffic_counters.md"},
    "cache_append": {"kernel": "singe_rotary_cache_write_chunks_bf16", "FETCH_SIZE": 44244, "WRITE_SIZE": 81920,
                     "source": "profiles/hbm_traffic_counters.md"},
}


def traffic(key):
    """(bytes per launch, where the counters were read) or (None, None) when no counter run covers the kernel."""
    entry = COUNTER_TRAFFIC.get(key)
    if entry is None:
        return None, None
    return entry["FETCH_SIZE"] * FETCH_UNIT_BYTES + entry["WRITE_SIZE"] * WRITE_UNIT_BYTES, entry["source"]


SECTIONS = ("decode", "decode_op", "prefill", "chunked_prefill", "fp8_decode", "dense_f32", "latent", "cache_append", "head_dim_64",
            "mfma_ceiling", "hbm_ceiling")


def parse():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=300)
    parser.add_argument("--warmup", type=int, default=30)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-extras", action="store_true", help="the headline decode section only")
    parser.add_argument("--workers", type=int, default=0, help="decode tuning override (0 = built-in choice)")
    parser.add_argument("--only", choices=SECTIONS, default=None,
                        help="run one section alone and print it (for profiler and counter runs of its kernel)")
    parser.add_argument("--few", action="store_true", help="with --only: a handful of launches, no warm-up (counter runs)")
    parser.add_argument("--full", action="store_true", help="print every section's detail as the one line (about 19 KB)")
    parser.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_detail.json"),
                        help="file that receives every section's detail beside the compact line ('' for none)")
    return parser.parse_args()


FEW = False


def measure(launch, group):
    """Per-launch time of `launch` in milliseconds: warm-up for WARMUP_SECONDS, then MIN_SAMPLES samples, each a pair of
    HIP events on torch's current stream (the stream every launch here goes to) around `group` back-to-back launches."""
    import torch

    samples = 3 if FEW else MIN_SAMPLES
    if not FEW:
        started = time.perf_counter()
        while time.perf_counter() - started < WARMUP_SECONDS:
            for _ in range(group):
                launch()
            torch.cuda.synchronize()
    begin = [torch.cuda.Event(enable_timing=True) for _ in range(samples)]
    finish = [torch.cuda.Event(enable_timing=True) for _ in range(samples)]
    for j in range(samples):
        begin[j].record()
        for _ in range(group):
            launch()
        finish[j].record()
    torch.cuda.synchronize()
    ms = sorted(b.elapsed_time(f) / group for b, f in zip(begin, finish))
    quartile = lambda q: ms[min(len(ms) - 1, int(round(q * (len(ms) - 1))))]
    return {"mean_ms": sum(ms) / len(ms), "median_ms": quartile(0.5), "p25_ms": quartile(0.25), "p75_ms": quartile(0.75),
            "iqr_ms": quartile(0.75) - quartile(0.25), "min_ms": ms[0], "samples": len(ms), "launches_per_sample": group}


def timing_fields(stats):
    return {"kernel_avg_us": stats["mean_ms"] * 1e3, "kernel_median_us": stats["median_ms"] * 1e3,
            "kernel_p25_us": stats["p25_ms"] * 1e3, "kernel_p75_us": stats["p75_ms"] * 1e3,
            "kernel_iqr_us": stats["iqr_ms"] * 1e3, "samples": stats["samples"],
            "launches_per_sample": stats["launches_per_sample"]}


def host_description():
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"cpu_model": model, "nproc": os.cpu_count() or 1, "usable_cores": usable}


def cpu_threads():
    return min(host_description()["usable_cores"], 16)


# ---- CPU baselines: the oracle (a C restatement of the reference's CPU functions) on a bounded sample -------------

def decode_cpu_baseline(work, budget_s=12.0, fp8=False):
    """The reference's CPU decode as written (one thread, weights re-evaluated per output dimension,
    singe-kernel/src/cpu/attention.rs:1172-1246), restated in the oracle, timed on as many leading sequences of the
    same workload as fit the budget; then the same sequences with the head rows over the host's cores and the
    weight of a (row, key) pair evaluated once, the way the reference's dense op spreads rows over threads
    (singe/src/backend/cpu/normalization/attention.rs:219-223); bit-identical outputs.  With an fp8 cache the
    oracle reads the cache dequantised to bf16_rne(value(code) * scale), one KV head of it."""
    import numpy as np
    import torch

    import oracle

    done_bytes, elapsed, used, parallel = 0, 0.0, 0, 0.0
    cores = cpu_threads()
    kv_heads = 1 if fp8 else work.kv_heads
    heads = work.heads // work.kv_heads * kv_heads
    for b in range(work.batch):
        length = int(work.seq_lens[b])
        n = (length + work.block_size - 1) // work.block_size
        index = torch.from_numpy(work.block_table[b, :n].astype(np.int64)).to(work.key_cache.device)
        if fp8:
            widen = lambda codes, scales: (codes[index][:, :, :1].view(torch.float8_e4m3fn).float()
                                           * scales[index][:, None, :1, None]).to(torch.bfloat16).float().cpu().numpy()
            kc, vc = widen(work.key_cache, work.key_scales), widen(work.value_cache, work.value_scales)
        else:
            kc, vc = work.key_cache[index].float().cpu().numpy(), work.value_cache[index].float().cpu().numpy()
        q = work.query[b:b + 1, :heads].float().cpu().numpy()
        table = np.arange(n, dtype=np.uint32).reshape(1, -1)
        shape = dict(batch=1, heads=heads, kv_heads=kv_heads, head_dim=work.head_dim, block_size=work.block_size,
                     block_table_batch_stride=max(n, 1), scale=work.scale)
        start = time.perf_counter()
        oracle.paged_kv_decode_attention_f32(q, kc, vc, [length], table, literal=True, **shape)
        elapsed += time.perf_counter() - start
        start = time.perf_counter()
        oracle.paged_kv_decode_attention_f32(q, kc, vc, [length], table, threads=cores, **shape)
        parallel += time.perf_counter() - start
        element = 1 if fp8 else 2
        done_bytes += length * 2 * kv_heads * work.head_dim * element + 2 * heads * work.head_dim * 2
        if fp8:
            done_bytes += 2 * n * kv_heads * 4
        used += 1
        if elapsed > budget_s:
            break
    what = f"first {used} of {work.batch} sequences" + (", one of its 8 KV heads (8 query heads)" if fp8 else "")
    return {
        "value": done_bytes / elapsed / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{what} of the same workload, reference loop shape (single thread, {elapsed:.1f} s); bytes counted "
                  f"as for the GPU figure",
        "row_parallel": {"value": done_bytes / parallel / 1e9, "unit": "GB/s", "cores": cores,
                         "sample": f"the same sequences, head rows over {cores} threads, weights hoisted ({parallel:.2f} s)"},
        "host": host_description(),
    }


def prefill_cpu_baseline(q, k, v, scale):
    """fmha_prefill_lse_f32 (singe-kernel/src/cpu/attention.rs:1758-1833) on one (batch, head) of the workload: rows
    1792..2303 as written (one thread, the weight re-evaluated per output dimension), extrapolated to the whole
    problem by the exact count of (query, key) pairs; then every row of two heads over the host's cores with the
    weights hoisted."""
    import numpy as np

    import oracle

    batch, seq, heads, dim = q.shape
    one = lambda t, h: np.ascontiguousarray(t[0, :, h:h + 1, :].float().cpu().numpy()[None])
    first, count = 1792, 512
    start = time.perf_counter()
    oracle.fmha_prefill_lse_f32_literal(one(q, 0), one(k, 0), one(v, 0), batch=1, query_len=seq, key_len=seq, heads=1,
                                        kv_heads=1, head_dim=dim, scale=scale, causal=True, row_first=first, row_count=count)
    elapsed = time.perf_counter() - start
    pairs = sum(r + 1 for r in range(first, first + count))
    cores = cpu_threads()
    two = lambda t: np.ascontiguousarray(t[0, :, 0:2, :].float().cpu().numpy()[None])
    start = time.perf_counter()
    oracle.fmha_prefill_lse_f32(two(q), two(k), two(v), batch=1, query_len=seq, key_len=seq, heads=2, kv_heads=2,
                                head_dim=dim, scale=scale, causal=True, threads=cores)
    parallel = time.perf_counter() - start
    parallel_pairs = 2 * seq * (seq + 1) // 2
    return {
        "value": 4 * dim * pairs / elapsed / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": f"rows {first}..{first + count - 1} of one (batch, head): {pairs} of the problem's "
                  f"{batch * heads * seq * (seq + 1) // 2} (query, key) pairs, reference loop shape (single thread, {elapsed:.1f} s)",
        "row_parallel": {"value": 4 * dim * parallel_pairs / parallel / 1e12, "unit": "TFLOP/s", "cores": cores,
                         "sample": f"all rows of two heads of one batch ({parallel_pairs} pairs), rows over {cores} threads, "
                                   f"weights hoisted ({parallel:.2f} s)"},
        "host": host_description(),
    }


def chunked_prefill_cpu_baseline(work):
    """attend_paged (singe/src/backend/cpu/normalization/attention.rs:424-538, serial in the reference) on the last 64
    new tokens of the first sequence over its whole prefix, one KV head (8 query heads): single thread, then the same
    rows over the host's cores."""
    import numpy as np
    import torch

    import oracle

    group = work.heads // work.kv_heads
    first, last = int(work.page_offsets[0]), int(work.page_offsets[1])
    index = torch.from_numpy(np.asarray(work.pages[first:last], dtype=np.int64)).to(work.key_cache.device)
    kc = work.key_cache[index][:, :, :1].float().cpu().numpy()
    vc = work.value_cache[index][:, :, :1].float().cpu().numpy()
    tokens = 64
    end = int(work.query_offsets[1])
    q = work.query[end - tokens:end, :group].float().cpu().numpy()
    keys = int(work.prefix[0]) + work.new_tokens
    paging = dict(query_offsets=[0, tokens], page_offsets=[0, last - first], pages=list(range(last - first)),
                  last_page_lengths=[int(work.last_page_lengths[0])])
    pairs = group * sum(keys - tokens + i + 1 for i in range(tokens))
    results = []
    for threads in (1, cpu_threads()):
        start = time.perf_counter()
        status, _, _ = oracle.paged_attention_f32(q, kc, vc, paging["query_offsets"], paging["page_offsets"], paging["pages"],
                                                  paging["last_page_lengths"], causal=True, threads=threads)
        results.append(time.perf_counter() - start)
        assert status == 0
    total_pairs = work.algorithmic_flops() // (4 * work.head_dim)
    return {
        "value": 4 * work.head_dim * pairs / results[0] / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": f"last {tokens} new tokens of sequence 0 over its {keys} keys, one KV head ({group} query heads): {pairs} of "
                  f"the problem's {total_pairs} (query, key) pairs, single thread ({results[0]:.1f} s)",
        "row_parallel": {"value": 4 * work.head_dim * pairs / results[1] / 1e12, "unit": "TFLOP/s", "cores": cpu_threads(),
                         "sample": f"the same rows over {cpu_threads()} threads ({results[1]:.2f} s)"},
        "host": host_description(),
    }


def dense_f32_cpu_baseline(q, k, v):
    """softcapped_window_attention_f32 (singe-kernel/src/cpu/attention.rs:1835-1925) on the whole first configuration:
    single thread, then rows over the host's cores (weights hoisted in both; the outputs are bit-identical to the
    reference loop's)."""
    import oracle

    batch, heads, seq, dim = q.shape
    operands = [t.cpu().numpy() for t in (q, k, v)]
    times = []
    for threads in (1, cpu_threads()):
        start = time.perf_counter()
        oracle.softcapped_window_attention_f32(*operands, batch=batch, query_len=seq, key_len=seq, heads=heads, kv_heads=heads,
                                               head_dim=dim, scale=0.125, causal=True, threads=threads)
        times.append(time.perf_counter() - start)
    return {"value": times[0] * 1e6, "unit": "us", "cores": 1, "kind": "port",
            "sample": "the whole configuration, single thread, weights hoisted",
            "row_parallel": {"value": times[1] * 1e6, "unit": "us", "cores": cpu_threads(), "sample": "rows over the host's cores"},
            "host": host_description()}


def latent_cpu_baseline(operands, keys, page, heads, sample=8):
    """Tensor::paged_mla_attention's CPU form (singe/src/backend/cpu/normalization/attention.rs:540-679, f64
    arithmetic, serial in the reference) on the first `sample` sequences of the decode workload, each with its pages
    gathered into a cache of their own: single thread, then the head rows over the host's cores."""
    import oracle

    latent_queries, positional_queries, latent_cache, positional_cache, table = operands
    count = (keys + page - 1) // page
    host = lambda tensor: tensor.float().cpu().numpy()
    times = {1: 0.0, cpu_threads(): 0.0}
    for sequence in range(sample):
        index = table[sequence * count:(sequence + 1) * count]
        inputs = (host(latent_queries[sequence:sequence + 1]), host(positional_queries[sequence:sequence + 1]), host(latent_cache[index]),
                  host(positional_cache[index]))
        for threads in times:
            start = time.perf_counter()
            status, _, _ = oracle.paged_mla_attention(*inputs, [0, 1], [0, count], list(range(count)), [keys - (count - 1) * page],
                                                      causal=True, threads=threads)
            times[threads] += time.perf_counter() - start
            assert status == 0
    nbytes = sample * (keys * 1152 + heads * (576 + 512) * 2)
    serial, spread = times[1], times[cpu_threads()]
    return {"value": nbytes / serial / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the first {sample} of the 256 sequences ({keys} keys, {heads} heads each), single thread ({serial:.1f} s); "
                      f"bytes counted as for the GPU figure",
            "row_parallel": {"value": nbytes / spread / 1e9, "unit": "GB/s", "cores": cpu_threads(),
                             "sample": f"the same sequences, head rows over {cpu_threads()} threads ({spread:.2f} s)"},
            "host": host_description()}


def cache_append_cpu_baseline(query, key, value, cos, sin, weights, page_slots, sample=4096):
    """The rotate-and-append step (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427; norm and rotation
    rotary_cache.rs:92-185) restated in the oracle, single thread, on the first `sample` tokens of the workload,
    appended to a cache that holds just their cells."""
    import numpy as np

    import oracle

    host = lambda tensor: tensor[:sample].float().cpu().numpy()
    q, k, v, c, s = host(query), host(key), host(value), host(cos), host(sin)
    groups, dim = k.shape[1:]
    pages = (sample + page_slots - 1) // page_slots
    caches = [np.zeros((pages, page_slots, groups, dim), dtype=np.float32) for _ in range(2)]
    cells = np.random.default_rng(4).permutation(pages * page_slots)[:sample]
    norms = [(1e-6, weight.float().cpu().numpy()) for weight in weights]
    start = time.perf_counter()
    status, _, _, _ = oracle.rotary_cache_write_f32(q, k, v, c, s, cells // page_slots, cells % page_slots, caches[0], caches[1],
                                                    query_norm=norms[0], key_norm=norms[1], in_place=True)
    elapsed = time.perf_counter() - start
    assert status == 0
    nbytes = 2 * sample * (q.shape[1] + 2 * groups) * dim * 2 + 2 * sample * (dim // 2) * 4 + 2 * sample * 4
    return {"value": nbytes / elapsed / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the first {sample} of the workload's {query.shape[0]} tokens, single thread ({elapsed:.2f} s); bytes "
                      f"counted as for the GPU figure (bf16 operands)",
            "host": host_description()}


# ---- GPU sections ----------------------------------------------------------------------------------------------------

def prefill_section(with_cpu=True, dim=128, key="prefill"):
    """Causal flash-attention prefill, batch 4, seq 4096, 32 heads, bf16 (the third benchmark configuration at
    head_dim 128)."""
    import torch

    import ctypes

    from singe_amd.kernel import attention as A

    from singe_amd import _native, synthetic

    batch, seq, heads = 4, 4096, 32
    q, k, v = (synthetic.portable_normal(f"{key}.{tensor}", (batch, seq, heads, dim), torch.bfloat16)
               for tensor in ("query", "key", "value"))
    out = torch.empty_like(q)
    scale = float(dim) ** -0.5
    config = A.FmhaPrefillConfig.contiguous(batch, seq, seq, heads, heads, dim, scale, True)
    stats = measure(lambda: A.fmha_prefill_bf16(None, out, q, k, v, config), 5)
    # (which of the two dense kernels the library gives this shape)
    rows_per_wave = int(_native.lib().singe_hip_dense_prefill_rows_per_wave(ctypes.byref(config._c())))
    kernel = f"singe_fmha_prefill_pair_bf16_d{dim}_causal" if rows_per_wave == 64 else f"singe_fmha_prefill_bf16_d{dim}_causal"
    flops = 4 * dim * batch * heads * (seq * (seq + 1) // 2)
    tflops = flops / (stats["mean_ms"] * 1e-3) / 1e12
    nbytes, source = traffic(key)
    if COUNTER_TRAFFIC.get(key, {}).get("kernel") != kernel:
        nbytes, source = None, None  # the counters were read on the other kernel
    result = {
        "workload": f"causal flash prefill: batch 4, seq 4096, 32 heads (MHA), head_dim {dim}, bf16 in/out, "
                    "fp32 softmax/accumulate" + (" (BASELINE config 3)" if dim == 128 else ""),
        "value": tflops, "unit": "TFLOP/s", "tokens_per_s": batch * seq / (stats["mean_ms"] * 1e-3),
        "ms_per_step": stats["mean_ms"], "ms_per_step_median": stats["median_ms"], "algorithmic_flops": flops,
        "pct_bf16_mfma_peak": 100.0 * tflops / MFMA_BF16_PEAK_TFLOPS,
        "roofline": {"bound": "mfma", "kernel": kernel, "rows_per_wave": rows_per_wave, "achieved": tflops,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": nbytes, "traffic_source": source, **timing_fields(stats)},
    }
    if dim == 128:
        # The same launch on all-zero tensors: the same instructions in the same order, but matrix-core operands
        # that never change a bit.  The device holds a higher clock there, so this figure is what the kernel's
        # instruction stream allows, and its distance to the figure above is what the data's switching costs.
        blank = torch.zeros_like(q)
        quiet = measure(lambda: A.fmha_prefill_bf16(None, out, blank, blank, blank, config), 5)
        quiet_tflops = flops / (quiet["mean_ms"] * 1e-3) / 1e12
        result["same_kernel_on_zero_inputs"] = {
            "what": "the same kernel and sizes on all-zero q, k, v (no operand bit changes: the clock is not held back)",
            "ms_per_step": quiet["mean_ms"], "tflops": quiet_tflops, "frac": quiet_tflops / MFMA_BF16_PEAK_TFLOPS,
            **timing_fields(quiet)}
    if with_cpu:
        result["cpu_baseline"] = prefill_cpu_baseline(q, k, v, scale)
    return result


def chunked_prefill_section(with_cpu=True):
    """Chunked paged prefill: 8 sequences, 512 new tokens each on prefixes U[1024, 16384], 64 query /
    8 KV heads, head_dim 128, page 16, bf16 (the fourth benchmark configuration), through the paged attention op."""
    import ctypes

    import numpy as np
    import torch

    from singe_amd import _native, neural, synthetic

    work = synthetic.chunked_prefill_workload(portable=True)
    index = lambda values: torch.from_numpy(np.asarray(values, dtype=np.int32)).cuda()
    paging = neural.Paging(index(work.query_offsets), index(work.page_offsets), index(work.pages), index(work.last_page_lengths))
    options = neural.AttentionOptions(causal=True)
    problem = neural._problem(work.query, work.key_cache, work.value_cache, paging, options)
    out = torch.empty_like(work.query)
    lse = torch.empty(work.query.shape[:2], device="cuda", dtype=torch.float32)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    handle = int(torch.cuda.current_stream().cuda_stream)
    scratch_bytes = int(_native.lib().singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem)))
    scratch = torch.empty(max(scratch_bytes, 1), device="cuda", dtype=torch.uint8)

    def launch():
        if scratch_bytes:
            code = _native.lib().singe_hip_paged_attention_scratch_bf16(
                handle, work.query.data_ptr(), work.key_cache.data_ptr(), work.value_cache.data_ptr(),
                paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(),
                paging.last_page_lengths.data_ptr(), out.data_ptr(), lse.data_ptr(), status.data_ptr(), scratch.data_ptr(),
                scratch.numel(), ctypes.byref(problem))
        else:
            code = _native.lib().singe_hip_paged_attention_bf16(
                handle, work.query.data_ptr(), work.key_cache.data_ptr(), work.value_cache.data_ptr(),
                paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(),
                paging.last_page_lengths.data_ptr(), out.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem))
        _native.check(code, "paged_attention")

    stats = measure(launch, 4)
    assert int(status.item()) == 0
    flops = work.algorithmic_flops()
    tflops = flops / (stats["mean_ms"] * 1e-3) / 1e12
    rows_per_wave = int(_native.lib().singe_hip_paged_attention_rows_per_wave(ctypes.byref(problem)))
    kernel = "singe_paged_attention_pair_bf16_d128_i32" if rows_per_wave == 64 else "singe_paged_attention_bf16_d128_i32_p16"
    nbytes, source = traffic("chunked_prefill")
    if COUNTER_TRAFFIC["chunked_prefill"]["kernel"] != kernel:
        nbytes, source = None, None  # the counters were read on the other kernel
    result = {
        "workload": "chunked paged prefill: 8 sequences x 512 new tokens on prefixes U[1024,16384], 64q/8kv heads, "
                    "head_dim 128, page 16, bf16 (BASELINE config 4); whole op (the attention kernel and, where the op "
                    "shares keys out, its merge)",
        "value": tflops, "unit": "TFLOP/s", "tokens_per_s": work.sequences * work.new_tokens / (stats["mean_ms"] * 1e-3),
        "ms_per_step": stats["mean_ms"], "ms_per_step_median": stats["median_ms"], "algorithmic_flops": flops,
        "algorithmic_bytes": work.algorithmic_bytes(), "key_splits_scratch_bytes": scratch_bytes,
        "roofline": {"bound": "mfma", "kernel": kernel, "rows_per_wave": rows_per_wave, "achieved": tflops,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": nbytes, "traffic_source": source, **timing_fields(stats)},
    }
    # The same launch on all-zero queries and caches: what the instruction stream allows where no operand bit changes
    # from one matrix instruction to the next and the clock is not held back (as in the dense prefill section).
    if rows_per_wave == 64:
        kept = (work.query, work.key_cache, work.value_cache)
        work.query, work.key_cache, work.value_cache = (torch.zeros_like(t) for t in kept)
        quiet = measure(launch, 4)
        work.query, work.key_cache, work.value_cache = kept
        quiet_tflops = flops / (quiet["mean_ms"] * 1e-3) / 1e12
        result["same_kernel_on_zero_inputs"] = {
            "what": "the same kernel, sizes and page table on all-zero queries and caches",
            "ms_per_step": quiet["mean_ms"], "tflops": quiet_tflops, "frac": quiet_tflops / MFMA_BF16_PEAK_TFLOPS,
            **timing_fields(quiet)}
    # The same attention with the query's RMS norm and rotation fused into the kernel (rotary_paged_attention): the
    # query is normalised, rotated and rounded on its way into the registers, which spares the two-step form's
    # write and re-read of the rotated query.
    tokens, half = work.query.shape[0], work.head_dim // 2
    position = np.concatenate([prefix + np.arange(work.new_tokens) for prefix in work.prefix]).astype(np.float64)
    angle = torch.from_numpy(position).cuda()[:, None] * (1e4 ** (-torch.arange(half, device="cuda").double() / half))[None, :]
    cos, sin = torch.cos(angle).float().contiguous(), torch.sin(angle).float().contiguous()
    weight = synthetic.portable_normal("chunked_prefill.query_weight", (work.head_dim,), torch.bfloat16)
    rotation = _native.QueryRotationC(neural._DATA_TYPES[torch.float32], 1, 1e-6)

    def launch_fused():
        _native.check(_native.lib().singe_hip_rotary_paged_attention_bf16(
            handle, work.query.data_ptr(), work.key_cache.data_ptr(), work.value_cache.data_ptr(),
            paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(),
            paging.last_page_lengths.data_ptr(), cos.data_ptr(), sin.data_ptr(), weight.data_ptr(), out.data_ptr(), lse.data_ptr(),
            status.data_ptr(), ctypes.byref(problem), ctypes.byref(rotation)), "rotary_paged_attention")

    fused = measure(launch_fused, 4)
    assert int(status.item()) == 0
    result["fused_query_rotation"] = {
        "workload": "the same attention with the query's RMS norm (with a weight) and rotation (f32 angles) done by the "
                    "attention kernel (rotary_paged_attention)",
        "kernel": ("singe_rotary_paged_attention_pair_bf16_d128_i32" if rows_per_wave == 64
                   else "singe_rotary_paged_attention_bf16_d128_i32_p16"), "ms_per_step": fused["mean_ms"],
        "ms_per_step_median": fused["median_ms"], "tflops": flops / (fused["mean_ms"] * 1e-3) / 1e12,
        "over_plain_attention_us": (fused["mean_ms"] - stats["mean_ms"]) * 1e3, **timing_fields(fused)}
    if with_cpu:
        result["cpu_baseline"] = chunked_prefill_cpu_baseline(work)
    return result


def latent_section(with_cpu=True):
    """Latent (MLA) attention over paged caches at DeepSeek's widths (latent 512, positional 64, 128 heads, bf16,
    page 64), beside the benchmark's configurations: a decode step (256 sequences of 4096 keys; every head reads
    the same 1152 bytes per key, so the step is priced against HBM and the matrix cores both) and a chunked
    prefill (8 x 512 new tokens on 8192 keys, priced against the dense bf16 MFMA peak).  Synthetic N(0,1) data."""
    import ctypes

    import numpy as np
    import torch

    from singe_amd import _native, neural, synthetic

    def case(sequences, group, heads=128, page=64):
        query_offsets, page_offsets, last, table, pages = [0], [0], [], [], 0
        for queries, keys in sequences:
            query_offsets.append(query_offsets[-1] + queries)
            count = (keys + page - 1) // page
            page_offsets.append(page_offsets[-1] + count)
            last.append(keys - (count - 1) * page)
            table += list(range(pages, pages + count))
            pages += count
        source = synthetic._PortableSource(synthetic.BASE_SEED, "cuda", f"latent_{len(sequences)}x{sequences[0][0]}")
        order = source.permutation("pages", pages)
        table = [int(order[entry]) for entry in table]
        tokens = query_offsets[-1]
        operands = tuple(source.normal(tensor, shape).to(torch.bfloat16) for tensor, shape in (
            ("latent_queries", (tokens, heads, 512)), ("positional_queries", (tokens, heads, 64)),
            ("latent_cache", (pages, page, 512)), ("positional_cache", (pages, page, 64))))
        index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
        paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
        # Through the C ABI with the output, the log-sum-exps, the status word and the scratch for key splits allocated
        # once, as a caller in a serving loop holds them.
        problem = _native.PagedMlaAttentionProblemC(tokens, heads, 512, 64, page, len(sequences), pages, len(table),
                                                    neural._DATA_TYPES[torch.bfloat16], 0, 1, 0, 0.0)
        out = torch.zeros_like(operands[0])
        lse = torch.full((tokens, heads), float("-inf"), device="cuda", dtype=torch.float32)
        status = torch.zeros(1, device="cuda", dtype=torch.int32)
        lib = _native.lib()
        scratch = torch.empty(max(int(lib.singe_hip_paged_mla_attention_scratch_bytes(ctypes.byref(problem))), 256), device="cuda",
                              dtype=torch.uint8)
        handle = int(torch.cuda.current_stream().cuda_stream)

        def launch():
            _native.check(lib.singe_hip_paged_mla_attention_scratch(
                handle, operands[0].data_ptr(), operands[1].data_ptr(), operands[2].data_ptr(), operands[3].data_ptr(),
                paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
                out.data_ptr(), lse.data_ptr(), status.data_ptr(), scratch.data_ptr(), scratch.numel(), ctypes.byref(problem)),
                "paged_mla_attention")

        stats = measure(launch, group)
        assert int(status.item()) == 0
        pairs = sum(sum(min(keys, max(keys - queries + i, 0) + 1) for i in range(queries)) for queries, keys in sequences)
        flops = pairs * heads * (576 + 512) * 2
        cache_bytes = sum(keys for _, keys in sequences) * 1152 + tokens * heads * (576 + 512) * 2
        return stats, flops, cache_bytes, (*operands, torch.tensor(table, device="cuda"))

    stats, flops, cache_bytes, decode_operands = case([(1, 4096)] * 256, 4)
    gbps, tflops = cache_bytes / (stats["mean_ms"] * 1e-3) / 1e9, flops / (stats["mean_ms"] * 1e-3) / 1e12
    nbytes, source = traffic("latent_decode")
    decode = {
        "workload": "latent attention decode: 256 sequences x 4096 keys, 128 heads, latent 512 + positional 64, page 64, bf16",
        "value": gbps, "unit": "GB/s", "tflops": tflops, "ms_per_step": stats["mean_ms"], "ms_per_step_median": stats["median_ms"],
        "algorithmic_bytes": cache_bytes, "algorithmic_flops": flops,
        "roofline": {"bound": "hbm", "kernel": "singe_paged_mla_attention_bf16_l512_p64", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": nbytes, "traffic_source": source,
                     "mfma_frac": tflops / MFMA_BF16_PEAK_TFLOPS, **timing_fields(stats)},
    }
    if with_cpu:
        decode["cpu_baseline"] = latent_cpu_baseline(decode_operands, 4096, 64, 128)
    del decode_operands
    # Fewer sequences than compute units: the op shares each one's keys out over the chip (given scratch) and merges.
    stats, flops, cache_bytes, _ = case([(1, 8192)] * 32, 4)
    gbps = cache_bytes / (stats["mean_ms"] * 1e-3) / 1e9
    few = {
        "workload": "latent attention decode over few sequences: 32 sequences x 8192 keys, 128 heads, latent 512 + positional 64, "
                    "page 64, bf16; whole op (the attention kernel on shares of each sequence's keys and its merge)",
        "value": gbps, "unit": "GB/s", "us_per_step": stats["mean_ms"] * 1e3, "us_per_step_median": stats["median_ms"] * 1e3,
        "algorithmic_bytes": cache_bytes, "algorithmic_flops": flops, "pct_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS,
        "tflops": flops / (stats["mean_ms"] * 1e-3) / 1e12, **timing_fields(stats)}
    stats, flops, cache_bytes, _ = case([(512, 8192)] * 8, 1)
    tflops = flops / (stats["mean_ms"] * 1e-3) / 1e12
    nbytes, source = traffic("latent_chunked_prefill")
    chunked = {
        "workload": "latent attention chunked prefill: 8 sequences x 512 new tokens on 8192 keys, 128 heads, latent 512 + "
                    "positional 64, page 64, bf16",
        "value": tflops, "unit": "TFLOP/s", "ms_per_step": stats["mean_ms"], "ms_per_step_median": stats["median_ms"],
        "algorithmic_flops": flops,
        "roofline": {"bound": "mfma", "kernel": "singe_paged_mla_attention_bf16_l512_p64", "achieved": tflops,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": nbytes, "traffic_source": source, **timing_fields(stats)},
    }
    return {"decode": decode, "decode_few_sequences": few, "chunked_prefill": chunked}


def cache_append_section(with_cpu=True):
    """The step before the chunked prefill of the fourth configuration: its 8 x 512 new tokens are normalised (RMS,
    with a weight, queries and keys), rotated (f32 angles) and the keys and values appended to the paged cache at the
    cells the page lists name, in one launch (rotary_cache_write): 64 query / 8 KV heads, head_dim 128, page 16, bf16.
    HBM bound: every operand is read once and every result written once."""
    import ctypes

    import numpy as np
    import torch

    from singe_amd import _native, neural, synthetic

    work = synthetic.chunked_prefill_workload(portable=True)
    tokens, heads, groups, dim = work.query.shape[0], work.heads, work.kv_heads, work.head_dim
    source = synthetic._PortableSource(synthetic.BASE_SEED, "cuda", "cache_append")
    key, value = (source.normal(tensor, (tokens, groups, dim)).to(torch.bfloat16) for tensor in ("key", "value"))
    weights = [source.normal(tensor, (dim,)).to(torch.bfloat16) for tensor in ("query_weight", "key_weight")]
    # Token j of a sequence is its key prefix + j: angles of that position, the cell its page list gives.
    position = np.concatenate([prefix + np.arange(work.new_tokens) for prefix in work.prefix]).astype(np.int64)
    sequence = np.repeat(np.arange(work.sequences), work.new_tokens)
    pages = np.asarray(work.pages)[np.asarray(work.page_offsets)[sequence] + position // work.page_size].astype(np.int32)
    slots = (position % work.page_size).astype(np.int32)
    angle = torch.from_numpy(position).cuda().double()[:, None] * (1e4 ** (-torch.arange(dim // 2, device="cuda").double() / (dim // 2)))[None, :]
    cos, sin = torch.cos(angle).float().contiguous(), torch.sin(angle).float().contiguous()
    pages, slots = torch.from_numpy(pages).cuda(), torch.from_numpy(slots).cuda()
    rotated = torch.empty_like(work.query)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    problem = _native.RotaryCacheProblemC(tokens, heads, groups, dim, work.key_cache.shape[0], work.page_size,
                                          neural._DATA_TYPES[torch.bfloat16], neural._DATA_TYPES[torch.float32], 0, 1, 1, 1e-6, 1e-6)
    stream = int(torch.cuda.current_stream().cuda_stream)

    def launch():
        _native.check(_native.lib().singe_hip_rotary_cache_write(
            stream, work.query.data_ptr(), key.data_ptr(), value.data_ptr(), cos.data_ptr(), sin.data_ptr(), pages.data_ptr(),
            slots.data_ptr(), weights[0].data_ptr(), weights[1].data_ptr(), rotated.data_ptr(), work.key_cache.data_ptr(),
            work.value_cache.data_ptr(), status.data_ptr(), ctypes.byref(problem)), "rotary_cache_write")

    stats = measure(launch, 4)
    assert int(status.item()) == 0
    nbytes = 2 * tokens * (heads + 2 * groups) * dim * 2 + 2 * tokens * (dim // 2) * 4 + 2 * tokens * 4 + 2 * dim * 2
    gbps = nbytes / (stats["mean_ms"] * 1e-3) / 1e9
    counted, source = traffic("cache_append")
    result = {
        "workload": "rotate and append (rotary_cache_write) for the fourth configuration's 4096 new tokens: 64 query / 8 KV "
                    "heads, head_dim 128, RMS norm with weights on queries and keys, f32 angles, page 16, bf16",
        "value": gbps, "unit": "GB/s", "us_per_step": stats["mean_ms"] * 1e3, "us_per_step_median": stats["median_ms"] * 1e3,
        "algorithmic_bytes": nbytes,
        "roofline": {"bound": "hbm", "kernel": "singe_rotary_cache_write_chunks_bf16", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": counted, "traffic_source": source,
                     **timing_fields(stats)},
    }
    if with_cpu:
        result["cpu_baseline"] = cache_append_cpu_baseline(work.query, key, value, cos, sin, weights, work.page_size)
    return result


def dense_f32_section(with_cpu=True):
    """The first benchmark configuration, the f32 accuracy anchor: causal dense attention, batch 1, 8 heads,
    512 x 512, head_dim 64, scale 1/8, tensors [batch, heads, len, dim].  Far too small for a roofline: the
    figure is microseconds per launch."""
    import torch

    from singe_amd.kernel import attention as A

    from singe_amd import synthetic

    batch, heads, seq, dim = 1, 8, 512, 64
    q, k, v = (synthetic.portable_normal(f"dense_f32.{tensor}", (batch, heads, seq, dim)) for tensor in ("query", "key", "value"))
    out = torch.empty_like(q)
    config = A.SoftcappedWindowAttentionConfig(A.bhsd_config(batch, heads, heads, seq, seq, dim, 0.125, True), 0, None)
    stats = measure(lambda: A.softcapped_window_attention_f32(None, out, q, k, v, config), 10)
    result = {
        "workload": "causal dense attention f32: batch 1, 8 heads, 512 x 512, head_dim 64, scale 0.125, BHSD "
                    "(BASELINE config 1, the accuracy anchor)",
        "value": stats["mean_ms"] * 1e3, "unit": "us", "us_per_step_median": stats["median_ms"] * 1e3,
        "algorithmic_flops": 4 * dim * heads * (seq * (seq + 1) // 2), "algorithmic_bytes": 4 * batch * heads * seq * dim * 4,
        "kernel": "singe_fmha_prefill_rows_f32_d64", **timing_fields(stats),
    }
    if with_cpu:
        result["cpu_baseline"] = dense_f32_cpu_baseline(q, k, v)
    return result


def fp8_decode_section(with_cpu=True):
    """Long-context decode over an fp8 e4m3 KV cache: batch 64, 64 query / 8 KV heads, head_dim 128,
    context 32768, block 16, one f32 scale per (block, kv head) (the fifth benchmark configuration); exact numerics."""
    import numpy as np
    import torch

    from singe_amd import synthetic
    from singe_amd.kernel import attention as A

    work = synthetic.paged_decode_fp8_workload(portable=True)
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                       work.block_size, work.physical_blocks,
                                                       work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")

    def launch(phases=3):
        A.paged_kv_decode_attention_f8e4m3kv_bf16(None, out, work.query, work.key_cache, work.value_cache, work.key_scales,
                                                  work.value_scales, lens, table, config, workspace, phases)

    step = measure(launch, 2)
    kernel = measure(lambda: launch(1), 2)
    used_blocks = int(np.sum((work.seq_lens.astype(np.int64) + work.block_size - 1) // work.block_size))
    nbytes = work.algorithmic_bytes(1) + 2 * used_blocks * work.kv_heads * 4  # + the scales of the used blocks
    gbps = nbytes / (step["mean_ms"] * 1e-3) / 1e9
    achieved = nbytes / (kernel["mean_ms"] * 1e-3) / 1e9
    counted, source = traffic("fp8_decode")
    result = {
        "workload": "paged decode, fp8 e4m3 KV: batch 64, 64q/8kv heads, head_dim 128, ctx 32768, block 16, "
                    "f32 scale per (block, kv head) (BASELINE config 5); split + reduce kernels",
        "value": gbps, "unit": "GB/s", "tokens_per_s": work.batch / (step["mean_ms"] * 1e-3),
        "ms_per_step": step["mean_ms"], "ms_per_step_median": step["median_ms"], "step_iqr_us": step["iqr_ms"] * 1e3,
        "pct_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS, "algorithmic_bytes": nbytes,
        "roofline": {"bound": "hbm", "kernel": "singe_paged_decode_f8kv_wide_d128_b16", "achieved": achieved, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": counted, "traffic_source": source,
                     **timing_fields(kernel)},
    }
    if with_cpu:
        result["cpu_baseline"] = decode_cpu_baseline(work, budget_s=2.0, fp8=True)
    return result


def head_dim_64_section():
    """The matrix-core kernels at head_dim 64, the other head dimension of the reference's own tests
    (singe/src/backend/cuda/kernel_plan/source/tests.rs:830-966): the third configuration's prefill and the second
    configuration's decode at that width; and the prefill at head_dim 96 and 32, which the dense and paged kernels are
    built for as well."""
    import numpy as np
    import torch

    from singe_amd import synthetic
    from singe_amd.kernel import attention as A

    prefill = prefill_section(with_cpu=False, dim=64, key="prefill_d64")
    work = synthetic.paged_decode_workload(head_dim=64, portable=True, name="paged_decode_d64")
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                       work.block_size, work.physical_blocks,
                                                       work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
    stats = measure(lambda: A.paged_kv_decode_attention_bf16(None, out, work.query, work.key_cache, work.value_cache, lens, table,
                                                             config, workspace), 6)
    nbytes = work.algorithmic_bytes()
    gbps = nbytes / (stats["mean_ms"] * 1e-3) / 1e9
    decode = {"workload": "paged decode: batch 32, 32q/8kv heads, head_dim 64, bf16, block 16, ctx U[512,4096]; split + reduce",
              "value": gbps, "unit": "GB/s", "ms_per_step": stats["mean_ms"], "algorithmic_bytes": nbytes,
              "pct_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS, **timing_fields(stats)}
    del work, out, workspace
    torch.cuda.empty_cache()
    # The dense prefill at the other widths the matrix-core kernels are built for.
    others = {f"prefill_d{dim}": prefill_section(with_cpu=False, dim=dim, key=f"prefill_d{dim}") for dim in (96, 32)}
    # The headline decode at eight and sixteen query heads per KV head (head_dim 128): the dense form of the decode
    # kernel, every query head a column of one product.
    for heads in (64, 128):
        work = synthetic.paged_decode_workload(heads=heads, portable=True, name=f"paged_decode_h{heads}")
        config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                           work.block_size, work.physical_blocks,
                                                           work.block_table_batch_stride, work.scale)
        lens = torch.from_numpy(work.seq_lens).cuda()
        table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
        out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
        workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
        step = lambda phases=3: A.paged_kv_decode_attention_bf16(None, out, work.query, work.key_cache, work.value_cache, lens,
                                                                 table, config, workspace, phases)
        whole, kernel = measure(step, 6), measure(lambda: step(1), 6)
        nbytes = work.algorithmic_bytes()
        rate = lambda stats: nbytes / (stats["mean_ms"] * 1e-3) / 1e9
        others[f"decode_{heads // 8}_heads_per_kv_head"] = {
            "workload": f"paged decode: batch 32, {heads}q/8kv heads, head_dim 128, bf16, block 16, ctx U[512,4096]; split + reduce",
            "value": rate(whole), "unit": "GB/s", "ms_per_step": whole["mean_ms"], "algorithmic_bytes": nbytes,
            "pct_hbm_peak": 100.0 * rate(whole) / HBM_PEAK_GBPS,
            "roofline": {"bound": "hbm", "kernel": "singe_paged_decode_bf16_wide_d128_b16", "achieved": rate(kernel), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": rate(kernel) / HBM_PEAK_GBPS, **timing_fields(kernel)}}
        del work, out, workspace
        torch.cuda.empty_cache()
    return {"prefill": prefill, "decode": decode, **others}


def mfma_ceiling_section():
    """What the matrix cores sustain with nothing else in the way: 512 workgroups of four waves, each wave a
    register-only loop of the prefill kernels' product (v_mfma_f32_32x32x16_bf16), on all-zero operands and on
    N(0, 1) operands from the same generator as the benchmark's tensors.  The clock under such a loop is set by
    power, and power by the operands' bits, so the second figure is the ceiling a prefill kernel has on data like
    the benchmark's."""
    import torch

    from singe_amd import _native

    workgroups, iterations = 512, 4000
    from singe_amd import synthetic

    operands = {"zeros": torch.zeros(1 << 22, device="cuda", dtype=torch.bfloat16),
                "normal": synthetic.portable_normal("mfma_ceiling.operands", (1 << 22,), torch.bfloat16)}
    out = torch.empty(workgroups * 256, device="cuda", dtype=torch.float32)
    handle = int(torch.cuda.current_stream().cuda_stream)
    flops = workgroups * 4 * iterations * 32 * 32768
    result = {"kernel": "singe_mfma_ceiling_bf16", "workgroups": workgroups, "iterations": iterations, "flops_per_launch": flops,
              "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s"}
    for name, data in operands.items():
        def launch():
            _native.check(_native.lib().singe_hip_mfma_ceiling(handle, data.data_ptr(), data.numel() * 2, out.data_ptr(),
                                                               out.numel(), workgroups, iterations, 0), "mfma_ceiling")
        stats = measure(launch, 1)
        tflops = flops / (stats["mean_ms"] * 1e-3) / 1e12
        result[name] = {"value": tflops, "frac_of_peak": tflops / MFMA_BF16_PEAK_TFLOPS, **timing_fields(stats)}
    return result


def hbm_ceiling_section():
    """What the memory system delivers to a kernel that only reads: one workgroup of 512 lanes per compute unit (the
    decode kernels' launch shape) streams buffers of the two decode workloads' sizes, 306 MB and 4.3 GB, once per
    launch with non-temporal loads; three buffers are rotated as the decode section rotates its KV pools."""
    import torch

    from singe_amd import _native

    workgroups = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.empty(workgroups * 512, device="cuda", dtype=torch.int32)
    handle = int(torch.cuda.current_stream().cuda_stream)
    result = {"kernel": "singe_hbm_stream_read", "workgroups": workgroups, "peak": HBM_PEAK_GBPS, "unit": "GB/s"}
    for name, nbytes, pools, group in (("decode_sized", DECODE_BYTES // 16 * 16, 3, 6), ("fp8_decode_sized", 4_305_977_600, 2, 2)):
        buffers = [torch.randint(0, 255, (nbytes,), device="cuda", dtype=torch.uint8) for _ in range(pools)]
        turn = [0]

        def launch():
            data = buffers[turn[0] % pools]
            turn[0] += 1
            _native.check(_native.lib().singe_hip_hbm_stream_read(handle, data.data_ptr(), nbytes, out.data_ptr(), out.numel(),
                                                                  workgroups), "hbm_stream_read")
        stats = measure(launch, group)
        gbps = nbytes / (stats["mean_ms"] * 1e-3) / 1e9
        result[name] = {"bytes": nbytes, "value": gbps, "frac_of_peak": gbps / HBM_PEAK_GBPS, **timing_fields(stats)}
        del buffers
        torch.cuda.empty_cache()
    return result


def decode_op_section():
    """The headline workload through the paged attention op in FlashInfer form (Operation::PagedAttention, the op a
    graph of the reference decodes with), its paging vectors i64 as the reference's DecodeStep writes them: one token a
    sequence, causal.  Given scratch the op checks the vectors, gives every token its page list and key count and runs
    the block-table decode kernels; with a fixed number of shares it stays on its row-tile kernel, timed beside it."""
    import ctypes

    import numpy as np
    import torch

    from singe_amd import _native, neural, synthetic

    work = synthetic.paged_decode_workload(portable=True)
    counts = (work.seq_lens.astype(np.int64) + work.block_size - 1) // work.block_size
    pages = np.concatenate([work.block_table[b, :n] for b, n in enumerate(counts)]).astype(np.int64)
    page_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    last = (work.seq_lens.astype(np.int64) - (counts - 1) * work.block_size)
    index = lambda values: torch.from_numpy(np.ascontiguousarray(values, dtype=np.int64)).cuda()
    paging = neural.Paging(index(np.arange(work.batch + 1)), index(page_offsets), index(pages), index(last))
    options = neural.AttentionOptions(causal=True, scale=work.scale)
    problem = neural._problem(work.query, work.key_cache, work.value_cache, paging, options)
    out = torch.empty_like(work.query)
    lse = torch.empty(work.query.shape[:2], device="cuda", dtype=torch.float32)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    handle = int(torch.cuda.current_stream().cuda_stream)
    lib = _native.lib()
    results = {}
    for name, shares in (("decode_kernels", 0), ("row_tile_kernel", 4)):
        lib.singe_hip_set_paged_attention_splits(shares)
        try:
            scratch = torch.empty(max(int(lib.singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem))), 256), device="cuda", dtype=torch.uint8)

            def launch():
                _native.check(lib.singe_hip_paged_attention_scratch_bf16(
                    handle, work.query.data_ptr(), work.key_cache.data_ptr(), work.value_cache.data_ptr(), paging.query_offsets.data_ptr(),
                    paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(), out.data_ptr(),
                    lse.data_ptr(), status.data_ptr(), scratch.data_ptr(), scratch.numel(), ctypes.byref(problem)), "paged_attention")

            stats = measure(launch, 6)
        finally:
            lib.singe_hip_set_paged_attention_splits(0)
        assert int(status.item()) == 0
        gbps = DECODE_BYTES / (stats["mean_ms"] * 1e-3) / 1e9
        results[name] = {"us_per_step": stats["mean_ms"] * 1e3, "us_per_step_median": stats["median_ms"] * 1e3, "value": gbps, "unit": "GB/s",
                         "pct_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS, "scratch_bytes": scratch.numel(), **timing_fields(stats)}
    return {"workload": "the headline decode step (BASELINE config 2) through the paged attention op in FlashInfer form, i64 paging, "
                        "causal; whole op under HIP events (every launch of it)",
            "algorithmic_bytes": DECODE_BYTES, **results}


def decode_section(args, with_cpu):
    """The headline: --warmup untimed steps (and on to 300 ms), exactly --steps timed steps between two synchronisations,
    then the split kernel alone under HIP events."""
    import numpy as np
    import torch

    from singe_amd import _native, synthetic
    from singe_amd.kernel import attention as A

    if args.workers:
        _native.lib().singe_hip_set_decode_workers(args.workers)
    work = synthetic.paged_decode_workload(portable=True)
    pools = [(work.key_cache, work.value_cache)]
    for extra in range(1, POOLS):
        other = synthetic.paged_decode_workload(portable=True, name=f"paged_decode_pool{extra}")
        pools.append((other.key_cache, other.value_cache))
        del other
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                       work.block_size, work.physical_blocks,
                                                       work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
    counter = [0]

    def step(phases=3):
        kc, vc = pools[counter[0] % POOLS]
        counter[0] += 1
        A.paged_kv_decode_attention_bf16(None, out, work.query, kc, vc, lens, table, config, workspace, phases)

    # Untimed warm-up: the steps asked for, and on until WARMUP_SECONDS have passed like every other figure of this
    # file (a handful of 55 us steps leaves the device's clocks where idling put them).
    warm_start = time.perf_counter()
    warm_steps = 0
    while warm_steps < args.warmup or time.perf_counter() - warm_start < WARMUP_SECONDS:
        step()
        warm_steps += 1
        if warm_steps % 64 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - start
    ms_per_step = seconds / args.steps * 1e3

    whole = measure(step, 6)               # the op under events: split + reduce
    kernel = measure(lambda: step(1), 6)   # the dominant kernel alone
    bytes_per_step = work.algorithmic_bytes()
    assert bytes_per_step == DECODE_BYTES, (bytes_per_step, DECODE_BYTES)
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    achieved = bytes_per_step / (kernel["mean_ms"] * 1e-3) / 1e9
    counted, source = traffic("decode") if not args.workers else (None, None)
    result = {
        "metric": "decode attn GB/s", "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "warmup_steps_run": warm_steps, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (splitmix64 counter streams, Box-Muller N(0,1), base seed 0x51A6E; singe_amd/synthetic.py portable=True)",
        "config": {
            "workload": "paged decode: batch 32, 32q/8kv heads, head_dim 128, bf16, block 16, "
                        "ctx U[512,4096], 16384-block pool (BASELINE config 2)",
            "total_keys": work.total_keys, "algorithmic_bytes": bytes_per_step, "algorithmic_flops": work.algorithmic_flops(),
            "workers": int(_native.lib().singe_hip_decode_workers(config._c())), "kv_pools_rotated": POOLS,
        },
        "tokens_per_s": work.batch / (ms_per_step * 1e-3),
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "step_under_events": {"mean_us": whole["mean_ms"] * 1e3, "median_us": whole["median_ms"] * 1e3,
                              "p25_us": whole["p25_ms"] * 1e3, "p75_us": whole["p75_ms"] * 1e3, "samples": whole["samples"],
                              "pct_hbm_peak": 100.0 * bytes_per_step / (whole["mean_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "roofline": {"bound": "hbm", "kernel": "singe_paged_decode_bf16_d128_g1_b16", "achieved": achieved, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": counted, "traffic_source": source,
                     **timing_fields(kernel)},
    }
    if with_cpu:
        result["cpu_baseline"] = decode_cpu_baseline(work)
    return result


def main():
    global FEW
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU exchange and every box here has one "
              "GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    with_cpu = not args.no_cpu_baseline
    FEW = bool(args.few and args.only)
    sections = {
        "decode_op": decode_op_section, "prefill": lambda: prefill_section(with_cpu), "chunked_prefill": lambda: chunked_prefill_section(with_cpu),
        "fp8_decode": lambda: fp8_decode_section(with_cpu), "dense_f32": lambda: dense_f32_section(with_cpu),
        "latent": lambda: latent_section(with_cpu), "cache_append": lambda: cache_append_section(with_cpu),
        "head_dim_64": head_dim_64_section, "mfma_ceiling": mfma_ceiling_section,
        "hbm_ceiling": hbm_ceiling_section,
    }
    if FEW:
        # A copy of known size beside the kernel, for the unit of the profiler's byte counters: torch's f32 -> bf16
        # copy of 2^28 elements reads 1 GiB and writes 512 MiB.
        torch.empty(1 << 28, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    if args.only and args.only != "decode":
        print(json.dumps({args.only: sections[args.only]()}), flush=True)
        return
    result = decode_section(args, with_cpu)
    if args.only == "decode" or args.no_extras:
        print(json.dumps(result), flush=True)
        return
    from singe_amd import error

    for name, run in sections.items():
        torch.cuda.empty_cache()
        try:
            result[name] = run()
        except error.UnsupportedWidth as refused:  # a width this build has no kernel for is said, not hidden
            result[name] = {"unsupported": str(refused)}
    ceiling = result["mfma_ceiling"]["normal"]["value"]
    for name in ("prefill", "chunked_prefill"):
        result[name]["roofline"]["frac_of_measured_ceiling"] = result[name]["roofline"]["achieved"] / ceiling
    result["roofline"]["frac_of_measured_ceiling"] = result["roofline"]["achieved"] / result["hbm_ceiling"]["decode_sized"]["value"]
    result["fp8_decode"]["roofline"]["frac_of_measured_ceiling"] = (result["fp8_decode"]["roofline"]["achieved"]
                                                                    / result["hbm_ceiling"]["fp8_decode_sized"]["value"])
    if args.full:
        print(json.dumps(result), flush=True)
        return
    if args.detail:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.detail)), exist_ok=True)
            with open(args.detail, "w") as handle:
                json.dump(result, handle)
        except OSError as problem:  # the detail file is a convenience; the line below is the result
            print(f"bench.py: detail file not written: {problem}", file=sys.stderr)
    print(json.dumps(compact(result), separators=(",", ":")), flush=True)


def _rounded(value, digits=4):
    if isinstance(value, float):
        return float(f"{value:.{digits}g}")
    return value


def _config_summary(section, ms=None):
    """The figures of one benchmark configuration that the compact line keeps: the kernel and its time, what it
    achieved against which peak (and against the ceiling measured in the same run), counter traffic, and the CPU
    baseline's value and core count."""
    roofline = section.get("roofline", {})
    baseline = section.get("cpu_baseline", {})
    if ms is None:
        ms = section.get("ms_per_step", section.get("value", 0.0) * 1e-3 if section.get("unit") == "us" else None)
    summary = {"kernel": roofline.get("kernel", section.get("kernel")), "ms_per_step": ms,
               "iqr_us": roofline.get("kernel_iqr_us", section.get("kernel_iqr_us")),
               "achieved": roofline.get("achieved"), "peak": roofline.get("peak"), "unit": roofline.get("unit"),
               "frac": roofline.get("frac"), "frac_of_measured_ceiling": roofline.get("frac_of_measured_ceiling"),
               "traffic": roofline.get("traffic"),
               "cpu_baseline": {"value": baseline.get("value"), "unit": baseline.get("unit"), "cores": baseline.get("cores"),
                                "row_parallel": baseline.get("row_parallel", {}).get("value"),
                                "row_parallel_cores": baseline.get("row_parallel", {}).get("cores")}}
    return {name: _rounded(value) if not isinstance(value, dict) else {k: _rounded(v) for k, v in value.items()}
            for name, value in summary.items()}


def compact(result):
    """The line the run ends with: the headline's fields as they are, and inside `roofline` one short object per
    further benchmark configuration (`configs`), the two measured ceilings, the whole decode op beside its dominant
    kernel, and the fraction of its roofline every other measured kernel reached (`others`).  Everything else is in
    the --detail file (or the --full line)."""
    line = {name: result[name] for name in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                            "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                                            "tokens_per_s", "pct_hbm_peak")}
    line["data"] = "synthetic (seeded splitmix64 N(0,1), base seed 0x51A6E)"
    roofline = {name: _rounded(value, 6) for name, value in result["roofline"].items() if name != "traffic_source"}
    roofline["whole_op_frac"] = _rounded(result["pct_hbm_peak"] / 100.0)
    roofline["whole_op_frac_under_events"] = _rounded(result["step_under_events"]["pct_hbm_peak"] / 100.0)
    roofline["ceilings"] = {
        "mfma_bf16_register_loop_normal_tflops": _rounded(result["mfma_ceiling"]["normal"]["value"]),
        "mfma_bf16_register_loop_zeros_tflops": _rounded(result["mfma_ceiling"]["zeros"]["value"]),
        "hbm_stream_read_decode_sized_gbps": _rounded(result["hbm_ceiling"]["decode_sized"]["value"]),
        "hbm_stream_read_fp8_decode_sized_gbps": _rounded(result["hbm_ceiling"]["fp8_decode_sized"]["value"])}
    configs = {}
    if "unsupported" not in result.get("dense_f32", {"unsupported": 1}):
        configs["1_dense_f32"] = _config_summary(result["dense_f32"])
    for label, name in (("3_prefill", "prefill"), ("4_chunked_prefill", "chunked_prefill"), ("5_fp8_decode", "fp8_decode")):
        if "unsupported" not in result.get(name, {"unsupported": 1}):
            configs[label] = _config_summary(result[name])
    if "same_kernel_on_zero_inputs" in result.get("prefill", {}) and "3_prefill" in configs:
        # (the same launch on all-zero tensors: what the instruction stream allows where the clock is not held back)
        configs["3_prefill"]["frac_on_zero_inputs"] = _rounded(result["prefill"]["same_kernel_on_zero_inputs"]["frac"])
    if "same_kernel_on_zero_inputs" in result.get("chunked_prefill", {}) and "4_chunked_prefill" in configs:
        configs["4_chunked_prefill"]["frac_on_zero_inputs"] = _rounded(result["chunked_prefill"]["same_kernel_on_zero_inputs"]["frac"])
    if "5_fp8_decode" in configs:
        configs["5_fp8_decode"]["whole_op_frac"] = _rounded(result["fp8_decode"]["pct_hbm_peak"] / 100.0)
    roofline["configs"] = configs
    others = {}

    def note(label, section):
        inner = section.get("roofline", {})
        if "frac" in inner:
            others[label] = _rounded(inner["frac"])
        elif "pct_hbm_peak" in section:
            others[label] = _rounded(section["pct_hbm_peak"] / 100.0)

    for name in ("latent", "head_dim_64", "decode_op"):
        for label, section in result.get(name, {}).items():
            if isinstance(section, dict):
                note(f"{name}.{label}", section)
                if "pct_hbm_peak" in section and "roofline" in section:
                    others[f"{name}.{label}.whole_op"] = _rounded(section["pct_hbm_peak"] / 100.0)
    if "roofline" in result.get("cache_append", {}):
        note("cache_append", result["cache_append"])
    roofline["others"] = others
    line["roofline"] = roofline
    baseline = result.get("cpu_baseline")
    if baseline:
        line["cpu_baseline"] = {"value": _rounded(baseline["value"]), "unit": baseline["unit"], "cores": baseline["cores"],
                                "kind": baseline["kind"], "sample": baseline["sample"],
                                "row_parallel": {k: _rounded(v) for k, v in baseline.get("row_parallel", {}).items()
                                                 if k != "sample"},
                                "host": baseline.get("host")}
    return line


if __name__ == "__main__":
    main()
