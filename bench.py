#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of paged decode attention (split kernel + split reduce) over one batch of the
headline decode workload: batch 32, 32 query / 8 KV heads, head_dim 128, bf16, block size 16,
context lengths uniform in [512, 4096], block tables from a seeded permutation of a 16384-block
pool.  Inputs are resident in HBM before the timed region; three independent KV pools are rotated so
consecutive steps cannot be served from the 256 MB Infinity Cache.

Prints one JSON line: whole-job GB/s of algorithmic bytes, the roofline of the dominant kernel
(measured with HIP events on the launch stream) and the CPU oracle timed on a bounded sample.  The
same line carries, under "prefill", the causal flash-attention prefill measurement (TFLOP/s against
the dense bf16 MFMA peak), under "chunked_prefill", "fp8_decode" and "dense_f32" the other three
benchmark configurations, and under "latent" latent (MLA) attention over paged caches (decode and chunked prefill).
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

# HBM bytes per launch of the decode split kernel at the headline workload, from rocprofv3 --pmc runs of
# this script: FETCH_SIZE 145768 x 2 KiB (the counter's unit, calibrated on a copy of known size) +
# WRITE_SIZE 4552 KiB.  Reported only for that kernel, workload and tuning.
DECODE_TRAFFIC_BYTES = (145766 * 2 + 4552) * 1024
# The same for the dense prefill kernel at batch 4 x seq 4096 x 32 heads: FETCH_SIZE 301283, WRITE_SIZE 131377.
PREFILL_TRAFFIC_BYTES = (311083 * 2 + 132590) * 1024
# The same for the latent attention kernel at its two workloads (--only-latent under rocprofv3 --pmc): decode
# FETCH_SIZE 608520, WRITE_SIZE 33047; chunked prefill FETCH_SIZE 1376200, WRITE_SIZE 526390.
LATENT_DECODE_TRAFFIC_BYTES = (608520 * 2 + 33047) * 1024
LATENT_CHUNKED_TRAFFIC_BYTES = (1376200 * 2 + 526390) * 1024
HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
POOLS = 3


def parse():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=300)
    parser.add_argument("--warmup", type=int, default=30)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement")
    parser.add_argument("--no-extras", action="store_true", help="skip the chunked-prefill and fp8-decode measurements")
    parser.add_argument("--prefill-steps", type=int, default=40)
    parser.add_argument("--workers", type=int, default=0, help="tuning override (0 = built-in choice)")
    parser.add_argument("--only-latent", action="store_true",
                        help="run the latent attention section alone and print it (for counter runs of its kernel)")
    return parser.parse_args()


def cpu_baseline(work, budget_s=12.0):
    """The reference's CPU decode as written (one thread, weights re-evaluated per output dimension),
    restated in the oracle, timed on as many leading sequences of the same workload as fit the budget."""
    import numpy as np

    import oracle

    order = list(range(work.batch))
    done_bytes, elapsed, used = 0, 0.0, 0
    cores = min(os.cpu_count() or 1, 16)
    parallel = 0.0
    for b in order:
        length = int(work.seq_lens[b])
        n = (length + work.block_size - 1) // work.block_size
        blocks = work.block_table[b, :n].astype(np.int64)
        import torch

        index = torch.from_numpy(blocks).to(work.key_cache.device)
        kc = work.key_cache[index].float().cpu().numpy()
        vc = work.value_cache[index].float().cpu().numpy()
        q = work.query[b:b + 1].float().cpu().numpy()
        table = np.arange(n, dtype=np.uint32).reshape(1, -1)
        start = time.perf_counter()
        oracle.paged_kv_decode_attention_f32(q, kc, vc, [length], table, batch=1, heads=work.heads,
                                             kv_heads=work.kv_heads, head_dim=work.head_dim,
                                             block_size=work.block_size, block_table_batch_stride=max(n, 1),
                                             scale=work.scale, literal=True)
        elapsed += time.perf_counter() - start
        # The same sequence with its independent head rows on every host core and the weight of a (row, key)
        # pair evaluated once: the way the reference's dense op spreads rows over threads
        # (singe/src/backend/cpu/normalization/attention.rs:219-223); bit-identical outputs.
        start = time.perf_counter()
        oracle.paged_kv_decode_attention_f32(q, kc, vc, [length], table, batch=1, heads=work.heads,
                                             kv_heads=work.kv_heads, head_dim=work.head_dim,
                                             block_size=work.block_size, block_table_batch_stride=max(n, 1),
                                             scale=work.scale, threads=cores)
        parallel += time.perf_counter() - start
        done_bytes += length * 2 * work.kv_heads * work.head_dim * 2 + 2 * work.heads * work.head_dim * 2
        used += 1
        if elapsed > budget_s:
            break
    return {
        "value": done_bytes / elapsed / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"first {used} of {work.batch} sequences of the same workload, reference loop shape "
                  f"(single thread, {elapsed:.1f} s)",
        "row_parallel": {"value": done_bytes / parallel / 1e9, "unit": "GB/s", "cores": cores,
                         "sample": f"the same sequences, head rows over {cores} threads, weights hoisted ({parallel:.2f} s)"},
    }


def prefill_section(steps):
    """Causal flash-attention prefill, batch 4, seq 4096, 32 heads, head_dim 128, bf16 (the
    third benchmark configuration): average kernel time from HIP events around back-to-back launches."""
    import torch

    from singe_amd.kernel import attention as A

    batch, seq, heads, dim = 4, 4096, 32, 128
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x51A6E + 3)
    q, k, v = (torch.randn((batch, seq, heads, dim), generator=gen, device="cuda").to(torch.bfloat16) for _ in range(3))
    out = torch.empty_like(q)
    config = A.FmhaPrefillConfig.contiguous(batch, seq, seq, heads, heads, dim, float(dim) ** -0.5, True)
    for _ in range(5):
        A.fmha_prefill_bf16(None, out, q, k, v, config)
    torch.cuda.synchronize()
    group = 5
    groups = max(steps // group, 4)
    begin = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    finish = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    for j in range(groups):
        begin[j].record()
        for _ in range(group):
            A.fmha_prefill_bf16(None, out, q, k, v, config)
        finish[j].record()
    torch.cuda.synchronize()
    ms = sorted(b.elapsed_time(f) / group for b, f in zip(begin, finish))
    avg = sum(ms) / len(ms)
    flops = 4 * dim * batch * heads * (seq * (seq + 1) // 2)
    tflops = flops / (avg * 1e-3) / 1e12
    return {
        "workload": "causal flash prefill: batch 4, seq 4096, 32 heads (MHA), head_dim 128, bf16 in/out, "
                    "fp32 softmax/accumulate (BASELINE config 3)",
        "value": tflops,
        "unit": "TFLOP/s",
        "tokens_per_s": batch * seq / (avg * 1e-3),
        "ms_per_step": avg,
        "algorithmic_flops": flops,
        "pct_bf16_mfma_peak": 100.0 * tflops / MFMA_BF16_PEAK_TFLOPS,
        "roofline": {
            "bound": "mfma",
            "kernel": "singe_fmha_prefill_bf16_d128_causal",
            "achieved": tflops,
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
            "traffic": PREFILL_TRAFFIC_BYTES,
            "kernel_avg_us": avg * 1e3,
            "kernel_median_us": ms[len(ms) // 2] * 1e3,
        },
    }


def time_launches(launch, steps, group):
    """Average milliseconds per launch from HIP events on the current stream around groups of
    back-to-back launches; returns (average, median)."""
    import torch

    groups = max(steps // group, 4)
    begin = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    finish = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    for j in range(groups):
        begin[j].record()
        for _ in range(group):
            launch()
        finish[j].record()
    torch.cuda.synchronize()
    ms = sorted(b.elapsed_time(f) / group for b, f in zip(begin, finish))
    return sum(ms) / len(ms), ms[len(ms) // 2]


def chunked_prefill_section(steps):
    """Chunked paged prefill: 8 sequences, 512 new tokens each on prefixes U[1024, 16384], 64 query /
    8 KV heads, head_dim 128, page 16, bf16 (the fourth benchmark configuration), through the paged attention op."""
    import ctypes

    import numpy as np
    import torch

    from singe_amd import _native, neural, synthetic

    work = synthetic.chunked_prefill_workload()
    index = lambda values: torch.from_numpy(np.asarray(values, dtype=np.int32)).cuda()
    paging = neural.Paging(index(work.query_offsets), index(work.page_offsets), index(work.pages), index(work.last_page_lengths))
    options = neural.AttentionOptions(causal=True)
    problem = neural._problem(work.query, work.key_cache, work.value_cache, paging, options)
    out = torch.empty_like(work.query)
    lse = torch.empty(work.query.shape[:2], device="cuda", dtype=torch.float32)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    handle = int(torch.cuda.current_stream().cuda_stream)

    def launch():
        code = _native.lib().singe_hip_paged_attention_bf16(
            handle, work.query.data_ptr(), work.key_cache.data_ptr(), work.value_cache.data_ptr(),
            paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(),
            paging.last_page_lengths.data_ptr(), out.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem))
        _native.check(code, "paged_attention")

    for _ in range(3):
        launch()
    torch.cuda.synchronize()
    avg, median = time_launches(launch, steps, 4)
    assert int(status.item()) == 0
    flops = work.algorithmic_flops()
    tflops = flops / (avg * 1e-3) / 1e12
    return {
        "workload": "chunked paged prefill: 8 sequences x 512 new tokens on prefixes U[1024,16384], 64q/8kv heads, "
                    "head_dim 128, page 16, bf16 (BASELINE config 4)",
        "value": tflops,
        "unit": "TFLOP/s",
        "tokens_per_s": work.sequences * work.new_tokens / (avg * 1e-3),
        "ms_per_step": avg,
        "algorithmic_flops": flops,
        "roofline": {"bound": "mfma", "kernel": "singe_paged_attention_bf16_d128_i32_p16", "achieved": tflops,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": None, "kernel_avg_us": avg * 1e3, "kernel_median_us": median * 1e3},
    }


def latent_section(steps):
    """Latent (MLA) attention over paged caches at DeepSeek's widths (latent 512, positional 64, 128 heads, bf16,
    page 64), beside the benchmark's configurations: a decode step (256 sequences of 4096 keys; every head reads
    the same 1152 bytes per key, so the step is priced against HBM and the matrix cores both) and a chunked
    prefill (8 x 512 new tokens on 8192 keys, priced against the dense bf16 MFMA peak).  Synthetic N(0,1) data."""
    import numpy as np
    import torch

    from singe_amd import neural

    def case(sequences, heads=128, page=64):
        query_offsets, page_offsets, last, table, pages = [0], [0], [], [], 0
        for queries, keys in sequences:
            query_offsets.append(query_offsets[-1] + queries)
            count = (keys + page - 1) // page
            page_offsets.append(page_offsets[-1] + count)
            last.append(keys - (count - 1) * page)
            table += list(range(pages, pages + count))
            pages += count
        order = np.random.default_rng(7).permutation(pages)
        table = [int(order[entry]) for entry in table]
        gen = torch.Generator(device="cuda")
        gen.manual_seed(11)
        rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
        tokens = query_offsets[-1]
        operands = (rand(tokens, heads, 512), rand(tokens, heads, 64), rand(pages, page, 512), rand(pages, page, 64))
        index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
        paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
        options = neural.AttentionOptions(causal=True)
        launch = lambda: neural.paged_mla_attention(*operands, paging, options, check=False)
        for _ in range(2):
            launch()
        torch.cuda.synchronize()
        avg, median = time_launches(launch, steps, 2)
        pairs = sum(sum(min(keys, max(keys - queries + i, 0) + 1) for i in range(queries)) for queries, keys in sequences)
        flops = pairs * heads * (576 + 512) * 2
        cache_bytes = sum(keys for _, keys in sequences) * 1152 + tokens * heads * (576 + 512) * 2
        return avg, median, flops, cache_bytes

    avg, median, flops, cache_bytes = case([(1, 4096)] * 256)
    gbps, tflops = cache_bytes / (avg * 1e-3) / 1e9, flops / (avg * 1e-3) / 1e12
    decode = {
        "workload": "latent attention decode: 256 sequences x 4096 keys, 128 heads, latent 512 + positional 64, page 64, bf16",
        "value": gbps, "unit": "GB/s", "tflops": tflops, "ms_per_step": avg, "ms_per_step_median": median,
        "algorithmic_bytes": cache_bytes, "algorithmic_flops": flops,
        "roofline": {"bound": "hbm", "kernel": "singe_paged_mla_attention_bf16_l512_p64", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": LATENT_DECODE_TRAFFIC_BYTES,
                     "mfma_frac": tflops / MFMA_BF16_PEAK_TFLOPS},
    }
    avg, median, flops, cache_bytes = case([(512, 8192)] * 8)
    tflops = flops / (avg * 1e-3) / 1e12
    chunked = {
        "workload": "latent attention chunked prefill: 8 sequences x 512 new tokens on 8192 keys, 128 heads, latent 512 + "
                    "positional 64, page 64, bf16",
        "value": tflops, "unit": "TFLOP/s", "ms_per_step": avg, "ms_per_step_median": median, "algorithmic_flops": flops,
        "roofline": {"bound": "mfma", "kernel": "singe_paged_mla_attention_bf16_l512_p64", "achieved": tflops,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": LATENT_CHUNKED_TRAFFIC_BYTES},
    }
    return {"decode": decode, "chunked_prefill": chunked}


def dense_f32_section(steps):
    """The first benchmark configuration, the f32 accuracy anchor: causal dense attention, batch 1, 8 heads,
    512 x 512, head_dim 64, scale 1/8, tensors [batch, heads, len, dim].  Far too small for a roofline: the
    figure is microseconds per launch."""
    import torch

    from singe_amd.kernel import attention as A

    batch, heads, seq, dim = 1, 8, 512, 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x51A6E + 1)
    q, k, v = (torch.randn((batch, heads, seq, dim), generator=gen, device="cuda") for _ in range(3))
    out = torch.empty_like(q)
    config = A.SoftcappedWindowAttentionConfig(A.bhsd_config(batch, heads, heads, seq, seq, dim, 0.125, True), 0, None)

    def launch():
        A.softcapped_window_attention_f32(None, out, q, k, v, config)

    for _ in range(5):
        launch()
    torch.cuda.synchronize()
    avg, median = time_launches(launch, steps, 10)
    return {
        "workload": "causal dense attention f32: batch 1, 8 heads, 512 x 512, head_dim 64, scale 0.125, BHSD "
                    "(BASELINE config 1, the accuracy anchor)",
        "value": avg * 1e3,
        "unit": "us",
        "us_per_step_median": median * 1e3,
        "algorithmic_flops": 4 * dim * heads * (seq * (seq + 1) // 2),
        "algorithmic_bytes": 4 * batch * heads * seq * dim * 4,
        "kernel": "singe_fmha_prefill_rows_f32_d64",
    }


def fp8_decode_section(steps):
    """Long-context decode over an fp8 e4m3 KV cache: batch 64, 64 query / 8 KV heads, head_dim 128,
    context 32768, block 16, one f32 scale per (block, kv head) (the fifth benchmark configuration); exact numerics."""
    import numpy as np
    import torch

    from singe_amd import synthetic
    from singe_amd.kernel import attention as A

    work = synthetic.paged_decode_fp8_workload()
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                       work.block_size, work.physical_blocks,
                                                       work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")

    def launch():
        A.paged_kv_decode_attention_f8e4m3kv_bf16(None, out, work.query, work.key_cache, work.value_cache, work.key_scales,
                                                  work.value_scales, lens, table, config, workspace)

    for _ in range(3):
        launch()
    torch.cuda.synchronize()
    avg, median = time_launches(launch, steps, 2)
    used_blocks = int(np.sum((work.seq_lens.astype(np.int64) + work.block_size - 1) // work.block_size))
    nbytes = work.algorithmic_bytes(1) + 2 * used_blocks * work.kv_heads * 4  # + the scales of the used blocks
    gbps = nbytes / (avg * 1e-3) / 1e9
    return {
        "workload": "paged decode, fp8 e4m3 KV: batch 64, 64q/8kv heads, head_dim 128, ctx 32768, block 16, "
                    "f32 scale per (block, kv head) (BASELINE config 5); split + reduce kernels",
        "value": gbps,
        "unit": "GB/s",
        "tokens_per_s": work.batch / (avg * 1e-3),
        "ms_per_step": avg,
        "algorithmic_bytes": nbytes,
        "roofline": {"bound": "hbm", "kernel": "singe_paged_decode_f8kv_wide_d128_b16", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": None, "step_avg_us": avg * 1e3,
                     "step_median_us": median * 1e3},
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU exchange and every box here has one "
              "GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from singe_amd import _native, synthetic
    from singe_amd.kernel import attention as A

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.only_latent:
        print(json.dumps({"latent": latent_section(4)}), flush=True)
        return
    if args.workers:
        _native.lib().singe_hip_set_decode_workers(args.workers)

    work = synthetic.paged_decode_workload()
    pools = [(work.key_cache, work.value_cache)]
    for extra in range(1, POOLS):
        other = synthetic.paged_decode_workload(seed=synthetic.BASE_SEED + 97 * extra)
        pools.append((other.key_cache, other.value_cache))
        del other
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                       work.block_size, work.physical_blocks,
                                                       work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")

    def step(i, phases=3):
        kc, vc = pools[i % POOLS]
        A.paged_kv_decode_attention_bf16(None, out, work.query, kc, vc, lens, table, config, workspace, phases)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - start
    ms_per_step = seconds / args.steps * 1e3

    # The dominant kernel alone (the split kernel): HIP events on its own stream around groups of
    # back-to-back launches (one per KV pool in turn), so the cost of recording an event is spread
    # over the group instead of being charged to one ~50 us launch.
    group = 6
    groups = max(args.steps // group, 5)
    begin = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    finish = [torch.cuda.Event(enable_timing=True) for _ in range(groups)]
    for j in range(groups):
        begin[j].record()
        for i in range(group):
            step(j * group + i, phases=1)
        finish[j].record()
    torch.cuda.synchronize()
    kernel_ms = sorted(b.elapsed_time(f) / group for b, f in zip(begin, finish))
    kernel_avg_ms = sum(kernel_ms) / len(kernel_ms)

    bytes_per_step = work.algorithmic_bytes()
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    achieved = bytes_per_step / (kernel_avg_ms * 1e-3) / 1e9
    result = {
        "metric": "decode attn GB/s",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "paged decode: batch 32, 32q/8kv heads, head_dim 128, bf16, block 16, "
                        "ctx U[512,4096], 16384-block pool (BASELINE config 2)",
            "total_keys": work.total_keys,
            "algorithmic_bytes": bytes_per_step,
            "algorithmic_flops": work.algorithmic_flops(),
            "workers": int(_native.lib().singe_hip_decode_workers(config._c())),
            "kv_pools_rotated": POOLS,
        },
        "tokens_per_s": work.batch / (ms_per_step * 1e-3),
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "roofline": {
            "bound": "hbm",
            "kernel": "singe_paged_decode_bf16_d128_g1_b16",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": DECODE_TRAFFIC_BYTES if not args.workers else None,
            "kernel_avg_us": kernel_avg_ms * 1e3,
            "kernel_median_us": kernel_ms[len(kernel_ms) // 2] * 1e3,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(work)
    if not args.no_prefill:
        del pools, workspace
        torch.cuda.empty_cache()
        result["prefill"] = prefill_section(args.prefill_steps)
    if not args.no_extras:
        try:
            del pools, workspace
        except NameError:
            pass
        torch.cuda.empty_cache()
        result["chunked_prefill"] = chunked_prefill_section(20)
        torch.cuda.empty_cache()
        result["fp8_decode"] = fp8_decode_section(10)
        torch.cuda.empty_cache()
        result["dense_f32"] = dense_f32_section(100)
        torch.cuda.empty_cache()
        result["latent"] = latent_section(8)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
