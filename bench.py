#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of the Q8_0 paged grouped-query decode attention (sdx_paged_attention: chunk kernel + merge) over
one batch of synthetic, HBM-resident inputs.  The default workload is BASELINE.json configs[1]: 32 sequences with
lengths drawn uniformly from [1024, 32768], 32 query heads over 4 K/V heads, head_dim 128, 256-token pages behind a
shuffled page table, FP16 queries and outputs.  The one JSON line also carries, under "also", the all-32768-token case
of the same shape (the north-star target), config 0, the chunked prefill of config 2 (MFMA-bound: TFLOP/s against the
dense FP16 peak), the verify span of config 3 and the sparse path of config 4.

    python bench.py --gpus 1 --steps 100 --warmup 200 [--workload config1|config1_32k|config0|config2|config3|config4]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SETTLE_MS = 60.0            # untimed device time of the same steps before every timed pass
HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense FP16/BF16 MFMA, published

# HBM bytes per launch of each workload's dominant kernel.  These are not measured in this run: they are the figures of the
# rocprofv3 counter runs summarised under profiles/ (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, the factors being what the same
# counters read for the library's 1 GiB copy kernel), kept here so that the bench line carries them; `traffic_source` names the
# summary.  A counter run cannot share a process with the timed passes.
PROFILED_TRAFFIC = {
    "config1": (626.8e6, "profiles/paged_attention_q8_d128_decode_config1.md"),
    "config1_32k": (1147.4e6, "profiles/paged_attention_q8_d128_decode_config1_32k.md"),
    "config0": (2.60e6, "profiles/paged_attention_q8_d128_decode_config0.md"),
    "config3": (1157.6e6, "profiles/paged_attention_q8_d128_verify_config3.md"),
    "config2": (117.3e6, "profiles/prefill_dense_d128_config2.md"),        # prefill_dense64_kernel, averaged over a prompt's four launches
    "config4": (278.0e6, "profiles/sparse_path_config4.md"),               # index_interval_kernel
}


def host_threads():
    """(logical cores of this host, threads the CPU baselines use): the oracle runs OpenMP over (sequence, K/V head) or over
    keys, on at most 16 threads (the box's CPU share for one GPU)."""
    cores = os.cpu_count() or 1
    try:
        cores_allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        cores_allowed = cores
    return cores, min(cores_allowed, 16)


def timed(gpu, step, steps, warmup):
    """(ms per step over the whole stream, ms per launch of the dominant kernel) for `steps` steps after `warmup`.  Two passes of
    the same `steps` steps: the first is bracketed by two events and nothing else (the step time), in the second the library
    also times every launch of the dominant kernel through the extended launch, whose events take the kernel's own start and
    end (the duration a tracer reports) -- the queue stalls for a few microseconds per such launch, which the step time
    should not carry."""
    for _ in range(warmup):
        step()
    gpu.synchronize()
    # The box's clocks settle under tens of milliseconds of the same load, whatever --warmup says: the same steps go on, untimed,
    # until SETTLE_MS of device time have passed (in stretches between two events, so that the queue never runs dry inside one).
    settled, settle_steps, stretch = 0.0, 0, 4
    while settled < SETTLE_MS and settle_steps < 20000:
        begin = gpu.event()
        for _ in range(stretch):
            step()
        end = gpu.event()
        took = gpu.elapsed_ms(begin, end)
        gpu.events_clear()
        settled += took
        settle_steps += stretch
        stretch = max(4, min(2000, int(stretch * 10.0 / max(took, 1e-3))))        # about 10 ms a stretch
    timed.settle_ms, timed.settle_steps = settled, settle_steps
    # A step of a few microseconds takes the host about as long to submit as the device to run: a host hiccup inside the timed
    # steps would then be measured as the device's.  Such steps are queued behind a few hundred microseconds of copying (untimed:
    # the first event comes after it in the stream), so that the device never waits for the host between the two events.
    head = None
    if settle_steps and settled / settle_steps < 0.04:
        head = (gpu.buffer(256 << 20), gpu.buffer(256 << 20))
        gpu.synchronize()
        for _ in range(3):
            gpu.copy(head[0].base(), head[1].base(), 256 << 20)
    begin = gpu.event()
    for _ in range(steps):
        step()
    end = gpu.event()
    total = gpu.elapsed_ms(begin, end)
    gpu.events_clear()
    if head:
        for buffer in head:
            gpu.release(buffer)
    gpu.profile(True)
    for _ in range(steps):
        step()
    kernel_ms, launches = gpu.profile_read()
    gpu.profile(False)
    return total / steps, (kernel_ms / launches if launches else None)


def measured_ceilings(gpu, size=1 << 30, repeats=10):
    """Measured GB/s of the library's plain copy kernel (read + write) and of its read-only streaming probe (coalesced
    16-byte non-temporal loads): what this box's HBM delivers to the simplest kernels."""
    a, b = gpu.buffer(size), gpu.buffer(size)
    rates = []
    for run, moved in ((lambda: gpu.copy(b.base(), a.base(), size), 2 * size), (lambda: gpu.read_probe(a.base(), size), size)):
        for _ in range(3):
            run()
        gpu.synchronize()
        begin = gpu.event()
        for _ in range(repeats):
            run()
        end = gpu.event()
        rates.append(moved / (gpu.elapsed_ms(begin, end) / repeats) / 1e6)
        gpu.events_clear()
    gpu.release(a); gpu.release(b)
    return rates


def measured_mfma_ceiling(gpu, live, trips=20000, repeats=5):
    """Measured TFLOP/s of back-to-back independent v_mfma_f32_16x16x32_f16 on every SIMD (two waves each): the dense FP16
    rate the box delivers at the clock it holds under that load -- for tame constant operands, or (live) for pseudo-random
    operands that change from product to product, as a kernel on real data presents them."""
    gpu.mfma_probe(trips, live)
    gpu.synchronize()
    begin = gpu.event()
    flops = sum(gpu.mfma_probe(trips, live) for _ in range(repeats))
    end = gpu.event()
    rate = flops / gpu.elapsed_ms(begin, end) / 1e9
    gpu.events_clear()
    return rate


def paged_result(gpu, work, steps, warmup):
    ms, kernel_ms = timed(gpu, work.step, steps, warmup)
    size = work.algorithmic_bytes()
    return {
        "ms_per_step": ms, "us_per_step": ms * 1e3, "kernel_us": None if kernel_ms is None else kernel_ms * 1e3,
        "algorithmic_bytes": size, "gbps": size / ms / 1e6, "frac_of_hbm_peak": size / ms / 1e6 / HBM_PEAK_GBPS,
        "kernel_gbps": None if kernel_ms is None else size / kernel_ms / 1e6,
        "tokens_per_s": work.seqs * work.span / (ms * 1e-3), "tflops": work.flops() / ms / 1e9,
        "settle_ms": timed.settle_ms, "settle_steps": timed.settle_steps,
    }


def cpu_baseline_paged(work, sample_seqs, threads, budget_seconds=12.0):
    """The CPU oracle on the first `sample_seqs` sequences of the same workload, timed on this host's cores: passes are
    repeated until about `budget_seconds` of wall time are spent and the fastest one counts.  Also returns the GPU-vs-oracle
    error on those sequences."""
    import oracle
    pool = work.read_pool()
    q = work.read_queries()[:sample_seqs]
    got = work.read_output()[:sample_seqs]
    table, positions = work.table[:sample_seqs], work.positions[:sample_seqs]
    best, spent, passes = None, 0.0, 0
    while passes < 2 or (spent < budget_seconds and passes < 200):
        start = time.perf_counter()
        want = oracle.paged_attention(pool, work.row_bytes, work.page_tokens, work.kv_heads, work.dim, table, positions, q, work.scale,
                                      threads=threads)
        seconds = time.perf_counter() - start
        best = seconds if best is None else min(best, seconds)
        spent += seconds
        passes += 1
    rows = int(work.lengths[:sample_seqs].sum()) * work.kv_heads * 2 * work.row_bytes
    error = float(np.abs(got - want).max())
    return {"value": rows / best / 1e9, "unit": "GB/s", "cores": threads, "host_cores": host_threads()[0], "kind": "port",
            "sample": f"{sample_seqs} of {work.seqs} sequences of the same workload ({int(work.lengths[:sample_seqs].sum())} cached tokens, "
                      f"{rows / 1e6:.0f} MB of K/V rows), fastest of {passes} passes in {spent:.1f} s, OpenMP over (sequence, K/V head)",
            "tokens_per_s": sample_seqs * work.span / best}, error


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    # (the memory and fabric clocks of the box take tens of milliseconds of sustained traffic to settle, and a pass timed after
    # 10 steps reads 1.5-4 % low: whatever --warmup is, every timed pass comes after SETTLE_MS more of the same steps)
    parser.add_argument("--steps", type=int, default=100)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--workload", default="config1")
    parser.add_argument("--no-also", action="store_true", help="measure only the named workload")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no second device); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    from straydog_amd.backend import Backend
    from straydog_amd import workloads

    gpu = Backend(0, 64 << 30)
    lengths = workloads.config1_lengths()
    builders = {
        "config1": lambda: workloads.PagedWorkload(gpu, lengths, seed=1),
        "config1_32k": lambda: workloads.PagedWorkload(gpu, [32768] * 32, seed=0x101),
        "config0": lambda: workloads.PagedWorkload(gpu, [4096], heads=16, kv_heads=2, seed=0, q_f16=False, out_f16=False),
        "config3": lambda: workloads.PagedWorkload(gpu, [65536 + 5] * 16, span=5, seed=3),
    }
    names = {
        "config1": "configs[1]: 32 seqs, len~U[1024,32768], 32q/4kv heads, d128, Q8_0 pages of 256, fp16 q/out",
        "config1_32k": "configs[1] shape with all 32 sequences at 32768 tokens",
        "config0": "configs[0]: 1 seq, ctx 4096, 16q/2kv heads, d128, fp32 q/out",
        "config3": "configs[3]: 16 seqs, ctx 65536 + span 5, 32q/4kv heads, d128, Q8_0 pages of 256",
        "config2": "configs[2]: 1 prompt of 8192 tokens prefilled in 4 chunks of 2048 (fp16 K/V appended as Q8_0, causal attention), 32q/4kv heads, d128",
        "config4": "configs[4]: batch 8, ctx 131072, 64x128 bf16 indexer, top-2048, 64 heads over bf16 latents 576/512",
    }
    copy_rate, read_rate = measured_ceilings(gpu)
    short_warmup = max(args.warmup // 5, 2)       # for the workloads whose steps are long or many launches: the same settling, fewer steps

    def run_paged(name, with_cpu, budget_seconds=12.0, warmup=None):
        work = builders[name]()
        result = paged_result(gpu, work, args.steps, args.warmup if warmup is None else warmup)
        result["warmup"] = args.warmup if warmup is None else warmup
        # what the same pool gives to the decode kernel's order of asking with the arithmetic left out (the pool holds a little
        # more than the batch's rows: whole pages)
        for _ in range(3):
            gpu.paged_stream_probe(work.pool)
        gpu.synchronize()
        begin = gpu.event()
        for _ in range(10):
            read = gpu.paged_stream_probe(work.pool)
        end = gpu.event()
        result["paged_stream_probe_gbps"] = read / (gpu.elapsed_ms(begin, end) / 10) / 1e6
        gpu.events_clear()
        baseline = None
        if with_cpu:
            threads = host_threads()[1]
            sample = {"config1": 32, "config1_32k": 4, "config0": 1, "config3": 1}[name]
            baseline, error = cpu_baseline_paged(work, min(sample, work.seqs), threads, budget_seconds)
            result["max_abs_error_vs_oracle_on_sample"] = error
        work.release()
        return result, baseline

    def cpu_baseline_sparse(work, b=0):
        """The oracle on sequence b of the batch: canonical index scores over every key, the top-k rule, the gather attention.
        One pass (about 131072 x 64 chains of 128 fused multiply-adds); also checks the GPU's indices and outputs of that sequence."""
        import oracle
        cores, threads = host_threads()
        bf16 = lambda bits: (np.asarray(bits).astype(np.uint32) << 16).view(np.float32)
        q = bf16(gpu.read_buffer(work.q_index, b * work.index_heads * work.index_dim * 2, np.uint16, work.index_heads * work.index_dim)).reshape(1, work.index_heads, -1)
        keys = bf16(gpu.read_buffer(work.keys, b * work.context * work.index_dim * 2, np.uint16, work.context * work.index_dim)).reshape(work.context, -1)
        weights = gpu.read_buffer(work.weights, b * work.index_heads * 4, np.float32, work.index_heads).reshape(1, -1)
        aq = bf16(gpu.read_buffer(work.q, b * work.heads * work.kdim * 2, np.uint16, work.heads * work.kdim)).reshape(1, work.heads, work.kdim)
        latents = gpu.read_buffer(work.latents, b * work.context * work.kdim * 2, np.uint16, work.context * work.kdim).reshape(work.context, work.kdim)
        start = time.perf_counter()
        scores = oracle.index_scores(q, keys, weights, np.array([work.context], np.int32), 1.0, threads=threads)
        chosen = oracle.top_k(scores, work.k)
        index_seconds = time.perf_counter() - start
        want = oracle.latent_attention(aq, None, None, 0, latents, chosen, None, work.vdim, work.scale)
        seconds = time.perf_counter() - start
        got_indices = gpu.read_buffer(work.indices, b * work.k * 4, np.int32, work.k)
        got = gpu.read_buffer(work.out, b * work.heads * work.vdim * 4, np.float32, work.heads * work.vdim).reshape(work.heads, work.vdim)
        return {"value": seconds * work.batch * 1e6, "unit": "us/step", "cores": threads, "host_cores": cores, "kind": "port",
                "sample": f"sequence {b} of {work.batch} (index scores over {work.context} keys in the canonical order, top-{work.k}, gather attention), one pass of "
                          f"{seconds:.2f} s ({index_seconds:.2f} s of it the indexer), scaled by {work.batch} to the step; OpenMP over keys",
                "indices_equal_oracle_on_sample": bool(np.array_equal(got_indices, chosen[0])),
                "max_abs_error_vs_oracle_on_sample": float(np.abs(got - want[0]).max())}

    def run_sparse(with_cpu=True):
        work = workloads.SparseWorkload(gpu)
        ms_index, bounds_ms = timed(gpu, work.step_index, max(args.steps // 5, 3), short_warmup)
        settle_ms = timed.settle_ms
        ms_attention, gather_ms = timed(gpu, work.step_attention, max(args.steps // 5, 3), short_warmup)
        settle_ms += timed.settle_ms
        size, keys = work.algorithmic_bytes(), work.batch * work.context * work.index_dim * 2
        sparse_baseline = cpu_baseline_sparse(work) if with_cpu and not args.no_cpu else None
        work.release()
        total = ms_index + ms_attention
        # the timed launches: the score bounds over all keys (index_interval_kernel), the gather kernel
        return {"us_per_step": total * 1e3, "index_topk_us": ms_index * 1e3, "gather_attention_us": ms_attention * 1e3,
                "kernel_us": None if bounds_ms is None else bounds_ms * 1e3, "key_bytes": keys,
                "gather_kernel_us": None if gather_ms is None else gather_ms * 1e3,
                "algorithmic_bytes": size, "gbps": size / total / 1e6, "frac_of_hbm_peak": size / total / 1e6 / HBM_PEAK_GBPS,
                "settle_ms": settle_ms, "cpu_baseline": sparse_baseline}

    def cpu_baseline_prefill(work, tokens=(2040, 4090, 6140, 8184), rows=8):
        """The oracle on `rows` consecutive query tokens near the end of each chunk (each attends the cache up to its own position),
        all heads: a stated part of the prompt's causal work, timed, and compared with the GPU's outputs of those tokens."""
        import oracle
        cores, threads = host_threads()
        out = work.read(work.out, work.tokens * work.heads * work.dim).reshape(work.tokens, work.heads, work.dim)
        q = work.read(work.q, work.tokens * work.heads * work.dim).reshape(work.tokens, work.heads, work.dim)
        pool = gpu.read_buffer(work.pool_buffer, 0, np.uint8, work.pool_buffer.size)
        wanted = [t + r for t in tokens for r in range(rows)]
        # every sampled token as a sequence of its own over the same pages: the oracle's threads run over (sequence, K/V head)
        table = np.repeat(work.table, len(wanted), axis=0)
        best, error = None, 0.0
        for _ in range(3):
            start = time.perf_counter()
            want = oracle.paged_attention(pool, work.row_bytes, work.page_tokens, work.kv_heads, work.dim, table, np.array(wanted, np.int32),
                                          q[wanted][:, None], work.scale, threads=threads)
            seconds = time.perf_counter() - start
            best = seconds if best is None else min(best, seconds)
        error = float(np.abs(out[wanted] - want[:, 0]).max())
        flops = 4 * work.heads * work.dim * sum(t + 1 for t in wanted)
        return {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "host_cores": cores, "kind": "port",
                "sample": f"{len(wanted)} of {work.tokens} query tokens ({rows} at each of positions {list(tokens)}), all {work.heads} heads, {flops / 1e9:.2f} GFLOP of the "
                          f"prompt's {work.flops() / 1e9:.0f}, fastest of 3 passes ({best:.2f} s), OpenMP over (token, K/V head)",
                "max_abs_error_vs_oracle_on_sample": error}

    def run_prefill(with_cpu=True):
        # a step = the prompt's four chunks through sdx_prefill_chunk (K/V append + attention in one call a chunk, the cached rows'
        # operand tiles kept between chunks); the same prompt through sdx_kv_write + sdx_paged_attention is timed beside it
        work = workloads.PrefillWorkload(gpu)
        steps = max(args.steps // 5, 3)
        separate_ms, _ = timed(gpu, work.step, steps, short_warmup)
        ms, kernel_ms = timed(gpu, work.step_chunks, steps, short_warmup)
        flops, size = work.flops(), work.algorithmic_bytes()
        prefill_baseline = cpu_baseline_prefill(work) if with_cpu and not args.no_cpu else None
        work.release()
        # the timed kernel launches are the 4 attention kernels of a step (not the kernel that appends the rows and builds the tiles)
        return {"ms_per_step": ms, "us_per_step": ms * 1e3, "kernel_us": None if kernel_ms is None else kernel_ms * 4e3, "flops": flops,
                "tflops": flops / ms / 1e9, "frac_of_mfma_peak": flops / ms / 1e9 / MFMA_PEAK_TFLOPS,
                "kernel_tflops": None if kernel_ms is None else flops / (4 * kernel_ms) / 1e9,
                "us_per_step_separate_calls": separate_ms * 1e3,
                "algorithmic_bytes": size, "gbps": size / ms / 1e6, "frac_of_hbm_peak": size / ms / 1e6 / HBM_PEAK_GBPS,
                "tokens_per_s": work.tokens / (ms * 1e-3), "settle_ms": timed.settle_ms, "cpu_baseline": prefill_baseline}

    def run_block_index():
        # Qwen's block indexer (scores + choice of 512 blocks) at 242K tokens: a decode row, and a prefill chunk of 256 rows
        out = {}
        for name, rows in (("decode_row", 1), ("verify_rows_5", 5), ("prefill_chunk_256", 256)):
            work = workloads.BlockIndexWorkload(gpu, rows)
            ms, kernel_ms = timed(gpu, work.step, max(args.steps // 5, 3), 2)
            out[name] = {"us_per_call": ms * 1e3, "us_per_token": ms * 1e3 / rows, "scores_kernel_us": None if kernel_ms is None else kernel_ms * 1e3,
                         "scores_gbps": None if kernel_ms is None else work.complete() * 512 / kernel_ms / 1e6,
                         "scores_fp32_tflops": None if kernel_ms is None else work.flops() / kernel_ms / 1e9}
            if rows > 8:
                # the same selection by intervals (sdx_qsa_index_interval): FP16 matrix products bound every score, only the blocks
                # around the 512th best are scored exactly; the second figure keeps the packed keys from the call before, as the
                # chunks of one prompt do
                work.with_interval()
                ms, kernel_ms = timed(gpu, work.step_interval, max(args.steps // 5, 3), 2)
                undecided = work.undecided()
                kept_ms, _ = timed(gpu, lambda: work.step_interval(True), max(args.steps // 5, 3), 2)
                out[name].update({"interval_us_per_call": ms * 1e3, "interval_us_per_token": ms * 1e3 / rows,
                                  "interval_scan_kernel_us": None if kernel_ms is None else kernel_ms * 1e3,
                                  "interval_scan_fp16_tflops": None if kernel_ms is None else work.flops() / kernel_ms / 1e9,
                                  "interval_kept_operands_us_per_call": kept_ms * 1e3, "interval_rows_left_to_exact_kernels": undecided})
            if True:
                # the attention over the rows' selections (24q/2kv heads, 256 columns, Q8_0 rows in the reference's state layout);
                # the 256 rows of a prompt chunk select overlapping rows, so their figure counts bytes the caches serve
                work.with_attention()
                ms, kernel_ms = timed(gpu, work.step_attention, max(args.steps // 5, 3), 2)
                out[name].update({"selected_attention_us": ms * 1e3, "selected_attention_kernel_us": None if kernel_ms is None else kernel_ms * 1e3,
                                  "selected_attention_gbps": work.attention_bytes() / ms / 1e6})
                if rows > 8:
                    # the same attention as a union walk (sdx_selected_attention_union), on these selections (independent queries:
                    # nothing to share) and on selections that overlap as consecutive prompt tokens' do (runs of 16 similar queries)
                    work.with_union()
                    ms, _ = timed(gpu, work.step_attention_union, 3, 1)
                    out[name]["selected_attention_union_us"] = ms * 1e3
                    work.similar_queries()
                    work.step()
                    ms, _ = timed(gpu, work.step_attention, 3, 1)
                    union_ms, _ = timed(gpu, work.step_attention_union, 3, 1)
                    out[name].update({"similar_queries_selected_attention_us": ms * 1e3, "similar_queries_selected_attention_union_us": union_ms * 1e3})
            work.release()
            if rows <= 8:
                stage = workloads.QwenStageWorkload(gpu, rows)
                ms, _ = timed(gpu, stage.step, max(args.steps // 5, 3), 2)
                out[name]["whole_stage_us"] = ms * 1e3        # norm + rope + K/V append + pooling, index, attention over the selection, gate
                stage.release()
        return out

    def run_host_resident():
        # the selection-list attention of rows at 242K tokens when the sequence's K/V rows are not in HBM: read over the bus entry by
        # entry (a pool in mapped host memory), or through the union of the selected blocks gathered into a VRAM stage first
        # (sdx_kv_cache_gather over a sequence parked in the cache's host tier); the same rows from HBM beside them, same bits
        out = {}
        for name, rows, similar in (("decode_row", 1, False), ("verify_rows_5", 5, False), ("prefill_chunk_256_similar_queries", 256, True)):
            work = workloads.HostResidentWorkload(gpu, rows, similar)
            resident_ms, _ = timed(gpu, work.step_resident, max(args.steps // 5, 3), 2)
            want = work.read_output()
            bus_ms, _ = timed(gpu, work.step_over_the_bus, 3, 1)
            same = bool(np.array_equal(work.read_output(), want))
            work.park()
            gathered_ms, _ = timed(gpu, work.step_gathered, 3, 1)
            same = same and bool(np.array_equal(work.read_output(), want))
            out[name] = {"rows": rows, "resident_in_hbm_us": resident_ms * 1e3, "read_over_the_bus_us": bus_ms * 1e3, "union_gathered_us": gathered_ms * 1e3,
                         "union_positions": work.union_positions, "gather_calls": work.gather_calls, "selected_positions": rows * 2051,
                         "same_bits_as_resident": same}
            work.release()
        return out

    if args.workload == "block_index":
        # the Qwen block indexer alone (what profiles/block_index_242k.md traces): not a BASELINE config, no headline metric
        print(json.dumps({"workload": "Qwen block indexer at 242K tokens", "steps": args.steps, **run_block_index(), "host_resident_242k": run_host_resident()}))
        gpu.close()
        return
    if args.workload == "config4":
        main_result = run_sparse()
        baseline = main_result.pop("cpu_baseline")
    elif args.workload == "config2":
        main_result = run_prefill()
        baseline = main_result.pop("cpu_baseline")
    else:
        main_result, baseline = run_paged(args.workload, not args.no_cpu)
    also = {}
    if not args.no_also:
        for name in ("config1_32k", "config0", "config3"):
            if name != args.workload:
                # each config's CPU baseline beside it: the oracle on a stated part of the same workload, a few seconds each
                # (30 untimed steps first: the clocks of a box move for the first ~25 launches of a heavy kernel, see
                # profiles/paged_attention_q8_d128_verify_config3.md; the figure is the rate the loop then keeps)
                also[name], also_baseline = run_paged(name, not args.no_cpu, budget_seconds=3.0, warmup=max(args.warmup, 30))
                also[name]["cpu_baseline"] = also_baseline
                also[name]["workload"] = names[name]
                also[name]["traffic"], also[name]["traffic_source"] = PROFILED_TRAFFIC[name]
                kernel = also[name]["kernel_us"] or also[name]["us_per_step"]
                also[name]["roofline"] = {"bound": "hbm", "achieved": also[name]["algorithmic_bytes"] / kernel / 1e3, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                          "frac": also[name]["algorithmic_bytes"] / kernel / 1e3 / HBM_PEAK_GBPS, "traffic": PROFILED_TRAFFIC[name][0],
                                          "kernel": "paged_attention_kernel<128,3,Q8_0>" if name == "config3" else "paged_attention_kernel<128,1,Q8_0>",
                                          "kernel_us": also[name]["kernel_us"]}
        if args.workload != "config2":
            also["config2"] = run_prefill()
            also["config2"]["workload"] = names["config2"]
            also["config2"]["traffic"], also["config2"]["traffic_source"] = PROFILED_TRAFFIC["config2"]
            achieved = also["config2"]["kernel_tflops"] or also["config2"]["tflops"]
            also["config2"]["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                                           "traffic": PROFILED_TRAFFIC["config2"][0], "kernel": "prefill_dense64_kernel<128>", "kernel_us": also["config2"]["kernel_us"]}
            also["config2"]["measured_mfma_tflops"] = measured_mfma_ceiling(gpu, False)
            also["config2"]["measured_mfma_tflops_live_operands"] = measured_mfma_ceiling(gpu, True)
        if args.workload != "config4":
            also["config4"] = run_sparse()
            also["config4"]["workload"] = names["config4"]
            also["config4"]["traffic"], also["config4"]["traffic_source"] = PROFILED_TRAFFIC["config4"]
            if also["config4"]["kernel_us"]:
                achieved = also["config4"]["key_bytes"] / also["config4"]["kernel_us"] / 1e3
                also["config4"]["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                                               "traffic": PROFILED_TRAFFIC["config4"][0], "kernel": "index_interval_kernel<64>", "kernel_us": also["config4"]["kernel_us"]}
        also["block_index_242k"] = run_block_index()
        also["block_index_242k"]["workload"] = "Qwen block indexer: 4x128 index heads, 60.5K complete blocks of a 262144-token context, top 512 blocks"
        also["host_resident_242k"] = run_host_resident()
        also["host_resident_242k"]["workload"] = "selection-list attention at 242K tokens (24q/2kv heads, 256 columns, Q8_0) over K/V rows that are not in HBM"

    kernel_us = main_result.get("kernel_us")
    achieved = main_result["algorithmic_bytes"] / (kernel_us * 1e-6) / 1e9 if kernel_us else main_result["gbps"]
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                "traffic": PROFILED_TRAFFIC[args.workload][0], "traffic_source": PROFILED_TRAFFIC[args.workload][1],
                "kernel": "paged_attention_kernel<128,3,Q8_0>" if args.workload == "config3" else "paged_attention_kernel<128,1,Q8_0>", "kernel_us": kernel_us, "measured_copy_gbps": copy_rate, "measured_read_gbps": read_rate,
                "measured_paged_stream_gbps": main_result.get("paged_stream_probe_gbps")}
    if args.workload == "config4" and kernel_us:
        # the dominant kernel reads every index key once: its algorithmic bytes are the keys
        achieved = main_result["key_bytes"] / (kernel_us * 1e-6) / 1e9
        roofline.update({"achieved": achieved, "frac": achieved / HBM_PEAK_GBPS, "kernel": "index_interval_kernel<64>"})
    if args.workload == "config2":
        achieved = main_result["kernel_tflops"] or main_result["tflops"]
        roofline = {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                    "traffic": PROFILED_TRAFFIC["config2"][0], "traffic_source": PROFILED_TRAFFIC["config2"][1], "kernel": "prefill_dense64_kernel<128>", "kernel_us": kernel_us,
                    "measured_mfma_tflops": measured_mfma_ceiling(gpu, False),
                    "measured_mfma_tflops_live_operands": measured_mfma_ceiling(gpu, True)}
    line = {
        "metric": "Q8_0 decode-attn HBM GB/s", "value": main_result["gbps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_ms": main_result.get("settle_ms"), "ms_per_step": main_result.get("ms_per_step", main_result["us_per_step"] / 1e3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8 K/V x fp16 MFMA, fp32 accumulate", "data": "synthetic",
        "config": {"workload": names[args.workload], "batch": 32 if args.workload.startswith("config1") else None},
        "tokens_per_s": main_result.get("tokens_per_s"), "frac_of_hbm_peak": main_result["frac_of_hbm_peak"],
        "roofline": roofline,
        "cpu_baseline": baseline, "host": {"cores": host_threads()[0], "cpu_threads_used": host_threads()[1]}, "detail": main_result, "also": also,
    }
    print(json.dumps(line))
    gpu.close()


if __name__ == "__main__":
    main()
