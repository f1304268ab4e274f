"""Shared helpers of the GPU parity tests: a Backend per test module, uploads, and the north-star tolerance."""
import numpy as np

ATOL, RTOL = 2e-3, 1e-2     # fp32-accumulated outputs: max-abs 2e-3 and relative 1e-2 of the oracle


def backend(budget=8 << 30):
    from straydog_amd.backend import Backend
    return Backend(0, budget)


def close_enough(got, want, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    error = np.abs(got - want)
    worst = float(error.max()) if error.size else 0.0
    scale = float(np.abs(want).max()) if want.size else 0.0
    relative = float(np.sqrt((error ** 2).sum() / max((want ** 2).sum(), 1e-300)))
    assert worst <= ATOL, f"{what}: max-abs error {worst:.3e} > {ATOL}"
    assert relative <= RTOL, f"{what}: relative L2 error {relative:.3e} > {RTOL}"
    assert np.all(error <= ATOL + RTOL * np.abs(want)), f"{what}: element outside atol+rtol"
    return worst, relative, scale


def make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes, spare_pages=2, dtype=np.float32):
    """A shuffled paged cache filled by the ORACLE's encoder (so attention tests do not depend on the GPU writer).
    Returns (pool struct, its buffer, host pool bytes, table array, table buffer)."""
    seqs = len(lengths)
    pages_per = [(n + page_tokens - 1) // page_tokens for n in lengths]
    total = sum(pages_per) + spare_pages
    order = rng.permutation(total)
    stride = max(pages_per)
    table = np.zeros((seqs, stride), dtype=np.int32)
    at = 0
    for s in range(seqs):
        table[s, :pages_per[s]] = order[at:at + pages_per[s]]
        at += pages_per[s]
    host = np.zeros(oracle.pool_bytes(total, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
    for s in range(seqs):
        k = rng.standard_normal((1, lengths[s], kv_heads, dim)).astype(dtype).astype(np.float32)
        v = rng.standard_normal((1, lengths[s], kv_heads, dim)).astype(dtype).astype(np.float32)
        oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, table[s:s + 1], np.zeros(1, np.int32), k, v)
    pool, buffer = gpu.kv_pool(total, page_tokens, kv_heads, dim, row_bytes)
    gpu.write_buffer(buffer, 0, host)
    table_buffer = gpu.upload(table)
    return pool, buffer, host, table, table_buffer
