"""Synthetic workloads of the attention path, built on the GPU through the C ABI (no host-side arithmetic):
the BASELINE configurations' shapes with seeded N(0,1) inputs, K/V quantised into the paged cache by the
library's own writer.  Used by bench.py, __graft_entry__.smoke() and the full-size GPU tests."""
import numpy as np

ROW_Q8 = {128: 136, 256: 272}


def stream(seed, index):
    """The seed of tensor `index` of a workload: every tensor is its own xorshift64 stream, (0x9e3779b97f4a7c15 ^ seed) + index,
    `seed` being the BASELINE config's number (the reference's habit, crates/straydog-engine/tests/attention_gpu.rs:91)."""
    return ((0x9e3779b97f4a7c15 ^ seed) + index) & 0xffffffffffffffff


class PagedWorkload:
    """A batch of sequences in a shuffled paged Q8_0 cache, with `span` query rows each."""

    def __init__(self, gpu, lengths, span=1, heads=32, kv_heads=4, dim=128, page_tokens=256, seed=1, q_f16=True, out_f16=True,
                 row_bytes=None, page_seed=None):
        self.gpu, self.span, self.heads, self.kv_heads, self.dim, self.page_tokens = gpu, span, heads, kv_heads, dim, page_tokens
        self.lengths = np.asarray(lengths, dtype=np.int64)            # cached tokens per sequence, the span's rows included
        self.seqs = len(lengths)
        self.row_bytes = row_bytes or ROW_Q8[dim]
        self.q_f16, self.out_f16 = q_f16, out_f16
        rng = np.random.default_rng(seed if page_seed is None else page_seed)     # where the pages lie; the rows are `seed`'s
        pages_per = (self.lengths + page_tokens - 1) // page_tokens
        self.page_count = int(pages_per.sum())
        self.table_stride = int(pages_per.max())
        order = rng.permutation(self.page_count).astype(np.int32)
        self.table = np.zeros((self.seqs, self.table_stride), dtype=np.int32)
        at = 0
        for s in range(self.seqs):
            self.table[s, :pages_per[s]] = order[at:at + pages_per[s]]
            at += int(pages_per[s])
        self.positions = (self.lengths - span).astype(np.int32)       # position of each sequence's first query row
        self.max_context = int(self.lengths.max())
        self.scale = float(1.0 / np.sqrt(np.float32(dim)))
        self.pool, self.pool_buffer = gpu.kv_pool(self.page_count, page_tokens, kv_heads, dim, self.row_bytes)
        self.table_buffer = gpu.upload(self.table)
        self.position_buffer = gpu.upload(self.positions)
        # K/V: N(0,1) generated on the device a sequence at a time, quantised by sdx_kv_write
        longest = int(self.lengths.max())
        stage_k = gpu.buffer(longest * kv_heads * dim * 4)
        stage_v = gpu.buffer(longest * kv_heads * dim * 4)
        zero = gpu.upload(np.zeros(1, dtype=np.int32))
        for s in range(self.seqs):
            n = int(self.lengths[s])
            gpu.fill_normal(stage_k.base(), n * kv_heads * dim, stream(seed, 2 * s + 1), 0)
            gpu.fill_normal(stage_v.base(), n * kv_heads * dim, stream(seed, 2 * s + 2), 0)
            gpu.kv_write(self.pool, self.table_buffer.at(s * self.table_stride * 4), self.table_stride, zero.base(), stage_k.base(),
                         stage_v.base(), False, 1, n)
        gpu.synchronize()
        for b in (stage_k, stage_v, zero):
            gpu.release(b)
        count = self.seqs * span * heads * dim
        self.q_buffer = gpu.buffer(count * (2 if q_f16 else 4))
        gpu.fill_normal(self.q_buffer.base(), count, stream(seed, 0), 1 if q_f16 else 0)
        self.out_buffer = gpu.buffer(count * (2 if out_f16 else 4))
        self.scratch = gpu.buffer(max(gpu.paged_attention_scratch(self.seqs, span, heads, dim, self.max_context), 4))
        gpu.synchronize()

    def step(self):
        g = self.gpu
        g.paged_attention(self.pool, self.table_buffer.base(), self.table_stride, self.position_buffer.base(), self.max_context,
                          self.q_buffer.base(), self.q_f16, self.seqs, self.span, self.heads, self.scale, self.out_buffer.base(),
                          self.out_f16, self.scratch)

    def algorithmic_bytes(self):
        """Bytes one step must move: every cached row of every K/V head once (keys and values), the page-table entries,
        the queries and the outputs."""
        rows = int(self.lengths.sum()) * self.kv_heads * 2 * self.row_bytes
        table = int(((self.lengths + self.page_tokens - 1) // self.page_tokens).sum()) * 4
        io = self.seqs * self.span * self.heads * self.dim * ((2 if self.q_f16 else 4) + (2 if self.out_f16 else 4))
        return rows + table + io

    def flops(self):
        # 2 products (QK^T and PV) x 2 flops per (query row, key, column)
        visible = sum(int(self.lengths[s] - self.span + r + 1) for s in range(self.seqs) for r in range(self.span))
        return 4 * self.heads * self.dim * visible

    def read_output(self):
        count = self.seqs * self.span * self.heads * self.dim
        out = self.gpu.read_buffer(self.out_buffer, 0, np.float16 if self.out_f16 else np.float32, count)
        return out.astype(np.float32).reshape(self.seqs, self.span, self.heads, self.dim)

    def read_queries(self):
        count = self.seqs * self.span * self.heads * self.dim
        q = self.gpu.read_buffer(self.q_buffer, 0, np.float16 if self.q_f16 else np.float32, count)
        return q.astype(np.float32).reshape(self.seqs, self.span, self.heads, self.dim)

    def read_pool(self):
        return self.gpu.read_buffer(self.pool_buffer, 0, np.uint8, self.pool_buffer.size)

    def release(self):
        for b in (self.pool_buffer, self.table_buffer, self.position_buffer, self.q_buffer, self.out_buffer, self.scratch):
            self.gpu.release(b)


class PrefillWorkload:
    """BASELINE config 2: one prompt prefilled in chunks.  A step appends each chunk's FP16 K/V rows to the Q8_0 cache and
    runs causal attention of the chunk's queries over the cache so far."""

    def __init__(self, gpu, tokens=8192, chunk=2048, heads=32, kv_heads=4, dim=128, page_tokens=256, seed=2):
        self.gpu, self.tokens, self.chunk, self.heads, self.kv_heads, self.dim, self.page_tokens = gpu, tokens, chunk, heads, kv_heads, dim, page_tokens
        self.row_bytes = ROW_Q8[dim]
        rng = np.random.default_rng(seed)
        self.page_count = (tokens + page_tokens - 1) // page_tokens
        self.table = rng.permutation(self.page_count).astype(np.int32).reshape(1, -1)
        self.scale = float(1.0 / np.sqrt(np.float32(dim)))
        self.pool, self.pool_buffer = gpu.kv_pool(self.page_count, page_tokens, kv_heads, dim, self.row_bytes)
        self.table_buffer = gpu.upload(self.table)
        self.starts = gpu.upload(np.arange(0, tokens, chunk, dtype=np.int32))          # position of each chunk's first token
        self.k = gpu.buffer(tokens * kv_heads * dim * 2)
        self.v = gpu.buffer(tokens * kv_heads * dim * 2)
        self.q = gpu.buffer(tokens * heads * dim * 2)
        self.out = gpu.buffer(tokens * heads * dim * 2)
        gpu.fill_normal(self.k.base(), tokens * kv_heads * dim, stream(seed, 1), 1)
        gpu.fill_normal(self.v.base(), tokens * kv_heads * dim, stream(seed, 2), 1)
        gpu.fill_normal(self.q.base(), tokens * heads * dim, stream(seed, 3), 1)
        self.scratch = gpu.buffer(max(gpu.paged_attention_scratch(1, chunk, heads, dim, tokens), 4))
        self.tiles = None
        gpu.synchronize()

    def step(self):
        g = self.gpu
        for c in range(self.tokens // self.chunk):
            kv_at, q_at = c * self.chunk * self.kv_heads * self.dim * 2, c * self.chunk * self.heads * self.dim * 2
            g.kv_write(self.pool, self.table_buffer.base(), self.table.shape[1], self.starts.at(4 * c), self.k.at(kv_at), self.v.at(kv_at),
                       True, 1, self.chunk)
            g.paged_attention(self.pool, self.table_buffer.base(), self.table.shape[1], self.starts.at(4 * c), self.tokens,
                              self.q.at(q_at), True, 1, self.chunk, self.heads, self.scale, self.out.at(q_at), True, self.scratch)

    def step_chunks(self):
        """The same prompt through sdx_prefill_chunk: K/V append and attention in one call a chunk, the cached rows' operand
        tiles kept between the chunks (everything before a chunk is valid: `valid` is the chunk's own position)."""
        g = self.gpu
        if self.tiles is None:
            self.tiles = g.buffer(g.prefill_tiles_bytes(1, self.kv_heads, self.dim, self.tokens))
        for c in range(self.tokens // self.chunk):
            kv_at, q_at = c * self.chunk * self.kv_heads * self.dim * 2, c * self.chunk * self.heads * self.dim * 2
            g.prefill_chunk(self.pool, self.table_buffer.base(), self.table.shape[1], self.starts.at(4 * c), self.tokens, self.k.at(kv_at),
                            self.v.at(kv_at), True, self.q.at(q_at), True, 1, self.chunk, self.heads, self.scale, self.out.at(q_at), True,
                            self.tiles, self.starts.at(4 * c))

    def flops(self):
        # causal only: 2 products x 2 flops per (query row, visible key, column)
        return 4 * self.heads * self.dim * (self.tokens * (self.tokens + 1) // 2)

    def algorithmic_bytes(self):
        # queries and outputs once, the chunk's K/V rows in and out, and the cache read once per chunk
        chunks = self.tokens // self.chunk
        cache = sum((c + 1) * self.chunk for c in range(chunks)) * self.kv_heads * 2 * self.row_bytes
        io = self.tokens * self.heads * self.dim * 4 + self.tokens * self.kv_heads * self.dim * 2 * 2 + self.tokens * self.kv_heads * 2 * self.row_bytes
        return cache + io

    def read(self, buffer, count):
        return self.gpu.read_buffer(buffer, 0, np.float16, count).astype(np.float32)

    def release(self):
        for b in (self.pool_buffer, self.table_buffer, self.starts, self.k, self.v, self.q, self.out, self.scratch, self.tiles):
            if b is not None:
                self.gpu.release(b)


class SparseWorkload:
    """BASELINE config 4: per sequence, index scores over BF16 keys -> top-k -> gather attention over BF16 latents."""

    def __init__(self, gpu, batch=8, context=131072, index_heads=64, index_dim=128, k=2048, heads=64, kdim=576, vdim=512, seed=4):
        self.gpu, self.batch, self.context, self.index_heads, self.index_dim = gpu, batch, context, index_heads, index_dim
        self.k, self.heads, self.kdim, self.vdim = k, heads, kdim, vdim
        self.scale = float(1.0 / np.sqrt(np.float32(kdim)))
        self.q_index = gpu.buffer(batch * index_heads * index_dim * 2)
        self.keys = gpu.buffer(batch * context * index_dim * 2)
        self.weights = gpu.buffer(batch * index_heads * 4)
        self.visible = gpu.upload(np.full(batch, context, dtype=np.int32))
        self.scores = gpu.buffer(batch * context * 4)
        self.indices = gpu.buffer(batch * k * 4)
        self.q = gpu.buffer(batch * heads * kdim * 2)
        self.latents = gpu.buffer(batch * context * kdim * 2)
        self.out = gpu.buffer(batch * heads * vdim * 4)
        gpu.fill_normal(self.q_index.base(), batch * index_heads * index_dim, stream(seed, 1), 2)
        gpu.fill_normal(self.keys.base(), batch * context * index_dim, stream(seed, 2), 2)
        gpu.fill_uniform(self.weights.base(), batch * index_heads, stream(seed, 3), 0.0, 1.0)
        gpu.fill_normal(self.q.base(), batch * heads * kdim, stream(seed, 4), 2)
        gpu.fill_normal(self.latents.base(), batch * context * kdim, stream(seed, 5), 2)
        gpu.synchronize()

    def step_index(self, keep_scores=False):
        g = self.gpu
        g.index_top_k(self.q_index.base(), self.keys.base(), self.weights.base(), self.visible.base(), self.batch, self.context,
                      self.index_heads, self.index_dim, 1.0, self.scores.base() if keep_scores else None, self.k, self.indices.base())

    def step_attention(self):
        g = self.gpu
        g.latent_attention(self.q.base(), self.latents.base(), self.indices.base(), self.batch, self.context, self.k, self.heads,
                           self.kdim, self.vdim, self.scale, self.out.base())

    def step(self):
        self.step_index()
        self.step_attention()

    def algorithmic_bytes(self):
        keys = self.batch * self.context * self.index_dim * 2
        gather = self.batch * self.k * self.kdim * 2
        small = self.batch * (self.index_heads * self.index_dim * 2 + self.index_heads * 4 + self.k * 4 + self.heads * self.kdim * 2 +
                              self.heads * self.vdim * 4)
        return keys + gather + small

    def release(self):
        for b in (self.q_index, self.keys, self.weights, self.visible, self.scores, self.indices, self.q, self.latents, self.out):
            self.gpu.release(b)


class BlockIndexWorkload:
    """Qwen's block indexer at the reference's long-context point (gpu/sparse_attention.hpp:403-437 is quoted at 242K tokens):
    `steps` rows at positions base.., 4 x 128 index queries each, pooled keys [128][context / 4 + 1] FP32."""

    def __init__(self, gpu, steps, base=242000, context=262144, seed=6):
        self.gpu, self.steps, self.base, self.pool = gpu, steps, base, context // 4 + 1
        self.queries = gpu.buffer(steps * 512 * 4)
        self.blocks = gpu.buffer(128 * self.pool * 4)
        self.scores = gpu.buffer(steps * self.pool * 4)
        self.indices = gpu.buffer(steps * 2052 * 4)
        self.counts = gpu.buffer(steps * 4)
        gpu.fill_normal(self.queries.base(), steps * 512, stream(seed, 1), 0)
        gpu.fill_normal(self.blocks.base(), 128 * self.pool, stream(seed, 2), 0)
        gpu.synchronize()

    def step(self):
        self.gpu.qsa_index(self.queries.base(), 512, self.blocks.base(), self.pool, self.base, self.steps, 2052, self.scores.base(),
                           self.indices.base(), self.counts.base())

    def with_interval(self):
        """Adds the selection by intervals (sdx_qsa_index_interval): its scratch, and the packed keys kept from call to call."""
        self.interval_scratch = self.gpu.buffer(self.gpu.qsa_index_interval_scratch(self.steps, self.pool))
        self.valid = [0]
        return self

    def step_interval(self, keep_operands=False):
        if not keep_operands:
            self.valid[0] = 0
        self.gpu.qsa_index_interval(self.queries.base(), 512, self.blocks.base(), self.pool, self.base, self.steps, 2052, self.scores.base(),
                                    self.indices.base(), self.counts.base(), self.interval_scratch, self.valid)

    def undecided(self):
        return self.gpu.qsa_index_interval_undecided(self.interval_scratch, self.steps, self.pool)

    def with_attention(self, heads=24, kv_heads=2, row_bytes=272, seed=7):
        """Adds the attention over each row's selection: Q8_0 rows of 256 columns in the reference's state layout."""
        gpu, context = self.gpu, (self.pool - 1) * 4
        self.heads, self.kv_heads, self.row_bytes = heads, kv_heads, row_bytes
        self.kv, self.kv_buffer = gpu.kv_pool(1, context, kv_heads, 256, row_bytes)
        k, table = gpu.buffer(8192 * kv_heads * 256 * 2), gpu.upload(np.zeros(1, dtype=np.int32))
        gpu.fill_normal(k.base(), 8192 * kv_heads * 256, stream(seed, 3), 1)
        for first in range(0, context, 8192):                # the cache is filled through the library's own writer
            start = gpu.upload(np.array([first], dtype=np.int32))
            gpu.kv_write(self.kv, table.base(), 1, start.base(), k.base(), k.base(), True, 1, 8192)
            gpu.release(start)
        self.q = gpu.buffer(self.steps * heads * 256 * 2)
        gpu.fill_normal(self.q.base(), self.steps * heads * 256, stream(seed, 4), 1)
        self.out = gpu.buffer(self.steps * heads * 256 * 2)
        self.scratch = gpu.buffer(gpu.selected_attention_scratch(self.steps, kv_heads, 2052))
        gpu.synchronize()
        gpu.release(k); gpu.release(table)
        return self

    def step_attention(self):
        self.gpu.selected_attention(self.kv, None, (self.pool - 1) * 4, self.base, self.indices.base(), 2052, self.counts.base(), self.q.base(), True,
                                    self.steps, self.heads, 0.0625, self.out.base(), True, self.scratch)

    def with_union(self):
        """Adds the union walk over the same selections (sdx_selected_attention_union); call after with_attention."""
        context = (self.pool - 1) * 4
        self.union_scratch = self.gpu.buffer(self.gpu.selected_attention_union_scratch(self.steps, self.heads, self.kv_heads, 2052, context))
        return self

    def step_attention_union(self):
        self.gpu.selected_attention_union(self.kv, None, (self.pool - 1) * 4, self.base, self.indices.base(), 2052, self.counts.base(), self.q.base(), True,
                                          self.steps, self.heads, 0.0625, self.out.base(), True, self.union_scratch)

    def similar_queries(self, alike=16, noise=0.05, seed=9):
        """Index queries as consecutive tokens of a prompt have them: runs of `alike` rows share a query up to a little noise, so
        their selections overlap; call step() afterwards to select with them."""
        rng = np.random.default_rng(seed)
        shared = rng.standard_normal(((self.steps + alike - 1) // alike, 512)).astype(np.float32)
        rows = np.repeat(shared, alike, axis=0)[:self.steps] + noise * rng.standard_normal((self.steps, 512)).astype(np.float32)
        self.gpu.write_buffer(self.queries, 0, rows.astype(np.float32).reshape(-1))

    def attention_bytes(self):
        # the selected rows of both planes of every K/V head, once per row
        return self.steps * 2051 * self.kv_heads * 2 * self.row_bytes

    def complete(self):
        return (self.base + self.steps) // 4

    def algorithmic_bytes(self):
        # the pooled keys of the complete blocks once, the scores out and in again, queries and the selection
        return self.complete() * 128 * 4 + 2 * self.steps * self.complete() * 4 + self.steps * (512 + 2052 + 1) * 4

    def flops(self):
        return 2 * 512 * self.steps * self.complete()

    def release(self):
        for b in (self.queries, self.blocks, self.scores, self.indices, self.counts):
            self.gpu.release(b)
        if hasattr(self, "kv_buffer"):
            for b in (self.kv_buffer, self.q, self.out, self.scratch):
                self.gpu.release(b)
        if hasattr(self, "interval_scratch"):
            self.gpu.release(self.interval_scratch)
        if hasattr(self, "union_scratch"):
            self.gpu.release(self.union_scratch)


class HostResidentWorkload:
    """A sparse (selection-list) pass over a Qwen-shaped sequence at 242K tokens whose K/V rows are not in HBM: the same rows'
    selections attended (a) from the pool in HBM, (b) from a pool in mapped host memory, every selected row read over the bus,
    (c) from a sequence parked in the cache's host tier, through the union of the selected blocks gathered into a VRAM stage
    (sdx_kv_cache_gather).  The selections are the block indexer's own (BlockIndexWorkload)."""

    def __init__(self, gpu, steps, similar=False, base=242000, heads=24, kv_heads=2, row_bytes=272, page_tokens=256, stage_positions=65536, seed=11):
        self.gpu, self.steps, self.base, self.heads, self.kv_heads = gpu, steps, base, heads, kv_heads
        self.context = base + steps
        pages = (self.context + page_tokens - 1) // page_tokens
        self.index = BlockIndexWorkload(gpu, steps, base=base)
        if similar:
            self.index.similar_queries()
        self.index.step()
        self.cache, *_ = gpu.kv_cache(pages, page_tokens, kv_heads, 256, row_bytes, 1, pages * page_tokens)
        gpu.kv_cache_host(self.cache, pages)
        gpu.kv_cache_reserve(self.cache, 0, self.context)
        self.pool, self.table, self.stride = gpu.kv_cache_view(self.cache)
        k, start = gpu.buffer(8192 * kv_heads * 256 * 2), gpu.buffer(4)
        for first in range(0, self.context, 8192):
            gpu.fill_normal(k.base(), 8192 * kv_heads * 256, stream(seed, 3 + first), 1)
            gpu.write_buffer(start, 0, np.array([first], dtype=np.int32))
            gpu.kv_write(self.pool, self.table, self.stride, start.base(), k.base(), k.base(), True, 1, min(8192, self.context - first))
        page_bytes = 2 * kv_heads * page_tokens * row_bytes
        # the same bytes in mapped host memory, under the same page table
        from . import abi
        self.mapped = gpu.host_state(pages * page_bytes)
        gpu.copy(self.mapped.base(), self.pool.pages, pages * page_bytes)
        self.mapped_pool = abi.KvPool(self.mapped.base(), pages, page_tokens, kv_heads, 256, row_bytes)
        self.stage = gpu.buffer(stage_positions // page_tokens * page_bytes)
        gpu.kv_stage(self.stage.base(), self.stage.size // 4096)
        self.q = gpu.buffer(steps * heads * 256 * 2)
        gpu.fill_normal(self.q.base(), steps * heads * 256, stream(seed, 4), 1)
        self.out = gpu.buffer(steps * heads * 256 * 2)
        self.renumbered = gpu.buffer(steps * 2052 * 4)
        self.scratch = gpu.buffer(gpu.selected_attention_scratch(steps, kv_heads, 2052))
        self.parked, self.union_positions, self.gather_calls = False, 0, 0
        gpu.synchronize()
        gpu.release(k); gpu.release(start)

    def _attend(self, pool, table, first=0, rows=None, indices=None):
        rows = self.steps if rows is None else rows
        indices = self.index.indices if indices is None else indices
        self.gpu.selected_attention(pool, table, self.context, self.base + first, indices.at(first * 2052 * 4), 2052, self.index.counts.at(first * 4),
                                    self.q.at(first * self.heads * 256 * 2), True, rows, self.heads, 0.0625, self.out.at(first * self.heads * 256 * 2), True,
                                    self.scratch)

    def step_resident(self):
        self._attend(self.pool, self.table)

    def step_over_the_bus(self):
        self._attend(self.mapped_pool, self.table)

    def park(self):
        self.gpu.kv_cache_park(self.cache, 0)
        self.parked = True

    def step_gathered(self):
        first, self.union_positions, self.gather_calls = 0, 0, 0
        while first < self.steps:
            taken, gathered, view, table, _ = self.gpu.kv_cache_gather(self.cache, 0, self.context, self.base, self.index.indices.base(), 2052,
                                                                      self.index.counts.base(), first, self.steps - first, self.renumbered.base())
            if not taken:
                raise RuntimeError("the stage does not hold one row's selection")
            self._attend(view, table, first, taken, self.renumbered)
            first += taken
            self.union_positions += gathered
            self.gather_calls += 1

    def read_output(self):
        return self.gpu.read_buffer(self.out, 0, np.float16, self.steps * self.heads * 256)

    def release(self):
        self.index.release()
        for b in (self.mapped, self.stage, self.q, self.out, self.renumbered, self.scratch):
            self.gpu.release(b)
        self.gpu.kv_cache_destroy(self.cache)


class QwenStageWorkload:
    """The whole attention stage of a Qwen decode / verification pass in one call (sdx_qsa_decode_attend) at 242K tokens:
    24 query / 2 K/V heads of 256 columns, Q8_0 rows in the reference's state layout, 4 x 128 index heads."""

    def __init__(self, gpu, steps, base=242000, context=262144, heads=24, kv_heads=2, row_bytes=272, seed=8):
        self.gpu, self.steps, self.heads = gpu, steps, heads
        pool = context // 4 + 1
        self.stride = heads * 512 + kv_heads * 512 + 640
        self.kv, self.kv_buffer = gpu.kv_pool(1, context, kv_heads, 256, row_bytes)
        k, table = gpu.buffer(8192 * kv_heads * 256 * 2), gpu.upload(np.zeros(1, dtype=np.int32))
        gpu.fill_normal(k.base(), 8192 * kv_heads * 256, stream(seed, 3), 1)
        for first in range(0, context, 8192):
            start = gpu.upload(np.array([first], dtype=np.int32))
            gpu.kv_write(self.kv, table.base(), 1, start.base(), k.base(), k.base(), True, 1, 8192)
            gpu.release(start)
        self.projections = gpu.buffer(steps * self.stride * 4)
        self.blocks, self.history = gpu.buffer(128 * pool * 4), gpu.buffer(16 * 128 * 4)
        self.norms = [gpu.buffer(n * 4) for n in (256, 256, 128, 128)]
        gpu.fill_normal(self.projections.base(), steps * self.stride, stream(seed, 1), 0)
        gpu.fill_normal(self.blocks.base(), 128 * pool, stream(seed, 2), 0)
        for i, n in enumerate((256, 256, 128, 128)):
            gpu.fill_uniform(self.norms[i].base(), n, stream(seed, 5 + i), 0.5, 1.5)
        self.positions = gpu.upload(np.arange(base, base + steps, dtype=np.uint32))
        self.state = gpu.qsa_state(self.kv, None, context, self.blocks.base(), self.history.base(), *[n.base() for n in self.norms], heads)
        self.scratch = gpu.buffer(gpu.qsa_decode_attend_scratch(steps, heads, kv_heads, context))
        self.attended = gpu.buffer(steps * heads * 256 * 4)
        gpu.synchronize()
        gpu.release(k); gpu.release(table)

    def step(self):
        # (the projections are normalised in place again on every call: values shrink towards the norm weights, the work is the same)
        self.gpu.qsa_decode_attend(self.state, self.projections.base(), self.stride, self.steps, self.positions.base(), self.positions.base(),
                                   self.scratch, self.attended.base())

    def release(self):
        for b in [self.kv_buffer, self.projections, self.blocks, self.history, self.positions, self.scratch, self.attended] + self.norms:
            self.gpu.release(b)


def config1_lengths(seed=0x9e3779b97f4a7c15 ^ 1, seqs=32, low=1024, high=32768):
    rng = np.random.default_rng(seed & 0xffffffff)
    return rng.integers(low, high + 1, size=seqs)
