"""Benchmark of the sparse-embedding hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload c4|c2] [--no-cpu-baseline]

Prints ONE JSON line. A "step" is one pass of the hot path over one batch of synthetic
input that is already resident in HBM. The default workload is benchmark config 4
(click-through-style merged table): feature ops (bucketize + mod) -> key tagging ->
dedup -> find-or-insert -> row gather -> sum pooling -> backward scatter -> fused sparse
Adam; `value` = id occurrences per second. Config 2 (standalone segment reduce, fwd + bwd
for sum / mean / max) is measured in the same run and reported under "workloads".

"roofline" describes the kernel that takes the largest share of the step: algorithmic
bytes per launch / mean launch time (HIP events on the launch stream) against the 8 TB/s
HBM peak. "cpu_baseline" is the reference's own CPU code (oracle/_ref, when built) on all host
cores of this box's share, on a bounded sample of the same workload; "cpu_baseline_reference_1core"
the same on one thread, "cpu_baseline_port_1core" the restated CPU path (oracle.cpu_path) on one
core. Without oracle/_ref, "cpu_baseline" is the port.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import workloads  # noqa: E402

HBM_PEAK_GBS = 8000.0


def _kernel_profile(fn, iters):
    """Per-kernel mean launch time in microseconds over `iters` calls of fn(), measured by the
    library's own HIP events around each kernel launch (on the launch stream)."""
    import ctypes

    from recis_amd import _lib
    lib = _lib.lib()
    fn()
    torch.cuda.synchronize()
    buf = ctypes.create_string_buffer(1 << 16)
    _lib.check(lib.recis_hip_profile_enable(1))
    _lib.check(lib.recis_hip_profile_report(buf, ctypes.c_int64(len(buf))))  # drop warm-up records
    for _ in range(iters):
        fn()
    _lib.check(lib.recis_hip_profile_report(buf, ctypes.c_int64(len(buf))))
    _lib.check(lib.recis_hip_profile_enable(0))
    out = {}
    for line in buf.value.decode().splitlines():
        name, calls, total_ms = line.split()
        out[name] = {"calls_per_step": int(calls) / iters, "us": float(total_ms) * 1e3 / int(calls)}
    return out


def _event_ms(fn, iters):
    """Mean time of fn() over `iters` launches, HIP events on the current stream."""
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


# --------------------------------------------------------------------- config 2
class Config2:
    """Standalone ragged segment_reduce on pre-materialised rows: 32 x 16384 segments,
    Poisson(30) lengths in [1, 200], D = 64 fp32, int32 offsets; forward + backward gradient
    scatter for the sum, mean and max combiners."""

    name = "c2_segment_reduce_32x16384_poisson30_d64_fp32"

    def __init__(self):
        from recis_amd import ops
        self.ops = ops
        c = workloads.config2()
        self.emb, self.off, self.grad = c["values"], c["offsets"], c["grad"]
        self.S, self.N, self.D = c["num_segments"], c["num_ids"], c["dim"]
        self.ids_per_step = 3 * self.N
        # algorithmic bytes of one pass: N rows of 256 B + 8 B index each, S rows of 256 B + offset
        self.pass_bytes = self.N * (self.D * 4 + 8) + self.S * (self.D * 4 + 4)
        self.rev = torch.arange(self.N, device="cuda")

    def step(self):
        o = self.ops
        for mode in ("sum", "mean"):
            o.segment_reduce_forward(self.emb, None, self.rev, self.off, mode)
            o.segment_reduce_backward(self.grad, None, self.rev, self.off, self.N, mode, rev_unique=True)
        _, arg = o.segment_reduce_forward(self.emb, None, self.rev, self.off, "max", return_argmax=True)
        o.segment_reduce_backward(self.grad, None, self.rev, self.off, self.N, "max", argmax=arg, rev_unique=True)

    def kernels(self):
        o = self.ops
        return {
            "seg_pool_fwd_kernel(sum)": (lambda: o.segment_reduce_forward(self.emb, None, self.rev, self.off, "sum"),
                                         self.pass_bytes),
            "seg_pool_bwd_kernel(sum)": (lambda: o.segment_reduce_backward(self.grad, None, self.rev, self.off,
                                                                          self.N, "sum", rev_unique=True),
                                         self.pass_bytes),
            "seg_max_fwd_kernel": (lambda: o.segment_reduce_forward(self.emb, None, self.rev, self.off, "max",
                                                                    return_argmax=True),
                                   self.pass_bytes + self.S * self.D * 4),
            "seg_max_bwd_kernel": (lambda: o.segment_reduce_backward(self.grad, None, self.rev, self.off, self.N,
                                                                     "max", argmax=self._argmax(), rev_unique=True),
                                   self.pass_bytes + self.S * self.D * 4),
        }

    def _argmax(self):
        if getattr(self, "_arg", None) is None:
            _, self._arg = self.ops.segment_reduce_forward(self.emb, None, self.rev, self.off, "max",
                                                           return_argmax=True)
        return self._arg

    def cpu_baseline(self, budget_s):
        import oracle
        k = 4096  # segments in the sample
        off = self.off[: k + 1].cpu().numpy().astype(np.int64)
        n = int(off[-1])
        emb = self.emb[:n].cpu().numpy()
        g = self.grad[:k].cpu().numpy()
        rev = np.arange(n)
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < budget_s:
            for mode in ("sum", "mean"):
                oracle.segment_reduce_forward(emb, None, rev, off, mode)
                oracle.segment_reduce_backward(g, None, rev, off, n, mode)
            _, arg = oracle.segment_max_forward(emb, rev, off)
            oracle.segment_max_backward(g, arg, rev, n)
            reps += 1
        dt = time.perf_counter() - t0
        return 3 * n * reps / dt, "first %d segments (%d ids) of config 2, fwd+bwd x (sum, mean, max)" % (k, n)


# --------------------------------------------------------------------- config 4
class Config4:
    """Click-through-style merged table: 26 id fields + 13 bucketized dense fields, batch 65536,
    dim 16 fp32, one coalesced table, fused dedup + lookup + sum pool + backward + sparse Adam
    (lr 1e-3, betas 0.9 / 0.999)."""

    name = "c4_ctr_merged_table_39x65536_d16_fp32_adam"

    def __init__(self, batch=65536, n_batches=8):
        from recis_amd import ops
        from recis_amd.nn.initializers import NormalInitializer
        from recis_amd.nn.modules import hashtable as ht
        self.ops, self.ht = ops, ht
        # the steps rotate over n_batches batches of the same fields, so that the table holds several
        # batches' worth of rows and a step touches a scattered part of it (one batch replayed would
        # keep the whole table in the caches)
        self.batches = [workloads.config4(batch=batch)] + [
            workloads.config4(batch=batch, data_seed=k) for k in range(1, n_batches)]
        self._turn = 0
        c = self.batches[0]
        self.c = c
        self.D = 16
        self.n_feat = len(c["sparse"]) + len(c["dense"])
        self.N = c["num_ids"]
        self.ids_per_step = self.N
        init = NormalInitializer(0.0, 0.01)
        init.set_shape([10240, self.D])
        init.set_dtype(torch.float32)
        # the table and the optimizer are the objects of recis.so (torch.classes.recis.HashtableImpl / SparseAdam),
        # the same ones the module layer drives
        self.table = ht.make_hashtable(10240, [self.D], torch.float32, torch.device("cuda"), True,
                                       ["f%d" % i for i in range(self.n_feat)], init.build().impl(),
                                       reserve_rows=int(self.N * 1.05) * n_batches)
        self.opt = torch.classes.recis.SparseAdam.make({"ctr": self.table}, 1e-3, 0.9, 0.999, 1e-8, 0.0, False)
        self.tags = list(range(self.n_feat))
        self.offsets = torch.arange(self.N + 1, dtype=torch.int32, device="cuda")
        g = torch.Generator(device="cuda").manual_seed(4)
        self.grad_out = torch.randn((self.N, self.D), device="cuda", generator=g)
        self.mods = [c["mod"]] * len(c["dense"])
        self.U = None
        for b in self.batches:  # admission of every batch's keys happens here, not in the timed steps
            self.c = b
            plan, _ = self.dedup(self.feature_ops())
            self.settle(plan)
        torch.cuda.synchronize()

    # the stages, also timed one by one for the breakdown
    def feature_ops(self):
        """The 39 id columns of the batch: the sparse ones as they are, the dense ones bucketized and
        reduced. They are tagged with their table (ids_encode) by the plan's own reads."""
        o = self.ops
        extra = o.fused_bucketized(self.c["dense"], self.c["boundaries"], mods=self.mods)   # Bucketize -> Mod, one pass
        return self.c["sparse"] + extra

    def dedup(self, ids):
        """Tagging, dedup and find-or-insert in one pass: the plan carries the row of every unique id.
        Every field holds one id per sample, so nothing per occurrence but the lists is asked for."""
        self.plan = self.ht.plan_lookup(self.table, ids, need_inverse=False, need_pos=False, tags=self.tags)
        return self.plan, None

    def lookup(self, plan):
        """The rows of the plan's unique ids: the full-length buffer the plan brought along (its first U entries
        count). Nothing waits for U: what follows takes it from device memory; settle() reads it once the whole
        step is queued."""
        return plan.index_buf

    def settle(self, plan):
        """The host's copy of the unique count (it arrived in pinned memory while the device went on) tells the id
        map how many ids the counted lookup held."""
        self.U = plan.U
        self.table.settle_count(self.U, plan)

    def pool_fwd(self, index, inv):
        # pooling reads the rows out of the table (no [U, D] copy); every field holds one id per
        # sample, so, as EmbeddingEngine does for dense [B] id tensors, each unique row is read
        # once and written to its occurrences
        return self.table.expand_rows(self.plan, index, None, None, None)

    def pool_bwd(self, inv):
        return self.ops.segment_reduce_backward_plan(self.grad_out, None, self.offsets, self.plan, "sum")

    def update(self, index, g):
        self.table.accept_grad_ex(index, g, True, 0)
        self.opt.step()
        self.opt.zero_grad()

    def bwd_update(self, index):
        """Backward of the pooling and the Adam step in one launch: the gradient of every unique row is
        summed over its occurrences and applied to the row by the lanes that summed it (the [U, D]
        gradient is not written). Bit for bit what pool_bwd + update give
        (tests/test_gpu_features.py::test_fused_gather_reduce_update_equals_the_two_calls)."""
        self.ht.accept_planned_grad(self.table, index, self.plan, self.grad_out, self.plan.occ)
        self.opt.step()       # sums the gradient it was handed unsummed and updates the rows, one launch
        self.opt.zero_grad()

    def next_batch(self):
        self.c = self.batches[self._turn % len(self.batches)]
        self._turn += 1

    def step(self):
        self.next_batch()
        ids = self.feature_ops()
        uniq, inv = self.dedup(ids)
        index = self.lookup(uniq)
        pooled = self.pool_fwd(index, inv)
        self.bwd_update(index)
        self.settle(uniq)
        return pooled

    def step_from_host(self):
        """The same step with the raw inputs starting in pinned host memory (26 id columns and 13
        float columns, 24 MB): what a caller that hands over host buffers would see."""
        if not hasattr(self, "_host"):
            self._host = [([t.cpu().pin_memory() for t in b["sparse"]], [t.cpu().pin_memory() for t in b["dense"]])
                          for b in self.batches]
        k = self._turn % len(self.batches)
        self._upload(k)
        return self.step()

    def _upload(self, k):
        b, host = self.batches[k], self._host[k]
        for dst, src in zip(b["sparse"] + b["dense"], host[0] + host[1]):
            dst.copy_(src, non_blocking=True)

    def step_from_host_overlapped(self):
        """step_from_host with the upload of the NEXT batch on a second stream (default priority)
        while this batch is worked: what a caller with two input buffers would see."""
        n = len(self.batches)
        if not hasattr(self, "_copy_stream"):
            self.step_from_host()  # makes the pinned copies
            torch.cuda.synchronize()
            self._copy_stream = torch.cuda.Stream()
            self._uploaded, self._worked = [None] * n, [None] * n
        main = torch.cuda.current_stream()
        k = self._turn % n
        if self._uploaded[k] is None:  # first call: nothing was prefetched
            self._upload(k)
        else:
            main.wait_event(self._uploaded[k])
            self._uploaded[k] = None
        nxt = (k + 1) % n
        with torch.cuda.stream(self._copy_stream):
            if self._worked[nxt] is not None:  # the step that last read these device buffers is done
                self._copy_stream.wait_event(self._worked[nxt])
            self._upload(nxt)
            self._uploaded[nxt] = torch.cuda.Event()
            self._uploaded[nxt].record(self._copy_stream)
        out = self.step()
        self._worked[k] = torch.cuda.Event()
        self._worked[k].record(main)
        return out

    def algorithmic_bytes(self):
        N, U, S, D = self.N, self.U, self.N, self.D
        feat = 13 * self.c["batch"] * (4 + 8)   # bucketize + mod in one pass (tagging: in the plan's reads)
        return {
            "feature_ops": feat,
            "dedup+lookup": N * (8 + 4) + U * 8 + U * (16 + 8),
            "pool_fwd": U * (8 + D * 4) + N * 4 + (U + 1) * 4 + S * D * 4,
            "pool_bwd+adam": S * D * 4 + N * 4 + (U + 1) * 4 + U * 8 + U * D * 4 * 6,
        }

    def fused_minimum_bytes(self):
        """The step's compulsory bytes with every intermediate counted as kept on chip (the [U, D]
        gradient between pooling backward and Adam among them): the lowest price of this config."""
        N, U, S = self.N, self.U, self.N
        return N * (8 + 4 + 4) + U * (16 + 8 + 384 + 8) + S * (64 + 64) + 13 * self.c["batch"] * (4 + 8 + 8 + 8)

    def kernel_bytes(self):
        """Algorithmic (compulsory) HBM bytes of one launch of each heavy kernel of the step."""
        N, U, S, D = self.N, self.U, self.N, self.D
        return {
            "plan_hist_kernel": 8 * N,                               # ids in
            "plan_scatter_kernel": 8 * N + 12 * N,                   # ids in; (id, position) out, by bucket
            # (id, position) in; list out; per unique id: the id, its list start, its row; one 16-byte slot of the map
            "plan_bucket_kernel": 12 * N + 4 * N + U * (8 + 4 + 8) + 16 * U,
            "csr_expand_kernel": U * (8 + D * 4) + 4 * N + 4 * (U + 1) + S * D * 4,
            # gradient rows in, list, list starts; per unique row: its index, parameter and two moments read and written
            "csr_rows_adam_kernel": S * D * 4 + 4 * N + 4 * U + U * (8 + D * 4 * 6),
        }

    def stage_times(self, iters):
        ids = self.feature_ops()
        uniq, inv = self.dedup(ids)
        index = self.lookup(uniq)
        self.settle(uniq)
        def dedup_lookup():
            self.settle(self.dedup(ids)[0])
        return {
            "feature_ops": _event_ms(self.feature_ops, iters),
            "dedup+lookup": _event_ms(dedup_lookup, iters),
            "pool_fwd": _event_ms(lambda: self.pool_fwd(index, inv), iters),
            "pool_bwd+adam": _event_ms(lambda: self.bwd_update(index), iters),
        }

    def cpu_baseline(self, budget_s):
        import oracle
        from oracle import cpu_path
        b = 8192
        sparse = [t[:b].cpu().numpy() for t in self.c["sparse"]]
        dense = [t[:b].cpu().numpy() for t in self.c["dense"]]
        bnd = self.c["boundaries"][0].cpu().numpy()
        n = b * self.n_feat
        off = np.arange(n + 1, dtype=np.int64)
        grad = self.grad_out[:n].cpu().numpy()
        table = cpu_path.CpuTable(self.D, 10240, lambda blk: np.zeros((10240, self.D), np.float32), "adam", 1e-3, 1e-8)
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < budget_s:
            extra = [oracle.uint64_mod(oracle.bucketize(d, bnd), self.c["mod"]) for d in dense]
            ids = oracle.ids_encode(sparse + extra, self.tags)
            cpu_path.train_step(table, ids, off, None, grad)
            reps += 1
        dt = time.perf_counter() - t0
        self._cpu_sample_ids = ids
        return n * reps / dt, "first %d samples (%d ids/step) of config 4, full step" % (b, n)

    def cpu_reference(self, budget_s, threads):
        """The reference's own CPU code (compiled from its sources into oracle/_ref) on the ids of
        cpu_baseline's sample, `threads` threads: ids_partition + Hashtable.EmbeddingLookup + sum
        pooling forward and backward as the reference's "torch" backend runs them on CPU tensors
        (index_select + index_add_: it has no CPU pooling operator) + AcceptGrad + SparseAdam.step.
        None when the reference build is absent."""
        from oracle import ref_ops
        if not ref_ops.available():
            return None
        ids = np.ascontiguousarray(self._cpu_sample_ids, dtype=np.int64)
        seg = np.arange(ids.size, dtype=np.int64)   # one id per sample and field
        params = np.array([10240, self.D, 1e-3, 0.9, 0.999, 1e-8, 0.0, budget_s, threads], np.float64)
        secs, steps, uniq = ref_ops.run("table_step_time", [params, ids, seg], threads=threads)[0]
        return {"value": ids.size * steps / secs, "unit": "ids/s", "cores": threads, "kind": "reference",
                "sample": "first %d samples (%d ids/step, %d distinct) of config 4: the reference's ids_partition + "
                          "EmbeddingLookup + torch-backend sum pooling fwd/bwd + AcceptGrad + SparseAdam.step "
                          "(feature ops left out)" % (ids.size // self.n_feat, ids.size, int(uniq))}



# --------------------------------------------------------------------- config 3
class Config3:
    """IDMap + EmbeddingBlocks at scale: 2e8 resident rows, dim 32 fp32 + two Adam state slots
    (~77 GB), 2e6 lookups per step, Zipf(1.1) over the resident keys with 10 % of the positions
    replaced by keys never seen before (admission inserts, on EVERY step: batches are never
    replayed); rows are expanded to one output row per lookup, the per-lookup gradients are
    reduced per key, fused sparse Adam; every looked-up row is stamped with the step; every
    `filter_interval` steps the sweep of the step filter evicts the keys not seen for `filter_step`
    steps (threshold = step - filter_step: recis/nn/modules/hashtable_hook_impl.py:527-551,
    recis/hooks/filter_hook.py:82-117), frees their rows and re-initialises them. The resident
    keys were last seen before step 0 (stamp -1)."""

    name = "c3_idmap_blocks_2e8rows_d32_fp32_adam_2e6ids_zipf1.1_10pct_new_evict50"

    def __init__(self, resident=200_000_000, ids_per_step=2_000_000, n_batches=48, filter_step=50,
                 filter_interval=50):
        from recis_amd import ops
        from recis_amd.nn.initializers import NormalInitializer
        from recis_amd.nn.modules import hashtable as ht
        self.ops, self.ht = ops, ht
        self.D, self.N, self.resident = 32, ids_per_step, resident
        self.ids_per_step = ids_per_step
        self.filter_step, self.filter_interval = filter_step, filter_interval
        init = NormalInitializer(0.0, 0.01)
        init.set_shape([10240, self.D])
        init.set_dtype(torch.float32)
        reserve = int(resident * 1.12) + 40 * ids_per_step // 10
        self.table = ht.make_hashtable(10240, [self.D], torch.float32, torch.device("cuda"), False, ["c3"],
                                       init.build().impl(), reserve_rows=reserve)
        self.table.append_step_filter_slot("step_filter", -1)
        self.opt = torch.classes.recis.SparseAdam.make({"c3": self.table}, 1e-3, 0.9, 0.999, 1e-8, 0.0, False)
        chunk = 25_000_000
        for lo in range(0, resident, chunk):
            ranks = torch.arange(lo, min(lo + chunk, resident), device="cuda")
            self.table.insert_lookup_index(workloads.splitmix64_torch(ranks))
        self.batches = []          # batch k = the lookups of step k; its new keys were never seen before
        self._gen = workloads.Config3Lookups(resident, ids_per_step)
        self.prepare(n_batches)
        g = torch.Generator(device="cuda").manual_seed(3)
        self.grad_out = torch.randn((ids_per_step, self.D), device="cuda", generator=g)
        self.span = torch.tensor([0, ids_per_step], dtype=torch.int64, device="cuda")
        self.step_no = 0
        self.step_t = torch.zeros(1, dtype=torch.int64, device="cuda")
        self.U = None
        self.sweeps = []           # (step, keys evicted, ms) of every sweep so far
        torch.cuda.synchronize()

    def prepare(self, steps):
        """Draws the lookups of the next `steps` steps (input generation, outside any timed region)."""
        done = getattr(self, "step_no", 0)
        while len(self.batches) < done + steps:
            self.batches.append(self._gen.batch(len(self.batches)))
        for k in range(max(0, done - 2)):   # batches of finished steps are not needed again
            self.batches[k] = None

    def step(self):
        o = self.ops
        if self.step_no >= len(self.batches):
            self.prepare(16)
        ids = self.batches[self.step_no]
        if self.step_no and self.step_no % self.filter_interval == 0:
            self.sweep(self.step_no - self.filter_step)
        self.step_no += 1
        plan = self.plan_of(ids)
        out = self.expand(plan)
        self.update(plan)
        self.step_t += 1
        self.settle(plan)
        return out

    # the stages of a step (tests look at the table between them)
    def plan_of(self, ids):
        """Dedup + find-or-insert, one pass; the plan brings the row of every unique id along (index_buf)."""
        return self.ht.plan_lookup(self.table, ids, need_inverse=False, need_pos=False)

    def expand(self, plan):
        """One row per lookup: every unique row is read once out of the table and written to its occurrences (no
        [U, D] copy, no second pass over it); the step filter's stamps of the rows go out in the same pass."""
        return self.table.expand_rows(plan, plan.index_buf, None, "step_filter", self.step_t)

    def update(self, plan):
        """The per-lookup gradients reduced per key and applied to the row in the same launch."""
        self.ht.accept_planned_grad(self.table, plan.index_buf, plan, self.grad_out, plan.occ, cover=self.span)
        self.opt.step()
        self.opt.zero_grad()

    def settle(self, plan):
        """The whole step is queued: the unique count has arrived in pinned memory meanwhile."""
        self.U = plan.U
        self.table.settle_count(self.U, plan)

    def sweep(self, threshold):
        """The eviction sweep of the step filter (one pass over the id map + re-initialisation of
        the freed rows); records (step, evicted keys, ms)."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        gone, _ = self.table.evict_older("step_filter", threshold)
        torch.cuda.synchronize()
        self.sweeps.append((self.step_no, int(gone.numel()), (time.perf_counter() - t0) * 1e3))
        return self.sweeps[-1]

    def run_to_next_sweep(self):
        """Steps (untimed by the caller) up to the next multiple of `filter_interval`, then that
        step with its sweep; returns the sweep's record."""
        before = len(self.sweeps)
        self.prepare(self.filter_interval + 1)
        while len(self.sweeps) == before:
            self.step()
        return self.sweeps[-1]

    def fused_minimum_bytes(self):
        N, U, D = self.N, self.U, self.D
        return U * (16 + 8 + 768 + 8) + int(0.1 * N) * 16 + N * (8 + 4 + 128 + 128)

    def algorithmic_bytes(self):
        N, U, D = self.N, self.U, self.D
        # dedup + lookup; rows read once and expanded per lookup; per-lookup gradients in; per unique row the
        # parameter and two moments read and written (the [U, D] gradient stays on chip); the stamp
        return N * (8 + 4) + U * 8 + U * (16 + 8) + int(0.1 * N) * 16 + U * D * 4 + N * (4 + D * 4) \
            + N * (4 + D * 4) + U * D * 4 * 6 + U * 8

    def kernel_bytes(self):
        """Algorithmic HBM bytes of one launch of each heavy kernel of the step (one row per lookup,
        so the segments are the occurrences)."""
        N, U, D = self.N, self.U, self.D
        return {
            "csr_expand_kernel": U * (8 + D * 4) + 4 * N + 4 * (U + 1) + N * D * 4,
            "csr_rows_adam_kernel": N * D * 4 + 4 * N + 4 * U + U * (8 + D * 4 * 6),
            "plan_bucket_kernel": 12 * N + 4 * N + U * (8 + 4 + 8) + 16 * U,
        }

    def cpu_baseline(self, budget_s):
        from oracle import cpu_path
        import oracle
        resident, n = 2_000_000, 200_000
        table = cpu_path.CpuTable(self.D, 10240, lambda blk: np.zeros((10240, self.D), np.float32), "adam", 1e-3, 1e-8)
        keys = workloads.splitmix64(np.arange(resident, dtype=np.uint64)).astype(np.int64)
        table.lookup(np.unique(keys))
        rng = np.random.default_rng(3)
        grad = rng.standard_normal((n, self.D)).astype(np.float32)
        span = np.array([0, n])
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < budget_s:
            ranks = workloads.bounded_zipf(rng, n, 1.1, resident)
            ranks[: n // 10] = resident + reps * (n // 10) + np.arange(n // 10)
            ids = workloads.splitmix64(ranks.astype(np.uint64)).astype(np.int64)
            uniq, inv = np.unique(ids, return_inverse=True)
            index, rows = table.lookup(uniq)
            oracle.gather(inv, rows)
            g = oracle.segment_reduce_backward(grad, None, inv, span, len(uniq), "tile")
            table.apply(index, g)
            reps += 1
        dt = time.perf_counter() - t0
        return n * reps / dt, "table scaled to %d resident rows, %d lookups/step (1/100 and 1/10 of config 3)" % (resident, n)


# --------------------------------------------------------------------- config 5
class Config5:
    """Long behaviour sequences: batch 2048 x 4 sequence fields, lognormal lengths (mean 200, max
    1000), Zipf(1.2) ids over 5e7 keys, dim 128, bf16 row storage with fp32 accumulation; mean
    pooling plus the unpooled gather padded to each field's longest sequence; backward of both
    into the unique rows, sparse Adagrad."""

    name = "c5_sequences_2048x4_lognormal200_d128_bf16_mean+padded_adagrad"

    def __init__(self):
        from recis_amd import ops
        from recis_amd.nn.initializers import NormalInitializer
        from recis_amd.nn.modules import hashtable as ht
        self.ops, self.ht = ops, ht
        c = workloads.config5()
        self.c = c
        self.D, self.N = 128, c["num_ids"]
        self.ids_per_step = self.N
        self.fields = c["fields"]
        self.batch = [c["batch"]] * len(self.fields)
        self.seq = [f["pad_len"] for f in self.fields]
        init = NormalInitializer(0.0, 0.01)
        init.set_shape([10240, self.D])
        init.set_dtype(torch.bfloat16)
        self.table = ht.make_hashtable(10240, [self.D], torch.bfloat16, torch.device("cuda"), True,
                                       ["s%d" % i for i in range(len(self.fields))], init.build().impl(),
                                       reserve_rows=int(self.N * 1.1))
        self.opt = torch.classes.recis.SparseAdagrad.make({"c5": self.table}, 0.01, 1e-8)
        self.S = sum(self.batch)
        self.pad_rows = sum(b * s for b, s in zip(self.batch, self.seq))
        g = torch.Generator(device="cuda").manual_seed(5)
        self.g_pool = torch.randn((self.S, self.D), device="cuda", generator=g)
        self.g_tile = torch.randn((self.pad_rows, self.D), device="cuda", generator=g).to(torch.bfloat16)
        self.offsets = ops.merge_offsets([f["offsets"] for f in self.fields], [f["num_ids"] for f in self.fields])
        self.U = None

    def step(self):
        o = self.ops
        # tagging (ids_encode), dedup and find-or-insert in one pass
        plan = self.ht.plan_lookup(self.table, [f["values"] for f in self.fields], tags=list(range(len(self.fields))))
        self.U = plan.U
        inv = plan.inverse
        index = self.table.settle_lookup(plan.index_buf, self.U, plan)
        chunks, chunk_rows = self.table.emb_blocks()
        rows = o.block_gather(index, chunks, chunk_rows, -1, False)
        pooled = o.segment_reduce_forward(rows, None, inv, self.offsets, "mean", out_dtype=torch.float32)
        padded, batch_seq = o.ragged_tile(self.batch, self.seq, inv, self.offsets, rows)
        self.bwd_update(plan, index)
        return pooled, padded

    def bwd_update(self, plan, index):
        """Backward of both outputs into the unique rows and the Adagrad update of those rows, one
        launch: the two gradients of an occurrence are summed where the row's gradient is summed."""
        src_p, coef_p, src_t = plan.src_for_pool_and_tile(self.offsets, None, True, self.batch, self.seq)
        self.ht.accept_planned_grad(self.table, index, plan, self.g_pool, src_p, coef_p, key=plan.serial)
        self.ht.accept_planned_grad(self.table, index, plan, self.g_tile, src_t, None, key=plan.serial)
        self.opt.step()       # both gradients of the plan summed and the rows updated in one launch
        self.opt.zero_grad()

    def fused_minimum_bytes(self):
        N, U, S, D = self.N, self.U, self.S, self.D
        return 12 * N + U * (24 + 1024) + S * (256 + 256) + self.pad_rows * 256

    def algorithmic_bytes(self):
        N, U, S, D = self.N, self.U, self.S, self.D
        return 12 * N + U * (24 + 4 * D * 2) + S * (D * 4 + D * 4) + 2 * self.pad_rows * D * 2 + 8 * N

    def kernel_bytes(self):
        """Algorithmic HBM bytes per launch: the padded gather runs once per field, the
        gather-reduce with the Adagrad update once over both gradients."""
        N, U, S, D = self.N, self.U, self.S, self.D
        n_fields = len(self.fields)
        return {
            "tile_fwd_kernel": (self.pad_rows * D * 2 + 4 * N + U * D * 2) // n_fields,  # distinct rows once
            # pooled gradients (fp32 rows, re-read out of the caches: one read per segment), padded
            # gradients (bf16 rows, one per occurrence inside its field's pad length), src + coef of
            # both inputs, list starts, row index, parameter and accumulator rows read and written
            "csr_rows_adagrad_kernel": S * D * 4 + N * D * 2 + (4 + 4 + 4) * N + (4 + 8) * U + 4 * U * D * 2,
            "seg_pool_fwd_kernel": U * D * 2 + 4 * N + 4 * (S + 1) + S * D * 4,
        }

    def cpu_baseline(self, budget_s):
        import oracle
        from oracle import cpu_path
        b = 128
        vals, offs = [], []
        for f in self.fields:
            off = f["offsets"][: b + 1].cpu().numpy().astype(np.int64)
            vals.append(f["values"][: int(off[-1])].cpu().numpy())
            offs.append(off)
        n = sum(len(v) for v in vals)
        offsets = oracle.merge_offsets(offs, [len(v) for v in vals])
        ids = oracle.ids_encode(vals, list(range(len(vals))))
        S = len(offsets) - 1
        g_pool = self.g_pool[:S].cpu().numpy()
        rows_pad = sum(b * s for s in self.seq)
        g_tile = np.ones((rows_pad, self.D), np.float32)
        table = cpu_path.CpuTable(self.D, 10240, lambda blk: np.zeros((10240, self.D), np.float32), "adagrad", 0.01, 1e-8)
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < budget_s:
            uniq, inv = np.unique(ids, return_inverse=True)
            index, rows = table.lookup(uniq)
            oracle.segment_reduce_forward(rows, None, inv, offsets, "mean")
            oracle.ragged_tile([b] * len(vals), self.seq, inv, offsets, rows)
            g = oracle.segment_reduce_backward(g_pool, None, inv, offsets, len(uniq), "mean")
            g += oracle.ragged_tile_back([b] * len(vals), self.seq, inv, offsets, g_tile, len(uniq))
            table.apply(index, g)
            reps += 1
        dt = time.perf_counter() - t0
        return n * reps / dt, "first %d of 2048 sequences per field (%d ids/step) of config 5, fp32 rows" % (b, n)


# --------------------------------------------------------------------- the same steps through the modules
class ModulePath4:
    """Config 4 through the drop-in layer: FeatureEngine (bucketize + mod of the 13 dense columns) ->
    EmbeddingEngine (39 features on one coalesced table) -> backward from one gradient per feature output ->
    SparseAdam.step, rotating over the same 8 batches as Config4. The work is Config4's: the engine returns
    one [B, 16] output per feature (views of the one pooled buffer) and backward receives one gradient per
    output, here 39 slices of one buffer, as Config4.grad_out is one buffer. (A dense tower that concatenates
    the outputs along the feature axis adds a 168 MB copy each way; that copy is the model's, not the table's,
    and is reported separately as module_path_with_concat_ms.)"""

    def __init__(self, n_batches=8, concat=False):
        from recis_amd.features import Bucketize, Feature, FeatureEngine, Mod, SelectField
        from recis_amd.nn import EmbeddingEngine, EmbeddingOption
        from recis_amd.nn.initializers import NormalInitializer
        from recis_amd.nn.modules.hashtable import HashtableRegister, filter_out_sparse_param
        from recis_amd.optim import SparseAdam
        HashtableRegister().clear()
        batches = [workloads.config4()] + [workloads.config4(data_seed=k) for k in range(1, n_batches)]
        c = batches[0]
        nd, ns = len(c["dense"]), len(c["sparse"])
        self.fe = FeatureEngine([Feature("d%d" % i).add_op(SelectField("d%d" % i)).add_op(Bucketize(c["boundaries"][i]))
                                 .add_op(Mod(c["mod"])) for i in range(nd)])
        self.names = ["s%d" % i for i in range(ns)] + ["d%d" % i for i in range(nd)]
        opts = {n: EmbeddingOption(embedding_dim=16, shared_name=n, combiner="sum", use_weight=False,
                                   initializer=NormalInitializer(0, 0.01),
                                   reserve_rows=int(c["num_ids"] * 1.05) * n_batches if k == 0 else 0)
                for k, n in enumerate(self.names)}
        self.eng = EmbeddingEngine(opts).cuda()
        self.eng.train()
        self.opt = SparseAdam(filter_out_sparse_param(self.eng), lr=1e-3)
        self.data = []
        for b in batches:
            d = {"s%d" % i: t.view(-1, 1) for i, t in enumerate(b["sparse"])}
            d.update({"d%d" % i: t for i, t in enumerate(b["dense"])})
            self.data.append(d)
        self.dense_of = {id(d): {k: v for k, v in d.items() if k[0] == "d"} for d in self.data}
        g = torch.Generator(device="cuda").manual_seed(4)
        self.concat = concat
        if concat:
            self.up = torch.randn((c["batch"], 16 * len(self.names)), device="cuda", generator=g)
        else:
            self.up = list(torch.randn((len(self.names) * c["batch"], 16), device="cuda", generator=g).split(c["batch"]))
        self._turn = 0
        for _ in range(n_batches + 2):
            self.step()
        torch.cuda.synchronize()

    def step(self):
        data = self.data[self._turn % len(self.data)]
        self._turn += 1
        x = dict(data)
        x.update(self.fe(self.dense_of[id(data)]))     # [B] id columns: the engine takes them as [B, 1]
        out = self.eng(x)
        if self.concat:
            torch.cat([out[n] for n in self.names], dim=1).backward(self.up)
        else:
            _HandGradients.apply(self.up, *[out[n] for n in self.names]).backward()
        self.opt.step()
        self.opt.zero_grad()


class _HandGradients(torch.autograd.Function):
    """Stands where a model's backward would be: a scalar whose backward hands each input its preset gradient
    (torch.autograd.backward with a list of 39 tensors and 39 gradients spends 0.1 ms of Python on checking
    them one by one, which no model's backward does)."""

    @staticmethod
    def forward(ctx, grads, *outs):
        ctx.grads = grads
        return outs[0].new_zeros(())

    @staticmethod
    def backward(ctx, _):
        return (None,) + tuple(ctx.grads)


class TorchLibraryPath4:
    """Config 4 through the reference's own boundary and its own call sequence, operator by operator
    (torch.ops.recis.* / torch.classes.recis.* of recis.so, nothing else): fused_bucketized -> fused_uint64_mod ->
    ids_encode -> ids_partition -> HashtableImpl.embedding_lookup -> segment_reduce_forward ->
    segment_reduce_backward -> HashtableImpl.accept_grad -> SparseAdam.step
    (recis/nn/modules/embedding_engine.py:627-675, csrc/embedding/hashtable.cc:153-165, adam.cc:98-135). Each
    operator materialises its result as the reference's does (the sorted unique ids, the [U, D] rows, the [U, D]
    gradient), so this is the unfused form of the step."""

    def __init__(self, n_batches=8):
        from recis_amd import torch_library
        torch_library.load()
        self.R = R = torch.ops.recis
        self.batches = [workloads.config4()] + [workloads.config4(data_seed=k) for k in range(1, n_batches)]
        c = self.batches[0]
        self.n_feat = len(c["sparse"]) + len(c["dense"])
        self.N, self.D = c["num_ids"], 16
        gen = torch.classes.recis.Generator.make_normal_generator([10240, self.D], torch.float32, 0.0, 0.01, None)
        self.table = R.make_hashtable(10240, [self.D], torch.float32, torch.device("cuda", 0), True,
                                      ["f%d" % i for i in range(self.n_feat)], gen, 0, 65536, 65536)
        self.table.reserve(int(self.N * 1.05) * n_batches)
        self.opt = torch.classes.recis.SparseAdam.make({"ctr": self.table}, 1e-3, 0.9, 0.999, 1e-8, 0.0, False)
        self.table_ids = torch.arange(self.n_feat, dtype=torch.int64)
        self.mods = torch.full((len(c["dense"]),), c["mod"], dtype=torch.int64)
        self.offsets = torch.arange(self.N + 1, dtype=torch.int32, device="cuda")
        g = torch.Generator(device="cuda").manual_seed(4)
        self.grad_out = torch.randn((self.N, self.D), device="cuda", generator=g)
        self._turn = 0
        for _ in range(n_batches + 2):
            self.step()
        torch.cuda.synchronize()

    def step(self):
        R = self.R
        c = self.batches[self._turn % len(self.batches)]
        self._turn += 1
        extra = R.fused_uint64_mod(R.fused_bucketized(c["dense"], c["boundaries"]), self.mods)
        ids = R.ids_encode(c["sparse"] + extra, self.table_ids)
        uniq, _, inverse = R.ids_partition(ids, 1)
        index, emb = self.table.embedding_lookup(uniq, False)
        pooled = R.segment_reduce_forward(emb, None, inverse, self.offsets, "sum")
        grad = R.segment_reduce_backward(self.grad_out, None, inverse, self.offsets, uniq.numel(), "sum")
        self.table.accept_grad(index, grad)
        self.opt.step()
        self.opt.zero_grad()
        return pooled


class ModulePath5:
    """Config 5 through the drop-in layer: each of the 4 sequence fields under two options of one
    shared name (mean pooling, and the rows kept and padded to the field's longest sequence), bf16
    table, backward of both, SparseAdagrad.step."""

    def __init__(self):
        from recis_amd.nn import EmbeddingEngine, EmbeddingOption
        from recis_amd.nn.initializers import NormalInitializer
        from recis_amd.nn.modules.hashtable import HashtableRegister, filter_out_sparse_param
        from recis_amd.optim import SparseAdagrad
        from recis_amd.ragged import RaggedTensor
        HashtableRegister().clear()
        c = workloads.config5()
        opts, self.data = {}, {}
        for i, f in enumerate(c["fields"]):
            rt = RaggedTensor(f["values"], f["offsets"])
            common = dict(embedding_dim=128, dtype=torch.bfloat16, shared_name="s%d" % i, use_weight=False,
                          initializer=NormalInitializer(0, 0.01), reserve_rows=int(f["num_ids"] * 1.1))
            opts["s%d_mean" % i] = EmbeddingOption(combiner="mean", **common)
            opts["s%d_rows" % i] = EmbeddingOption(combiner="tile", combiner_kwargs={"tile_len": f["pad_len"]},
                                                   **common)
            self.data["s%d_mean" % i] = rt
            self.data["s%d_rows" % i] = rt
        self.eng = EmbeddingEngine(opts).cuda()
        self.eng.train()
        self.opt = SparseAdagrad(filter_out_sparse_param(self.eng), lr=0.01)
        g = torch.Generator(device="cuda").manual_seed(5)
        out = self.eng(self.data)
        self.ups = {k: torch.randn(v.shape, device="cuda", generator=g).to(v.dtype) for k, v in out.items()}
        del out
        for _ in range(5):
            self.step()
        torch.cuda.synchronize()

    def step(self):
        out = self.eng(self.data)
        torch.autograd.backward([out[k] for k in out], [self.ups[k] for k in out])
        self.opt.step()
        self.opt.zero_grad()


# HBM bytes per launch by workload and kernel, from hardware-counter runs of this file
# (rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE, with --workload W --calib-copy): each
# counter is scaled by what it reads for the calibration kernel that moves 1 GiB each way
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).
MEASURED_TRAFFIC = {
    "c4": {"csr_rows_adam_kernel": 733263974, "csr_expand_kernel": 267866214, "plan_bucket_kernel": 192615833,
           "plan_scatter_kernel": 60778086, "plan_hist_kernel": 23677952, "bucketize_kernel": 10267238,
           "plan_colscan_kernel": 3305881, "csr_hot_finish_kernel": 1179648, "plan_assign_new_kernel": 60825},
    "c3": {"csr_rows_adam_kernel": 768038502, "csr_expand_kernel": 386756403, "plan_bucket_kernel": 200619008,
           "plan_scatter_kernel": 49669427, "plan_assign_new_kernel": 23479500, "plan_hist_kernel": 19194368},
    "c5": {"tile_fwd_kernel": 549505638, "csr_rows_adagrad_kernel": 769052876, "seg_pool_fwd_kernel": 93497753,
           "block_gather_kernel": 109106995, "plan_bucket_kernel": 95373721, "plan_scatter_kernel": 46198784},
    "c2": {"seg_pool_fwd_kernel(sum)": 4319621529, "seg_pool_bwd_kernel(sum)": 4321946419,
           "seg_max_fwd_kernel": 4453851545, "seg_max_bwd_kernel": 4453874585},
}


def _measured_traffic(wl):
    if "_variant_" in wl.name:   # the counters were read on the named configurations only
        return {}
    return MEASURED_TRAFFIC.get(type(wl).__name__.lower().replace("config", "c"), {})


# Requests per launch that leave the compute units' first-level caches for the L2, reads + writes
# (rocprofv3 --pmc TCP_TCC_READ_REQ_sum TCP_TCC_WRITE_REQ_sum of this file with --workload W; a read
# request carries up to 128 bytes, a write request up to 64). The kernels of these steps touch rows
# of 64-256 bytes at random places, so what they wait for is the number of requests, not the bytes:
# see _random_request_ceiling.
MEASURED_REQUESTS = {
    "c4": {"csr_rows_adam_kernel": 7283000, "csr_expand_kernel": 3640000, "plan_bucket_kernel": 3408000,
           "plan_scatter_kernel": 1006000, "plan_hist_kernel": 692000, "plan_assign_new_kernel": 198000,
           "bucketize_kernel": 134000, "plan_colscan_kernel": 47000, "csr_hot_finish_kernel": 11000},
    "c3": {"csr_rows_adam_kernel": 8435000, "csr_expand_kernel": 5635000, "plan_bucket_kernel": 3292000,
           "plan_scatter_kernel": 934000, "plan_hist_kernel": 647000, "plan_assign_new_kernel": 400000,
           "plan_colscan_kernel": 46000, "csr_hot_finish_kernel": 11000},
    "c5": {"csr_rows_adagrad_kernel": 9528000, "plan_bucket_kernel": 1780000, "seg_pool_fwd_kernel": 1710000,
           "block_gather_kernel": 1272000, "plan_scatter_kernel": 1090000, "plan_hist_kernel": 574000},
}


def _random_request_ceiling(slot_mb=4096, n=1 << 24):
    """Requests per second this device serves when every lane asks for another random line: the
    step filter's own kernel (recis_block_filter: one 8-byte read at a random row of an int64 slot
    per thread, one byte written per thread in order). Measured live; it reads 5.0-5.3e10/s over a
    64 MB - 1 GB slot and 4.2-4.4e10/s over 4 - 8 GB, whatever is fetched per request (8 bytes here,
    64-byte rows in the steps), while requests that follow one another in memory are served at
    1.1e11/s (config 5's padded gather): every random request opens another page of the memory, and
    that rate, not the bytes, is what a step of 64- or 128-byte rows at random places runs into."""
    from recis_amd import ops
    rows = slot_mb * 2**20 // 8
    slot = torch.zeros(rows, 1, dtype=torch.int64, device="cuda")
    idx = torch.randint(0, rows, (n,), device="cuda")
    ms = _event_ms(lambda: ops.block_filter(idx, [slot], rows, 1), 10)
    return n / ms * 1e3


def request_ceiling_probe():
    """What this device does with random accesses, by the product's own row movers (--workload probe):
    requests per second of recis_block_filter (8 bytes per request) over slots of several sizes, and
    rows per second of recis_gather (random rows in, one output row each) for 64- and 128-byte rows,
    next to the same calls with the rows in order."""
    from recis_amd import ops
    out = {"metric": "random requests per second", "block_filter_8B_reads": {}, "gather_rows": {}}
    n = 1 << 24
    for mb in (64, 1024, 4096, 8192):
        out["block_filter_8B_reads"]["%d_MB_slot" % mb] = round(_random_request_ceiling(mb, n) / 1e9, 2)
    n = 1 << 22
    for D in (16, 32):
        rows = (4 << 30) // (4 * D)
        table = torch.zeros(rows, D, device="cuda")
        idx = torch.randint(0, rows, (n,), device="cuda")
        seq = torch.arange(n, device="cuda")
        t_rand = _event_ms(lambda: ops.gather(idx, table), 10)
        t_seq = _event_ms(lambda: ops.gather(seq, table), 10)
        out["gather_rows"]["%d_byte_rows_4096_MB" % (4 * D)] = {
            "random_G_rows_per_s": round(n / t_rand / 1e6, 2), "in_order_G_rows_per_s": round(n / t_seq / 1e6, 2),
            "random_GBps_read": round(n * 4 * D / t_rand / 1e6, 1), "in_order_GBps_read": round(n * 4 * D / t_seq / 1e6, 1)}
        del table, idx, seq
        torch.cuda.empty_cache()
    # the bare probe: rows at random places and nothing else (recis_hip_probe_random_rows)
    from recis_amd import _lib
    lib, i64, ptr = _lib.lib(), _lib.i64, _lib.ptr
    sink = torch.zeros(4096, dtype=torch.int32, device="cuda")
    n = 1 << 23
    out["bare_rows"] = {}
    for mb in (256, 4096, 16384):
        table = torch.zeros(mb << 18, dtype=torch.int32, device="cuda")
        for row_bytes in (64, 128, 256):
            rows = (mb << 20) // row_bytes
            rand = torch.randint(0, rows, (n,), device="cuda", dtype=torch.int32)
            seq = (torch.arange(n, device="cuda", dtype=torch.int32) % rows).contiguous()
            res = {}
            for name, idx, in_flight, write in (("random_read", rand, 1, 0), ("random_read_4_in_flight", rand, 4, 0),
                                                ("random_write", rand, 1, 1), ("in_order_read", seq, 1, 0),
                                                ("in_order_write", seq, 1, 1)):
                def call():
                    _lib.check(lib.recis_hip_probe_random_rows(ptr(table), i64(rows), i64(row_bytes), ptr(idx), i64(n),
                                                               in_flight, write, ptr(sink), _lib.stream_ptr(table.device)))
                ms = _event_ms(call, 10)
                res[name] = {"G_rows_per_s": round(n / ms / 1e6, 1), "GBps": round(n * row_bytes / ms / 1e6)}
            out["bare_rows"]["%d_MB_table_%d_byte_rows" % (mb, row_bytes)] = res
            del rand, seq
        del table
        torch.cuda.empty_cache()
    out["unit"] = "G requests/s (block_filter), G rows/s (gather, bare_rows)"
    return out


def _request_roofline(wl, kernels_us, ms_per_step, ceiling):
    """The step against the random-request ceiling: requests per launch (MEASURED_REQUESTS) over
    the launch times measured in this run, per kernel and for the whole step."""
    req = MEASURED_REQUESTS.get(type(wl).__name__.lower().replace("config", "c"))
    if not req or "_variant_" in wl.name:
        return None
    per_kernel = {k: round(req[k] / kernels_us[k] / 1e3, 1) for k in req if kernels_us.get(k)}
    dom = max((k for k in per_kernel), key=lambda k: kernels_us[k])
    out = {"bound": "random requests to memory", "unit": "G requests/s", "peak": round(ceiling / 1e9, 1),
           "peak_source": "recis_block_filter at random rows of a 64 MB slot (4.3e10/s over 4 GB), this run",
           "kernel": dom, "achieved": per_kernel[dom], "frac": round(per_kernel[dom] * 1e9 / ceiling, 3),
           "requests_per_launch": req[dom], "kernels_g_requests_per_s": per_kernel}
    if type(wl).__name__ in ("Config3", "Config4"):   # steps whose every kernel of weight works at random places
        total = sum(req.values())
        out.update({"step_requests": total, "step_floor_ms": round(total / ceiling * 1e3, 4),
                    "step_frac": round(total / ceiling * 1e3 / ms_per_step, 3)})
    return out


def checkpoint_round_trip(rows=8 << 20, dim=16, parallel=8):
    """Save and load of one table with Adam state (rows x (8 B key + 3 x dim x 4 B)) through the
    checkpoint directory layout, to a scratch directory under TMPDIR. Not part of the step metric."""
    import shutil
    import tempfile

    from recis_amd.nn import HashTable
    from recis_amd.nn.modules.hashtable import HashtableRegister, filter_out_sparse_param
    from recis_amd.optim import SparseAdam
    from recis_amd.serialize import Loader, Saver

    def make(name):
        HashtableRegister().clear()
        ht = HashTable([dim], block_size=10240, device="cuda", name=name, children=["ckpt_bench"])
        SparseAdam(filter_out_sparse_param(ht), lr=1e-3)
        return ht

    ht = make("ckpt_bench_src")
    ids = torch.randperm(4 * rows, device="cuda")[:rows]
    ht._hashtable_impl.insert(ids, torch.randn(rows, dim, device="cuda"))
    nbytes = rows * (8 + 3 * dim * 4)
    path = tempfile.mkdtemp(prefix="recis_ckpt_")
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        Saver(0, 1, parallel, path, hashtables={"t": ht}).save()
        t_save = time.perf_counter() - t0
        dst = make("ckpt_bench_dst")
        t0 = time.perf_counter()
        Loader(path, hashtables={"t": dst}, parallel=parallel).load()
        torch.cuda.synchronize()
        t_load = time.perf_counter() - t0
        ok = dst._hashtable_impl.ids_num() == rows
    finally:
        shutil.rmtree(path, ignore_errors=True)
    return {"metric": "table checkpoint round trip", "rows": rows, "bytes": nbytes, "files": parallel,
            "save_s": round(t_save, 3), "save_GBps": round(nbytes / t_save / 1e9, 2),
            "load_s": round(t_load, 3), "load_GBps": round(nbytes / t_load / 1e9, 2), "loaded_all_rows": ok,
            "directory": os.path.dirname(path)}


def _timed_steps(wl, steps, warmup):
    if hasattr(wl, "prepare"):
        wl.prepare(steps + warmup)
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        wl.step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t) / steps * 1e3


def _kernel_roofline(wl, iters):
    """Per-kernel launch times of wl.step() (the library's HIP events on the launch stream) and the
    roofline object of the kernel with the largest share: algorithmic bytes per launch / mean launch
    time against the HBM peak."""
    if hasattr(wl, "prepare"):
        wl.prepare(iters + 2)
    kern = _kernel_profile(wl.step, iters)
    kb = wl.kernel_bytes()
    dom = max((k for k in kern if k in kb), key=lambda k: kern[k]["us"] * kern[k]["calls_per_step"])
    ach = kb[dom] / kern[dom]["us"] / 1e3
    roof = {"bound": "hbm", "kernel": dom, "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": ach / HBM_PEAK_GBS, "traffic": _measured_traffic(wl).get(dom), "launch_us": round(kern[dom]["us"], 2),
            "launches_per_step": kern[dom]["calls_per_step"], "algorithmic_bytes_per_launch": kb[dom]}
    kernels_us = {k: round(v["us"], 2) for k, v in sorted(kern.items(), key=lambda kv: -kv[1]["us"])}
    kernels_gbs = {k: round(kb[k] / kern[k]["us"] / 1e3, 1) for k in kern if kb.get(k)}
    return roof, kernels_us, kernels_gbs


def _step_roofline(wl, ms):
    """Whole-step fractions of the HBM peak, by the bytes the kernels as built must move and by the
    lowest price of the same config (every intermediate kept on chip)."""
    nbytes = wl.algorithmic_bytes()
    nbytes = sum(nbytes.values()) if isinstance(nbytes, dict) else nbytes
    out = {"algorithmic_bytes": nbytes, "achieved": nbytes / ms / 1e6, "frac": nbytes / ms / 1e6 / HBM_PEAK_GBS,
           "unit": "GB/s"}
    if hasattr(wl, "fused_minimum_bytes"):
        sb = wl.fused_minimum_bytes()
        out["fused_minimum_bytes"] = sb
        out["fused_minimum_frac"] = sb / ms / 1e6 / HBM_PEAK_GBS
    return out


def _c3_eviction(wl, step_ms):
    """Runs config 3 on to its next sweep of the step filter (every 50 steps, threshold step - 50)
    and reports it: the keys it evicted, its time, and the step time with the sweep spread over
    the 50 steps it serves. New keys per step come from the id map's own counters."""
    live0, idn0, _, _ = wl.table.id_map_stats()
    step0 = wl.step_no
    at, evicted, ms = wl.run_to_next_sweep()
    live1, idn1, _, _ = wl.table.id_map_stats()
    steps = wl.step_no - step0
    out = {"sweep_at_step": at, "evicted_per_sweep": evicted, "sweep_ms": round(ms, 3),
           "sweep_interval_steps": wl.filter_interval, "live_keys_before": live0, "live_keys_after": live1,
           "new_keys_per_step": round((live1 + evicted - live0) / max(steps, 1), 1),
           "ms_per_step_with_sweep": round(step_ms + ms / wl.filter_interval, 4)}
    # The first sweep removes the rows the table was loaded with and nobody looked up since (most of
    # the table). The one after it is what a long run sees: the keys of one interval's steps that did
    # not come back within the next.
    at2, evicted2, ms2 = wl.run_to_next_sweep()
    out["steady_sweep"] = {"sweep_at_step": at2, "evicted": evicted2, "sweep_ms": round(ms2, 3),
                           "live_keys_after": wl.table.id_map_stats()[0],
                           "ms_per_step_with_sweep": round(step_ms + ms2 / wl.filter_interval, 4)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c4", choices=["c4", "c2", "c3", "c5", "ckpt", "probe", "c4_unfused"],
                    help="c4_unfused: config 4 through the reference's own operator sequence alone (the torch_library_path_ms "
                         "leg of the default run), for a kernel trace of that sequence")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--batch", type=int, default=0,
                    help="config 4 with another number of samples per step (default 65536): a smaller table")
    ap.add_argument("--rotate", type=int, default=0,
                    help="config 4 rotating over this many batches (default 8): the table holds that many batches' keys")
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-stages", action="store_true",
                    help="skip the stage-by-stage timings, so that every kernel launch of the run belongs to a "
                         "full step (the form a kernel trace is compared with kernels_us in)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch a plain elementwise kernel that reads 1 GiB and writes 1 GiB "
                         "(scale for hardware-counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU that owns the whole table; --gpus %d is not supported "
              "(every GPU box of this build has one GPU; a sharded table would exchange ids and rows per step)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    os.environ.setdefault("OMP_NUM_THREADS", "1")

    if args.workload == "ckpt":
        print(json.dumps(checkpoint_round_trip()))
        return
    if args.workload == "probe":
        print(json.dumps(request_ceiling_probe()))
        return
    if args.workload == "c4_unfused":
        wl = TorchLibraryPath4()
        ms = _timed_steps(wl, args.steps, args.warmup)
        print(json.dumps({"workload": "config 4 through ids_encode -> ids_partition -> embedding_lookup -> "
                                      "segment_reduce_forward -> segment_reduce_backward -> accept_grad -> SparseAdam.step",
                          "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
                          "ids_per_s": wl.N / ms * 1e3}))
        return
    classes = {"c4": Config4, "c2": Config2, "c3": Config3, "c5": Config5}
    if args.workload == "c4" and (args.batch or args.rotate):   # a variant for experiments, named as such
        main_wl = Config4(batch=args.batch or 65536, n_batches=args.rotate or 8)
        main_wl.name += "_variant_batch%d_rotate%d" % (args.batch or 65536, args.rotate or 8)
        args.no_extra = args.no_cpu_baseline = True
    else:
        main_wl = classes[args.workload]()
    # part of set-up, before the W warm-up steps: the first steps of a process pay for the device
    # allocations of the step's outputs (config 5: 2 GB blocks, tens of ms)
    if hasattr(main_wl, "prepare"):
        main_wl.prepare(10 + args.warmup + args.steps)
    for _ in range(10):
        main_wl.step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        main_wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        main_wl.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = main_wl.ids_per_step / (dt / args.steps)

    out = {
        "metric": "embedding ids/sec (lookup+pool+bwd+sparse opt) at 1 GPU",
        "value": value, "unit": "ids/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": main_wl.name, "ids_per_step": main_wl.ids_per_step},
    }

    def c2_summary(wl):
        res = {}
        for kname, (fn, nbytes) in wl.kernels().items():
            ms = _event_ms(fn, 10)
            res[kname] = {"ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
                          "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_launch": nbytes,
                          "traffic": _measured_traffic(wl).get(kname)}
        return res

    def step_summary(wl, ms, iters):
        """One entry of "workloads": step time, ids/s, whole-step and dominant-kernel rooflines."""
        roof, kernels_us, _ = _kernel_roofline(wl, iters)
        nbytes = wl.algorithmic_bytes()
        nbytes = sum(nbytes.values()) if isinstance(nbytes, dict) else nbytes
        res = {"ms_per_step": round(ms, 4), "ids_per_s": wl.ids_per_step / ms * 1e3,
               "unique_ids_per_step": wl.U, "step_roofline": _step_roofline(wl, ms), "roofline": roof,
               "kernels_us": kernels_us}
        if out.get("request_roofline"):
            res["request_roofline"] = _request_roofline(wl, kernels_us, ms, out["request_roofline"]["peak"] * 1e9)
        return res

    if args.calib_copy:
        src = torch.zeros(1 << 28, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    extras = {}
    if args.workload == "c2":
        res = c2_summary(main_wl)
        dom = max(res, key=lambda k: res[k]["ms"])
        out["roofline"] = {"bound": "hbm", "kernel": dom, "achieved": res[dom]["gbs"], "peak": HBM_PEAK_GBS,
                           "unit": "GB/s", "frac": res[dom]["frac"], "traffic": res[dom]["traffic"],
                           "launch_us": round(res[dom]["ms"] * 1e3, 2),
                           "algorithmic_bytes_per_launch": res[dom]["algorithmic_bytes_per_launch"]}
        out["stages_ms"] = {k: v["ms"] for k, v in res.items()}
    else:
        stages = None
        if args.workload == "c4" and not args.no_stages:
            stages = main_wl.stage_times(max(5, args.steps))
        roof, kernels_us, kernels_gbs = _kernel_roofline(main_wl, max(5, args.steps))
        out["config"]["unique_ids_per_step"] = main_wl.U
        out["roofline"] = roof
        out["kernels_us"] = kernels_us
        out["kernels_gbs"] = kernels_gbs
        out["step_roofline"] = _step_roofline(main_wl, ms_per_step)
        ceiling = _random_request_ceiling(64)
        out["request_roofline"] = _request_roofline(main_wl, kernels_us, ms_per_step, ceiling)
        if stages is not None:
            ab = main_wl.algorithmic_bytes()
            out["stages_ms"] = {k: round(v, 4) for k, v in stages.items()}
            out["stages_gbs"] = {k: round(ab[k] / stages[k] / 1e6, 1) for k in stages}
            host_ms = _event_ms(main_wl.step_from_host, max(5, args.steps))
            out["inputs_from_pinned_host"] = {"ms_per_step": round(host_ms, 4),
                                              "ids_per_s": main_wl.N / host_ms * 1e3}
            over_ms = _event_ms(main_wl.step_from_host_overlapped, max(5, args.steps))
            torch.cuda.synchronize()
            out["inputs_from_pinned_host"]["overlapped_ms_per_step"] = round(over_ms, 4)
            out["inputs_from_pinned_host"]["overlapped_ids_per_s"] = main_wl.N / over_ms * 1e3
        if args.workload == "c3":
            out["eviction"] = _c3_eviction(main_wl, ms_per_step)
    if not args.no_extra:
        if args.workload != "c4":
            del main_wl
            main_wl = None
            torch.cuda.empty_cache()
        for key, cls in classes.items():
            if key == args.workload:
                continue
            wl = cls()
            if key == "c2":
                extras[wl.name] = c2_summary(wl)
                extras[wl.name]["ids_per_s"] = wl.ids_per_step / _event_ms(wl.step, 5) * 1e3
            else:
                extras[wl.name] = step_summary(wl, _timed_steps(wl, 8, 5), 8)
                if key == "c3":
                    extras[wl.name]["eviction"] = _c3_eviction(wl, extras[wl.name]["ms_per_step"])
            del wl
            torch.cuda.empty_cache()
        # the same steps through the drop-in module layer (EmbeddingEngine + sparse optimizer)
        for key, cls, name in (("c4", ModulePath4, Config4.name), ("c5", ModulePath5, Config5.name)):
            mp = cls()
            ms = _timed_steps(mp, 20, 5)
            target = out if key == args.workload else extras.get(name)
            if target is not None:
                target["module_path_ms"] = round(ms, 4)
            del mp
            torch.cuda.empty_cache()
        if args.workload == "c4":
            for key, make in (("module_path_with_concat_ms", lambda: ModulePath4(concat=True)),
                              ("torch_library_path_ms", TorchLibraryPath4)):
                wl = make()
                out[key] = round(_timed_steps(wl, 20, 5), 4)
                del wl
                torch.cuda.empty_cache()
        if main_wl is None and not args.no_cpu_baseline:
            main_wl = classes[args.workload]()
    if extras:
        out["workloads"] = extras

    if not args.no_cpu_baseline:
        cores = min(16, os.cpu_count() or 1)
        v, sample = main_wl.cpu_baseline(10.0)
        port = {"value": v, "unit": "ids/s", "cores": 1, "kind": "port", "sample": sample}
        ref = main_wl.cpu_reference(8.0, cores) if hasattr(main_wl, "cpu_reference") else None
        if ref is not None:   # the reference's own CPU code, all host cores of this box's share
            out["cpu_baseline"] = ref
            out["cpu_baseline_port_1core"] = port
            ref1 = main_wl.cpu_reference(4.0, 1)
            if ref1 is not None:
                out["cpu_baseline_reference_1core"] = ref1
        else:
            out["cpu_baseline"] = port
    from recis_amd import _lib
    out["device_errors"] = _lib.poll_device_errors()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
