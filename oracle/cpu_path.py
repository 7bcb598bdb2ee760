"""The reference's CPU embedding path restated end to end from the oracle's pieces:
TEST INFRASTRUCTURE (parity checker and timed CPU baseline), never product code.

One training step, as the reference runs it on a CPU-resident table:
  1. ``ids.unique(return_inverse=True)``               recis/nn/modules/hashtable.py:278
  2. ``CpuIdMap::Lookup`` + allocator                   csrc/embedding/cpu_id_map.cc:73-90
  3. block growth ``(id_num + bs) / bs``                csrc/embedding/hashtable.cc:255-261
  4. ``block_gather`` of the unique rows                csrc/ops/block_ops.cc:186-221
  5. pooling over the occurrences (torch backend: ``emb[idx] * w`` + ``index_add_``;
     the arithmetic of embedding_ops.py:59-66,109-125 / the segment-reduce kernel)
  6. backward scatter to the unique rows (transpose of 5; duplicates summed, /world=1)
  7. fused row update: ``block_apply_adamw``            csrc/ops/block_apply_adamw_op.cc:9-132
     or Adagrad (no reference counterpart)
  8. optional last-seen-step stamp and eviction         hashtable_hook_impl.py:487-551
"""
import numpy as np

from . import (IdMap, block_apply_adagrad, block_apply_adamw, block_filter, block_gather, block_insert,
               segment_reduce_backward, segment_reduce_forward)


class CpuTable:
    def __init__(self, dim, block_size, init_block, optimizer="adagrad", lr=0.01, eps=1e-8, beta1=0.9,
                 beta2=0.999, decay=1.0, beta_dtype=np.float64, step_filter=False):
        """``init_block(block_index) -> [block_size, dim] float32``: the rows a new block starts with."""
        self.dim, self.bs, self.init_block = dim, block_size, init_block
        self.optimizer, self.lr, self.eps = optimizer, lr, eps
        self.beta1, self.beta2, self.decay = beta1, beta2, decay
        self.idmap = IdMap()
        self.emb, self.s0, self.s1 = [], [], []
        self.b1t, self.b2t = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
        self.stamp = [] if step_filter else None
        self.global_step = 0

    def _grow(self):
        want = (self.idmap.id_num() + self.bs) // self.bs
        while len(self.emb) < want:
            self.emb.append(np.ascontiguousarray(self.init_block(len(self.emb)), dtype=np.float32))
            self.s0.append(np.zeros((self.bs, self.dim), np.float32))
            self.s1.append(np.zeros((self.bs, self.dim), np.float32))
            if self.stamp is not None:
                self.stamp.append(np.zeros((self.bs, 1), np.int64))

    def lookup(self, unique_ids):
        index = self.idmap.lookup(unique_ids)
        self._grow()
        rows = block_gather(index, self.emb, self.bs)
        if self.stamp is not None:
            block_insert(index, np.array([[self.global_step]], np.int64), self.stamp, self.bs)
        return index, rows

    def apply(self, index, grad):
        if self.optimizer == "adagrad":
            block_apply_adagrad(index, grad, self.emb, self.s0, self.lr, self.eps, self.bs)
        else:
            block_apply_adamw(index, grad, self.emb, self.b1t, self.b2t, self.s0, self.s1, self.lr, self.beta1,
                              self.beta2, self.decay, self.eps, self.bs)

    def evict_older_than(self, filter_step):
        """GlobalStepFilter: drop keys with stamp < global_step - filter_step; freed rows are
        re-initialised (here: zero state, embedding from ``reinit``) and recycled."""
        ids, index = self.idmap.snapshot()
        mask = block_filter(index, self.stamp, self.bs, self.global_step - filter_step)
        self.idmap.delete(ids[mask], index[mask])
        return ids[mask], index[mask]

    def rows_of(self, ids):
        index = self.idmap.lookup_readonly(ids)
        return index, block_gather(index, self.emb, self.bs)


def train_step(table, ids, offsets, weight, grad_out, combiner="sum"):
    """One full step; returns (pooled output, unique ids, their row index)."""
    uniq, inverse = np.unique(ids, return_inverse=True)
    index, rows = table.lookup(uniq)
    pooled = segment_reduce_forward(rows, weight, inverse, offsets, combiner)
    g_unique = segment_reduce_backward(grad_out, weight, inverse, offsets, len(uniq), combiner)
    table.apply(index, g_unique)
    table.global_step += 1
    return pooled, uniq, index
