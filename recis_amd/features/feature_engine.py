"""``FeatureEngine``: runs a list of features step by step, batching the same-typed ops
of one step into ONE fused HIP launch (mirror of ``recis.features.feature_engine``,
feature_engine.py:107-284, with the fused implementations of fused_op_impl.py:113-516
for Mod, Bucketize, Hash, IDMultiHash and SequenceTruncate). Features with identical op chains are computed
once and shared."""
from collections import defaultdict
from typing import Dict, List

import torch
from torch import nn

from .. import ops
from ..ragged.tensor import RaggedTensor
from .feature import Feature
from .op import Bucketize, Hash, IDMultiHash, Mod, SequenceTruncate, _values, _with_values, sequence_truncate


def _fused_mod(op_list, inputs):
    outs = ops.fused_uint64_mod([_values(x).cuda() for x in inputs], [op.mod_value for op in op_list])
    return [_with_values(x, o) for x, o in zip(inputs, outs)]


def _fused_bucketize(op_list, inputs):
    outs = ops.fused_bucketized([_values(x).cuda().float() for x in inputs], [op.boundary.cuda() for op in op_list])
    return [_with_values(x, o) for x, o in zip(inputs, outs)]


def _fused_bucketize_mod(op_list, inputs):
    """Bucketize followed by Mod of the same feature: one pass (``op_list``: (Bucketize, Mod) pairs)."""
    vals = [_values(x) for x in inputs]
    if all(v.is_cuda and v.dtype == torch.float32 for v in vals):
        # the common case needs no conversions: one call of the registered operator
        outs = ops.recis_ops().fused_bucketized_mod(vals, [b.boundary_on(v.device) for (b, _), v in zip(op_list, vals)],
                                                    [m.mod_value for _, m in op_list])
        outs = [o if v.dim() == 1 else o.view(v.shape) for o, v in zip(outs, vals)]
    else:
        outs = ops.fused_bucketized([v.cuda().float() for v in vals], [b.boundary.cuda() for b, _ in op_list],
                                    mods=[m.mod_value for _, m in op_list])
    return [_with_values(x, o) for x, o in zip(inputs, outs)]


def _fused_hash(op_list, inputs):
    results = [None] * len(inputs)
    for kind in ("farm", "murmur"):
        idx = [i for i, op in enumerate(op_list) if op.hash_type == kind]
        if not idx:
            continue
        outs = ops.fused_hash([inputs[i].values().cuda() for i in idx],
                              [inputs[i].offsets()[-1].cuda() for i in idx], kind)
        for i, o in zip(idx, outs):
            rest = [t.cuda() for t in inputs[i].offsets()[:-1]]
            if not rest:
                import torch
                rest = [torch.arange(o.numel() + 1, device=o.device)]
            results[i] = RaggedTensor(o, rest, None)
    return results


def _fused_multi_hash(op_list, inputs):
    outs = ops.fused_multi_hash([_values(x).cuda() for x in inputs], [op.muls for op in op_list],
                                [op.primes for op in op_list], [op.num_buckets for op in op_list])
    results, k = [], 0
    for op, x in zip(op_list, inputs):
        n = len(op.muls)
        results.append({"%s_%d" % (op.prefix, j): _with_values(x, outs[k + j]) for j in range(n)})
        k += n
    return results


_CHAIN = "bucketize+mod"   # a Bucketize whose feature goes on with a Mod: both in one launch
_FUSED = {Mod: _fused_mod, Bucketize: _fused_bucketize, Hash: _fused_hash, IDMultiHash: _fused_multi_hash,
          SequenceTruncate: sequence_truncate, _CHAIN: _fused_bucketize_mod}


class FeatureEngine(nn.Module):
    def __init__(self, feature_list: List[Feature]):
        super().__init__()
        self._features = nn.ModuleDict()
        self._alias = {}
        by_hash = defaultdict(list)
        for f in feature_list:
            by_hash[f.get_hash()].append(f)
        for group in by_hash.values():
            primary = group[0]
            if primary.name in self._features:
                raise ValueError("Duplicate feature name: %s" % primary.name)
            if primary.compiled:
                raise ValueError("feature %s has been compiled" % primary.name)
            primary.compiled_(True)
            self._features[primary.name] = primary
            for dup in group[1:]:
                self._alias[dup.name] = primary.name
        # step k = the k-th op of every feature that has one, grouped by op class
        self._steps = []
        feats = list(self._features.values())
        depth = max((len(f.ops) for f in feats), default=0)
        done_early = set()  # (feature, k): op k of the feature was applied together with op k - 1
        for k in range(depth):
            groups = defaultdict(list)
            for f in feats:
                if k < len(f.ops) and (f.name, k) not in done_early:
                    op = f.ops[k]
                    nxt = f.ops[k + 1] if k + 1 < len(f.ops) else None
                    if type(op) is Bucketize and type(nxt) is Mod and 0 < nxt.mod_value and \
                            not (nxt._forward_hooks or nxt._forward_pre_hooks or op._forward_hooks or op._forward_pre_hooks):
                        groups[_CHAIN].append((f.name, (op, nxt)))
                        done_early.add((f.name, k + 1))
                        continue
                    groups[type(op) if type(op) in _FUSED else ("single", f.name)].append((f.name, op))
            self._steps.append(groups)

    def forward(self, data: Dict, remain_no_use_data: bool = True) -> Dict:
        assert isinstance(data, dict), "data must be a dict"
        state = {}
        for step_idx, groups in enumerate(self._steps):
            for key, members in groups.items():
                names = [n for n, _ in members]
                op_list = [op for _, op in members]
                inputs = [state[n] if step_idx > 0 else data for n in names]
                if key in _FUSED and (len(members) > 1 or key == _CHAIN):
                    outs = _FUSED[key](op_list, inputs)
                else:
                    # Module.__call__ costs several microseconds of hook bookkeeping per op, which is
                    # most of a SelectField; ops with no hooks registered are called directly
                    outs = [op(x) if (op._forward_hooks or op._forward_pre_hooks) else op.forward(x)
                            for op, x in zip(op_list, inputs)]
                for n, o in zip(names, outs):
                    state[n] = o
        results = dict(data) if remain_no_use_data else {}
        for name, out in state.items():
            if isinstance(out, dict):
                results.update(out)
            else:
                results[name] = out
        for dup, primary in self._alias.items():
            results[dup] = results[primary]
        return results
