"""The few ``BatchedDataDict`` methods the driver-side mirrors need (``size``, ``select_indices``,
``slice``, ``from_batches``; ``nemo_rl/distributed/batched_data_dict.py:191-330, 885-906, 1018-1060``).

The mirrors only call these methods, so a real NeMo-RL ``BatchedDataDict`` works in their place; this
class exists so that they can run and be tested without NeMo-RL.  Values are tensors (batch along
dim 0) or lists with one entry per sample.
"""

from __future__ import annotations

from typing import Any, Mapping, Optional, Sequence

import torch


class BatchedDataDict(dict):
    @property
    def size(self) -> int:
        if not self:
            return 0
        first = next(iter(self.values()))
        return first.shape[0] if torch.is_tensor(first) else len(first)

    def select_indices(self, indices) -> "BatchedDataDict":
        out = type(self)()
        for k, v in self.items():
            if torch.is_tensor(v):
                out[k] = v[indices]
            elif isinstance(v, list):
                out[k] = [v[i] for i in indices]
            else:
                raise TypeError(f"Unsupported type {type(v)} for index selection in BatchedDataDict")
        return out

    def slice(self, start: int, end: int) -> "BatchedDataDict":
        out = type(self)()
        for k, v in self.items():
            if torch.is_tensor(v):
                assert end <= v.shape[0], f"end: {end} is greater than the shape of the tensor: {v.shape[0]} for key: {k}"
            out[k] = v[start:end]
        return out

    @classmethod
    def from_batches(cls, batches: Sequence[Mapping[Any, Any]], pad_value_dict: Optional[dict] = None,
                     **_ignored) -> "BatchedDataDict":
        """Concatenate along the batch; tensors with a sequence axis are right-padded to the longest."""
        out = cls()
        pad_value_dict = pad_value_dict or {}
        if not batches:
            return out
        for k in batches[0]:
            vals = [b[k] for b in batches]
            if torch.is_tensor(vals[0]):
                if vals[0].dim() >= 2:
                    width = max(v.shape[1] for v in vals)
                    vals = [torch.nn.functional.pad(v, [0, 0] * (v.dim() - 2) + [0, width - v.shape[1]],
                                                    value=pad_value_dict.get(k, 0)) for v in vals]
                out[k] = torch.cat(vals, dim=0)
            else:
                out[k] = [x for v in vals for x in v]
        return out
