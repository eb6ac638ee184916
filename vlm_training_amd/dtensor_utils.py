"""Strip and restore DTensor wrapping around the kernels (models/qwen3_5/utils.py:13-42).

Under the reference's tensor parallelism the projections are column-parallel, so an attention layer holds q, k, v
as DTensors sharded by head; the HIP kernels take plain local tensors (``Hq/tp`` and ``Hkv/tp`` heads over the
whole packed row) and need no collective.  ``_dtensor_unwrap`` hands out the local shards and remembers mesh and
placements of the first tensor, ``_dtensor_rewrap`` puts a kernel's output back under them.
"""
from __future__ import annotations

import torch

try:                                                     # torch builds without distributed support have no DTensor
    from torch.distributed.tensor import DTensor
except Exception:                                        # pragma: no cover
    DTensor = None


def _is_dtensor(t) -> bool:
    return DTensor is not None and isinstance(t, DTensor)


@torch.compiler.disable(recursive=True)
def _dtensor_unwrap(*tensors):
    """``(local_tensors, wrap_info)``: ``wrap_info`` is None when the first tensor is a plain tensor, else its
    ``(device_mesh, placements)``."""
    first = tensors[0]
    if _is_dtensor(first):
        wrap = (first.device_mesh, first.placements)
        return tuple(t.to_local() if _is_dtensor(t) else t for t in tensors), wrap
    return tensors, None


@torch.compiler.disable(recursive=True)
def _dtensor_rewrap(tensor, wrap_info):
    if wrap_info is None:
        return tensor
    mesh, placements = wrap_info
    return DTensor.from_local(tensor, device_mesh=mesh, placements=placements, run_check=False)


def _local(param):
    """The local shard of a parameter, DTensor or plain."""
    return param.to_local() if _is_dtensor(param) else param
