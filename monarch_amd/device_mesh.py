"""``DeviceMesh``: which ranks form the reduce group of the named mesh dimensions.

Mirror of monarch_tensor_worker/src/device_mesh.rs:58-177, relative to one owning rank.
The group size is the ``N`` that Avg divides by and that scatter splits into
(monarch_tensor_worker/src/lib.rs:899,911).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Sequence

from ._lib import check, lib, u64_array
from .ndslice import Slice


@dataclass(frozen=True)
class Dim:
    name: str
    rank: int          # position of the owning rank inside the dimension
    size: int
    members: List[int]  # members[rank] is the owning rank


class DeviceMesh:
    def __init__(self, names: Sequence[str], ranks: Slice, rank: int):
        if len(names) != ranks.ndim:
            raise ValueError(f"names and coordinates mismatch in length: names={list(names)}")
        self.names = list(names)
        self.ranks = ranks
        self.rank = rank
        self.dims: Dict[str, Dim] = {}
        for d, name in enumerate(self.names):
            members = u64_array([0] * ranks.sizes[d])
            dim_rank = C.c_uint64()
            rc = lib().mhip_mesh_dim_members(C.byref(ranks.c), rank, d, members, C.byref(dim_rank))
            if rc:
                raise ValueError(f"value {rank} not in slice")
            self.dims[name] = Dim(name, dim_rank.value, ranks.sizes[d], list(members)[: ranks.sizes[d]])
        self.all_ranks = list(ranks)

    def sizes(self) -> Dict[str, int]:
        return {n: d.size for n, d in self.dims.items()}

    def get_ranks_for_dim_slice(self, names: Sequence[str]) -> List[int]:
        for n in names:
            if n not in self.dims:
                raise KeyError(f"no dim with name {n}")
        idx = [self.names.index(n) for n in names]
        cap = 1
        for i in idx:
            cap *= self.ranks.sizes[i]
        out = u64_array([0] * cap)
        count = C.c_uint64()
        arr = (C.c_uint32 * max(1, len(idx)))(*idx)
        check(lib().mhip_mesh_ranks_for_dims(C.byref(self.ranks.c), self.rank, arr, len(idx), out, cap, C.byref(count)))
        return list(out)[: count.value]

    def group_size(self, names: Sequence[str]) -> int:
        return len(self.get_ranks_for_dim_slice(names))
