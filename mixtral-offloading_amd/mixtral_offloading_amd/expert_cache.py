"""LRU cache of experts over fixed device slots, fed from pinned host slabs.

Same surface as the reference's ``ExpertCache`` (``src/expert_cache.py``):
``ExpertCache(make_module, main_size, offload_size, buffer_size)``,
``add_expert(uid, module, eviction_group, offload)``, and
``load_experts(*uids, unordered)`` yielding ``(uid, module)`` pairs that are
only valid inside the loop.  What is different underneath:

* the policy (which expert a miss evicts, hit / miss counts) is the host-only
  C++ object ``hqq_lru`` of the library, one per eviction group;
* every expert keeps a pinned host copy for its whole life, so an eviction
  copies nothing back (the reference copies the victim device-to-host,
  ``src/expert_cache.py:189``; weights are immutable, the copy is redundant);
* host-to-device loads are ``hipMemcpyAsync`` from pinned memory on a side
  stream (``hqq_slab_h2d_async``), ordered against the compute stream with
  events in both directions, so they overlap whatever the compute stream is
  doing (the reference copies on the current stream, ``:188``);
* a miss loads into a spare device slot and the victim's slot becomes the next
  spare (the reference's buffer rotation, ``:186-194``), so a load never waits
  for the victim's last use."""
from __future__ import annotations

import ctypes
from collections import deque
from dataclasses import dataclass
from typing import Any, Dict, Iterator, List, Optional, Tuple

import torch

from . import _lib
from .expert_wrapper import MixtralExpertWrapper

ExpertUID = Any
_MAX_GROUP_EXPERTS = 4096


@dataclass
class ExpertInfo:
    uid: ExpertUID
    eviction_group: int
    index: int  # index of the expert inside its eviction group
    host_slab: torch.Tensor  # pinned uint8 copy, kept for the life of the cache

    @property
    def offloaded(self) -> bool:
        return self._group.slot_of(self.index) < 0


class EvictionGroup:
    """One ``hqq_lru`` plus the map from its local slots to global device slots."""

    def __init__(self, slots_cap: int):
        self._lru = _lib.lib.hqq_lru_create(_MAX_GROUP_EXPERTS, slots_cap)
        if not self._lru:
            raise MemoryError("hqq_lru_create failed")
        self.members: List[ExpertInfo] = []
        self.global_slot: List[int] = []  # local slot -> global device slot

    def __del__(self):
        if getattr(self, "_lru", None):
            _lib.lib.hqq_lru_destroy(self._lru)
            self._lru = None

    @property
    def hits(self) -> int:
        return _lib.lib.hqq_lru_hits(self._lru)

    @property
    def misses(self) -> int:
        return _lib.lib.hqq_lru_misses(self._lru)

    def slot_of(self, index: int) -> int:
        return _lib.lib.hqq_lru_slot_of(self._lru, index)

    def add_resident(self, index: int, global_slot: int) -> None:
        local = _lib.lib.hqq_lru_add_resident(self._lru, index)
        if local < 0:
            raise ValueError("Cache is full")
        assert local == len(self.global_slot)
        self.global_slot.append(global_slot)

    def plan(self, indices: List[int]):
        n = len(indices)
        arr = (ctypes.c_int32 * n)(*indices)
        order, slot, victim = (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)()
        rc = _lib.lib.hqq_lru_plan(self._lru, arr, n, order, slot, victim)
        if rc != 0:
            raise ValueError("No evictable experts" if not self.global_slot else "invalid expert request")
        return list(order), list(slot), list(victim)


class ExpertCache:
    def __init__(self, make_module: callable, main_size: int, offload_size: int, buffer_size: int):
        """Dynamically loads an array of modules with identical hyperparameters."""
        self.module_type = self.module_size = self.device = None
        self.active = False
        self.registered_experts: Dict[ExpertUID, ExpertInfo] = dict()
        self.main_size, self.offload_size, self.buffer_size = main_size, offload_size, buffer_size

        # device slots: main_size resident places plus buffer_size spares that misses load into
        self.slots: List[MixtralExpertWrapper] = [self._check_module(make_module()) for _ in range(main_size + buffer_size)]
        assert self.module_size is not None
        self.free_main = deque(range(main_size))
        self.spare = deque(range(main_size, main_size + buffer_size))
        self.group_infos: Dict[int, EvictionGroup] = dict()
        self.n_offloaded = 0

        assert self.device.type == "cuda", "experts are cached on a GPU"
        self.copy_stream = torch.cuda.Stream(device=self.device)  # default priority
        self.ready = [torch.cuda.Event() for _ in self.slots]  # load into the slot finished (copy stream)
        self.released = [torch.cuda.Event() for _ in self.slots]  # last use of the slot finished (compute stream)
        self._used = [False] * len(self.slots)
        self.bytes_copied = 0

    def _check_module(self, module: MixtralExpertWrapper):
        assert isinstance(module.storage, torch.UntypedStorage)
        if self.module_type is None:
            self.module_type = type(module)
            self.module_size = len(module.storage)
            self.device = module.storage.device
        else:
            assert isinstance(module, self.module_type)
            assert len(module.storage) == self.module_size
            assert module.storage.device == self.device
        return module

    def _group(self, g: int) -> EvictionGroup:
        if g not in self.group_infos:
            self.group_infos[g] = EvictionGroup(self.main_size + self.buffer_size)
        return self.group_infos[g]

    def add_expert(self, uid: ExpertUID, module: MixtralExpertWrapper, eviction_group: int = 0,
                   offload: Optional[bool] = None):
        """Register an expert to the cache and associate it with uid."""
        assert self.module_type is not None
        assert isinstance(module, self.module_type)
        return self.add_expert_storage(uid, module.storage, eviction_group=eviction_group, offload=offload)

    def add_expert_storage(self, uid: ExpertUID, storage: torch.UntypedStorage, eviction_group: int = 0,
                           offload: Optional[bool] = None):
        assert uid not in self.registered_experts, f"expert {uid} already registered"
        assert isinstance(storage, torch.UntypedStorage)
        assert len(storage) == self.module_size
        group = self._group(eviction_group)
        to_device = (offload is None or not offload) and len(self.free_main) > 0
        if not to_device:
            if offload is False or self.n_offloaded >= self.offload_size:
                raise ValueError("Cache is full")
        host = torch.empty(self.module_size, dtype=torch.uint8, pin_memory=True)
        host.copy_(torch.as_tensor(storage, dtype=torch.uint8, device=storage.device))
        info = ExpertInfo(uid, eviction_group, len(group.members), host)
        info._group = group
        group.members.append(info)
        self.registered_experts[uid] = info
        if to_device:
            slot = self.free_main.popleft()
            self.slots[slot].storage.copy_(storage)
            group.add_resident(info.index, slot)
        else:
            self.n_offloaded += 1

    def load_experts(self, *uids: ExpertUID, unordered: bool = False) -> Iterator[Tuple[ExpertUID, MixtralExpertWrapper]]:
        """
        :example:
        >>> for uid, expert in expert_cache.load_experts(*list_of_uids, unordered=True):
        >>>     result += expert(x) * get_moe_weight(uid)

        :param uids: iterate over the specified expert uids. Same uids as in add_expert
        :param unordered: if True, allows cache to iterate experts in arbitrary order
            (resident experts first, so that loads overlap their computation)
        :returns: an iterator that yields (uid, expert) pairs, only usable inside the for loop
        """
        assert len(set(uids)) == len(uids)
        assert not self.active, "already loading experts; buffers are busy"
        infos = [self.registered_experts[uid] for uid in uids]
        if not infos:
            return
        assert len(set(info.eviction_group for info in infos)) == 1, "experts must be in the same evicton group"
        group = self.group_infos[infos[0].eviction_group]
        order, local_slots, victims = group.plan([info.index for info in infos])
        compute = torch.cuda.current_stream(self.device)
        miss = {idx: victim >= 0 for idx, victim in zip(order, victims)}
        local_of = dict(zip(order, local_slots))
        to_load = deque(idx for idx in order if miss[idx])  # in the order the policy evicted for them
        slot_for: Dict[int, int] = {idx: group.global_slot[local_of[idx]] for idx in order if not miss[idx]}
        waiting = set()  # device slots holding an expert of this call that has not been handed out yet

        def issue_loads():
            # Start as many loads as there are spare slots, on the side stream.  A spare that still holds an expert
            # of this call (evicted again by a later miss of the same call) is not touched until that expert has
            # been handed out; it is always ahead in the sequence, so this cannot stall.
            while to_load and self.spare and self.spare[0] not in waiting:
                idx = to_load.popleft()
                dst = self.spare.popleft()
                local = local_of[idx]
                self.spare.append(group.global_slot[local])  # the victim's slot is the next spare
                group.global_slot[local] = dst
                if self._used[dst]:  # its last reader on the compute stream must be done before it is overwritten
                    self.copy_stream.wait_event(self.released[dst])
                self._copy_in(group.members[idx], dst)
                slot_for[idx] = dst
                waiting.add(dst)

        try:
            self.active = True
            if to_load and not self.spare:
                raise ValueError("No free device buffer: buffer_size must be at least 1")
            issue_loads()
            sequence = order if unordered else [info.index for info in infos]
            for idx in sequence:
                if idx not in slot_for:
                    issue_loads()
                    if idx not in slot_for:
                        raise RuntimeError("internal error: caching algorithm failed")
                slot = slot_for[idx]
                if miss[idx]:
                    compute.wait_event(self.ready[slot])
                yield (group.members[idx].uid, self.slots[slot])
                self.released[slot].record(compute)
                self._used[slot] = True
                waiting.discard(slot)
                issue_loads()
        finally:
            self.active = False

    def _copy_in(self, info: ExpertInfo, slot: int) -> None:
        dst = self.slots[slot].storage
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib.hqq_slab_h2d_async(dst.data_ptr(), info.host_slab.data_ptr(), self.module_size,
                                                   self.copy_stream.cuda_stream, None), "hqq_slab_h2d_async")
            self.ready[slot].record(self.copy_stream)
        self.bytes_copied += self.module_size

    def resident_group(self, eviction_group: int) -> Optional[List[MixtralExpertWrapper]]:
        """The device modules of every expert of a group, in expert order, when all of them are resident and none
        can be evicted (no expert of the cache is offloaded); else None."""
        if self.n_offloaded > 0 or eviction_group not in self.group_infos:
            return None
        group = self.group_infos[eviction_group]
        out = []
        for info in group.members:
            local = _lib.lib.hqq_lru_slot_of(group._lru, info.index)
            if local < 0:
                return None
            out.append(self.slots[group.global_slot[local]])
        return out

    # convenience counters (the reference keeps hits / misses per EvictionGroupInfo)
    def stats(self) -> Dict[str, int]:
        return {"hits": sum(g.hits for g in self.group_infos.values()),
                "misses": sum(g.misses for g in self.group_infos.values()), "bytes_copied": self.bytes_copied}
