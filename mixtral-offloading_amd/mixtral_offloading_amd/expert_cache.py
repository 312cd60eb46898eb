"""LRU cache of experts over fixed device slots, fed from pinned host slabs.

Same surface as the reference's ``ExpertCache`` (``src/expert_cache.py``):
``ExpertCache(make_module, main_size, offload_size, buffer_size)``,
``add_expert(uid, module, eviction_group, offload)``, and
``load_experts(*uids, unordered)`` yielding ``(uid, module)`` pairs that are
only valid inside the loop.  What is different underneath:

* the policy (which expert a miss evicts, hit / miss counts) is the host-only
  C++ object ``hqq_lru`` of the library, one per eviction group;
* every expert that can be evicted (any expert of a group with an offloaded
  member) keeps a pinned host copy for its whole life, so an eviction
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
    # pinned uint8 copy, kept for the life of the cache; None while the expert cannot be evicted (no expert of its
    # group is offloaded), so that a fully resident model pins nothing
    host_slab: Optional[torch.Tensor]

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
        self.evictable = False  # true once an expert of the group is offloaded: residents can then be evicted
        self.last_request: set = set()  # the experts of the group's latest real request
        self.last_guess: set = set()    # the experts of the latest guess, until the next real request scores it

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

    def plan_guess(self, indices: List[int], keep: List[int]):
        """The policy's part of a speculative load: which of the guessed experts are loaded, where, and whom they evict
        (never an expert of `keep`); resident experts are left alone and nothing is counted."""
        n, nk = len(indices), len(keep)
        arr, kp = (ctypes.c_int32 * n)(*indices), (ctypes.c_int32 * max(nk, 1))(*keep)
        order, slot, victim = (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)()
        count = ctypes.c_int32(0)
        rc = _lib.lib.hqq_lru_plan_guess(self._lru, arr, n, kp, nk, order, slot, victim, ctypes.byref(count))
        if rc != 0:
            raise ValueError("invalid expert request")
        k = count.value
        return list(order[:k]), list(slot[:k]), list(victim[:k])


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

        self._init_device_side()
        self._used = [False] * len(self.slots)
        self.bytes_copied = 0
        self._copy_pending = set()  # slots filled by a copy that the compute stream has not been made to wait for yet
        # speculative prefetches: experts loaded on a guess and not asked for yet, and how the guesses turned out
        self._speculative = set()
        self.prefetch_loads = 0   # copies started on a guess
        self.prefetch_useful = 0  # of those, experts that a real request then found on the device
        self.prefetch_skipped_busy = 0       # guesses dropped because the copy stream still had work (host link busy)
        self.prefetch_skipped_protected = 0  # guesses dropped because only the latest request's experts could have made room
        # how often a guessed expert is asked for next, and how often an expert of a request is asked for again by the
        # next request of its group: every guess is scored, acted on or not
        self.prefetch_backlog = 0  # unfinished copies a guess may queue behind (0: only on an idle link)
        # Guesses are acted on only while the link is found busy in less than this share of the recent prefetch calls:
        # when loads bound the step (measured: busy at 80 - 96 % of the calls with a random router), tokens per second
        # go with the bytes copied and every wrong guess costs its slab, even one started on a momentarily idle link.
        self.prefetch_busy_limit = 0.25
        self._busy_share = 1.0  # running mean of "the link had unfinished copies" over prefetch calls
        self._inflight: set = set()  # slots whose copy may still be running
        self.guess_scored = self.guess_right = 0
        self.reuse_scored = self.reuse_right = 0
        self.copy_trace = None    # a list: (uid, start event, end event, kind) of every copy, for tests that look at overlap
        self._copy_kind = "demand"

    # ---- the device side, kept apart so that the scheduling above it can be driven on a machine without a GPU
    def _init_device_side(self) -> None:
        assert self.device.type == "cuda", "experts are cached on a GPU"
        self.copy_stream = torch.cuda.Stream(device=self.device)  # default priority
        self.ready = [torch.cuda.Event() for _ in self.slots]  # load into the slot finished (copy stream)
        self.released = [torch.cuda.Event() for _ in self.slots]  # last use of the slot finished (compute stream)

    def _compute_stream(self):
        return torch.cuda.current_stream(self.device)

    def _link_backlog(self) -> int:
        """Copies given to the copy stream that have not finished yet (host-side event queries, no synchronisation)."""
        self._inflight = {slot for slot in self._inflight if not self.ready[slot].query()}
        return len(self._inflight)

    def _alloc_host(self, nbytes: int) -> torch.Tensor:
        return torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)

    def _copy_in(self, info: ExpertInfo, slot: int) -> None:
        dst = self.slots[slot].storage
        with torch.cuda.device(self.device):
            if self.copy_trace is not None:
                t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                t0.record(self.copy_stream)
            _lib.check(_lib.lib.hqq_slab_h2d_async(dst.data_ptr(), info.host_slab.data_ptr(), self.module_size,
                                                   self.copy_stream.cuda_stream, None), "hqq_slab_h2d_async")
            self.ready[slot].record(self.copy_stream)
            self._inflight.add(slot)
            if self.copy_trace is not None:
                t1.record(self.copy_stream)
                self.copy_trace.append((info.uid, t0, t1, self._copy_kind))

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

    def _pin(self, source: torch.UntypedStorage) -> torch.Tensor:
        host = self._alloc_host(self.module_size)
        host.copy_(torch.as_tensor(source, dtype=torch.uint8, device=source.device))
        return host

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
        # Host copies are pinned only for experts that can leave the device: an expert can be evicted once any expert
        # of its group is offloaded (a miss of that group then takes a resident one's place).
        if not to_device and not group.evictable:
            group.evictable = True
            for member in group.members:
                member.host_slab = self._pin(self.slots[group.global_slot[group.slot_of(member.index)]].storage)
        info = ExpertInfo(uid, eviction_group, len(group.members), self._pin(storage) if group.evictable else None)
        info._group = group
        group.members.append(info)
        self.registered_experts[uid] = info
        if to_device:
            slot = self.free_main.popleft()
            self.slots[slot].storage.copy_(storage)
            group.add_resident(info.index, slot)
        else:
            self.n_offloaded += 1

    def expert_bytes(self, uid: ExpertUID) -> torch.Tensor:
        """The slab of a registered expert as a uint8 tensor: its pinned host copy, or (an expert that cannot be
        evicted has none) a view of the device slot it lives in."""
        info = self.registered_experts[uid]
        if info.host_slab is not None:
            return info.host_slab
        group = self.group_infos[info.eviction_group]
        storage = self.slots[group.global_slot[group.slot_of(info.index)]].storage
        return torch.as_tensor(storage, dtype=torch.uint8, device=storage.device)

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
        request = {info.index for info in infos}
        if group.last_guess:
            self.guess_scored += len(group.last_guess)
            self.guess_right += len(group.last_guess & request)
            group.last_guess = set()
        if group.last_request:
            self.reuse_scored += len(group.last_request)
            self.reuse_right += len(group.last_request & request)
        group.last_request = request
        compute = self._compute_stream()
        miss = {idx: victim >= 0 for idx, victim in zip(order, victims)}
        self._settle_speculation(group, order, victims, real=True)
        local_of = dict(zip(order, local_slots))
        sequence = order if unordered else [info.index for info in infos]
        rank = {idx: i for i, idx in enumerate(sequence)}
        to_load = deque(idx for idx in order if miss[idx])  # in the order the policy evicted for them
        slot_for: Dict[int, int] = {idx: group.global_slot[local_of[idx]] for idx in order if not miss[idx]}
        # Device slots whose content is an expert of this call that has not been handed out yet -- hits included: the
        # policy marks every requested expert used and then lets later misses of the same call evict the earlier ones
        # (a call may ask for more experts than the group has places).  Nothing is copied into such a slot.
        holder: Dict[int, int] = {slot: idx for idx, slot in slot_for.items()}
        copied = set()  # experts whose slot is filled by a copy of this call: the compute stream waits for it
        again = set()   # experts whose slot had to be given up before their turn (ordered iteration only)

        def copy_to(idx: int, dst: int) -> None:
            if self._used[dst]:  # its last reader on the compute stream must be done before it is overwritten
                self.copy_stream.wait_event(self.released[dst])
            self._copy_in(group.members[idx], dst)
            self.bytes_copied += self.module_size
            self._copy_pending.add(dst)
            slot_for[idx] = dst
            holder[dst] = idx
            copied.add(idx)

        def give_up(candidates) -> int:
            # every candidate holds an expert that this call still has to hand out, all of them later in the sequence
            # (ordered iteration asked for a miss before hits that the policy evicted for it): the one needed last
            # loses its place and is copied in again from its host slab when its turn comes
            dst = max(candidates, key=lambda s: rank[holder[s]])
            bumped = holder.pop(dst)
            del slot_for[bumped]
            again.add(bumped)
            return dst

        def start_load(idx: int, force: bool) -> bool:
            # A miss goes into a spare slot and its victim's slot becomes the next spare (so the copy never waits for
            # the victim's last use), or, with no spare free, into the victim's own slot.
            local = local_of[idx]
            home = group.global_slot[local]
            dst = next((s for s in self.spare if s not in holder), None)
            if dst is None and home not in holder:
                dst = home
            if dst is None:
                if not force:
                    return False
                dst = give_up([home] + list(self.spare))
            if dst != home:
                self.spare.remove(dst)
                self.spare.append(home)
                group.global_slot[local] = dst
            copy_to(idx, dst)
            return True

        def issue_loads() -> None:
            while to_load and start_load(to_load[0], force=False):
                to_load.popleft()

        try:
            self.active = True
            issue_loads()
            for idx in sequence:
                if idx not in slot_for:
                    issue_loads()
                if idx not in slot_for and idx in again:
                    # evicted by the policy within this call: it only passes through a spare slot
                    if not self.spare:
                        raise RuntimeError("internal error: caching algorithm failed")
                    dst = next((s for s in self.spare if s not in holder), None)
                    copy_to(idx, dst if dst is not None else give_up(list(self.spare)))
                elif idx not in slot_for:
                    if not to_load or to_load[0] != idx:
                        raise RuntimeError("internal error: caching algorithm failed")
                    start_load(to_load.popleft(), force=True)
                slot = slot_for[idx]
                if slot in self._copy_pending:  # filled by this call, or by a prefetch nobody has waited for yet
                    compute.wait_event(self.ready[slot])
                    self._copy_pending.discard(slot)
                yield (group.members[idx].uid, self.slots[slot])
                self.released[slot].record(compute)
                self._used[slot] = True
                del holder[slot]
                issue_loads()
        finally:
            # a caller that leaves the loop early: the policy already counts the remaining misses as resident
            holder.clear()
            while to_load:
                start_load(to_load.popleft(), force=True)
            self.active = False

    def _settle_speculation(self, group: EvictionGroup, order, victims, real: bool) -> None:
        """Book-keeping of guesses after a plan: a real request that finds a speculatively loaded expert makes that
        guess useful; an expert evicted before anyone asked for it was a wasted one."""
        gid = id(group)
        for idx, victim in zip(order, victims):
            if victim >= 0:
                self._speculative.discard((gid, victim))
            if real and (gid, idx) in self._speculative:
                self._speculative.discard((gid, idx))
                if victim < 0:
                    self.prefetch_useful += 1

    def prefetch(self, *uids: ExpertUID) -> int:
        """Start loading the given experts of one eviction group on a guess (the reference lists speculative loading
        as not yet available, README.md:24-26).  Nothing is handed out and hits / misses are not counted: the copies
        run on the side stream, a loaded guess becomes the group's most recently used expert, and whoever asks for it
        later finds it on the device.  Returns the number of copies started.

        Two rules keep a guess from costing a real request anything.  A guess is only acted on while the host link
        is idle (every copy given to the copy stream has finished; `prefetch_backlog` allows that many unfinished
        ones) and has mostly been idle at the recent calls (`prefetch_busy_limit`): on a saturated link an early copy
        only displaces a needed one and every wrong guess adds a slab to the queue.  And a guess does not evict an expert of the group's latest real request (the ones the current token
        may ask for again) unless guesses have proved the better bet: every guess is scored against the next real
        request of its group, every request against the one before it, and the latest request's experts are
        protected until at least eight of each have been scored and guessed experts are asked for more often than
        repeated ones.  Guesses that only protected experts could make room for are dropped.  Guessed experts that
        are resident already are left alone (no change of their place in the eviction order)."""
        assert not self.active, "already loading experts; buffers are busy"
        infos = [self.registered_experts[uid] for uid in dict.fromkeys(uids)]
        if not infos:
            return 0
        assert len(set(info.eviction_group for info in infos)) == 1, "experts must be in the same evicton group"
        group = self.group_infos[infos[0].eviction_group]
        group.last_guess = {info.index for info in infos}
        absent = sum(1 for info in infos if group.slot_of(info.index) < 0)
        if not absent:
            return 0
        backlog = self._link_backlog()
        self._busy_share = 0.9 * self._busy_share + 0.1 * (1.0 if backlog > 0 else 0.0)
        if backlog > self.prefetch_backlog or self._busy_share > self.prefetch_busy_limit:
            self.prefetch_skipped_busy += absent
            return 0
        guesses_win = (self.guess_scored >= 8 and self.reuse_scored >= 8 and
                       self.guess_right * self.reuse_scored > self.reuse_right * self.guess_scored)
        order, local_slots, victims = group.plan_guess([info.index for info in infos],
                                                       [] if guesses_win else sorted(group.last_request))
        self.prefetch_skipped_protected += absent - len(order)
        if not order:
            return 0
        self._settle_speculation(group, order, victims, real=False)
        started = 0
        for idx, local, victim in zip(order, local_slots, victims):
            if victim < 0:
                continue
            home = group.global_slot[local]
            if self.spare:
                dst = self.spare.popleft()
                self.spare.append(home)
                group.global_slot[local] = dst
            else:
                dst = home
            if self._used[dst]:
                self.copy_stream.wait_event(self.released[dst])
            self._copy_kind = "prefetch"
            try:
                self._copy_in(group.members[idx], dst)
            finally:
                self._copy_kind = "demand"
            self.bytes_copied += self.module_size
            self._copy_pending.add(dst)
            self._speculative.add((id(group), idx))
            started += 1
        self.prefetch_loads += started
        return started

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
                "misses": sum(g.misses for g in self.group_infos.values()), "bytes_copied": self.bytes_copied,
                "prefetch_loads": self.prefetch_loads, "prefetch_useful": self.prefetch_useful,
                "prefetch_skipped_busy": self.prefetch_skipped_busy,
                "prefetch_skipped_protected": self.prefetch_skipped_protected,
                "guess_scored": self.guess_scored, "guess_right": self.guess_right,
                "reuse_scored": self.reuse_scored, "reuse_right": self.reuse_right}
