"""Expert pool: keep N of E experts per layer resident in HBM and resolve the rest on demand.

Host-side mirror of the reference's pooled MoE path (paths relative to the reference's root):

  ExpertPool (LRU slot bookkeeping)                                 src/zero-tvm/expert-pool.ts:33-148
  SLAB_TENSORS, makeLayerPool, fillSlots, the device slot map       src/zero-tvm/engine-core.ts:1063-1257, :2455-2483, :2704-2725
  moe_slot_translate                                                src/compiler/shaders/moe_slot_translate.wgsl

The kernels do not change: the gathered GEMV reads its row base from ids[], so a buffer that holds SLOTS
experts with ids[] holding SLOT indices is the code path it already runs. The whole feature is buffer size
plus this bookkeeping. On a 288 GB part a pool is a choice rather than a need (a 35B-A3B checkpoint fits
many times over); it is here so that an engine written against the reference's pooled surface binds
unchanged, and so that several models can share one GPU's memory.
"""
from dataclasses import dataclass, field

import numpy as np

MISS = 0xFFFFFFFF


@dataclass
class PoolResolution:
    slots: np.ndarray            # int32, one slot per requested expert, in request order
    misses: list = field(default_factory=list)   # [(expert, slot)] the caller must upload before dispatching
    evicted: list = field(default_factory=list)  # expert ids dropped to make room


class ExpertPool:
    """LRU map of expert ids onto a fixed number of slots. Pure and synchronous: I/O and GPU work belong to
    the caller."""

    @staticmethod
    def min_slots(per_request, pinned=0):
        """Smallest pool that can serve a request of `per_request` distinct experts while `pinned` slots are
        held permanently: a pinned slot is not available to the request."""
        return per_request + pinned

    def __init__(self, slots, pin=()):
        if slots < 1:
            raise ValueError("expert pool needs at least one slot, got %d" % slots)
        self.slots = slots
        self._expert_of = [-1] * slots
        self._slot_of = {}
        self._used_at = [0] * slots
        self._clock = 0
        self._free = list(range(slots - 1, -1, -1))     # popped from the end: slot 0 is handed out first
        self._pinned = set()
        self.hits = 0
        self.requests = 0
        for e in pin:
            if not self._free:
                raise ValueError("cannot pin %d: pool of %d is full" % (e, slots))
            slot = self._free.pop()
            self._expert_of[slot] = e
            self._slot_of[e] = slot
            self._pinned.add(e)

    def slot_for(self, expert):
        return self._slot_of.get(expert, -1)

    def resolve(self, experts):
        """Map one request's expert choices onto slots, evicting as needed. Every requested expert is resident
        on return; duplicates inside a request share a slot and are loaded once; nothing this request touched
        (and nothing pinned) can be evicted by it."""
        experts = [int(e) for e in experts]
        out = np.empty(len(experts), np.int32)
        res = PoolResolution(out)
        held = set()
        for i, e in enumerate(experts):
            self.requests += 1
            slot = self._slot_of.get(e)
            if slot is not None:
                self.hits += 1
            else:
                slot = self._take(held, res.evicted)
                self._expert_of[slot] = e
                self._slot_of[e] = slot
                res.misses.append((e, slot))
            self._clock += 1
            self._used_at[slot] = self._clock
            held.add(e)
            out[i] = slot
        return res

    def _take(self, held, evicted):
        if self._free:
            return self._free.pop()
        victim, oldest = -1, None
        for s in range(self.slots):
            e = self._expert_of[s]
            if e < 0:
                return s
            if e in held or e in self._pinned:
                continue
            if oldest is None or self._used_at[s] < oldest:
                oldest, victim = self._used_at[s], s
        if victim < 0:
            raise RuntimeError("expert pool of %d slots (%d pinned) cannot serve this request — size it with "
                               "ExpertPool.min_slots(per_request, pinned)" % (self.slots, len(self._pinned)))
        evicted.append(self._expert_of[victim])
        del self._slot_of[self._expert_of[victim]]
        return victim

    @property
    def hit_rate(self):
        return self.hits / self.requests if self.requests else 0.0


def slab_tensors(d, ffn, bits=4):
    """The nine stacked tensors of a MoE layer and their bytes per expert (engine-core.ts:1168-1185):
    (field, proj, kind, stride)."""
    w_gu, s_gu = ffn * (d * bits // 32) * 4, ffn * (d // 64) * 2
    w_dn, s_dn = d * (ffn * bits // 32) * 4, d * (ffn // 64) * 2
    return (("gateWeights", "gate", "w", w_gu), ("gateScales", "gate", "s", s_gu), ("gateBiases", "gate", "b", s_gu),
            ("upWeights", "up", "w", w_gu), ("upScales", "up", "s", s_gu), ("upBiases", "up", "b", s_gu),
            ("downWeights", "down", "w", w_dn), ("downScales", "down", "s", s_dn), ("downBiases", "down", "b", s_dn))


class ArraySlabSource:
    """A slab source over host arrays {(layer, proj, kind): uint8 [experts, stride]}: slab_bytes() and read(),
    the two calls a pool makes on the reference's SlabSource (src/zero-tvm/slab-source.ts)."""

    def __init__(self, slabs):
        self._slabs = {k: np.ascontiguousarray(v).view(np.uint8).reshape(v.shape[0], -1) for k, v in slabs.items()}
        self.reads = 0

    def slab_bytes(self, layer, proj, kind):
        return self._slabs[(layer, proj, kind)].shape[1]

    def read(self, layer, proj, kind, expert):
        self.reads += 1
        return self._slabs[(layer, proj, kind)][expert]


class LayerPool:
    """One MoE layer's pool: the SLOTS-row buffers the MoE bind groups bind, and (optimistic recorder) the
    device-resident expert -> slot map the translate kernel reads (engine-core.ts:1187-1219)."""

    def __init__(self, device, layer, d, ffn, experts, pool_slots, source, shared_expert_index=-1, per_token_slots=None,
                 optimistic=False, bits=4):
        pinned = 1 if shared_expert_index >= 0 else 0
        if per_token_slots is not None and pool_slots < ExpertPool.min_slots(per_token_slots, pinned):
            raise ValueError("expertPool %d is below the pool's minimum %d (%d slots per token%s) — one token's experts "
                             "could not all be resident at once"
                             % (pool_slots, ExpertPool.min_slots(per_token_slots, pinned), per_token_slots,
                                " + 1 pinned shared expert" if pinned else ""))
        self.device, self.layer, self.source = device, layer, source
        self.expert_rows = experts + pinned
        self.slabs = []
        self.buffers = {}
        for fld, proj, kind, stride in slab_tensors(d, ffn, bits):
            declared = source.slab_bytes(layer, proj, kind)
            if declared != stride:
                raise ValueError("layer %d %s is %d B per expert by the spec and %d B in the checkpoint" % (layer, fld, stride, declared))
            if stride % 4:
                raise ValueError("%s stride %d is not a multiple of 4" % (fld, stride))
            buf = device.create_buffer(pool_slots * stride, "%s.slots" % fld)
            self.slabs.append((buf, stride, proj, kind))
            self.buffers[fld] = buf
        pin = [shared_expert_index] if pinned else []
        self.pool = ExpertPool(pool_slots, pin)
        self.map_buf = self.cpu_map = None
        if optimistic:
            self.cpu_map = np.full(self.expert_rows, MISS, np.uint32)
            for e in pin:
                self.cpu_map[e] = self.pool.slot_for(e)
            self.map_buf = device.create_buffer(self.expert_rows * 4, "moeSlotMap_%d" % layer)
            device.write_buffer(self.map_buf, 0, self.cpu_map)
        # the pinned shared expert is uploaded once, up front
        self.fill_slots([(e, self.pool.slot_for(e)) for e in pin])

    def fill_slots(self, misses):
        """Fill the missed slots from the slab source: every slab of every miss (engine-core.ts:1248-1257)."""
        for expert, slot in misses:
            for buf, stride, proj, kind in self.slabs:
                self.device.write_buffer(buf, slot * stride, self.source.read(self.layer, proj, kind, expert))

    def resolve(self, expert_ids):
        """Serial pooled path: expert ids (read back from the router) -> slot ids, misses uploaded on return.
        Returns the uint32 slot ids to write into the ids buffer the matmuls bind."""
        r = self.pool.resolve(expert_ids)
        self.fill_slots(r.misses)
        if self.cpu_map is not None:
            for e in r.evicted:
                self.cpu_map[e] = MISS
            for e, slot in r.misses:
                self.cpu_map[e] = slot
            if r.misses or r.evicted:
                self.device.write_buffer(self.map_buf, 0, self.cpu_map)
        return r.slots.astype(np.uint32), r

    def missed(self, expert_ids):
        """Optimistic recorder: was the device map wrong for this token AS OF SUBMIT, i.e. before resolve()
        mutates it (engine-core.ts:2467-2471)? Then the token replays from this layer."""
        return any(self.cpu_map[int(e)] == MISS for e in expert_ids)

    def translate(self, ids_out, ids_in, n):
        """Optimistic recorder: rewrite expert ids into slot ids on the device through the resident map; a miss
        becomes slot 0 and the token replays once the readback names it."""
        self.device.ctx.moe_slot_translate(ids_out.addr, ids_in.addr, self.map_buf.addr, n, self.expert_rows)

    def destroy(self):
        for buf, *_ in self.slabs:
            buf.destroy()
        if self.map_buf is not None:
            self.map_buf.destroy()
