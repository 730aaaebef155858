"""Stand-ins for the wire.  The hot path of this package is the *local* half of
every primitive (pack, unpack, shard compute); what the reference sends through
MPI or NCCL between those halves is supplied here by one of two transports:

``LoopbackTransport``
    every rank of a :class:`SimWorld` runs in its own thread of this process and
    messages are handed over through a mailbox, device buffer to device buffer.
    Semantics are those of the reference's exchange (post receives, pack, send,
    unpack), so whole layers can be checked against their sequential
    counterparts without MPI.

``SoloTransport``
    one live rank; peers are absent.  Receive buffers keep whatever the caller
    seeded them with, gathers return registered peer contributions (or mirror
    the live rank), and metadata assumes that every peer holds a shard shaped
    like the live rank's.  This is the configuration timed by the benchmark:
    exactly one rank's share of the work.
"""

import threading
import weakref

import numpy as np


class TransportError(RuntimeError):
    pass


def broadcast_partner(small_shape, small_index, big_shape, big_index, transpose_small=False, transpose_big=False):
    """Whether the worker at ``small_index`` of the smaller partition is the one
    the worker at ``big_index`` of the larger partition receives a broadcast
    from (sends its part of a sum to).  The rule of the reference
    (backends/common/partition.py:552-604, :745-794): either shape may be
    reversed first, the smaller one is then padded with ones on the left, a
    dimension takes part where the two extents agree, and must have extent 1 in
    the smaller partition where they do not."""
    small_shape = [int(n) for n in small_shape]
    small_index = [int(i) for i in small_index]
    big_shape = [int(n) for n in big_shape]
    big_index = [int(i) for i in big_index]
    if transpose_small:
        small_shape, small_index = small_shape[::-1], small_index[::-1]
    if transpose_big:
        big_shape, big_index = big_shape[::-1], big_index[::-1]
    pad = len(big_shape) - len(small_shape)
    if pad < 0:
        raise TransportError("broadcast: the source partition has more dimensions than the destination")
    small_shape, small_index = [1] * pad + small_shape, [0] * pad + small_index
    for d, (a, b) in enumerate(zip(small_shape, big_shape)):
        if a == b:
            if small_index[d] != big_index[d]:
                return False
        elif a != 1:
            raise TransportError(f"broadcast: extents {a} and {b} of dimension {d} neither agree nor is the smaller one 1")
    return True


# ---------------------------------------------------------------------------
# Solo
# ---------------------------------------------------------------------------

class SoloTransport:

    # Receive buffers are filled before a layer runs, so a layer may consume all
    # ghost slabs of all dimensions in one fused pass.
    ghosts_preloaded = True

    def __init__(self, world):
        self.world = world
        self._gather_providers = {}
        self._constant = set()       # tags whose provider stands for peers that contribute the same on every call
        self._seeded = {}            # tag -> weak reference to the buffer whose peer slots a constant provider has filled
        self._shape_provider = None

    # -- configuration by tests / benchmarks --------------------------------

    def set_gather_provider(self, tag, fn, constant=False):
        """``fn(P, tensor) -> list of P.size tensors`` supplies what the peers
        would contribute to a gather carrying ``tag`` (entry ``P.rank`` is
        replaced by the live tensor).  It is asked on every gather, unless
        ``constant`` says that the peers' parts do not depend on the call: an
        in-place gather then asks once per buffer and the parts stay in its
        slots (seeded peers, as a benchmark of one rank's share has them)."""
        self._gather_providers[tag] = fn
        self._constant.discard(tag)
        if constant:
            self._constant.add(tag)
        self._seeded.pop(tag, None)

    def _is_seeded(self, tag, buffer):
        ref = self._seeded.get(tag)
        return ref is not None and ref() is buffer

    def set_peer_shape_provider(self, fn):
        """``fn(P, index, my_shape) -> shape`` of the shard held by the peer at
        Cartesian ``index``; default: same as the live rank's."""
        self._shape_provider = fn

    # -- metadata -----------------------------------------------------------

    def subtensor_shapes(self, P, local_shape):
        from ...utilities.slicing import range_index
        table = np.zeros(list(P.shape) + [P.dim], dtype=int)
        mine = np.asarray(local_shape, dtype=int)
        for index in range_index(P.shape):
            if self._shape_provider is not None and tuple(index) != tuple(P.index):
                table[tuple(index)] = np.asarray(self._shape_provider(P, index, mine), dtype=int)
            else:
                table[tuple(index)] = mine
        return table

    def broadcast_data(self, P, data, root, P_data):
        if data is None:
            raise TransportError("solo transport: this rank does not hold the data being broadcast")
        return data

    def allgather_data(self, P, data):
        return np.stack([np.asarray(data)] * P.size)

    def allreduce_data(self, P, data, op):
        data = np.asarray(data)
        if op == "sum":
            return data * P.size
        return data

    # -- tensors ------------------------------------------------------------

    def exchange(self, P, sends, recvs):
        """Nothing leaves and nothing arrives: receive buffers hold what the
        caller seeded them with."""
        return None

    def allgather(self, P, tensor, tag=None):
        import torch
        fn = self._gather_providers.get(tag)
        if fn is None:
            parts = [tensor] * P.size
        else:
            parts = list(fn(P, tensor))
            if len(parts) != P.size:
                raise TransportError(f"gather provider for {tag!r} returned {len(parts)} parts for {P.size} workers")
            parts[P.rank] = tensor
        return torch.stack(parts)

    def allgather_into(self, P, buffer, tag=None):
        """In-place all-gather: ``buffer`` is ``[P.size, ...]`` and slot
        ``P.rank`` already holds this worker's part.  Without a provider the
        absent workers hold what the live one holds (as in :meth:`allgather`);
        a provider supplies their parts on every call, a constant one once per
        buffer object."""
        fn = self._gather_providers.get(tag)
        if fn is None:
            for p in range(P.size):
                if p != P.rank:
                    buffer[p].copy_(buffer[P.rank])
            return buffer
        if tag in self._constant and self._is_seeded(tag, buffer):
            return buffer
        parts = list(fn(P, buffer[P.rank]))
        if len(parts) != P.size:
            raise TransportError(f"gather provider for {tag!r} returned {len(parts)} parts for {P.size} workers")
        for p, part in enumerate(parts):
            if p != P.rank:
                buffer[p].copy_(part)
        if tag in self._constant:
            self._seeded[tag] = weakref.ref(buffer)
        return buffer

    def peers_gathered_ahead(self, P, buffer, tag=None):
        """True when the slots of ``buffer`` other than ``P.rank`` hold the
        peers' parts before the live rank's part exists -- a constant provider
        has filled them on an earlier call -- so that one kernel may produce the
        live part and consume the others."""
        return tag in self._constant and self._is_seeded(tag, buffer)

    def broadcast(self, P_src, P_dst, tensor, transpose_src=False, transpose_dst=False, tag=None):
        if P_src.active:
            return tensor
        raise TransportError("solo transport: the live rank is not a source of this broadcast")

    def broadcast_adjoint(self, P_src, P_dst, grad, transpose_src=False, transpose_dst=False, tag=None):
        """Sum-reduce from ``P_dst`` onto ``P_src``.  The live rank owns the
        data; the contributions of the absent workers are absent too."""
        return grad if P_src.active else None

    def gather_list(self, P, tensor, tag=None):
        """The tensors of all workers of ``P`` in rank order.  The absent
        workers hold what the live one holds unless a provider says otherwise."""
        fn = self._gather_providers.get(tag)
        if fn is None:
            return [tensor] * P.size
        parts = list(fn(P, tensor))
        if len(parts) != P.size:
            raise TransportError(f"gather provider for {tag!r} returned {len(parts)} parts for {P.size} workers")
        parts[P.rank] = tensor
        return parts

    def release(self, P, tag=None):
        return None


# ---------------------------------------------------------------------------
# Loopback
# ---------------------------------------------------------------------------

class _Mailbox:

    def __init__(self, timeout):
        self.cv = threading.Condition()
        self.slots = {}
        self.failed = None
        self.timeout = timeout

    def put(self, key, value, readers=1):
        with self.cv:
            if key in self.slots:
                raise TransportError(f"mailbox key {key!r} posted twice")
            self.slots[key] = [value, readers]
            self.cv.notify_all()

    def take(self, key):
        with self.cv:
            ok = self.cv.wait_for(lambda: key in self.slots or self.failed is not None, timeout=self.timeout)
            if self.failed is not None:
                raise TransportError(f"another rank failed: {self.failed!r}")
            if not ok:
                raise TransportError(f"timed out waiting for {key!r}")
            slot = self.slots[key]
            slot[1] -= 1
            if slot[1] == 0:
                del self.slots[key]
            return slot[0]

    def fail(self, exc):
        with self.cv:
            if self.failed is None:
                self.failed = exc
            self.cv.notify_all()


class LoopbackTransport:

    ghosts_preloaded = False

    def __init__(self, world, timeout=120.0):
        self.world = world
        self.mail = _Mailbox(timeout)
        self._seq = {}
        self._seq_lock = threading.Lock()

    @classmethod
    def run(cls, world, fn, timeout=120.0):
        transport = cls(world, timeout)
        previous = world.transport
        world.transport = transport
        results = [None] * world.size
        errors = [None] * world.size

        def body(rank):
            import torch
            try:
                # Backward passes of GPU tensors normally all run on the single
                # autograd thread of the device; a rank blocking there for a
                # message would stall every other rank.  With multithreading
                # off, each rank's backward runs on its own thread.
                with torch.autograd.set_multithreading_enabled(False):
                    results[rank] = fn(world.partition(rank))
            except BaseException as exc:  # noqa: B902 - re-raised below
                errors[rank] = exc
                transport.mail.fail(exc)

        threads = [threading.Thread(target=body, args=(r,), name=f"sim-rank-{r}") for r in range(world.size)]
        try:
            for t in threads:
                t.start()
            for t in threads:
                t.join()
        finally:
            world.transport = previous
        for rank, exc in enumerate(errors):
            if exc is not None and not isinstance(exc, TransportError):
                raise exc
        for exc in errors:
            if exc is not None:
                raise exc
        return results

    def _next(self, me, group, kind):
        key = (me, group, kind)
        with self._seq_lock:
            n = self._seq.get(key, 0)
            self._seq[key] = n + 1
        return n

    # -- collectives on host data ---------------------------------------------

    def _allgather_obj(self, P, obj, kind):
        group = P._ranks
        seq = self._next(P._me, group, kind)
        self.mail.put((kind, group, seq, P._me), obj, readers=len(group))
        return [self.mail.take((kind, group, seq, r)) for r in group]

    def subtensor_shapes(self, P, local_shape):
        shapes = self._allgather_obj(P, tuple(int(s) for s in local_shape), "shapes")
        table = np.zeros(list(P.shape) + [P.dim], dtype=int)
        for rank, shape in enumerate(shapes):
            table[tuple(P.index_of_rank(rank))] = np.asarray(shape, dtype=int)
        return table

    def broadcast_data(self, P, data, root, P_data):
        if P_data is not None:
            source = P_data._ranks[0] if P_data._ranks is not None else getattr(P_data, "_ranks_released", (None,))[0]
        else:
            source = P._ranks[root]
        everyone = self._allgather_obj(P, data, "bcast")
        return everyone[P._ranks.index(source)]

    def allgather_data(self, P, data):
        return np.stack([np.asarray(d) for d in self._allgather_obj(P, data, "gather")])

    def allreduce_data(self, P, data, op):
        parts = [np.asarray(d) for d in self._allgather_obj(P, data, "reduce")]
        if op == "sum":
            return np.sum(parts, axis=0)
        if op == "max":
            return np.max(parts, axis=0)
        if op == "min":
            return np.min(parts, axis=0)
        raise ValueError(f"unknown reduction {op!r}")

    # -- tensors ------------------------------------------------------------

    def exchange(self, P, sends, recvs):
        """``sends`` / ``recvs``: lists of ``(peer_rank_in_P, tensor, tag)``.
        All sends are posted, then receives are completed in list order (the
        copy is enqueued on the current stream, after the sender's pack), then
        the sender waits until every peer has taken its message so that the
        buffer may be reused."""
        group = P._ranks
        me = P._me
        acks = []
        for peer, tensor, tag in sends:
            dst = group[peer]
            seq = self._next(me, group, ("send", dst, tag))
            self.mail.put(("p2p", group, me, dst, tag, seq), tensor)
            acks.append(("ack", group, me, dst, tag, seq))
        for peer, tensor, tag in recvs:
            src = group[peer]
            seq = self._next(me, group, ("recv", src, tag))
            payload = self.mail.take(("p2p", group, src, me, tag, seq))
            if tuple(payload.shape) != tuple(tensor.shape) or payload.dtype != tensor.dtype:
                raise TransportError(f"message {tuple(payload.shape)}/{payload.dtype} does not fit receive buffer "
                                     f"{tuple(tensor.shape)}/{tensor.dtype}")
            tensor.copy_(payload)
            self.mail.put(("ack", group, src, me, tag, seq), True)
        for key in acks:
            self.mail.take(key)

    def allgather(self, P, tensor, tag=None):
        import torch
        parts = self._allgather_obj(P, tensor, ("tgather", tag))
        out = torch.stack(parts)
        # Nobody may overwrite its contribution before everyone has stacked it.
        self._allgather_obj(P, None, ("tgather-done", tag))
        return out

    def peers_gathered_ahead(self, P, buffer, tag=None):
        """Peers compute their parts while this worker computes its own: never
        ahead."""
        return False

    def allgather_into(self, P, buffer, tag=None):
        """In-place all-gather: ``buffer`` is ``[P.size, ...]`` and slot
        ``P.rank`` already holds this worker's part; the other slots are filled
        from the peers' buffers (copies enqueued on the shared stream)."""
        buffers = self._allgather_obj(P, buffer, ("tgather-into", tag))
        for p, theirs in enumerate(buffers):
            if p != P.rank:
                buffer[p].copy_(theirs[p])
        # Nobody may overwrite its own slot before everyone has copied it.
        self._allgather_obj(P, None, ("tgather-into-done", tag))
        return buffer

    def _shapes_of(self, union, P_src, P_dst, kind, tag):
        """The shapes of both partitions, known to every worker of the union
        (a worker outside a partition does not know that partition's shape)."""
        mine = (tuple(int(n) for n in P_src.shape) if P_src.active else None,
                tuple(int(n) for n in P_dst.shape) if P_dst.active else None)
        everyone = self._allgather_obj(union, mine, (kind, tag))
        src_shape = next(a for a, _ in everyone if a is not None)
        dst_shape = next(b for _, b in everyone if b is not None)
        return src_shape, dst_shape

    def broadcast(self, P_src, P_dst, tensor, transpose_src=False, transpose_dst=False, tag=None):
        """Every worker of ``P_dst`` receives the tensor held by the worker of
        ``P_src`` that shares its index in the dimensions ``P_src`` spans
        (weights stored on a sub-grid, used on the full grid); see
        :func:`broadcast_partner`."""
        union = P_src.create_partition_union(P_dst)
        key = ("tbcast", tag)
        src_shape, dst_shape = self._shapes_of(union, P_src, P_dst, "tbcast-shapes", tag)
        payload = (tuple(int(i) for i in P_src.index), tensor) if P_src.active else None
        everyone = self._allgather_obj(union, payload, key)
        out = tensor
        if P_dst.active:
            mine = [int(i) for i in P_dst.index]
            match = None
            for item in everyone:
                if item is None:
                    continue
                index, t = item
                if broadcast_partner(src_shape, index, dst_shape, mine, transpose_src, transpose_dst):
                    match = t
                    break
            if match is None:
                raise TransportError("broadcast: no source worker matches this destination index")
            out = tensor if match is tensor else match.clone()
        self._allgather_obj(union, None, ("tbcast-done", tag))
        return out

    def gather_list(self, P, tensor, tag=None):
        """The tensors of all workers of ``P`` in rank order (shapes may differ).
        They are the peers' own tensors: read them, then call :meth:`release`."""
        return self._allgather_obj(P, tensor, ("tlist", tag))

    def release(self, P, tag=None):
        """Every worker of ``P`` has enqueued its reads of the tensors handed
        out by :meth:`gather_list`; the rank threads share one stream, so the
        owners may reuse them from here on."""
        self._allgather_obj(P, None, ("tlist-done", tag))

    def broadcast_adjoint(self, P_src, P_dst, grad, transpose_src=False, transpose_dst=False, tag=None):
        """Sum-reduce: every worker of ``P_src`` receives the sum of the
        tensors held by the workers of ``P_dst`` it would broadcast to, added in
        rank order; the other workers receive None."""
        from ... import hip_ops
        union = P_src.create_partition_union(P_dst)
        src_shape, dst_shape = self._shapes_of(union, P_src, P_dst, "tbcast-adj-shapes", tag)
        payload = (tuple(int(i) for i in P_dst.index), grad) if P_dst.active else None
        everyone = self._allgather_obj(union, payload, ("tbcast-adj", tag))
        out = None
        if P_src.active:
            mine = [int(i) for i in P_src.index]
            # In the order of the workers' ranks in the world, whatever the order of the union.
            for _, item in sorted(zip(union._ranks, everyone), key=lambda pair: pair[0]):
                if item is None:
                    continue
                index, g = item
                if not broadcast_partner(src_shape, mine, dst_shape, index, transpose_src, transpose_dst):
                    continue
                if out is None:
                    out = g.clone()
                else:
                    full = [slice(0, int(n)) for n in g.shape]
                    hip_ops.copy_box(g, full, out, full, accumulate=True)
        # Nobody may reuse its gradient buffer before every source has summed it.
        self._allgather_obj(union, None, ("tbcast-adj-done", tag))
        return out
