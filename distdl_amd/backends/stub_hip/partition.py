"""Single-process stand-ins for the reference's MPI partitions.

The reference describes teams of workers with MPI groups and communicators
(backends/common/partition.py:19-146, 976-1142).  On one GPU there is one
process, so a partition here is an explicit, ordered tuple of *world ranks*
plus the world rank this object speaks for.  All group algebra (inclusive
sub-partitions, unions, Cartesian topologies and sub-topologies, neighbours) is
then local arithmetic; anything that needs another worker's data goes through
the world's transport (``transport.py``), which is either an in-process
loopback between rank threads or a solo stub with seeded peers.

Only the attributes and factories the hot-path layers use are provided:
``active, rank, size, shape, index, dim, device`` and the ``create_*`` /
``neighbor_ranks`` / ``*_data`` methods.
"""

import numpy as np

from ...utilities.slicing import range_index

PROC_NULL = -1


class SimWorld:
    """A team of ``size`` simulated workers inside one process.

    ``world.partition(rank)`` is what ``MPIPartition(MPI.COMM_WORLD)`` is on
    that rank in the reference.
    """

    def __init__(self, size, device=None, transport=None):
        from .device import get_device
        from .transport import SoloTransport
        self.size = int(size)
        self.device = get_device() if device is None else device
        self.transport = SoloTransport(self) if transport is None else transport

    def partition(self, rank=0):
        return Partition(self, tuple(range(self.size)), int(rank))

    def run(self, fn, timeout=120.0):
        """Runs ``fn(P_world)`` once per rank, each in its own thread, with a
        loopback transport that really moves data between them.  Returns the
        list of results in rank order."""
        from .transport import LoopbackTransport
        return LoopbackTransport.run(self, fn, timeout=timeout)


class Partition:
    """Unstructured team of workers (reference: MPIPartition,
    backends/common/partition.py:19-146)."""

    def __init__(self, world=None, ranks=None, me=None, device=None):
        self._world = world
        self._ranks = None if ranks is None else tuple(int(r) for r in ranks)
        self._me = me
        self._seq = {}
        if world is not None and self._ranks is not None and me in self._ranks:
            self.active = True
            self.rank = self._ranks.index(me)
            self.size = len(self._ranks)
            self.index = self.rank
        else:
            self.active = False
            self.rank = PROC_NULL
            self.size = -1
            self.index = None
        self.shape = np.array([self.size], dtype=int)
        self.dim = 1
        if device is not None:
            self.device = device
        elif world is not None:
            self.device = world.device
        else:
            from .device import get_device
            self.device = get_device()

    # -- identity -----------------------------------------------------------

    def __eq__(self, other):
        """Same team, same order, seen from the same worker (reference :187-217);
        inactive partitions never compare equal."""
        if not isinstance(other, Partition) or not self.active or not other.active:
            return False
        return (self._world is other._world and self._ranks == other._ranks and
                self._me == other._me and self.device == other.device)

    def __ne__(self, other):
        return not self.__eq__(other)

    __hash__ = object.__hash__

    def __repr__(self):
        return f"{type(self).__name__}(active={self.active}, rank={self.rank}, shape={list(self.shape)})"

    def initialize_backend_comm(self):
        """Nothing to create: there is no communicator library behind the stub."""
        return None

    def deactivate(self):
        """Releases the team (reference :151-185).  Shapes of Cartesian
        partitions survive, as in the reference."""
        self.active = False
        self.rank = PROC_NULL
        self.size = -1
        self.shape = np.array([self.size], dtype=int)
        self.dim = 1
        self.index = self.rank
        self._ranks_released = self._ranks
        self._ranks = None

    # -- factories ----------------------------------------------------------

    def _group(self):
        return self._ranks if self._ranks is not None else ()

    def create_partition_inclusive(self, ranks):
        """New team from the listed ranks *of this partition*, in the listed
        order (reference :224-251)."""
        if self._ranks is None:
            return Partition(self._world, None, self._me, device=self.device)
        ranks = [int(r) for r in np.atleast_1d(np.asarray(ranks))]
        for r in ranks:
            if r < 0 or r >= len(self._ranks):
                raise ValueError(f"rank {r} is not in a partition of size {len(self._ranks)}")
        return Partition(self._world, tuple(self._ranks[r] for r in ranks), self._me, device=self.device)

    def create_partition_union(self, other, initialize_backend_comm=False):
        """This team followed by the members of ``other`` not already in it
        (reference :253-290)."""
        if self._world is not other._world and self._world is not None and other._world is not None:
            raise Exception("partitions of different worlds cannot be united")
        world = self._world if self._world is not None else other._world
        mine = self._group()
        ranks = tuple(mine) + tuple(r for r in other._group() if r not in mine)
        me = self._me if self._me is not None else other._me
        return Partition(world, ranks if ranks else None, me, device=self.device)

    def create_cartesian_topology_partition(self, shape, **options):
        """Same team with a row-major Cartesian layout (reference :292-329)."""
        shape = np.asarray(shape).astype(int)
        if self._ranks is not None and int(np.prod(shape)) != len(self._ranks):
            raise Exception(f"Cartesian shape {shape.tolist()} does not match a team of {len(self._ranks)}")
        return CartesianPartition(self._world, self._ranks, self._me, shape, device=self.device)

    def create_broadcast_partition_to(self, P_dest, transpose_src=False, transpose_dest=False,
                                      initialize_backend_comm=False):
        """``(P_send, P_recv)`` of a broadcast from this partition to ``P_dest``
        (reference :490-632).  The reference builds one communicator per source
        worker; here both partitions are the union of the two teams seen from
        this worker -- ``P_send`` active on the workers of the source, ``P_recv``
        on those of the destination -- and carry the route (the two Cartesian
        partitions and their transposes), from which the transport finds every
        worker's partner by the reference's broadcast rule."""
        return _route_partitions(Route("broadcast", self, P_dest, bool(transpose_src), bool(transpose_dest)))

    def create_reduction_partition_to(self, P_dest, transpose_src=False, transpose_dest=False,
                                      initialize_backend_comm=False):
        """``(P_send, P_recv)`` of a sum-reduction from this partition onto
        ``P_dest`` (reference :683-823): the broadcast rule read backwards, this
        partition being the larger one."""
        return _route_partitions(Route("reduction", self, P_dest, bool(transpose_src), bool(transpose_dest)))

    # -- small host data exchanges -------------------------------------------

    def _next_seq(self, kind):
        n = self._seq.get(kind, 0)
        self._seq[kind] = n + 1
        return n

    def broadcast_data(self, data, root=0, P_data=None):
        """Every active worker gets the ``data`` held by the workers of
        ``P_data`` (or by ``root``) (reference :825-902)."""
        if not self.active:
            return None
        return self._world.transport.broadcast_data(self, data, root, P_data)

    def allgather_data(self, data):
        """Stack of every worker's ``data`` in rank order (reference :904-930)."""
        if not self.active:
            return None
        return self._world.transport.allgather_data(self, data)

    def allreduce_data(self, data, op="sum"):
        """Element-wise reduction of every worker's array (reference :932-973)."""
        if not self.active:
            return None
        return self._world.transport.allreduce_data(self, data, op)


class CartesianPartition(Partition):
    """Team with a Cartesian topology, ranks in row-major order of the index
    (reference: MPICartesianPartition, backends/common/partition.py:976-1142)."""

    def __init__(self, world, ranks, me, shape, device=None):
        super().__init__(world, ranks, me, device=device)
        self.shape = np.asarray(shape).astype(int)
        self.dim = len(self.shape)
        self.index = self.cartesian_index(self.rank) if self.active else None

    def deactivate(self):
        shape = self.shape
        super().deactivate()
        self.shape = np.asarray(shape).astype(int)
        self.dim = len(self.shape)
        self.index = None

    def cartesian_index(self, rank):
        if not self.active:
            raise Exception("inactive partition has no Cartesian index")
        return np.asarray(np.unravel_index(int(rank), tuple(int(s) for s in self.shape)), dtype=int)

    def _rank_of(self, index):
        return int(np.ravel_multi_index(tuple(int(i) for i in index), tuple(int(s) for s in self.shape)))

    def neighbor_ranks(self, rank):
        """(left, right) neighbour ranks per dimension, PROC_NULL at the edges
        (reference :1110-1142)."""
        if not self.active:
            raise Exception("inactive partition has no neighbours")
        index = self.cartesian_index(rank)
        out = []
        for i in range(self.dim):
            left = right = PROC_NULL
            if index[i] - 1 >= 0:
                j = index.copy()
                j[i] -= 1
                left = self._rank_of(j)
            if index[i] + 1 < self.shape[i]:
                j = index.copy()
                j[i] += 1
                right = self._rank_of(j)
            out.append((left, right))
        return out

    def create_cartesian_subtopology_partition(self, remain_shape):
        """Sub-grid through this worker along the kept dimensions, like
        ``MPI_Cart_sub`` (reference :1056-1089)."""
        if not self.active:
            return Partition(self._world, None, self._me, device=self.device)
        keep = [bool(k) for k in remain_shape]
        sub_shape = [int(s) for s, k in zip(self.shape, keep) if k]
        ranks = []
        for sub_index in range_index(sub_shape):
            full = self.index.copy()
            it = iter(sub_index)
            for d in range(self.dim):
                if keep[d]:
                    full[d] = next(it)
            ranks.append(self._ranks[self._rank_of(full)])
        return CartesianPartition(self._world, tuple(ranks), self._me, sub_shape, device=self.device)

    def create_allreduction_partition(self, axes_reduce, initialize_backend_comm=False):
        """The workers that share this worker's index outside ``axes_reduce``,
        in row-major order of the reduced axes, with extent 1 in every other
        dimension (reference :634-681)."""
        if not self.active:
            return Partition(self._world, None, self._me, device=self.device)
        axes = [int(a) for a in axes_reduce]
        for a in axes:
            if a >= self.dim:
                raise ValueError(f"Dimension {a} in axes_reduce exceeds partition dimesion.")
        sub = self.create_cartesian_subtopology_partition([d in axes for d in range(self.dim)])
        shape = [int(self.shape[d]) if d in axes else 1 for d in range(self.dim)]
        return CartesianPartition(self._world, sub._ranks, self._me, shape, device=self.device)

    # Geometry of the team seen from any member; used by the solo transport to
    # answer for absent peers.
    def index_of_rank(self, rank):
        return np.asarray(np.unravel_index(int(rank), tuple(int(s) for s in self.shape)), dtype=int)


class Route:
    """What a pair of broadcast / reduction partitions stands for: data moves
    from ``P_src`` to ``P_dest`` (``kind`` "broadcast": copies from the smaller
    partition; "reduction": sums onto the smaller one), either partition
    transposed first."""

    __slots__ = ("kind", "P_src", "P_dest", "transpose_src", "transpose_dest")

    def __init__(self, kind, P_src, P_dest, transpose_src, transpose_dest):
        self.kind, self.P_src, self.P_dest = kind, P_src, P_dest
        self.transpose_src, self.transpose_dest = transpose_src, transpose_dest


def _route_partitions(route):
    P_src, P_dest = route.P_src, route.P_dest
    world = P_src._world if P_src._world is not None else P_dest._world
    me = P_src._me if P_src._me is not None else P_dest._me
    union = tuple(P_src._group()) + tuple(r for r in P_dest._group() if r not in P_src._group())
    P_send = Partition(world, union if P_src.active else None, me, device=P_src.device)
    P_recv = Partition(world, union if P_dest.active else None, me, device=P_dest.device)
    P_send._route = P_recv._route = route
    return P_send, P_recv
