"""Simulated-rank communicator group (include/flagcx_amd/fx_sim.h) for tests
and the benchmark.  Every rank posts the same collective; the last post runs it."""
import ctypes as C

from . import _native as N

lib = N.lib

ALGO, ORDER, NSLICES, NREDSLICES, REDSLICESIZE, SYNC, SCRATCH_BYTES, ARITH = 0, 1, 2, 3, 4, 5, 6, 7
ALGO_DIRECT, ALGO_RING = 0, 1
ORDER_RANK, ORDER_RING, ORDER_TREE, ORDER_HOST = 0, 1, 2, 3
SYNC_GROUP, SYNC_RENDEZVOUS = 0, 1
ARITH_DEFAULT, ARITH_ELEMENT = 0, 1


def _szs(v):
    return (C.c_size_t * max(len(v), 1))(*[int(x) for x in v])


class SimGroup:
    def __init__(self, nranks, **config):
        self.n = nranks
        self.comms = (C.c_void_p * nranks)()
        N.check(lib.fxSimCommInitAll(self.comms, nranks), "fxSimCommInitAll")
        self.configure(**config)

    def configure(self, algo=None, order=None, nslices=None, nredslices=None, redslicesize=None, sync=None,
                  scratch_bytes=None, arith=None):
        for key, val in ((ALGO, algo), (ORDER, order), (NSLICES, nslices), (NREDSLICES, nredslices),
                         (REDSLICESIZE, redslicesize), (SYNC, sync), (SCRATCH_BYTES, scratch_bytes), (ARITH, arith)):
            if val is not None:
                N.check(lib.fxSimCommConfig(self.comms[0], key, val), f"fxSimCommConfig({key})")

    def destroy(self):
        if self.comms is not None:
            lib.fxSimCommDestroyAll(self.comms, self.n)
            self.comms = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.destroy()

    # each method posts for every rank in turn and returns the LAST call's code
    def _each(self, fn, streams):
        rc = N.SUCCESS
        for r in range(self.n):
            s = streams[r] if isinstance(streams, (list, tuple)) else streams
            rc = fn(r, s)
            if rc != N.SUCCESS:
                return rc
        return rc

    def all_reduce(self, sends, recvs, count, dtype, op, streams):
        return self._each(lambda r, s: lib.flagcxAllReduce(sends[r], recvs[r], count, dtype, op, self.comms[r], s),
                          streams)

    def custom_all_reduce(self, sends, recvs, count, dtype, op, streams):
        return self._each(
            lambda r, s: lib.flagcxCustomAllReduceImpl(sends[r], recvs[r], count, dtype, op, self.comms[r], s), streams)

    def reduce(self, sends, recvs, count, dtype, op, root, streams):
        return self._each(
            lambda r, s: lib.flagcxReduce(sends[r], recvs[r], count, dtype, op, root, self.comms[r], s), streams)

    def reduce_scatter(self, sends, recvs, recvcount, dtype, op, streams):
        return self._each(
            lambda r, s: lib.flagcxReduceScatter(sends[r], recvs[r], recvcount, dtype, op, self.comms[r], s), streams)

    def all_gather(self, sends, recvs, sendcount, dtype, streams):
        return self._each(lambda r, s: lib.flagcxAllGather(sends[r], recvs[r], sendcount, dtype, self.comms[r], s),
                          streams)

    def all_to_allv(self, sends, sendcounts, sdispls, recvs, recvcounts, rdispls, dtype, streams):
        return self._each(
            lambda r, s: lib.flagcxAlltoAllv(sends[r], _szs(sendcounts[r]), _szs(sdispls[r]), recvs[r],
                                             _szs(recvcounts[r]), _szs(rdispls[r]), dtype, self.comms[r], s), streams)

    def progress(self, rank):
        """(launch count when `rank`'s latest collective call was accepted, launch count now)."""
        joined, launched = C.c_uint64(), C.c_uint64()
        N.check(lib.fxSimCommProgress(self.comms[rank], C.byref(joined), C.byref(launched)), "fxSimCommProgress")
        return joined.value, launched.value

    def register_windows(self, windows, nbytes):
        arr = (C.c_void_p * self.n)(*windows) if windows else None
        return lib.fxSimRegisterWindows(self.comms[0], arr, nbytes)


class HostStaged:
    """The reference's host-staged reducing collectives over n simulated ranks
    (include/flagcx_amd/fx_host_staged.h): D2H, the bootstrap ring on the host, H2D,
    with the reference's per-phase timers."""

    def __init__(self, nranks, device_memcpy=None):
        self.n = nranks
        self.h = C.c_void_p()
        fn = C.cast(device_memcpy, C.c_void_p) if device_memcpy is not None else None
        N.check(lib.fxHostStagedCreate(C.byref(self.h), nranks, fn), "fxHostStagedCreate")

    def _run(self, call):
        t = (C.c_uint64 * (self.n * len(N.TIMER_NAMES)))()
        rc = call(t)
        k = len(N.TIMER_NAMES)
        return rc, [dict(zip(N.TIMER_NAMES, t[r * k:(r + 1) * k])) for r in range(self.n)]

    def _ptrs(self, v):
        return (C.c_void_p * self.n)(*v)

    def all_reduce(self, sends, recvs, count, dtype, op):
        """Returns (result code, per-rank dicts of phase nanoseconds)."""
        return self._run(lambda t: lib.fxHostStagedAllReduce(self.h, self._ptrs(sends), self._ptrs(recvs), count,
                                                             dtype, op, t))

    def reduce(self, sends, recvs, count, dtype, op, root):
        """recvs[r] is used for r == root only."""
        return self._run(lambda t: lib.fxHostStagedReduce(self.h, self._ptrs(sends), self._ptrs(recvs), count,
                                                          dtype, op, root, t))

    def reduce_scatter(self, sends, recvs, recvcount, dtype, op):
        return self._run(lambda t: lib.fxHostStagedReduceScatter(self.h, self._ptrs(sends), self._ptrs(recvs),
                                                                 recvcount, dtype, op, t))

    def destroy(self):
        if self.h:
            lib.fxHostStagedDestroy(self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.destroy()
