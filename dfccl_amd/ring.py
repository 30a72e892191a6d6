"""Drives n virtual ranks of one GPU from one host thread: the pattern the tests
and the benchmark use (each rank context is what one process of the reference's
caller would own)."""
import threading
import time

import torch

from . import api

KINDS = ("all_reduce", "reduce_scatter", "all_gather", "reduce", "broadcast")


class VirtualRing:
    def __init__(self, nranks):
        self.n = nranks
        self.ctxs = [api.RankCtx(r) for r in range(nranks)]
        self.comms = {}   # coll_id -> [VirtualComm per rank]
        self.kinds = {}
        self.done = {}    # (rank, coll_id) -> threading.Event
        self.t_submit = {}
        self.t_done = {}
        self.finalized = False

    # -- registration -----------------------------------------------------------
    def prepare(self, coll_id, kind, count, dtype, op=api.ncclSum, root=0, premul=None, premul_device=None):
        """premul: the bytes of one element, or a list with one such scalar per rank; every rank then makes a
        PreMulSum operator with its scalar on its communicator handle and registers the collective with it (op is
        ignored).  premul_device: a list with one device address per rank instead (ncclScalarDevice)."""
        comms = api.VirtualComm.create_all(self.n)
        for r, ctx in enumerate(self.ctxs):
            if premul_device is not None:
                op = comms[r].create_premul_sum(dtype, device_ptr=premul_device[r])
            elif premul is not None:
                op = comms[r].create_premul_sum(dtype, premul[r] if isinstance(premul, (list, tuple)) else premul)
            if kind == "all_reduce":
                ctx.prepare_all_reduce(count, dtype, op, comms[r], coll_id)
            elif kind == "reduce_scatter":
                ctx.prepare_reduce_scatter(count, dtype, op, comms[r], coll_id)
            elif kind == "all_gather":
                ctx.prepare_all_gather(count, dtype, comms[r], coll_id)
            elif kind == "reduce":
                ctx.prepare_reduce(count, dtype, op, root, comms[r], coll_id)
            elif kind == "broadcast":
                ctx.prepare_broadcast(count, dtype, root, comms[r], coll_id)
            else:
                raise ValueError(kind)
            self.done[(r, coll_id)] = threading.Event()
        self.comms[coll_id] = comms
        self.kinds[coll_id] = kind

    def finalize(self):
        for ctx in self.ctxs:
            ctx.finalize()
        self.finalized = True

    # -- submission -------------------------------------------------------------
    def submit(self, rank, coll_id, send, recv):
        ev = self.done[(rank, coll_id)]
        ev.clear()
        key = (rank, coll_id)

        def cb(_cid, key=key, ev=ev):
            self.t_done[key] = time.perf_counter()
            ev.set()

        ctx = self.ctxs[rank]
        run = getattr(ctx, "run_" + self.kinds[coll_id])
        run(send, recv, coll_id, cb)
        self.t_submit[key] = time.perf_counter()

    def run(self, coll_id, sends, recvs, timeout=60.0):
        """Submit coll_id on every rank (rank order) and wait for all callbacks."""
        for r in range(self.n):
            self.submit(r, coll_id, sends[r], recvs[r])
        self.wait([(r, coll_id) for r in range(self.n)], timeout)

    def wait(self, keys, timeout=60.0):
        deadline = time.monotonic() + timeout
        for key in keys:
            left = deadline - time.monotonic()
            if left <= 0 or not self.done[key].wait(left):
                missing = [k for k in keys if not self.done[k].is_set()]
                try:
                    stats = self.stats()
                    self.ctxs[0].dump_state()
                except Exception as e:  # the counters are a diagnosis aid only
                    stats = repr(e)
                raise TimeoutError(f"collective {key[1]} on rank {key[0]} did not complete within {timeout}s; "
                                   f"(rank, collective) still waited for: {missing}; daemon counters: {stats}")

    def stats(self):
        total = {}
        for ctx in self.ctxs:
            for k, v in ctx.stats().items():
                total[k] = max(total.get(k, 0), v) if k == "daemonLaunches" else total.get(k, 0) + v
        return total

    def destroy(self):
        for ctx in self.ctxs:
            ctx.destroy()
        for comms in self.comms.values():
            for c in comms:
                c.destroy()
        self.comms.clear()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()
        return False


def sync_inputs():
    """Make earlier torch work on the current stream visible before a submission.
    (Never torch.cuda.synchronize(): that would wait for the resident daemon.)"""
    torch.cuda.current_stream().synchronize()
