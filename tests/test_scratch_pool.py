"""``ScratchPool`` (the per-(device, stream, thread) scratch that inference frames reuse) stays bounded: the pool of a thread
that has ended is dropped, and with a byte cap the least recently used pools go first.  Runs on CPU tensors: the pool's
bookkeeping does not depend on the device."""
import threading

import torch

from htgs_amd.torch_bindings.rasterization import ScratchPool

CPU = torch.device("cpu")


def setup_function(_):
    ScratchPool.clear()
    ScratchPool.max_bytes = None


def teardown_function(_):
    ScratchPool.clear()
    ScratchPool.max_bytes = None


def test_buffers_are_reused_and_only_grow():
    pool = ScratchPool.current(CPU)
    a = pool.get("x", 100, torch.int32, CPU)
    assert pool.get("x", 50, torch.int32, CPU) is a and ScratchPool.current(CPU) is pool
    b = pool.get("x", 200, torch.int32, CPU, headroom=0.125)
    assert b is not a and b.numel() == 225 and pool.nbytes() == 900


def test_pools_of_ended_threads_are_dropped():
    def frame():
        ScratchPool.current(CPU).get("x", 1 << 16, torch.float32, CPU)
    for _ in range(5):
        t = threading.Thread(target=frame)
        t.start()
        t.join()
    # the next look-up that creates a pool drops those of the threads that have ended
    ScratchPool.current(CPU).get("x", 16, torch.float32, CPU)
    assert len(ScratchPool._pools) == 1 and ScratchPool.total_bytes() == 64


def test_byte_cap_drops_the_least_recently_used_pools():
    ScratchPool.max_bytes = 3000
    ready, done = threading.Barrier(4), threading.Event()

    def frame():
        ScratchPool.current(CPU).get("x", 250, torch.float32, CPU)        # 1000 bytes each
        ready.wait()
        done.wait()                                                       # stay alive: only the cap can drop this pool
    threads = [threading.Thread(target=frame) for _ in range(3)]
    for t in threads:
        t.start()
    ready.wait()
    assert ScratchPool.total_bytes() == 3000
    mine = ScratchPool.current(CPU)
    mine.get("x", 500, torch.float32, CPU)                                # 2000 bytes more: 5000 held
    assert ScratchPool.current(CPU) is mine                               # the look-up enforces the cap, never on the pool asked for
    assert ScratchPool.total_bytes() <= 3000 and mine.nbytes() == 2000 and len(ScratchPool._pools) == 2
    done.set()
    for t in threads:
        t.join()
