"""Device memory behind the DeviceMemory interface (aion runtime/device_memory.zig:36-108): the context's pool.
A freed block serves the next request of its size class in stream order; nothing the pool does may change what a
buffer holds while it is live."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_freed_blocks_are_reused_by_size_class(gpu):
    gpu.trim()
    live0, cached0 = gpu.memory_stats()
    assert cached0 == 0
    a = gpu.alloc(1000)
    live1, _ = gpu.memory_stats()
    assert live1 - live0 == 1024                     # classes below 2 KiB are multiples of 256 bytes
    h = a.handle
    a.free()
    assert gpu.memory_stats() == (live0, 1024)
    b = gpu.alloc(900)                               # same class: the cached block comes back
    assert b.handle == h and gpu.memory_stats() == (live0 + 1024, 0)
    c = gpu.alloc(5000)                              # another class: a block of its own
    assert c.handle != h
    live2, _ = gpu.memory_stats()
    assert 5000 <= live2 - live0 - 1024 <= 5000 * 1.125 + 256
    b.free(); c.free()
    _, cached = gpu.memory_stats()
    assert cached == live2 - live0
    gpu.trim()
    assert gpu.memory_stats() == (live0, 0)


def test_reuse_is_ordered_behind_the_last_use(gpu):
    """A block is freed while work that reads it is still in the stream, and handed out again at once: the new owner's
    writes are enqueued behind that work, so the copy made from the old contents is intact."""
    n = 1 << 20
    src = np.arange(n, dtype=np.float32)
    a = gpu.upload(src)
    dst = gpu.alloc(n * 4)
    gpu._check(gpu._lib.aionhip_d2d(gpu._ctx, dst.handle, 0, a.handle, 0, n * 4))      # reads `a`, asynchronous
    h = a.handle
    a.free()
    b = gpu.alloc(n * 4)
    assert b.handle == h
    gpu._check(gpu._lib.aionhip_memset(gpu._ctx, b.handle, 0, 0, n * 4))                  # overwrites the block
    assert np.array_equal(dst.numpy(np.float32, (n,)), src)
    assert not gpu.download(b, np.float32, (n,)).any()
    b.free(); dst.free()


def test_large_blocks_alignment_and_foreign_handles(gpu):
    gpu.trim()
    live0, _ = gpu.memory_stats()
    big = gpu.alloc((64 << 20) + 4096)               # above the pool's block limit: released on free, not cached
    big.free()
    assert gpu.memory_stats() == (live0, 0)
    al = gpu.alloc(3000, alignment=4096)
    assert al.handle % 4096 == 0
    h = al.handle
    al.free()
    again = gpu.alloc(3000, alignment=4096)
    assert again.handle == h                         # the cached block meets the alignment: it is the one handed out
    again.free()
    with pytest.raises(Exception):
        gpu.alloc(100, alignment=48)                 # not a power of two
    gpu.trim()


def test_program_recorded_before_a_work_buffer_grows_is_refused(orc):
    """A recorded program's launches address the context's work buffers. A later eager step that needs a larger one
    replaces it; the old program must then be refused (nothing launched) instead of replaying on freed memory, and
    recording the steps again gives a program that runs."""
    from aion_amd import backend as be
    from aion_amd import hip
    g = be.HipBackend(0)                              # a context of its own: the scratch sizes are what is under test
    try:
        rng = np.random.default_rng(9)
        n, k = 256, 512
        wf = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
        blocks = be.quantize_blocks(be.Q4_0, wf, 0)
        w = g.upload_weight(be.Q4_0, be.KMAJOR_KN, n, k, blocks)
        a4 = rng.standard_normal((4, k)).astype(np.float32)
        a_buf, c_buf = g.upload(a4), g.zeros(4 * n * 4)
        g.step_matmul(w, a_buf, 4, c_buf)             # eager once: the prepared-activation scratch gets its size for 4 rows
        prog = g.record_program(lambda: g.step_matmul(w, a_buf, 4, c_buf))
        assert g.program_is_current(prog)
        g.program_execute(prog)
        want = orc.matmul_q_packed(be.Q4_0, a4, blocks, n, threads=4)
        assert np.abs(g.download(c_buf, np.float32, (4, n)) - want).max() <= 1e-5 * np.sqrt((want.astype(np.float64) ** 2).mean())
        big = g.upload(rng.standard_normal((64, k)).astype(np.float32))
        big_c = g.zeros(64 * n * 4)
        g.step_matmul(w, big, 64, big_c)              # 64 rows: the scratch is replaced by a larger one
        assert not g.program_is_current(prog)
        with pytest.raises(be.AionHipError) as e:
            g.program_execute(prog)
        assert e.value.status == hip.INVALID_ARGUMENT and "stale program" in str(e.value)
        g.program_destroy(prog)
        prog = g.record_program(lambda: g.step_matmul(w, a_buf, 4, c_buf))
        g._check(g._lib.aionhip_memset(g._ctx, c_buf.handle, 0, 0, 4 * n * 4))
        g.program_execute(prog)
        assert np.abs(g.download(c_buf, np.float32, (4, n)) - want).max() <= 1e-5 * np.sqrt((want.astype(np.float64) ** 2).mean())
        g.program_destroy(prog)
        for t in (a_buf, c_buf, big, big_c):
            t.free()
        w.free()
    finally:
        g.close()
