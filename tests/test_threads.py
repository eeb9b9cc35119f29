"""Entry points called from several host threads: the library serialises them with one lock.  Without a GPU this
exercises the compile-only mode (descriptor validation, kernel cache, error text per thread)."""
import ctypes
import threading

from jittor_amd import _lib as L


def test_entry_points_from_several_threads():
    lib = L.init(-1)
    P = 0x100000
    errors = []

    def worker(i):
        try:
            for j in range(20):
                x = L.tensor(P, "float32", [64 + i, 128]); y = L.tensor(P, "float32", [64 + i])
                rc = lib.mjt_reduce(ctypes.byref(x), ctypes.byref(y), L.OP_CODE["add"], 2)
                assert rc == 0, lib.mjt_last_error()
                bad = L.tensor(P, "float32", [3])                      # wrong result shape: an error, with this thread's text
                rc = lib.mjt_reduce(ctypes.byref(x), ctypes.byref(bad), L.OP_CODE["add"], 2)
                assert rc < 0 and (b"x[%d,128" % (64 + i)) in lib.mjt_last_error()   # this thread's own message
        except Exception as e:                                          # noqa: BLE001 - reported below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
