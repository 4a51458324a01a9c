"""CPU emulation of libksq.so for the tests: the library's own kernel sources built for the host
(tests/emu/build_emu.py) and run one fiber per lane (tests/emu/emu_runtime.cpp).

``session()`` points ksanallm_amd.capi at the emulated library for the length of a ``with`` block, so the same
helpers that drive the GPU tests (tests/ksq_testlib.py) run on CPU tensors; every tensor handed to the C ABI is
announced to the emulator, which checks buffer-resource loads against it.  Only tests use this module.
"""
import contextlib
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# KSQ_EMU_ASAN=1 selects the AddressSanitizer build (tests/emu/build_emu.py --asan); the process then has to be started
# with the sanitizer's runtime preloaded (tests/test_emu_asan.py does that for a subprocess)
LIB_PATH = os.path.join(HERE, "libksq_emu_asan.so" if os.environ.get("KSQ_EMU_ASAN") == "1" else "libksq_emu.so")

_emu = None


def library():
    """The emulated library, built on first use if it is not there."""
    global _emu
    if _emu is None:
        if not os.path.exists(LIB_PATH):
            from tests.emu import build_emu

            build_emu.build()
        from ksanallm_amd import capi

        L = capi._bind(ctypes.CDLL(LIB_PATH))
        L.ksq_emu_register.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        L.ksq_emu_register.restype = None
        L.ksq_emu_unregister.argtypes = [ctypes.c_void_p]
        L.ksq_emu_unregister.restype = None
        L.ksq_emu_clear_registry.restype = None
        L.ksq_emu_set_block_sample.argtypes = [ctypes.c_int]
        L.ksq_emu_set_block_sample.restype = None
        L.ksq_emu_error_count.restype = ctypes.c_long
        L.ksq_emu_partial_rendezvous_count.restype = ctypes.c_long
        L.ksq_emu_error_string.argtypes = [ctypes.c_int]
        L.ksq_emu_error_string.restype = ctypes.c_char_p
        L.ksq_emu_clear_errors.restype = None
        _emu = L
    return _emu


def _nbytes(x):
    if hasattr(x, "data_ptr"):
        return x.numel() * x.element_size()
    if hasattr(x, "ctypes"):
        return x.nbytes
    return None


def errors():
    L = library()
    n = L.ksq_emu_error_count()
    return n, [L.ksq_emu_error_string(i).decode() for i in range(min(n, 64))]


def assert_clean(what=""):
    n, msgs = errors()
    library().ksq_emu_clear_errors()
    assert n == 0, f"{what}: {n} out-of-bounds accesses reported by the emulator, first: {msgs[:3]}"


@contextlib.contextmanager
def session(sample_blocks=0):
    """capi talks to the emulated library inside the block.  sample_blocks > 0 runs only that many positions of each
    grid (bounds checks on large shapes; outputs are then incomplete)."""
    from ksanallm_amd import capi

    L = library()
    saved_lib, saved_addr = capi._lib, capi._addr

    def addr(x):
        a = saved_addr(x)
        n = _nbytes(x)
        if a is not None and n:
            L.ksq_emu_register(a, n)
        return a

    capi._lib, capi._addr = L, addr
    L.ksq_emu_clear_errors()
    L.ksq_emu_set_block_sample(sample_blocks)
    try:
        yield L
    finally:
        capi._lib, capi._addr = saved_lib, saved_addr
        L.ksq_emu_set_block_sample(0)
        L.ksq_emu_clear_registry()
