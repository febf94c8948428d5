"""The HAL executable plugin, driven the way IREE's plugin manager drives one
(runtime/src/iree/hal/local/executable_plugin_manager.c and
plugins/system_library_plugin.c of the reference): dlopen, query, load with a
host allocator, resolve import names, call the imports with a pointer to the
parameter struct, unload. The CPU tests cover the protocol; the GPU test calls
the three imports on host buffers and checks them against the oracle."""
import ctypes as C
import os

import numpy as np
import pytest

import ukref
from iree_amd import _lib
from iree_amd import flags as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "iree_amd", "plugin", "libmi355x_uk_plugin.so")


class Header(C.Structure):
    _fields_ = [("version", C.c_uint32), ("name", C.c_char_p), ("description", C.c_char_p),
                ("features", C.c_uint32), ("sanitizer", C.c_int32), ("reserved", C.c_uint64 * 8)]


CTL = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.POINTER(C.c_void_p))


class Allocator(C.Structure):
    _fields_ = [("self", C.c_void_p), ("ctl", CTL)]


class Environment(C.Structure):
    _fields_ = [("host_allocator", Allocator)]


class StringView(C.Structure):
    _fields_ = [("data", C.c_char_p), ("size", C.c_size_t)]


class StringPair(C.Structure):
    _fields_ = [("key", StringView), ("value", StringView)]


class ResolveParams(C.Structure):
    _fields_ = [("count", C.c_size_t), ("symbol_names", C.POINTER(C.c_char_p)),
                ("out_fn_ptrs", C.POINTER(C.c_void_p)), ("out_fn_contexts", C.POINTER(C.c_void_p))]


LOAD = C.CFUNCTYPE(C.c_void_p, C.POINTER(Environment), C.c_size_t, C.POINTER(StringPair),
                   C.POINTER(C.c_void_p))
UNLOAD = C.CFUNCTYPE(None, C.c_void_p)
RESOLVE = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.POINTER(ResolveParams), C.POINTER(C.c_uint32))
IMPORT = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_void_p)


class PluginV0(C.Structure):
    _fields_ = [("header", C.POINTER(Header)), ("load", LOAD), ("unload", UNLOAD), ("resolve", RESOLVE)]


class Host:
    """A minimal plugin host: counts allocations so leaks show."""

    def __init__(self):
        self.libc = C.CDLL(None)
        self.libc.malloc.restype = C.c_void_p
        self.libc.malloc.argtypes = [C.c_size_t]
        self.libc.free.argtypes = [C.c_void_p]
        self.live = 0

        def ctl(_self, command, params, inout_ptr):
            if command in (0, 1):      # malloc / calloc
                n = C.cast(params, C.POINTER(C.c_size_t))[0]
                p = self.libc.malloc(n)
                if command == 1:
                    C.memset(p, 0, n)
                inout_ptr[0] = p
                self.live += 1
                return 0
            if command == 3:           # free
                self.libc.free(inout_ptr[0])
                self.live -= 1
                return 0
            return 12                  # realloc: unimplemented in this host
        self.ctl = CTL(ctl)
        self.lib = C.CDLL(PLUGIN)
        self.lib.iree_hal_executable_plugin_query.restype = C.POINTER(PluginV0)
        self.lib.iree_hal_executable_plugin_query.argtypes = [C.c_uint32, C.c_void_p]

    def query(self, max_version=1):
        return self.lib.iree_hal_executable_plugin_query(max_version, None)

    def load(self, plugin, params=()):
        env = Environment(Allocator(None, self.ctl))
        pairs = (StringPair * max(1, len(params)))()
        for i, (k, v) in enumerate(params):
            pairs[i] = StringPair(StringView(k, len(k)), StringView(v, len(v)))
        out_self = C.c_void_p()
        status = plugin.load(C.byref(env), len(params), pairs, C.byref(out_self))
        return status or 0, out_self

    def resolve(self, plugin, self_ptr, names):
        n = len(names)
        arr = (C.c_char_p * n)(*names)
        fns = (C.c_void_p * n)()
        ctxs = (C.c_void_p * n)()
        res = C.c_uint32(0xFFFFFFFF)
        rp = ResolveParams(n, arr, fns, ctxs)
        status = plugin.resolve(self_ptr, C.byref(rp), C.byref(res))
        return status or 0, res.value, list(fns), list(ctxs)


@pytest.fixture(scope="module")
def host():
    if not os.path.exists(PLUGIN):
        pytest.fail(f"{PLUGIN} is not built (run __graft_entry__.build())")
    return Host()


def test_query_reports_version_and_refuses_newer_hosts(host):
    p = host.query(1)
    assert p and p.contents.header.contents.version == 1
    assert p.contents.header.contents.name == b"mi355x_uk"
    assert p.contents.header.contents.features == 0        # a system plugin, not standalone
    assert p.contents.header.contents.sanitizer == 0
    assert not host.query(2)                                 # host asks for a newer interface


@pytest.mark.parametrize("flags,kind", [([], 0), (["-fsanitize=address"], 1), (["-fsanitize=thread"], 3)])
def test_header_names_the_sanitizer_it_was_compiled_with(flags, kind):
    """The header's sanitizer field is whatever the compiler says is in force
    for the plugin's translation unit (the reference runtime refuses a plugin
    built with a sanitizer it does not run itself,
    runtime/src/iree/hal/local/executable_plugin.h:76-121): the macro the
    plugin initialises the field with, expanded by the preprocessor under each
    sanitizer switch."""
    import shutil
    import subprocess
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    src = '#include "iree_amd_hal_plugin_abi.h"\nKIND_IS IREE_AMD_HAL_PLUGIN_SANITIZER_KIND\n'
    compilers = [c for c in ("gcc", "/opt/rocm/llvm/bin/clang") if shutil.which(c)]
    assert compilers
    for cc in compilers:
        out = subprocess.run([cc, "-E", "-P", "-x", "c", "-I", include, *flags, "-"], input=src, text=True,
                             capture_output=True, check=True).stdout
        line = [l for l in out.splitlines() if l.startswith("KIND_IS")][0]
        assert line.split()[1] == str(kind), (cc, flags, line)
    with open(os.path.join(os.path.dirname(PLUGIN), "mi355x_uk_plugin.c")) as f:
        assert ".sanitizer = IREE_AMD_HAL_PLUGIN_SANITIZER_KIND" in f.read()


def test_load_resolve_unload_protocol(host):
    plugin = host.query().contents
    status, self_ptr = host.load(plugin, [(b"uk_library", _lib.library_path().encode())])
    assert status == 0 and self_ptr.value
    assert host.live == 1
    names = [b"iree_uk_mmt4d", b"iree_uk_pack", b"iree_uk_unpack", b"mi355x_uk_mmt4d",
             b"?mi355x_uk_pack", b"?not_there"]
    status, resolution, fns, ctxs = host.resolve(plugin, self_ptr, names)
    assert status == 0
    assert resolution == 1                                   # one optional import missing
    assert all(fns[:5]) and fns[5] is None
    assert all(c == self_ptr.value for c in ctxs[:5])
    assert fns[0] != fns[3]                                  # two parameter layouts, see the GPU test
    # a required unknown import: NOT_FOUND, the known ones still resolved
    status, resolution, fns, _ = host.resolve(plugin, self_ptr, [b"iree_uk_mmt4d", b"other_symbol"])
    assert status == 5 and fns[0] and fns[1] is None
    plugin.unload(self_ptr)
    assert host.live == 0


def test_load_fails_cleanly_without_the_library(host):
    plugin = host.query().contents
    status, self_ptr = host.load(plugin, [(b"uk_library", b"/nonexistent/libiree_amd_uk.so")])
    assert status == 14 and not self_ptr.value               # UNAVAILABLE
    assert host.live == 0


@pytest.mark.gpu
def test_imports_run_pack_mmt4d_unpack_on_host_buffers(host, uk, cuda):
    """linalg.matmul i8 x i8 -> i32 as the compiler would emit it with data
    tiling: two packs, mmt4d, unpack, every call through a plugin import with
    the reference's parameter structs on HOST memory. Bit-exact."""
    plugin = host.query().contents
    status, self_ptr = host.load(plugin, [(b"uk_library", _lib.library_path().encode())])
    assert status == 0
    status, _, fns, ctxs = host.resolve(plugin, self_ptr,
                                        [b"mi355x_uk_pack", b"iree_uk_mmt4d", b"mi355x_uk_unpack"])
    assert status == 0
    pack_fn, mmt4d_r_fn, unpack_fn = (IMPORT(f) for f in fns)

    class Mmt4dWithResult(C.Structure):      # the llvm-cpu lowering's form: i32 result first
        _fields_ = [("result", C.c_int32), ("params", _lib.Mmt4dParams)]
    assert Mmt4dWithResult.params.offset == 8

    def mmt4d_fn(addr, ctx, reserved):
        w = Mmt4dWithResult(-1, C.cast(addr, C.POINTER(_lib.Mmt4dParams)).contents)
        rc = mmt4d_r_fn(C.addressof(w), ctx, reserved)
        assert w.result == 0
        return rc
    M, N, K = 100, 70, 150
    M0, N0, K0 = 32, 32, 16
    M1, N1, K1 = -(-M // M0), -(-N // N0), -(-K // K0)
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    b = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    lhs = np.full(M1 * K1 * M0 * K0, 0x55, np.int8)
    rhs = np.full(N1 * K1 * N0 * K0, 0x55, np.int8)
    acc = np.full(M1 * N1 * M0 * N0, -1, np.int32)
    c = np.full((M, N), -7, np.int32)
    ptr = lambda x: x.ctypes.data_as(C.c_void_p)  # noqa: E731
    p = _lib.PackParams(ptr(a), 0, K, 1, ptr(lhs), 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0,
                        0, F.PACK_TYPE_I8I8, None)
    assert pack_fn(C.addressof(p), ctxs[0], None) == 0
    p = _lib.PackParams(ptr(b), 0, N, 1, ptr(rhs), 0, K1 * N0 * K0, N0 * K0, K, N, N1, K1, N0, K0,
                        0, F.PACK_TYPE_I8I8 | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER, None)
    assert pack_fn(C.addressof(p), ctxs[0], None) == 0
    m = _lib.Mmt4dParams(ptr(lhs), 0, K1 * M0 * K0, ptr(rhs), 0, K1 * N0 * K0, ptr(acc), 0,
                         N1 * M0 * N0, M1, N1, K1, M0, N0, K0,
                         F.MMT4D_TYPE_S8S8S32 | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION, None)
    assert mmt4d_fn(C.addressof(m), ctxs[1], None) == 0
    u = _lib.UnpackParams(ptr(acc), 0, N1 * M0 * N0, M0 * N0, ptr(c), 0, N, 1, M1, N1, M0, N0, M, N,
                          F.UNPACK_TYPE_I32I32, None)
    assert unpack_fn(C.addressof(u), ctxs[2], None) == 0
    want = np.zeros((M, N), np.int32)
    assert ukref.oracle().oracle_matmul_rowmajor(ukref.ptr(a), ukref.ptr(b), ukref.ptr(want),
                                                 M, N, K, F.MMT4D_TYPE_S8S8S32) == 0
    assert np.array_equal(c, want)
    # an invalid call surfaces as a non-zero import result, not a crash
    m.flags = 0x0C
    assert mmt4d_fn(C.addressof(m), ctxs[1], None) != 0
    plugin.unload(self_ptr)
    assert host.live == 0


@pytest.mark.gpu
def test_plain_c_host_program_drives_the_plugin(cuda):
    """plugin_host_check.c: the same protocol from a C program with no Python or
    torch in the process (dlopen, query, load, resolve, three imports, unload)."""
    import subprocess
    exe = os.path.join(ROOT, "iree_amd", "plugin", "plugin_host_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} is not built (run __graft_entry__.build())")
    r = subprocess.run([exe, PLUGIN, _lib.library_path()], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "OK:" in r.stdout


@pytest.mark.gpu
def test_imports_called_from_many_host_threads_at_once(host, uk, cuda):
    """The contract of an import: "called from arbitrary threads concurrently"
    (samples/custom_dispatch/cpu/plugin/system_plugin.c:21-25 of the reference).
    12 host threads (more than the pool has slots, so some calls wait for one)
    each run pack, pack, mmt4d, unpack on buffers of their own, several times,
    with shapes that make the pool's buffers grow; every result is the exact
    integer product."""
    import threading
    plugin = host.query().contents
    status, self_ptr = host.load(plugin, [(b"uk_library", _lib.library_path().encode())])
    assert status == 0
    status, _, fns, ctxs = host.resolve(plugin, self_ptr,
                                        [b"mi355x_uk_pack", b"mi355x_uk_mmt4d", b"mi355x_uk_unpack"])
    assert status == 0
    pack_fn, mmt4d_fn, unpack_fn = (IMPORT(f) for f in fns)
    ptr = lambda x: x.ctypes.data_as(C.c_void_p)  # noqa: E731
    M0, N0, K0 = 32, 32, 16
    errors = []

    def worker(t):
        try:
            rng = np.random.default_rng(100 + t)
            for rep in range(3):
                M, N, K = 40 + 37 * t + 5 * rep, 200 - 11 * t + rep, 64 + 48 * ((t + rep) % 5)
                M1, N1, K1 = -(-M // M0), -(-N // N0), -(-K // K0)
                a = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
                b = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
                lhs = np.full(M1 * K1 * M0 * K0, 0x55, np.int8)
                rhs = np.full(N1 * K1 * N0 * K0, 0x55, np.int8)
                acc = np.full(M1 * N1 * M0 * N0, -1, np.int32)
                c = np.full((M, N), -7, np.int32)
                p = _lib.PackParams(ptr(a), 0, K, 1, ptr(lhs), 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0,
                                    0, F.PACK_TYPE_I8I8, None)
                assert pack_fn(C.addressof(p), ctxs[0], None) == 0
                p = _lib.PackParams(ptr(b), 0, N, 1, ptr(rhs), 0, K1 * N0 * K0, N0 * K0, K, N, N1, K1, N0, K0,
                                    0, F.PACK_TYPE_I8I8 | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER, None)
                assert pack_fn(C.addressof(p), ctxs[0], None) == 0
                m = _lib.Mmt4dParams(ptr(lhs), 0, K1 * M0 * K0, ptr(rhs), 0, K1 * N0 * K0, ptr(acc), 0,
                                     N1 * M0 * N0, M1, N1, K1, M0, N0, K0, F.MMT4D_TYPE_S8S8S32, None)
                assert mmt4d_fn(C.addressof(m), ctxs[1], None) == 0
                u = _lib.UnpackParams(ptr(acc), 0, N1 * M0 * N0, M0 * N0, ptr(c), 0, N, 1, M1, N1, M0, N0,
                                      M, N, F.UNPACK_TYPE_I32I32, None)
                assert unpack_fn(C.addressof(u), ctxs[2], None) == 0
                want = a.astype(np.int32) @ b.astype(np.int32)
                assert np.array_equal(c, want), (t, rep, M, N, K)
        except BaseException as e:  # noqa: BLE001
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(12)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=300)
    assert not any(th.is_alive() for th in threads), "a worker thread did not finish"
    assert not errors, errors
    plugin.unload(self_ptr)
    assert host.live == 0
