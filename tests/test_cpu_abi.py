"""Host-side checks that need no GPU: the shared libraries load, export every
symbol the headers declare, the plugin passes the reference loader's validation,
and the host arithmetic (partition, trigger layout, synthetic data) agrees with
the oracle."""
import ctypes as C
import glob
import itertools
import os
import re

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import adaptor
from flagcx_amd import kernels as K
from oracle import fx_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "flagcx_amd", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        text = text.split("struct flagcxDeviceAdaptor_v1")[0]          # function POINTERS are not exports
        for m in re.finditer(r"^(?!typedef)[A-Za-z_][\w \*]*?\b(\w+)\s*\([^;{]*\)\s*;", text, flags=re.M):
            names.add(m.group(1))
    return names


# Declared with C++ linkage, as the reference declares it (flagcx_kernel_internal.h:56): exported under its mangled name.
CXX_LINKAGE = {"flagcxLaunchCollectiveKernel": "_Z28flagcxLaunchCollectiveKernelPvmmP12flagcxStream"}


def test_kernel_library_exports_every_declared_symbol():
    declared = _declared_functions()
    assert {"fx_reduce_copy", "fx_reduce_slices", "fx_pack", "flagcxAllReduce", "flagcxCustomAllReduceImpl",
            "fx_synth_fill", "fx_part_ring_ar", "fx_reduce_ordered", "flagcxLaunchCollectiveKernel"} <= declared
    missing = [n for n in sorted(declared) if not hasattr(N.lib, CXX_LINKAGE.get(n, n))]
    assert not missing, f"declared in include/ but not exported: {missing}"
    assert set(N.exported_symbols()) <= declared          # the binding uses nothing undeclared


def test_kernels_only_library_exports_fx_and_nothing_flagcx():
    """The library a FlagCX build links into libflagcx.so must not bring a second
    flagcxAllReduce: it exports every fx_* function of the kernel header and of
    the partition API, the reference-named consumer launcher, and no other
    dynamic symbol."""
    import subprocess
    path = os.path.join(N.LIB_DIR, "libflagcx-kernels-mi355x.so")
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    launcher = CXX_LINKAGE["flagcxLaunchCollectiveKernel"]   # the one symbol FlagCX's scheduler calls by name
    assert launcher in exported
    assert all(s.startswith("fx_") for s in exported - {launcher}), sorted(exported)[:10]
    wanted = {n for n in _declared_functions() if n.startswith("fx_") and n != "fx_synth_fill"}
    assert wanted <= exported, sorted(wanted - exported)
    lib = C.CDLL(path)
    lib.fx_version.restype = C.c_char_p
    assert lib.fx_version().startswith(b"flagcx_amd")


def test_plugin_passes_the_reference_loader_checks():
    t = adaptor.load_plugin()
    assert t.name == b"MI355X"
    # name[32] + 48 pointers (flagcx_device_adaptor.h:30-116)
    assert C.sizeof(adaptor.DeviceAdaptorV1) == 32 + 48 * C.sizeof(C.c_void_p)
    assert len(adaptor.REQUIRED) == 32
    for f in adaptor.REQUIRED:
        assert getattr(t, f), f
    # the hot path additionally needs these two (uni_runner_impl.cc:1815; core/group.cc:451-453)
    assert t.hostGetDevicePointer and t.launchDeviceFunc
    assert t.getDeviceProperties and t.getDevicePciBusId and t.getDeviceByPciBusId and t.dmaSupport
    # only the plugin symbol is exported
    out = os.popen(f"nm -D --defined-only {N.PLUGIN_LIB}").read()
    syms = [l.split()[-1] for l in out.splitlines() if " D " in l or " T " in l]
    assert syms == ["flagcxDeviceAdaptorPlugin_v1"]


def test_ccl_plugin_passes_the_reference_loader_checks():
    from flagcx_amd import ccl_adaptor
    t = ccl_adaptor.load_plugin()
    assert t.name == b"MI355X-SIM"
    # name pointer + 34 function pointers (flagcx_ccl_adaptor.h:42-122), all required (ccl_plugin_load.cc:64-81)
    assert C.sizeof(ccl_adaptor.CCLAdaptorV1) == 35 * C.sizeof(C.c_void_p)
    assert len(ccl_adaptor._FIELDS) == 34
    out = os.popen(f"nm -D --defined-only {ccl_adaptor.CCL_PLUGIN_LIB}").read()
    syms = [l.split()[-1] for l in out.splitlines() if " D " in l or " T " in l or " B " in l]
    assert syms == ["flagcxCCLAdaptorPlugin_v1"]          # nothing that could clash with libflagcx.so
    v = C.c_int()
    assert t.getVersion(C.byref(v)) == N.SUCCESS and t.getVersion(None) == N.INVALID_ARGUMENT
    assert t.getErrorString(9) == b"not supported"
    assert t.commCount(None, C.byref(v)) == N.INVALID_ARGUMENT
    assert t.commDestroy(None) == N.INVALID_ARGUMENT
    assert t.allReduce(0x1000, 0x1000, 4, N.DT_FP32, N.OP_SUM, None, None) == N.INVALID_ARGUMENT
    with pytest.raises(ImportError):
        ccl_adaptor.load_plugin(N.KERNEL_LIB)


def test_loader_rejects_bad_plugins(tmp_path):
    with pytest.raises(ImportError):
        adaptor.load_plugin(str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):                       # a library without the versioned symbol
        adaptor.load_plugin(N.KERNEL_LIB)


def test_host_argument_guards_of_the_plugin():
    t = adaptor.load_plugin()
    assert t.getDevice(None) == N.INVALID_ARGUMENT
    assert t.getDeviceCount(None) == N.INVALID_ARGUMENT
    assert t.getVendor(None) == N.INVALID_ARGUMENT
    v = C.create_string_buffer(128)
    assert t.getVendor(v) == N.SUCCESS and v.value == b"AMD"
    assert t.hostGetDevicePointer(None, None) == N.INVALID_ARGUMENT
    assert t.eventElapsedTime(None, None, None) == N.INVALID_ARGUMENT
    assert t.ipcMemHandleGet(None, None) == N.INVALID_ARGUMENT
    assert t.ipcMemHandleClose(None) == N.INVALID_ARGUMENT
    assert t.getDevicePciBusId(None, 16, 0) == N.INVALID_ARGUMENT
    assert t.getDeviceProperties(None, 0) == N.INVALID_ARGUMENT
    assert t.getDeviceByPciBusId(None, None) == N.INVALID_ARGUMENT
    assert t.streamFree(None) == N.SUCCESS and t.streamDestroy(None) == N.SUCCESS
    assert t.eventDestroy(None) == N.SUCCESS
    h, sz = C.c_void_p(), C.c_size_t()
    assert t.ipcMemHandleCreate(C.byref(h), C.byref(sz)) == N.SUCCESS and h.value and sz.value == 64
    assert t.ipcMemHandleFree(h) == N.SUCCESS
    dma = C.c_bool(True)
    assert t.dmaSupport(C.byref(dma)) == N.SUCCESS and dma.value is False


def test_dtype_sizes():
    # flagcx/flagcx.cc:35-66
    want = {0: 1, 1: 1, 2: 4, 3: 4, 4: 8, 5: 8, 6: 2, 7: 4, 8: 8, 9: 2, 10: 0, -1: 0}
    for dt, sz in want.items():
        assert N.lib.fx_dtype_size(dt) == sz
        if sz and dt in (2, 6, 7, 9):
            assert O.lib.oracle_dtype_size(dt) == sz


def test_split_and_nredslices_match_oracle():
    for total, parts in itertools.product([0, 1, 5, 63, 64, 65, 1000003, 33554432, 2**33 + 7], [1, 2, 3, 7, 8, 64]):
        for idx in {0, 1, parts // 2, parts - 1}:
            if idx < parts:
                assert K.split(total, parts, idx) == O.split(total, parts, idx)
    for count, n, S, R, sz in itertools.product([0, 1, 5, 524288, 524289, 33554432, 10**9], [1, 2, 8], [1, 3, 8],
                                                [0, 4], [0, 1, 65536, 262144]):
        assert N.lib.fx_nredslices(count, n, S, R, sz) == O.lib.oracle_nredslices(count, n, S, R, sz)


def _nodes(fn, *args):
    n = fn(*args, None)
    arr = (N.RedNode * max(n, 1))()
    assert fn(*args, arr) == n
    return [arr[i] for i in range(n)]


def _same(a, b):
    f = ["step", "rank", "in1_buf", "in2_buf", "out_buf", "slice", "in1_off", "in2_off", "out_off", "count"]
    return all(getattr(a, x) == getattr(b, x) for x in f)


@pytest.mark.parametrize("count,n,S,R", [(33554432, 8, 8, 2), (1000003, 8, 3, 2), (17, 4, 2, 3), (5, 8, 1, 1),
                                          (64, 2, 1, 1), (12345, 3, 4, 5), (0, 4, 2, 2)])
def test_partition_plans_match_oracle(count, n, S, R):
    for rank in range(n):
        a, b = _nodes(N.lib.fx_part_ring_ar, count, n, rank, S, R), O.plan_ring_ar(count, n, rank, S, R)
        assert len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
        a, b = _nodes(N.lib.fx_part_ring_rs, count, n, rank, S, R), O.plan_ring_rs(count, n, rank, S, R)
        assert len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
        a, b = _nodes(N.lib.fx_part_locred, count, n, rank, S), O.plan_locred(count, n, rank, S)
        assert len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
    assert N.lib.fx_part_ring_ar(count, 1, 0, S, R, None) == 0


def test_trigger_set_get_round_trip_and_oracle_layout():
    rng = np.random.default_rng(2)
    for _ in range(200):
        in1, in2, out = (int(x) for x in rng.integers(0, 2**63, 3))
        count, nth = int(rng.integers(0, 2**32)), int(rng.integers(0, 2**16))
        dt, op, st = int(rng.integers(0, 16)), int(rng.integers(0, 16)), int(rng.integers(0, 4))
        t = K.make_trigger(in1, in2, out, count, nth, dt, op, st)
        assert list(t.value) == O.trigger_encode(in1, in2, out, count, nth, dt, op, st)
        assert K.trigger_fields(t) == dict(in1=in1, in2=in2, out=out, count=count, nthreads=nth, dtype=dt, op=op,
                                           state=st)
    assert C.sizeof(N.ReduceTrigger) == 32 and C.sizeof(N.SliceDesc) == 80


def test_synth_is_deterministic_and_thread_independent():
    for dtype, dist, a, b in ((N.DT_FP32, K.SYNTH_UNIFORM, -1, 1), (N.DT_BF16, K.SYNTH_NORMAL, 0, 1),
                              (N.DT_FP16, K.SYNTH_NORMAL, 0, 1), (N.DT_INT32, K.SYNTH_UNIFORM_INT, -2**20, 2**20)):
        x1 = K.synth(100001, dtype, dist, a, b, seed=5, stream=2, threads=1)
        x8 = K.synth(100001, dtype, dist, a, b, seed=5, stream=2, threads=8)
        assert np.array_equal(x1, x8)
        assert np.array_equal(x1[:777], K.synth(777, dtype, dist, a, b, seed=5, stream=2))   # prefix property
        assert not np.array_equal(x1, K.synth(100001, dtype, dist, a, b, seed=5, stream=3))
        assert not np.array_equal(x1, K.synth(100001, dtype, dist, a, b, seed=6, stream=2))
    u = K.synth(400000, N.DT_FP32, K.SYNTH_UNIFORM, -1, 1, seed=0)
    assert -1 <= u.min() and u.max() < 1 and abs(u.mean()) < 0.01 and abs(u.std() - 3 ** -0.5) < 0.01
    g = K.synth(400000, N.DT_FP64, K.SYNTH_NORMAL, 0, 0.02, seed=4)
    assert abs(g.mean()) < 2e-4 and abs(g.std() - 0.02) < 2e-4
    i = K.synth(400000, N.DT_INT32, K.SYNTH_UNIFORM_INT, -2**20, 2**20, seed=2)
    assert i.min() >= -2**20 and i.max() <= 2**20 and i.min() < -2**20 + 100 and i.max() > 2**20 - 100
    # 16-bit outputs are correctly rounded versions of the same fp32 stream
    f = K.synth(50000, N.DT_FP32, K.SYNTH_NORMAL, 0, 1, seed=1)
    h = K.synth(50000, N.DT_FP16, K.SYNTH_NORMAL, 0, 1, seed=1)
    bf = K.synth(50000, N.DT_BF16, K.SYNTH_NORMAL, 0, 1, seed=1)
    assert np.array_equal(h, f.astype(np.float16).view(np.uint16))
    assert np.array_equal(bf, np.array([O.lib.oracle_f32_to_bf16(float(x)) for x in f], np.uint16))


def test_argument_screening_needs_no_gpu():
    """Rejections happen before any device call, so they are testable here."""
    p = 0x1000
    rc = lambda **kw: K.reduce_copy(kw.get("out", p), kw.get("ins", [p, p]), kw.get("n", 4), kw.get("dtype", N.DT_FP32),
                                    kw.get("op", N.OP_SUM), kw.get("first", 0))
    assert rc(op=N.OP_AVG, out=None) == N.INVALID_ARGUMENT           # every FlagCX type and op is carried; what is left
    assert rc(dtype=N.DT_FP64, op=5) == N.INVALID_ARGUMENT             # to reject lies outside the enums
    assert rc(dtype=N.DT_INT64, out=p + 4) == N.INVALID_ARGUMENT      # 8-byte elements need 8-byte alignment
    assert rc(dtype=10) == N.INVALID_ARGUMENT and rc(dtype=-1) == N.INVALID_ARGUMENT
    assert rc(op=5) == N.INVALID_ARGUMENT
    assert rc(first=2) == N.INVALID_ARGUMENT and rc(first=-1) == N.INVALID_ARGUMENT
    assert rc(out=None) == N.INVALID_ARGUMENT
    assert rc(out=p + 1) == N.INVALID_ARGUMENT
    assert rc(dtype=N.DT_BF16, ins=[p, p + 1]) == N.INVALID_ARGUMENT
    assert rc(ins=[p] * 65) == N.INVALID_ARGUMENT
    assert rc(n=0, out=None, ins=[None]) == N.SUCCESS
    assert K.reduce_slices([], 2, N.DT_FP32, N.OP_SUM) == N.SUCCESS
    assert K.reduce_slices([([p, p], p, 4)], 9, N.DT_FP32, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.reduce_slices([([p, None], p, 4)], 2, N.DT_FP32, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.copy_slices([(None, p, 4)]) == N.INVALID_ARGUMENT
    assert K.copy_slices([(None, None, 0)]) == N.SUCCESS
    assert K.pack(p, p, [1], [0], 10) == N.INVALID_ARGUMENT
    assert K.pack(None, None, [0, 0], [0, 0], N.DT_FP32) == N.SUCCESS
    assert N.lib.fxSimCommInitAll(None, 2) == N.INVALID_ARGUMENT
    comms = (C.c_void_p * 2)()
    assert N.lib.fxSimCommInitAll(comms, 0) == N.INVALID_ARGUMENT
    assert N.lib.flagcxAllReduce(p, p, 4, N.DT_FP64, 5, None, None) == N.INVALID_ARGUMENT
    assert N.lib.flagcxAllReduce(p, p, 4, N.DT_FP32, N.OP_SUM, None, None) == N.INVALID_ARGUMENT


def test_reduce_fifo_host_protocol():
    """enqueue / full ring / slot-not-collected behaviour of the host side
    (flagcx_reduce_kernel_host.cc:55-70), with no consumer running."""
    nbytes = N.lib.fx_fifo_bytes(2)
    buf = (C.c_uint64 * (nbytes // 8))()
    N.check(N.lib.fx_fifo_init(buf, 2))
    idx = C.c_int()
    for want in (0, 1):
        N.check(N.lib.fx_fifo_enqueue(buf, 1, 2, 3, 4, 32, N.DT_FP32, N.OP_SUM, C.byref(idx)))
        assert idx.value == want and N.lib.fx_fifo_poll_state(buf, want) == 1
    N.check(N.lib.fx_fifo_enqueue(buf, 1, 2, 3, 4, 32, N.DT_FP32, N.OP_SUM, C.byref(idx)))
    assert idx.value == -1                                           # full: produced - consumed >= capacity
    buf[1] = 1                                                       # the consumer took one ...
    N.check(N.lib.fx_fifo_enqueue(buf, 1, 2, 3, 4, 32, N.DT_FP32, N.OP_SUM, C.byref(idx)))
    assert idx.value == -1                                           # ... but slot 0 is not Available yet
    N.check(N.lib.fx_fifo_set_state(buf, 0, 3))
    N.check(N.lib.fx_fifo_set_state(buf, 0, 0))
    N.check(N.lib.fx_fifo_enqueue(buf, 9, 8, 7, 6, 32, N.DT_BF16, N.OP_MAX, C.byref(idx)))
    assert idx.value == 0 and buf[2] == 3 and buf[4] == 9 and buf[6] == 7
    assert (buf[7] >> 48) & 0xf == N.DT_BF16 and (buf[7] >> 52) & 0xf == N.OP_MAX and buf[7] & 0xffffffff == 6
    assert N.lib.fx_fifo_init(buf, 0) == N.INVALID_ARGUMENT and N.lib.fx_fifo_init(buf, 2000) == N.INVALID_ARGUMENT
    assert N.lib.fx_fifo_poll_state(buf, 5) == -1


def test_reduce_fifo_producer_loop_against_a_host_side_consumer():
    """fx_fifo_run_batch (the scheduler's enqueue-and-collect loop) with a Python
    thread playing the consumer on the same ring: 200 triggers through 8 slots are
    all delivered once, in order, with the fields they were given; with nobody
    consuming, the loop gives up after its spin limit."""
    import threading
    cap, total = 8, 200
    buf = (C.c_uint64 * (N.lib.fx_fifo_bytes(cap) // 8))()
    N.check(N.lib.fx_fifo_init(buf, cap))
    trig = (N.ReduceTrigger * total)()
    for i in range(total):
        N.lib.fx_trigger_set(C.byref(trig[i]), 1000 + i, 2000 + i, 3000 + i, i, 32, i % 10, i % 5, 1)
    seen, stop = [], threading.Event()

    def consumer():                                   # the protocol of flagcx_reduce_kernel_device.cu:53-186, in Python
        taken = 0
        while not stop.is_set() and taken < total:
            if buf[2] > taken:                        # produced
                w = 4 + 4 * (taken % cap)
                seen.append((buf[w], buf[w + 1], buf[w + 2], buf[w + 3] & 0xffffffff, (buf[w + 3] >> 48) & 0xf,
                             (buf[w + 3] >> 52) & 0xf))
                taken += 1
                buf[1] = taken                        # consumed
                buf[w + 3] |= 3 << 56                 # Complete
    t = threading.Thread(target=consumer)
    t.start()
    try:
        assert N.lib.fx_fifo_run_batch(buf, trig, total, 2_000_000_000) == N.SUCCESS
    finally:
        stop.set()
        t.join(timeout=30)
    assert seen == [(1000 + i, 2000 + i, 3000 + i, i, i % 10, i % 5) for i in range(total)]
    assert buf[2] == total and all((buf[4 + 4 * s + 3] >> 56) & 3 == 0 for s in range(cap))     # every slot handed back
    assert N.lib.fx_fifo_run_batch(buf, trig, 1, 1000) == N.INTERNAL_ERROR                       # nobody consumes
    assert N.lib.fx_fifo_run_batch(buf, None, 1, 1000) == N.INVALID_ARGUMENT
    assert N.lib.fx_fifo_run_batch(buf, trig, 0, 1000) == N.SUCCESS


def test_scheduler_stand_in_takes_one_symbol_from_the_kernel_library(tmp_path):
    """tests/unirunner_client.cc declares flagcxLaunchCollectiveKernel exactly as
    the reference's header does and carries its own host side of the ring, as
    libflagcx.so does: linked against libflagcx-kernels-mi355x.so alone it must
    leave no symbol undefined, and the launcher must be the only symbol it takes
    from that library.  (The GPU tests run the copy of it that the build made.)"""
    import shutil
    import subprocess
    if not shutil.which("g++"):
        pytest.skip("no g++")
    exe = tmp_path / "unirunner_client"
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-Werror", f"-I{ROOT}/include",
                    f"{ROOT}/tests/unirunner_client.cc", "-o", str(exe), f"-L{N.LIB_DIR}", "-lflagcx-kernels-mi355x",
                    "-ldl", "-Wl,--no-undefined", f"-Wl,-rpath,{N.LIB_DIR}", "-Wl,-rpath-link,/opt/rocm/lib"], check=True)
    out = subprocess.run(["nm", "-D", "--undefined-only", str(exe)], check=True, capture_output=True, text=True).stdout
    undefined = {line.split()[-1].split("@")[0] for line in out.splitlines() if line.strip()}
    ours = {u for u in undefined if u.startswith("fx_") or "flagcx" in u}
    assert ours == {CXX_LINKAGE["flagcxLaunchCollectiveKernel"]}, sorted(ours)
    src = open(f"{ROOT}/tests/unirunner_client.cc").read()
    ref = "/root/reference/flagcx/include/flagcx_kernel_internal.h"
    if os.path.exists(ref):          # the prototype is the reference's, token for token
        want = re.search(r"void flagcxLaunchCollectiveKernel\([^;]*;", open(ref).read(), flags=re.S).group(0)
        assert " ".join(want.split()) in " ".join(src.split())
    built = os.path.join(N.LIB_DIR, "unirunner_client")
    assert os.path.exists(built), "the build did not leave flagcx_amd/lib/unirunner_client for the GPU tests"


def test_reference_named_launcher_refuses_a_missing_ring_without_touching_the_device(capfd):
    """flagcxLaunchCollectiveKernel has no result to return (the reference's signature is void): a call it cannot
    serve says so on stderr and enqueues nothing.  No GPU needed for the first check it makes."""
    lib = C.CDLL(os.path.join(N.LIB_DIR, "libflagcx-kernels-mi355x.so"))
    fn = getattr(lib, CXX_LINKAGE["flagcxLaunchCollectiveKernel"])
    fn.restype, fn.argtypes = None, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
    fn(None, 32, 1, None)
    assert "flagcxLaunchCollectiveKernel: no ring" in capfd.readouterr().err


def test_headers_are_plain_c_and_a_c_client_links(tmp_path):
    """The boundary is a C ABI: every header compiles as strict C11, a C program
    links against the kernel library and the host-only entry points answer."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "client.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "flagcx_amd/fx_types.h"
#include "flagcx_amd/fx_kernels.h"
#include "flagcx_amd/fx_sim.h"
#include "flagcx_amd/fx_synth.h"
#include "flagcx_amd/fx_device_adaptor.h"
#include "flagcx_amd/fx_ccl_adaptor.h"
#include "flagcx_amd/fx_host_staged.h"
#include "flagcx_amd/fx_handle.h"
_Static_assert(sizeof(struct flagcxDeviceHandle) == 28 * sizeof(void *), "device handle: 28 operations (flagcx.h:143-185)");
_Static_assert(sizeof(fxReduceTrigger) == 32, "trigger is 32 bytes");
_Static_assert(sizeof(struct flagcxDeviceAdaptor_v1) == 32 + 48 * sizeof(void *), "v1 device adaptor layout");
_Static_assert(sizeof(struct flagcxCCLAdaptor_v1) == 35 * sizeof(void *), "v1 ccl adaptor layout");
_Static_assert(sizeof(flagcxUniqueId) == 256, "unique id");
int main(void) {
  size_t cnt, off;
  fxReduceTrigger t;
  int dt, op, st, version;
  uint64_t c;
  flagcxUniqueId a, b;
  fx_split(10, 3, 0, &cnt, &off);
  if (cnt != 4 || off != 0) return 1;
  fx_trigger_set(&t, 1, 2, 3, 77, 32, flagcxBfloat16, flagcxMax, fxTriggerEnqueued);
  fx_trigger_get(&t, NULL, NULL, NULL, &c, NULL, &dt, &op, &st);
  if (c != 77 || dt != flagcxBfloat16 || op != flagcxMax || st != fxTriggerEnqueued) return 2;
  if (fx_dtype_size(flagcxFloat64) != 8 || fx_dtype_size(99) != 0) return 3;
  if (fx_reduce_copy(NULL, NULL, 2, 4, flagcxFloat32, flagcxNumRedOps, 0, NULL) != flagcxInvalidArgument) return 4;
  if (strcmp(flagcxGetErrorString(flagcxInvalidArgument), "invalid argument")) return 5;
  if (flagcxGetVersion(&version) != flagcxSuccess || version != FX_SIM_VERSION) return 6;
  if (flagcxGetUniqueId(&a) != flagcxSuccess || flagcxGetUniqueId(&b) != flagcxSuccess) return 7;
  if (!memcmp(&a, &b, sizeof(a))) return 8;
  /* housekeeping calls that need no GPU: argument screening and the fixed answers */
  {
    void *p = NULL, *h = NULL;
    flagcxWindow_t w;
    if (flagcxMemAlloc(NULL, 16, flagcxMemCCL) != flagcxInvalidArgument) return 9;
    if (flagcxMemAlloc(&p, 0, flagcxMemCCL) != flagcxInvalidArgument) return 10;
    if (flagcxMemAlloc(&p, 16, flagcxMemSHMEM) != flagcxInternalError) return 11;
    if (flagcxMemFree(NULL, flagcxMemCCL) != flagcxSuccess) return 12;
    if (flagcxCommRegister(NULL, NULL, 16, &h, flagcxMemCCL) != flagcxInvalidArgument) return 13;
    if (flagcxCommRegister(NULL, &a, 16, &h, flagcxMemCCL) != flagcxSuccess || h != (void *)&a) return 14;
    if (flagcxCommDeregister(NULL, NULL, flagcxMemCCL) != flagcxSuccess) return 15;
    if (flagcxCommWindowRegister(NULL, &a, 16, &w, FLAGCX_WIN_COLL_SYMMETRIC, flagcxMemCCL) != flagcxNotSupported) return 16;
    if (flagcxCommSuspend(NULL) != flagcxInvalidArgument || flagcxCommFinalize(NULL) != flagcxInvalidArgument) return 17;
    if (strcmp(flagcxGetLastError(NULL), "Undefined: flagcxComm is not fully initialized.")) return 18;
    if (flagcxDeviceHandleInit(NULL) != flagcxInvalidArgument || flagcxHandleFree(NULL) != flagcxSuccess) return 19;
  }
  printf("%s\n", fx_version());
  return 0;
}
''')
    exe = tmp_path / "client"
    libdir = os.path.join(root, "flagcx_amd", "lib")
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{root}/include", str(src), "-o",
                    str(exe), f"-L{libdir}", "-lflagcx_amd", "-lflagcx-kernels-mi355x", f"-Wl,-rpath,{libdir}",
                    "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "flagcx_amd" in out


def test_kernel_index_arithmetic_on_the_host(tmp_path):
    """tests/host_tiling_check.hip drives fx::planTiles and fx::laneOfTile -- the
    functions the kernels themselves call -- over 14,168 (address, length, element
    size, unroll, hand-out, die shift) cases and checks that every vector of a segment
    is handled exactly once, the unchecked path only ever sees whole in-segment
    vectors, and nothing outside the segment is touched; then the host's decisions
    around them: which segments are striped, and which batches of copies count as
    reading their sources more than once (fx::rereadHint)."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = tmp_path / "host_tiling_check"
    subprocess.run([hipcc, "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-O2",
                    "-std=c++17", f"-I{root}/include",
                    f"-I{root}/flagcx_amd/csrc", f"{root}/tests/host_tiling_check.hip", "-o", str(exe)], check=True,
                   capture_output=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.startswith("ok"), out.stdout


def test_fifo_share_arithmetic_on_the_host(tmp_path):
    """tests/host_fifo_check.cc drives fx::fifoGridFor and fx::shareFor -- the very
    functions the FIFO consumer uses to size its grid and to decide which
    workgroups take which tiles of a trigger -- on the CPU: the grid never exceeds
    what the device holds at once, every taker index has exactly one workgroup,
    workgroup 0 computes only when it is alone."""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = tmp_path / "host_fifo_check"
    subprocess.run([gxx, "-O1", "-std=c++17", f"-I{root}/flagcx_amd/csrc", f"{root}/tests/host_fifo_check.cc", "-o",
                    str(exe)], check=True, capture_output=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.startswith("ok"), out.stdout


def test_bench_refuses_more_than_one_gpu():
    """Nothing in this build uses a second GPU; the benchmark says so instead of
    pretending to scale."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "--gpus must be 1" in r.stderr and r.stdout == ""


def test_torch_backend_module_loads_and_fails_loudly_without_a_gpu():
    """The c10d backend module imports against the installed torch, exports its
    factory, and a rank that cannot reach a GPU raises instead of falling back."""
    torch = pytest.importorskip("torch")
    import torch.distributed as dist
    import flagcx_amd.torch_backend as fxb
    ext = fxb.extension()
    assert callable(ext.create_backend)
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible: the refusal cannot be shown")
    with pytest.raises(RuntimeError, match="flagcxCommInitRank failed"):
        fxb.new_backend(dist.HashStore(), 0, 2)


REFERENCE = "/root/reference/flagcx"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference's headers are not on this machine")
def test_headers_agree_with_the_reference_headers(tmp_path):
    """A translation unit that includes the reference's own flagcx.h and adaptor
    headers first and this library's headers after them must compile: C++
    rejects a second declaration of an extern "C" function whose types differ,
    so every entry point declared here has the reference's signature.  The
    structures that cross the boundary have the same size either way."""
    import shutil
    import subprocess
    if not shutil.which("g++"):
        pytest.skip("no g++")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    inc = [f"-I{REFERENCE}/include", f"-I{REFERENCE}/adaptor/include", f"-I{REFERENCE}/core", f"-I{root}/include"]
    ours = "\n".join(f'#include "flagcx_amd/{h}"' for h in
                     ["fx_types.h", "fx_device_adaptor.h", "fx_ccl_adaptor.h", "fx_sim.h", "fx_handle.h", "fx_kernels.h"])
    theirs = '#include <cstring>\n#include "flagcx.h"\n#include "flagcx_device_adaptor.h"\n#include "flagcx_ccl_adaptor.h"\n'
    sizes = r'''
#include <cstdio>
int main() {
  /* the unique ids as test/unittest/service/test_unique_id.cpp pins them: 256 bytes in public, 4120 inside, 8-aligned */
  static_assert(sizeof(flagcxUniqueId) == 256 && sizeof(flagcxInnerUniqueId) == 4120, "unique id sizes");
  static_assert(alignof(flagcxInnerUniqueId) >= alignof(uint64_t), "inner unique id alignment");
  printf("%zu %zu %zu %zu %zu %zu %d %d %d %d\n", sizeof(flagcxDeviceAdaptor_v1), sizeof(flagcxCCLAdaptor_v1),
         sizeof(flagcxDeviceHandle), sizeof(flagcxHandlerGroup), sizeof(flagcxUniqueId), sizeof(flagcxInnerUniqueId),
         (int)flagcxBfloat16, (int)flagcxAvg, (int)flagcxNotSupported, (int)flagcxMemcpyDeviceToDevice);
  return 0;
}
'''
    out = []
    for name, text in (("both", theirs + ours + sizes), ("ours", "#include <cstring>\n" + ours + sizes)):
        src = tmp_path / f"{name}.cc"
        src.write_text(text)
        exe = tmp_path / name
        subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", *inc[-1 if name == "ours" else 0:], str(src), "-o", str(exe)],
                       check=True)
        out.append(subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout)
    assert out[0] == out[1], out
