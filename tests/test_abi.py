"""CPU-side checks of the C-ABI library: it loads, exports every function include/drone_hip.h declares,
the Python mirror binds each of them, struct layouts match the reference's, and host-only entry points
(generators, argument validation) behave.  No GPU work happens here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from drone_amd import _lib, rmat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "drone_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef struct \w+ \{.*?\} \w+;", "", text, flags=re.S)
    text = re.sub(r"enum \w+ \{.*?\};", "", text, flags=re.S)
    names = re.findall(r"\b([A-Za-z_]\w*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert "build_graph" in names and "PR_IncEVal" in names and "drone_pr_run_f64" in names
    handle = C.CDLL(_lib.library_path())
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, f"declared in drone_hip.h but not exported: {missing}"


def test_python_mirror_binds_every_declared_symbol():
    assert sorted(_lib.SIGNATURES) == declared_functions()
    _lib.lib()


def test_struct_layouts_match_reference():
    # common.h:23-27: 6 int + 2 float, returned by value over cgo
    assert C.sizeof(_lib.Response) == 32
    assert _lib.Response.VisitedSize.offset == 16 and _lib.Response.CalTime.offset == 24
    # graph.h:40-43: two pointers
    assert C.sizeof(_lib.Comm) == 16
    # graph.h:16-38 field offsets on LP64 (ext appended after GID)
    g = _lib.Graph
    assert (g.Global2Local.offset, g.Local2Global.offset, g.MasterWorkerIndex.offset, g.Master2Workers.offset) == (0, 8, 16, 24)
    assert (g.MasterSize.offset, g.MirrorWorkerSize.offset, g.Mirror2Worker.offset, g.MirrorSize.offset) == (32, 36, 40, 48)
    assert (g.index.offset, g.dst.offset, g.edgeLen.offset) == (56, 64, 72)
    assert (g.localVertexSize.offset, g.globalVertexSize.offset, g.edgeSize.offset) == (80, 88, 96)
    assert (g.gridSize.offset, g.blockSize.offset, g.active.offset, g.updateByMessage.offset, g.GID.offset) == (104, 108, 112, 120, 128)
    # pr.h:7-16: ten pointers, then ext
    assert _lib.PRValues.outDegree.offset == 72 and _lib.PRValues.ext.offset == 80
    # cc.h:17-25 / sssp.h:17-25: five pointers, then ext
    assert _lib.CCValues.ccValue.offset == 32 and _lib.CCValues.ext.offset == 40
    assert _lib.SSSPValues.distance.offset == 32 and _lib.SSSPValues.ext.offset == 40


ABI_STRUCTS = [("Graph", _lib.Graph), ("Comm", _lib.Comm), ("Response", _lib.Response), ("PRValues", _lib.PRValues),
               ("CCValues", _lib.CCValues), ("SSSPValues", _lib.SSSPValues)]


def test_header_layouts_compiled_by_a_c_compiler(tmp_path):
    """The layouts a C (or cgo) caller gets from include/drone_hip.h, taken from the header itself: a C program that
    includes it prints sizeof and every field's offsetof; they must equal the ctypes mirrors the tests call through,
    the sizes the library was compiled with (drone_abi_sizes), and - for the leading fields - the reference's layouts
    (pr.h:7-16 is ten pointers = 80 bytes; cc.h / sssp.h:17-25 five pointers; graph.h:16-38 ends with GID)."""
    import shutil
    import subprocess
    cc = shutil.which("gcc") or shutil.which("cc")
    assert cc, "no C compiler"
    lines = ["#include <stddef.h>", "#include <stdio.h>", '#include "drone_hip.h"',
             '_Static_assert(sizeof(Response) == 32, "Response is 6 int + 2 float, returned by value");',
             '_Static_assert(sizeof(Comm) == 2 * sizeof(void *), "Comm is two pointers");',
             '_Static_assert(offsetof(PRValues, ext) == 10 * sizeof(void *), "ext follows the reference\'s ten pointers");',
             '_Static_assert(offsetof(CCValues, ext) == 5 * sizeof(void *) && offsetof(SSSPValues, ext) == 5 * sizeof(void *), "ext");',
             '_Static_assert(offsetof(Graph, ext) >= offsetof(Graph, GID) + sizeof(int), "ext follows GID");',
             "int main(void) {"]
    for name, cls in ABI_STRUCTS:
        lines.append(f'    printf("{name} size %zu\\n", sizeof({name}));')
        for field, _ in cls._fields_:
            lines.append(f'    printf("{name} {field} %zu\\n", offsetof({name}, {field}));')
    lines += ["    return 0;", "}"]
    src = tmp_path / "abi.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "abi"
    subprocess.check_call([cc, "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = {}
    for line in subprocess.check_output([str(exe)], text=True).splitlines():
        name, field, value = line.split()
        got[(name, field)] = int(value)
    count = C.c_int(16)
    sizes = (C.c_size_t * 16)()
    assert _lib.lib().drone_abi_sizes(C.byref(count), sizes) == 0 and count.value == len(ABI_STRUCTS)
    for i, (name, cls) in enumerate(ABI_STRUCTS):
        assert got[(name, "size")] == C.sizeof(cls) == sizes[i], name
        for field, _ in cls._fields_:
            assert got[(name, field)] == getattr(cls, field).offset, (name, field)
    assert got[("PRValues", "size")] == 88 and got[("CCValues", "size")] == got[("SSSPValues", "size")] == 48


def test_version_and_error_channel():
    L = _lib.lib()
    assert b"gfx950" in L.drone_version()
    # invalid arguments are rejected on the host before anything touches a device
    rc = L.drone_rmat_edges(0, 10, 0.57, 0.19, 0.19, 1, 0, None, None)
    assert rc == -1 and L.drone_last_error() == -1 and b"scale" in L.drone_last_error_string()
    h = C.c_void_p()
    assert L.drone_pr_plan_create(C.byref(h), 0, 0, None, None, None, None) == -1
    assert L.drone_pr_bytes_per_iteration(10, 100) == 4 * 100 + 32 * 10 + 8


def test_rmat_generator_is_a_pure_function_of_seed_and_index():
    s, d = rmat.rmat_edges(10, 5000, seed=7)
    s2, d2 = rmat.rmat_edges(10, 3000, seed=7, first_edge=2000)
    np.testing.assert_array_equal(s[2000:], s2)
    np.testing.assert_array_equal(d[2000:], d2)
    s3, _ = rmat.rmat_edges(10, 5000, seed=8)
    assert (s != s3).any()
    assert s.max() < 1024 and d.max() < 1024


def test_rmat_quadrant_probabilities():
    # one level: the four quadrants appear with probabilities a, b, c, d
    s, d = rmat.rmat_edges(1, 400000, a=0.57, b=0.19, c=0.19, seed=3)
    q = np.bincount(s.astype(int) * 2 + d.astype(int), minlength=4) / 400000.0
    np.testing.assert_allclose(q, [0.57, 0.19, 0.19, 0.05], atol=4e-3)


@pytest.mark.parametrize("seed,expect", [(1, None)])
def test_rmat_checksums_are_stable(seed, expect):
    """Edge count and a 64-bit hash of the cleaned, sorted edge list for scale 10 with each benchmark seed:
    the GPU box must generate exactly these graphs."""
    import json
    gold = json.load(open(os.path.join(ROOT, "tests", "golden", "rmat_checksums.json")))
    for entry in gold:
        s, d = rmat.rmat_edges(10, 1024 * entry["edge_factor"], a=entry["a"], b=entry["b"], c=entry["c"], seed=entry["seed"])
        src, dst = rmat.clean_directed_np(s, d)
        key = (dst.astype(np.uint64) << np.uint64(32)) | src.astype(np.uint64)
        h = np.uint64(1469598103934665603)
        with np.errstate(over="ignore"):
            acc = np.bitwise_xor.reduce(key * np.uint64(1099511628211) + np.arange(len(key), dtype=np.uint64))
        assert len(key) == entry["edges"]
        assert int(acc ^ h) == entry["hash"]


def test_fill_generators():
    x = rmat.uniform_f32((1000, 7), seed=3)
    assert x.min() >= -1 and x.max() < 1 and abs(x.mean()) < 0.05
    y = rmat.normal_f32(200000, seed=4)
    assert abs(y.mean()) < 0.01 and abs(y.std() - 1) < 0.01
    z = rmat.randint_i32(100000, seed=5, bound=41)
    assert z.min() == 0 and z.max() == 40
    np.testing.assert_array_equal(rmat.uniform_f32(50, seed=3), x.ravel()[:50])


def test_gcn_entry_points_validate_arguments_on_the_host():
    """Bad arguments are rejected before any device work (runs without a GPU)."""
    L = _lib.lib()
    h = C.c_void_p()
    assert L.drone_spmm_plan_create(C.byref(h), -1, 4, 0, None, None, None, 16, None) == -1
    assert L.drone_spmm_plan_create(C.byref(h), 4, 4, 0, None, None, None, 16, None) == -1      # null row_ptr
    assert L.drone_spmm_csr_f32(None, None, None, None, None, 1, None, 1, 1, 1.0, 0.0, None) == -1
    assert b"plan" in L.drone_last_error_string()
    assert L.drone_sgemm_rm_f32(0, 0, 4, 4, 4, 1.0, None, 2, None, 4, 0.0, None, 4, None) == -1  # lda < K
    assert L.drone_sgemm_rm_f32(0, 0, 0, 4, 4, 1.0, None, 4, None, 4, 0.0, None, 4, None) == 0   # empty product
    assert L.drone_cross_entropy_f32(0, 3, None, 3, None, None, 3, 1.0, None, None, None) == -1
    assert L.drone_dropout_mask(None, 0, 1, 0, 1.5, None) == -1                                   # p out of range
    assert L.drone_adam_step_f32(None, None, None, None, 0, 0, 0.0, 0.01, 0.9, 0.999, 1e-8, 0, None) == -1
    assert L.drone_spmm_bytes(10, 100, 8) == 4 * 11 + 8 * 100 + 8 * 10 * 8
    assert L.drone_sgemm_flops(3, 4, 5) == 120
    cfg = _lib.GcnConfig(0, 1, 1, 1, 0.5, 0.01, 0.0, 0, 1, 0, 1)
    assert L.drone_gcn_create(C.byref(h), C.byref(cfg), 0, None, None, None, None, None, 1, None, None, None, None, None) == -1
    assert L.drone_pr_plan_create_ex(C.byref(h), 10, 0, None, None, None, 4, None) == -1


class _Transport(C.Structure):
    """drone_transport of include/drone_hip.h"""
    _EX = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                      C.c_void_p, C.c_void_p, C.c_int, C.c_void_p)
    _AR = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p)
    _fields_ = [("ctx", C.c_void_p), ("exchange", _EX), ("allreduce_sum_f32", _AR)]


def test_loopback_transport_times_out_instead_of_hanging():
    """A worker whose peer never arrives gets an error after timeout_ms; the group then stays broken.  Runs
    without a GPU: the barrier comes before any device call."""
    L = _lib.lib()
    grp = C.c_void_p()
    assert L.drone_loopback_create(C.byref(grp), 0, 10) == -1
    assert L.drone_loopback_create(C.byref(grp), 2, -1) == -1
    assert L.drone_loopback_create(C.byref(grp), 2, 50) == 0
    comm = _lib.Comm()
    assert L.drone_loopback_attach(grp, 2, C.byref(comm)) == -1      # workerId out of range
    assert L.drone_loopback_attach(grp, 0, C.byref(comm)) == 0
    tr = C.cast(comm.comm, C.POINTER(_Transport)).contents
    send_len = (C.c_int * 2)(0, 0)
    send_index = (C.c_int * 3)(0, 0, 0)
    recv_len = (C.c_int * 2)(7, 7)
    send = (C.c_void_p * 2)(None, None)
    recv = (C.c_void_p * 2)(None, None)
    elem = (C.c_size_t * 2)(4, 4)
    args = (send_len, send_index, 2, send, recv, elem, recv_len, 1, None)
    rc = tr.exchange(tr.ctx, 0, 2, *args)
    assert rc == -1 and b"did not arrive" in L.drone_last_error_string()
    assert tr.exchange(tr.ctx, 0, 2, *args) == -1                    # broken for good
    assert tr.exchange(tr.ctx, 0, 3, *args) == -1                    # wrong worker count
    assert tr.exchange(tr.ctx, 0, 2, send_len, send_index, 9, send, recv, elem, recv_len, 1, None) == -1
    assert L.drone_loopback_destroy(grp) == 0
