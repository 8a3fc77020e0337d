"""The C ABI: structure layout against the reference's header (golden numbers written
by tests/golden/make_abi_layout.py from the reference's own thnets.h), and that the
built library exports every symbol include/thnets_hip.h declares.  No GPU needed."""
import ctypes as C
import json
import os
import re
import subprocess

import pytest

from thnets_amd import abi, api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = json.load(open(os.path.join(ROOT, "tests", "golden", "abi_layout.json")))
HEADER = os.path.join(ROOT, "include", "thnets_hip.h")


@pytest.mark.parametrize("variant", ["default", "lowp"])
def test_ctypes_mirror_matches_reference_layout(variant):
    lay = (abi.ABI if variant == "default" else abi.ABI_LOWP).layout()
    for k, v in lay.items():
        assert GOLDEN[variant][k] == v, k


def test_enum_values_match_reference():
    g = GOLDEN["default"]
    assert len(abi.MODULE_TYPES) == g["n_module_types"]
    assert abi.MT["MT_Linear"] == g["MT_Linear"]
    assert abi.MT["MT_CAddTable"] == g["MT_CAddTable"]
    assert abi.MT["MT_SpatialBatchNormalization"] == g["MT_SpatialBatchNormalization"]
    assert abi.ENGINE_LOWP == g["ENGINE_LOWP"]
    assert abi.ENGINE_HIP == g["ENGINE_LOWP"] + 1


PROBE = r'''
#include <stdio.h>
#include <stddef.h>
#include "thnets_hip.h"
int main(void)
{
	printf("{\"sizeof_THFloatStorage\": %zu, \"sizeof_THFloatTensor\": %zu, \"sizeof_module\": %zu,"
		"\"off_module_union\": %zu, \"off_module_output\": %zu, \"off_module_net\": %zu,"
		"\"off_module_inputs\": %zu, \"sizeof_SpatialConvolution\": %zu, \"off_conv_nOutputPlane\": %zu,"
		"\"sizeof_SpatialMaxPooling\": %zu, \"off_maxpool_indices\": %zu, \"off_bn_eps\": %zu,"
		"\"sizeof_network\": %zu, \"sizeof_THNETWORK\": %zu, \"off_thnetwork_net\": %zu,"
		"\"off_thnetwork_out\": %zu, \"off_thnetwork_mean\": %zu, \"off_thnetwork_std\": %zu,"
		"\"sizeof_SpatialFullConvolution\": %zu, \"off_fullconv_adjW\": %zu, \"off_fullconv_ones\": %zu,"
		"\"n_module_types\": %d, \"MT_Linear\": %d, \"MT_CAddTable\": %d, \"ENGINE_LOWP\": %d}\n",
		sizeof(THFloatStorage), sizeof(THFloatTensor), sizeof(struct module),
		offsetof(struct module, SpatialConvolution), offsetof(struct module, output), offsetof(struct module, net),
		offsetof(struct module, inputs), sizeof(struct SpatialConvolution),
		offsetof(struct SpatialConvolution, nOutputPlane), sizeof(struct SpatialMaxPooling),
		offsetof(struct SpatialMaxPooling, indices), offsetof(struct SpatialBatchNormalization, eps),
		sizeof(struct network), sizeof(THNETWORK), offsetof(THNETWORK, net), offsetof(THNETWORK, out),
		offsetof(THNETWORK, mean), offsetof(THNETWORK, std), sizeof(struct SpatialFullConvolution),
		offsetof(struct SpatialFullConvolution, adjW), offsetof(struct SpatialFullConvolution, ones),
		MT_Transpose + 1, MT_Linear, MT_CAddTable, ENGINE_LOWP);
	return 0;
}
'''


def test_c_header_matches_reference_layout(tmp_path):
    src = tmp_path / "probe.c"
    src.write_text(PROBE)
    exe = tmp_path / "probe"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)])
    got = json.loads(subprocess.check_output([str(exe)]).decode())
    for k, v in got.items():
        assert GOLDEN["default"][k] == v, k


def test_golden_layout_is_current_when_reference_is_mounted(tmp_path):
    ref = "/root/reference"
    if not os.path.exists(os.path.join(ref, "thnets.h")):
        pytest.skip("reference tree not mounted")
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_abi_layout", os.path.join(ROOT, "tests", "golden",
                                                                                  "make_abi_layout.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.probe(ref, []) == GOLDEN["default"]
    assert mod.probe(ref, ["-DLOWP"]) == GOLDEN["lowp"]


def _object_lists():
    """The object lists INTEGRATION.md gives a thnets maintainer: the HIP=1 block of the
    Makefile fragment, and the objects that stand in for gemm8.o under LOWP=1."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    m = re.search(r"LIBOBJS \+= ((?:\w+\.o ?)+)", text)
    engine = m.group(1).split()
    m = re.search(r"link `((?:\w+\.o ?)+)` instead", text)
    lowpgemm = m.group(1).split()
    return engine, lowpgemm


def _nm(path, undefined):
    out = subprocess.check_output(["nm", "-u" if undefined else "--defined-only", path]).decode()
    return set(line.split()[-1] for line in out.splitlines() if line.strip())


# what the system provides: libc / libm / libstdc++ / compiler runtime / the HIP runtime
SYSTEM = re.compile(r"^(GOMP_|omp_|hip[A-Z]|__hip|_Z(?!\d+thhip)|__cxa|__gxx|_Unwind|__stack_chk|__dso_handle|_GLOBAL_|__truncsfhf2|"
                    r"__extendhfsf2|mem(cpy|set|move)$|__mem\w+_chk|malloc$|calloc$|realloc$|free$|exit$|abort$|atexit$|"
                    r"f?printf$|__\w*printf_chk|v?fprintf$|snprintf$|fputs$|fputc$|fwrite$|fflush$|puts$|stderr$|stdout$|"
                    r"getenv$|atoi$|strcmp$|strlen$|qsort$|clock_gettime$|log$|logf$|sqrt$|sqrtf$|roundf$|floorf$|ceilf$|"
                    r"expf$|fmaxf$|fminf$)")


def test_makefile_and_integration_name_the_same_kernel_objects():
    mk = open(os.path.join(ROOT, "thnets_amd", "csrc", "Makefile")).read()
    hip_srcs = re.search(r"^HIP_SRCS = (.*)$", mk, flags=re.M).group(1).split()
    engine, _ = _object_lists()
    assert sorted(o for o in engine if o not in ("th_engine.o", "th_io.o")) == sorted(f[:-4] + ".o" for f in hip_srcs)


@pytest.mark.parametrize("flags", [[], ["-DLOWP"]])
def test_in_tree_object_list_links(tmp_path, flags):
    """The engine as a thnets maintainer would link it (Makefile's HIP=1 option modelled on
    Makefile:152-178): th_engine.c and th_io.c compile with -DTHNETS_IN_TREE, warning-free,
    with the reference's flags (-Wall -fopenmp, Makefile:28) against its own unmodified thnets.h (default and -DLOWP layout), and the
    object list INTEGRATION.md gives is closed - every symbol those objects leave undefined
    is defined by another of them, by the reference's library (tensor helpers, THError) or
    by the system.  The same for the objects that replace gemm8.o (lowpgemm,
    lowp_basic.c:290-297).  The kernel objects are the ones the library was built from."""
    ref = "/root/reference"
    if not os.path.exists(os.path.join(ref, "thnets.h")):
        pytest.skip("reference tree not mounted")
    csrc = os.path.join(ROOT, "thnets_amd", "csrc")
    engine, lowpgemm = _object_lists()
    assert "th_engine.o" in engine and "th_io.o" in engine and len(engine) >= 11
    paths = {}
    for o in engine:
        src = os.path.join(csrc, o[:-2] + ".c")
        if os.path.exists(src):
            paths[o] = str(tmp_path / o)
            r = subprocess.run(["gcc", "-std=gnu11", "-Wall", "-Werror", "-Wno-unused-function", "-fopenmp", "-c",
                                "-DTHNETS_IN_TREE"] + flags + ["-I", ref, src, "-o", paths[o]], capture_output=True, text=True)
            assert r.returncode == 0, r.stderr
        else:
            assert os.path.exists(os.path.join(csrc, o[:-2] + ".hip")), o
            paths[o] = os.path.join(csrc, "build", o)
            if not os.path.exists(paths[o]):
                pytest.fail("%s missing: build the library first (python __graft_entry__.py)" % paths[o])
    reflib = os.path.join(ROOT, "oracle", "_ref", "libthnets_ref_lowp.so" if flags else "libthnets_ref.so")
    if not os.path.exists(reflib):
        pytest.skip("oracle/_ref not built")
    provided = _nm(reflib, False)
    for objs, must_define in ((engine, ["THHip_ToHip", "thhip_forward", "thhip_process_float", "thhip_process_images",
                                        "THHipTensor_newFromFloatTensor", "THFloatTensor_newFromHipTensor",
                                        "thhip_free_network", "thhip_free"]),
                              (lowpgemm, ["lowpgemm"])):
        defined, undefined = set(), set()
        for o in objs:
            defined |= _nm(paths[o], False)
            undefined |= _nm(paths[o], True)
        for name in must_define:
            assert name in defined, name
        open_ = sorted(u for u in undefined - defined if not SYSTEM.match(u))
        missing = [u for u in open_ if u not in provided]
        assert not missing, "%s leave undefined: %s" % (objs, missing)
        # what does come from the reference's library are its tensor helpers and THError
        assert all(u.startswith("TH") for u in open_), open_
    # nothing of the stand-alone host files is needed
    assert "th_api.o" not in engine and "th_tensor.o" not in engine


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^[A-Za-z_][A-Za-z0-9_ \*]*?\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", text, flags=re.M)
    return sorted(set(n for n in names if not n.startswith("(")))


def test_library_exports_every_declared_symbol():
    lib = api.load_library()
    names = declared_functions()
    assert "THCreateHipNetwork" in names and "thhip_conv2d" in names and "lowpgemm" in names
    assert len(names) >= 55
    for n in names:
        assert hasattr(lib, n), "libthnets_hip.so does not export %s" % n
    for v in ("th_debug", "th_profile", "th_minmax"):
        C.c_int.in_dll(lib, v)
    for n in names:
        assert n in api.PROTOTYPES, "no ctypes prototype for %s" % n


def test_thhip_half_float_switch_contract():
    lib = api.load_library()
    assert lib.THHipHalfFloat(1) == 0
    assert lib.THHipHalfFloat(2) == 0
    assert lib.THHipHalfFloat(3) == -3      # ERR_NOTIMPLEMENTED, like THCudaHalfFloat without fp16
    assert lib.THHipHalfFloat(0) == 0


def test_pool_outsize_is_host_only_and_follows_reference_rule(oracle):
    lib = api.load_library()
    for (H, W, k, d, p, ceil) in [(55, 55, 3, 2, 0, 0), (13, 13, 3, 2, 0, 1), (112, 112, 3, 2, 1, 0), (7, 9, 2, 2, 1, 1),
                                  (6, 6, 3, 3, 1, 1), (5, 5, 2, 2, 1, 1)]:
        oh, ow = C.c_int(), C.c_int()
        lib.thhip_pool_outsize(H, W, k, k, d, d, p, p, ceil, C.byref(oh), C.byref(ow))
        assert (oh.value, ow.value) == oracle.pool_outsize(H, W, k, k, d, d, p, p, ceil)
