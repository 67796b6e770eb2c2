"""CPU-side checks of the C-ABI boundary: the built library loads, exports every symbol that
include/infr_hip.h declares, the Python mirror's struct layouts match the header's, and the
host-side error paths that need no GPU behave like the reference's error values."""
import ctypes as C
import os
import re
import subprocess

import pytest

import moe4all_amd as M
from moe4all_amd import backend as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "infr_hip.h")
PROBE_HEADER = os.path.join(ROOT, "include", "infr_hip_probe.h")
SYNTH_HEADER = os.path.join(ROOT, "include", "infr_synth.h")


def declared_symbols(path=HEADER, prefix="infr_hip_"):
    src = open(path).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", src)))


def test_header_declares_the_backend_trait_surface():
    syms = declared_symbols()
    for required in ("infr_hip_create", "infr_hip_destroy", "infr_hip_name", "infr_hip_capabilities_get",
                     "infr_hip_alloc", "infr_hip_alloc_uninit", "infr_hip_buffer_len", "infr_hip_buffer_free",
                     "infr_hip_upload", "infr_hip_download", "infr_hip_upload_range", "infr_hip_download_range",
                     "infr_hip_copy_buffer", "infr_hip_compile", "infr_hip_plan_free", "infr_hip_execute",
                     "infr_hip_sync", "infr_hip_last_error"):
        assert required in syms


def test_library_exports_every_declared_symbol():
    lib = M.load_library()
    boundary, probes = declared_symbols(), declared_symbols(PROBE_HEADER)
    for s in boundary + probes:
        assert hasattr(lib, s), f"{s} declared in include/ but not exported"
    # the boundary header holds no measurement call, and the Python mirror binds exactly the declared set
    assert not [s for s in boundary if "_probe_" in s or "_prof_" in s]
    assert sorted(B._SIGNATURES) == sorted(set(boundary + probes))
    synth = declared_symbols(SYNTH_HEADER, "infr_synth_")
    assert len(synth) == 4
    for s in synth:
        assert hasattr(lib, s), f"{s} declared in include/infr_synth.h but not exported"


def test_struct_layouts_match_the_header(tmp_path):
    """Compile a tiny C program against the header and compare sizeof/offsetof with ctypes."""
    prog = tmp_path / "layout.c"
    prog.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "infr_hip_probe.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(infr_tensor_decl), sizeof(infr_op_moe_ffn), sizeof(infr_op),
         sizeof(infr_graph), sizeof(infr_binding), sizeof(infr_hip_capabilities), sizeof(infr_hip_config),
         sizeof(infr_hip_prof_entry), offsetof(infr_op, u));
  printf("%zu %zu %zu %zu\n", offsetof(infr_op_moe_ffn, scale), offsetof(infr_op_moe_ffn, gating),
         offsetof(infr_op_moe_ffn, expert_ids), offsetof(infr_op_gated_act, swiglu_clamp));
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(prog), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode().split()
    got = [int(v) for v in out]
    want = [C.sizeof(B._TensorDecl), C.sizeof(B._OpMoeFfn), C.sizeof(B._Op), C.sizeof(B._Graph), C.sizeof(B._Binding),
            C.sizeof(B._Caps), C.sizeof(B._Config), C.sizeof(B._ProfEntry), B._Op.u.offset,
            B._OpMoeFfn.scale.offset, B._OpMoeFfn.gating.offset, B._OpMoeFfn.expert_ids.offset,
            B._OpGatedAct.swiglu_clamp.offset]
    assert got == want


def test_dtype_ordinals_follow_the_reference_enum():
    # crates/infr-core/src/tensor.rs:7-57
    names = ["F32", "F16", "Bf16", "I32", "U32", "Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q8_0", "Q2K", "Q3K", "Q4K", "Q5K", "Q6K",
             "Iq1S", "Iq1M", "Iq2Xxs", "Iq2Xs", "Iq2S", "Iq3Xxs", "Iq3S", "Iq4Nl", "Iq4Xs", "Tq1_0", "Tq2_0", "I2S", "Q2_0",
             "Mxfp4", "Nvfp4"]
    assert [d.name for d in M.DType] == names and [int(d) for d in M.DType] == list(range(30))
    assert [int(u) for u in M.BufferUsage] == list(range(6))
    assert [k.name for k in M.TensorKind] == ["Input", "Weight", "Internal", "Output"]


def _gpu_present():
    try:
        M.Backend(0).close()
        return True
    except M.BackendError:
        return False


def test_no_device_is_an_error_not_a_fallback():
    if _gpu_present():
        pytest.skip("a device is present; the no-device path is exercised on CPU-only hosts")
    with pytest.raises(M.BackendError) as e:
        M.Backend(0)
    assert "no CPU fallback" in str(e.value)


def test_null_and_foreign_handles_are_errors():
    lib = M.load_library()
    assert lib.infr_hip_buffer_len(None) == 0
    assert lib.infr_hip_name(None) == b""
    assert lib.infr_hip_sync(None) == 4  # INFR_ERR_INVALID
    assert b"bad handle" in lib.infr_hip_last_error()
    h = C.c_void_p()
    assert lib.infr_hip_alloc(None, 16, 0, C.byref(h)) == 4
    lib.infr_hip_buffer_free(None)
    lib.infr_hip_plan_free(None)
    lib.infr_hip_destroy(None)


def test_every_status_returning_entry_point_catches_exceptions():
    """No exception may cross the C ABI (the header promises it): every extern "C" function that returns a status is a
    function-try-block in the sources, and the void ones that free objects swallow what their bodies throw."""
    for name in ("backend.cpp", "gguf.cpp"):
        src = open(os.path.join(ROOT, "moe4all_amd", "csrc", name)).read()
        heads = re.findall(r'^extern "C" infr_status (\w+)\((?:[^;{]|\n)*?\)\s*(try)?\s*\{', src, flags=re.M)
        assert len(heads) >= 10
        missing = [n for n, t in heads if not t]
        assert not missing, f"{name}: {missing} can let an exception escape"
        assert src.count("catch (...) { return guard_fail(") >= len(heads)
