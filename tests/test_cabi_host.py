"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol the
header declares, and the ctypes table covers exactly those symbols."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cuda_mace_hip.h")
LIB = os.path.join(ROOT, "cuda-mace_amd", "cuda_mace", "lib", "libcuda_mace_hip.so")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.isfile(LIB), "build the library first: python cuda-mace_amd/build.py"
    lib = ctypes.CDLL(LIB)
    names = _declared()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), name


def test_ctypes_table_matches_header():
    from cuda_mace import _cabi

    assert sorted(_cabi.SIGNATURES) == _declared()


def test_host_side_validation_needs_no_gpu():
    lib = ctypes.CDLL(LIB)
    lib.cm_last_error.restype = ctypes.c_char_p
    assert lib.cm_abi_version() >= 1
    assert lib.cm_channels_supported(128) == 1 and lib.cm_channels_supported(48) == 0
    lib.cm_mp_forward.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    rc = lib.cm_mp_forward(None, None, None, None, None, 10, 10, 48, None, None)
    assert rc == -22 and b"multiple of 32" in lib.cm_last_error()
    rc = lib.cm_mp_forward(None, None, None, None, None, 10, 10, 64, None, None)
    assert rc == -22 and b"NULL" in lib.cm_last_error()
    lib.cm_stable_key_sort_workspace.restype = ctypes.c_size_t
    lib.cm_stable_key_sort_workspace.argtypes = [ctypes.c_int64, ctypes.c_int64]
    assert lib.cm_stable_key_sort_workspace(100, 10) >= 4 * 120


def test_binding_rejects_host_tensors():
    import pytest
    import torch
    from cuda_mace import _cabi

    with pytest.raises(RuntimeError, match="GPU"):
        _cabi.sh_forward(torch.zeros(4, 3))


def test_profiler_ranges_are_off_unless_asked_for():
    """cm_trace_* do nothing by default; with CUDA_MACE_TRACE=1 the marker library is found at run time and push / pop
    can be called without a profiler attached.  The switch is read once per process, hence the child processes."""
    import subprocess
    import sys

    code = (
        "import ctypes; lib = ctypes.CDLL(%r); lib.cm_trace_push.argtypes = [ctypes.c_char_p]; lib.cm_trace_push.restype = None;"
        "lib.cm_trace_pop.restype = None; lib.cm_trace_push(b'cuda_mace:test'); lib.cm_trace_pop(); print(lib.cm_trace_enabled())" % LIB
    )
    seen = {}
    for value in (None, "0", "1"):
        env = {k: v for k, v in os.environ.items() if k != "CUDA_MACE_TRACE"}
        if value is not None:
            env["CUDA_MACE_TRACE"] = value
        res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
        assert res.returncode == 0, res.stderr
        seen[value] = int(res.stdout.split()[-1])
    assert seen[None] == 0 and seen["0"] == 0
    have_markers = any(os.path.exists(os.path.join(d, n)) for d in ("/opt/rocm/lib", "/opt/rocm/lib64")
                       for n in ("librocprofiler-sdk-roctx.so", "libroctx64.so"))
    assert seen["1"] == (1 if have_markers else 0)


def test_edge_range_clamp_arithmetic(tmp_path):
    """cm::clamp_edge_range, which every kernel applies to the CSR offsets it reads, compiled for the host and run on
    valid, reversed, out-of-range and random offsets (tests/host/clamp_edge_range_check.cpp)."""
    import shutil
    import subprocess

    import pytest

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    exe = tmp_path / "clamp_check"
    src = os.path.join(ROOT, "tests", "host", "clamp_edge_range_check.cpp")
    res = subprocess.run([hipcc, "--cuda-host-only", "-x", "hip", "-O1", "-I" + os.path.join(ROOT, "include"),
                          "-I" + os.path.join(ROOT, "cuda-mace_amd", "csrc"), src, "-o", str(exe)],
                         capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr


def test_build_refuses_scratch_in_hand_scheduled_kernels():
    """The build parses the compiler's resource-usage remarks and fails when a kernel whose loads are issued from inline
    assembly spills registers (its correctness depends on loaded registers staying where the load put them)."""
    import importlib.util

    import pytest

    spec = importlib.util.spec_from_file_location("_cm_build", os.path.join(ROOT, "cuda-mace_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    line = "csrc/linear.hip:1:1: remark: %s [-Rpass-analysis=kernel-resource-usage]"
    ok = "\n".join(line % t for t in ("Function Name: _ZN2cm18linear_ring_kernelILi4ELb0EEE", "    VGPRs: 216",
                                      "    ScratchSize [bytes/lane]: 0", "    SGPRs Spill: 0", "    VGPRs Spill: 0",
                                      "Function Name: _ZN2cm13linear_kernelILi8ELb1EEE", "    ScratchSize [bytes/lane]: 100"))
    build._check_no_scratch("linear.hip", ok)  # the plain kernel may spill, the ring kernel does not
    bad = ok.replace("ScratchSize [bytes/lane]: 0", "ScratchSize [bytes/lane]: 100", 1)
    with pytest.raises(RuntimeError, match="ScratchSize"):
        build._check_no_scratch("linear.hip", bad)
    with pytest.raises(RuntimeError, match="VGPRs Spill"):
        build._check_no_scratch("linear.hip", ok.replace("VGPRs Spill: 0", "VGPRs Spill: 24"))
    with pytest.raises(RuntimeError, match="no resource-usage remark"):
        build._check_no_scratch("mp.hip", ok)


def test_build_refuses_copies_into_landing_registers():
    """The resident-weights linear kernel lands its loads in accumulator-file registers named at issue time; the build
    scans the device assembly and fails if anything but a load writes one of those registers inside such a kernel."""
    import importlib.util

    import pytest

    spec = importlib.util.spec_from_file_location("_cm_build", os.path.join(ROOT, "cuda-mace_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    ok = ["_ZN2cm13linear_kernelILi8ELb1EEE:  ; @x", "\tv_accvgpr_write_b32 a3, v7", ".Lfunc_end0:",
          "_ZN2cm22linear_resident_kernelILi128ELi4ELb0EEE:  ; @y", "\tglobal_load_dwordx4 a[64:67], v[2:3], off nt",
          "\tv_accvgpr_read_b32 v5, a64", "\tv_accvgpr_write_b32 a0, 0", "\tv_accvgpr_write_b32 a130, v9", ".Lfunc_end1:"]
    build._scan_landing_registers("linear.hip", ok)  # other kernels may copy; so may this one outside its landing registers
    for bad in ("\tv_accvgpr_write_b32 a66, v84", "\tv_accvgpr_mov_b32 a64, a12"):
        with pytest.raises(RuntimeError, match="copies into a landing register"):
            build._scan_landing_registers("linear.hip", ok[:5] + [bad] + ok[5:])
    with pytest.raises(RuntimeError, match="no code found"):
        build._scan_landing_registers("linear.hip", ok[:3])
    with pytest.raises(RuntimeError, match="no load into the accumulator file"):
        build._scan_landing_registers("linear.hip", ok[:4] + ok[5:])


def test_build_refuses_use_of_a_register_before_its_load_has_landed():
    """Kernels that issue loads from inline assembly and wait for them later: the build walks their generated code with
    the hardware's rule (vector-memory operations retire in order; s_waitcnt vmcnt(n) leaves the newest n out) and fails
    on any instruction that touches a register while a load into it is in flight -- the copy a compiler may place where
    such a register crosses a loop's back edge, which reads the register before the data is there."""
    import importlib.util

    import pytest

    spec = importlib.util.spec_from_file_location("_cm_build", os.path.join(ROOT, "cuda-mace_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    head = ["_ZN2cm13other_kernelEv:  ; @x", "\tglobal_load_dword v5, v[2:3], off", "\tv_mov_b32_e32 v6, v5", ".Lfunc_end0:",
            "_ZN2cm25mp_backward_sender_kernelILi128ELi1ELb0EEE:  ; @y"]
    tail = ["\ts_endpgm", ".Lfunc_end1:"]
    ok = ["\tglobal_load_dword v5, v[2:3], off", "\tv_add_u32_e32 v9, v8, v7", "\ts_waitcnt vmcnt(0)", "\tv_mov_b32_e32 v6, v5",
          ".LBB1_1:  ; loop", "\tv_add_f32_e32 v10, v6, v10",
          "\tglobal_load_dword v5, v[2:3], off", "\tglobal_load_lds_dwordx4 v[20:21], off nt", "\tglobal_load_dword v12, v[2:3], off",
          "\tv_add_u32_e32 v20, 4, v20",                       # the address of a load that lands in LDS is free at once
          "\ts_waitcnt vmcnt(1) lgkmcnt(0)", "\tv_mov_b32_e32 v6, v5",  # the older load has landed, the newest may be out
          "\t;;#ASMSTART", "\t; landed v12", "\t;;#ASMEND", "\tv_mov_b32_e32 v13, v12",  # the source says so: taken at its word
          "\ts_cbranch_scc1 .LBB1_1"]
    assert build._scan_in_flight_registers("mp.hip", head + ok + tail) == 1  # kernels not named may do as they like

    def scan(body):
        build._scan_in_flight_registers("mp.hip", head + body + tail)

    with pytest.raises(RuntimeError, match="v_mov_b32_e32 v14, v12.*touches v12"):  # newest load still out at vmcnt(1)
        scan(ok[:12] + ["\tv_mov_b32_e32 v14, v12"] + ok[12:])
    with pytest.raises(RuntimeError, match="touches v5"):  # written, not read: the load would land on top of it
        scan(ok[:7] + ["\tv_mov_b32_e32 v5, 0"] + ok[7:])
    with pytest.raises(RuntimeError, match="touches v5"):  # used as an address
        scan(ok[:7] + ["\tglobal_load_dword v30, v[4:5], off"] + ok[7:])
    # issued at the bottom of the loop, waited for at its top: the copy across the back edge reads too early ...
    loop = [".LBB1_1:", "\ts_waitcnt vmcnt(0)", "\tv_add_f32_e32 v10, v38, v10", "\tglobal_load_dword v46, v[2:3], off",
            "\tv_mov_b32_e32 v38, v46", "\ts_cbranch_scc1 .LBB1_1"]
    with pytest.raises(RuntimeError, match="v_mov_b32_e32 v38, v46.*touches v46"):
        scan(loop)
    scan(loop[:4] + loop[5:])  # ... without it the register is first read behind the wait at the top
    # ... and a use that only the way round the back edge makes too early is found as well
    with pytest.raises(RuntimeError, match="v_add_f32_e32 v10, v46, v10.*touches v46"):
        scan([".LBB1_1:", "\tv_add_f32_e32 v10, v46, v10", "\ts_waitcnt vmcnt(0)", "\tglobal_load_dword v46, v[2:3], off",
              "\ts_cbranch_scc1 .LBB1_1"])
    # a wait on one side of a branch only does not count for the other side
    with pytest.raises(RuntimeError, match="touches v5"):
        scan(["\tglobal_load_dword v5, v[2:3], off", "\ts_cbranch_scc1 .LBB1_2", "\ts_waitcnt vmcnt(0)", ".LBB1_2:", "\tv_mov_b32_e32 v6, v5"])
    scan(["\tglobal_load_dword v5, v[2:3], off", "\ts_cbranch_scc1 .LBB1_2", "\ts_waitcnt vmcnt(0)", "\ts_branch .LBB1_3", ".LBB1_2:",
          "\ts_waitcnt vmcnt(0)", ".LBB1_3:", "\tv_mov_b32_e32 v6, v5"])
    with pytest.raises(RuntimeError, match="no code found"):
        build._scan_in_flight_registers("mp.hip", head[:4])


def test_header_is_valid_c_and_cpp(tmp_path):
    """The boundary is a C ABI: the header must compile as plain C (what cgo, a Fortran binding generator or LAMMPS'
    C glue would include) and as C++, on its own."""
    import shutil
    import subprocess

    import pytest

    for compiler, lang, std in (("gcc", "c", "-std=c99"), ("g++", "c++", "-std=c++11")):
        exe = shutil.which(compiler)
        if exe is None:
            pytest.skip("no " + compiler)
        src = tmp_path / ("use_header." + ("c" if lang == "c" else "cpp"))
        src.write_text('#include "cuda_mace_hip.h"\nint main(void) { cm_mace_weights w; cm_mace_graph g; (void)w; (void)g; '
                       'return (int)sizeof(cm_stream_t) == 0; }\n')
        res = subprocess.run([exe, std, "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I" + os.path.join(ROOT, "include"),
                              str(src)], capture_output=True, text=True, timeout=120)
        assert res.returncode == 0, res.stderr
