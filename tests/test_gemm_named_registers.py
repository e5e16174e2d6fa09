"""The MXFP8 GEMM's split of the register file between the compiler and the registers its loop names, checked in the
compiler's assembly (llmp_amd/csrc/check_named_registers.py, also a step of the build). Needs hipcc, no GPU; fails,
not skips, where hipcc is missing: a build that cannot be checked is not a build."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_compiler_keeps_off_the_registers_the_gemm_names():
    spec = importlib.util.spec_from_file_location(
        "check_named_registers", os.path.join(ROOT, "llmp_amd", "csrc", "check_named_registers.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    assert os.path.exists(module.HIPCC), "hipcc is missing: the GEMM's register split cannot be checked"
    module.check()
