"""The MXFP8 GEMM (and its F16 sibling, the same loop) names the registers of its loop (fragments, scales and sums) in its instructions and holds the
compiler to the registers below them. Nothing in the language enforces that split, so this build step reads the
compiler's assembly of the kernel: no instruction that the compiler wrote may touch a named register, nothing may
spill, and the kernel's register counts must cover the named ones. Needs hipcc, no GPU. Run by the library's build
(__graft_entry__.build) and by tests/test_gemm_named_registers.py; `python check_named_registers.py` runs it alone."""
import os
import re
import shutil
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
# kernel -> (the compiler's registers v0 .. below this, the highest named register, the sums' registers)
SHAPES = {"GemmKernel192": (64, 252, 192), "GemmKernel128": (64, 216, 128),
          "GemmKernelHalf192": (64, 252, 192), "GemmKernelHalf128": (64, 216, 128)}


def kernels(assembly):
    """name -> body of every GemmKernel instance."""
    found = {}
    for m in re.finditer(r"^(_ZN\S*GemmKernel\S*):", assembly, re.M):
        end = assembly.index("s_endpgm", m.end())
        found[m.group(1)] = assembly[m.end():end]
    return found


def check():
    """Raises AssertionError (or the compiler's error) unless the split holds in every GEMM kernel."""
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "mxfp8.s")
        subprocess.run(
            [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-I" + HERE,
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S", "-o", out,
             os.path.join(HERE, "mxfp8.hip")],
            check=True, capture_output=True, timeout=600)
        with open(out) as f:
            assembly = f.read()
    bodies = kernels(assembly)
    assert len(bodies) == len(SHAPES), "the kernels were not found"
    for name, body in bodies.items():
        COMPILER_VGPRS, TOP_VGPR, SUMS = next(v for k, v in SHAPES.items() if k in name)
        own = False  # inside an instruction sequence that the source wrote
        products = 0
        for line in body.split("\n"):
            text = line.strip()
            if "#ASMSTART" in text:
                own = True
                continue
            if "#ASMEND" in text:
                own = False
                continue
            if not text or text[0] in ";." or text.endswith(":"):
                continue
            products += "v_mfma_scale" in text or "v_mfma_f32_16x16x32_f16" in text
            if own:
                continue
            code = text.split(";")[0]
            high = [int(b) for _, b in re.findall(r"\bv\[(\d+):(\d+)\]", code)] + [int(v) for v in re.findall(r"\bv(\d+)\b", code)]
            assert not [v for v in high if v >= COMPILER_VGPRS], f"{name}: the compiler wrote `{text}`"
            assert not re.search(r"\ba\[?\d+", code), f"{name}: the compiler wrote `{text}`"
        assert products > 0
        meta = assembly[assembly.index(".amdhsa_kernel " + name):]
        meta = meta[:meta.index(".end_amdhsa_kernel")]
        field = lambda key: int(re.search(r"\.amdhsa_%s (\d+)" % key, meta).group(1))
        assert field("private_segment_fixed_size") == 0, f"{name} spills"
        assert field("accum_offset") > TOP_VGPR, "the sums' registers start inside the named ones"
        assert field("next_free_vgpr") >= field("accum_offset") + SUMS


if __name__ == "__main__":
    check()
    print("the compiler keeps off the registers the GEMM names")
