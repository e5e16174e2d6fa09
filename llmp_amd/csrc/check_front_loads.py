"""The one-token block product (vecq_flat.h; and the one-token expert layer, moe_token.hip) loads its activations' first blocks by instructions the compiler does
not track, so that it can wait for them by count after the first tile's loads are queued. Between such a load and
that wait the destination registers hold nothing yet, and the compiler, which takes them for ordinary values, is free
to copy or spill them. Nothing in the language forbids that, so this build step reads the compiler's assembly of every
kernel that has such loads: from a load to the wait that follows it, no instruction may name a register the load
writes, and nothing may spill. Needs hipcc, no GPU. Run by the library's build (__graft_entry__.build) and by
tests/test_front_loads.py; `python check_front_loads.py` runs it alone."""
import os
import re
import shutil
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
SOURCES = ("vecq_flat_q4k.hip", "vecq_flat_q8.hip", "vecq_flat_q5k.hip", "vecq_flat_q6k.hip", "moe_token.hip")
# The first instruction of the wait's chain, or (the one-token expert layer's second launch) a plain wait for all.
WAIT = re.compile(r"s_cmp_lt_u32 s\d+, 10\b|^s_waitcnt vmcnt\(0\)$")


def registers(code):
    """The vector registers an instruction names."""
    named = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", code):
        named.update(range(int(a), int(b) + 1))
    named.update(int(v) for v in re.findall(r"\bv(\d+)\b", code))
    return named


def check_kernel(name, body):
    """The number of tracked loads; raises AssertionError on a register named between a load and its wait."""
    pending = {}  # register -> the load that writes it
    own = False
    loads = 0
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
        code = text.split(";")[0]
        if own and re.match(r"global_load_dword(x2|x4)?\s", code):
            destination = code.split(",")[0]
            for r in registers(destination):
                pending[r] = code
            loads += 1
            continue
        if own and WAIT.search(code.strip()):
            pending = {}
            continue
        if own and pending and re.match(r"s_(cmp|cbranch|waitcnt|branch)", code):
            continue  # the rest of the wait's chain
        # Address registers of later loads may be rewritten; what matters is a read or a write of a pending one.
        touched = registers(code) & set(pending)
        assert not touched, f"{name}: `{code}` names v{sorted(touched)} before the wait for `{pending[min(touched)]}`"
    assert not pending, f"{name}: a load without a wait after it"
    assert loads == 0 or "scratch_" not in body, f"{name}: spills"
    return loads


def check():
    """Raises AssertionError (or the compiler's error) unless every such load is left alone until its wait."""
    kernels = 0
    for source in SOURCES:
        with tempfile.TemporaryDirectory() as tmp:
            out = os.path.join(tmp, "flat.s")
            subprocess.run(
                [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-I" + HERE,
                 "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S", "-o", out,
                 os.path.join(HERE, source)],
                check=True, capture_output=True, timeout=1200)
            with open(out) as f:
                assembly = f.read()
        for m in re.finditer(r"^(_ZN\S*(?:VecQFlat|MoeTokenKernel)\S*):", assembly, re.M):
            body = assembly[m.end():assembly.index("s_endpgm", m.end())]
            if check_kernel(m.group(1), body) > 0:
                kernels += 1
    assert kernels >= 4, f"only {kernels} kernels with such loads were found"
    return kernels


if __name__ == "__main__":
    print(f"{check()} kernels load their activations' first blocks by instructions; nothing touches the registers before the wait")
