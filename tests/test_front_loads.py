"""The one-token block product's activations are loaded by instructions the compiler does not track and waited for by
count; the compiler's assembly is read for anything that names their registers before that wait
(llmp_amd/csrc/check_front_loads.py, also a step of the build). Needs hipcc, no GPU; fails, not skips, where hipcc is
missing."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_nothing_touches_the_front_loads_registers_before_their_wait():
    spec = importlib.util.spec_from_file_location(
        "check_front_loads", os.path.join(ROOT, "llmp_amd", "csrc", "check_front_loads.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    assert os.path.exists(module.HIPCC), "hipcc is missing: the front loads cannot be checked"
    assert module.check() >= 4
