"""The part of the C++ front-end test that needs no GPU, run to a normal return from main.

The process has libh2x.so (and with it the HIP runtime, not initialised), the CPU oracle and
its OpenMP team loaded, and leaves through exit handlers and static destructors, which is
what this test is about; it also checks that the host headers keep no object of static
storage duration that would free device memory in its destructor."""
import os
import re
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
EXE = os.path.join(HERE, "cpp", "build", "test_h2_frontend")
HEADERS = os.path.join(ROOT, "dihydrogen_amd", "host", "include")


def test_front_end_host_arms_return_from_main():
    assert os.path.exists(EXE), f"{EXE} is missing: run `make -C tests/cpp`"
    for _ in range(3):
        r = subprocess.run([EXE, "--host-only"], capture_output=True, text=True, timeout=60)
        assert r.returncode == 0, f"exit status {r.returncode}\n{r.stdout[-2000:]}{r.stderr[-2000:]}"
        assert r.stdout.rstrip().endswith("test_h2_frontend: host-only ok")


def test_no_static_object_owns_device_memory():
    owners = r"(Memory\s*<|Workspace\b|Tensor\s*<|ShufflePlan\b|HaloExchange|Shuffler)"
    pattern = re.compile(r"^\s*(inline\s+)?static\s+(?!constexpr|inline\s+constexpr)[^;(]*" + owners + r"[^;(]*\s+\w+\s*(;|=|\{)")
    offenders = []
    for folder, _, files in os.walk(HEADERS):
        for name in files:
            path = os.path.join(folder, name)
            for number, line in enumerate(open(path), 1):
                if pattern.search(line):
                    offenders.append(f"{path}:{number}: {line.strip()}")
    assert not offenders, "\n".join(offenders)
