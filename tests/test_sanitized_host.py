"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer, on the CPU only.

Two programs are built with g++ -fsanitize=address,undefined and run here:

* tests/sanitize/planner_bounds.cpp: the multi-tensor planner (csrc/gm_planner.cpp) laid out over random
  lists (tensors of 0 to 2^28 elements, misaligned views, short buffers, both segments, every chunk size,
  lane width and workgroup size the library can launch), every descriptor walked lane by lane through the
  same lane_share function the kernels index with: chunks tile each tensor exactly once, every descriptor
  stays inside its allocation, grid x slice covers the chunk, grouped accesses are aligned.  Small lists are
  really read and written through the descriptors, in exact-length heap blocks.
  Perturbations tried while writing it, each caught: a chunk count one too long for tensors whose tail is
  257 elements (check 2 fails), and lane_share ignoring the alignment flags (check 4 fails).
* tests/sanitize/host_mirror_driver.cpp: every entry point of the host-side mirror of the Go packages
  (go-metal_amd/host/*.cpp) on a CPU stand-in of the device ABI, including malformed and truncated state
  documents, out-of-range counts and non-finite state.

Neither program is ever run on the GPU box (not marked gpu); the sanitizers watch host code only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "sanitize")
BUILD = os.path.join(SRC, "_build")
FLAGS = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
         "-static-libasan", "-static-libubsan", "-Wall", "-I", os.path.join(ROOT, "include")]
PLANNER = os.path.join(ROOT, "go-metal_amd", "csrc", "gm_planner.cpp")


def build(name, sources, extra=()):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++ on this machine")
    os.makedirs(BUILD, exist_ok=True)
    out = os.path.join(BUILD, name + ".bin")
    import glob
    headers = glob.glob(os.path.join(ROOT, "go-metal_amd", "*", "*.hpp")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    newest = max(os.path.getmtime(s) for s in list(sources) + headers)
    if not os.path.exists(out) or os.path.getmtime(out) < newest:
        subprocess.check_call([gxx] + FLAGS + list(extra) + list(sources) + ["-o", out, "-lpthread"])
    return out


def run(binary, *args):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([binary] + list(args), env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=600)
    text = proc.stdout
    assert proc.returncode == 0, text[-4000:]
    assert "AddressSanitizer" not in text and "runtime error" not in text and "LeakSanitizer" not in text, text[-4000:]
    return text


def test_planner_bounds_under_sanitizers():
    binary = build("planner_bounds", [os.path.join(SRC, "planner_bounds.cpp"), PLANNER], extra=["-O2"])
    text = run(binary, "90", "0x6d657461")
    assert ", 0 failures" in text, text[-2000:]


def test_host_mirror_under_sanitizers():
    import glob
    sources = [os.path.join(SRC, "host_mirror_driver.cpp"), os.path.join(SRC, "cpu_device.cpp"), PLANNER]
    sources += sorted(glob.glob(os.path.join(ROOT, "go-metal_amd", "host", "*.cpp")))
    text = run(build("host_mirror_driver", sources))
    assert "host_mirror_driver: 0 failures" in text, text[-2000:]
