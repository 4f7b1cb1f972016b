"""Build the CPU checker (oracle/gsx_oracle.cpp, oracle/fastgs_oracle.cpp) into oracle/libgsx_oracle.so.

Test infrastructure only: nothing in the shipped package imports this.

The reference itself cannot be built here (CUDA 12.8 + glm + LibTorch, gsplat/CMakeLists.txt), so
there is no oracle/_ref build; the checker is the restatement in gsx_oracle.cpp.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRCS = [os.path.join(HERE, "gsx_oracle.cpp"), os.path.join(HERE, "fastgs_oracle.cpp")]
OUT = os.path.join(HERE, "libgsx_oracle.so")
MATH_INC = os.path.join(ROOT, "lichtfeld-studio_amd", "csrc")

# x86-64-v3 = AVX2 + FMA: gsx::fma must be the hardware instruction, and the binary has to run on
# the GPU box's host CPU as well as here, so no -march=native.
FLAGS = ["-O2", "-march=x86-64-v3", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-shared", "-fPIC",
         "-fvisibility=hidden", "-std=c++17", "-Wall", "-Wno-unknown-pragmas"]


def build(force=True):
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= max(
            *[os.path.getmtime(s) for s in SRCS],
            *[os.path.getmtime(os.path.join(MATH_INC, h)) for h in ("gsx_math.h", "gsx_camera.h", "gsx_record.h")]):
        return OUT
    cmd = ["g++", *FLAGS, "-I", MATH_INC, *SRCS, "-o", OUT]
    subprocess.run(cmd, check=True)
    return OUT


def sanitize():
    """The checker's sources and oracle/sanitize_driver.cpp as one executable under AddressSanitizer and
    UndefinedBehaviorSanitizer (host code only), run once: a small training iteration through the C entry points with
    exactly sized heap buffers.  Returns the driver's output; raises when the build or the run fails."""
    exe = os.path.join(HERE, "sanitize_check")
    flags = ["-O1", "-g", "-march=x86-64-v3", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-std=c++17",
             "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
             "-Wno-unknown-pragmas"]
    subprocess.run(["g++", *flags, "-I", MATH_INC, *SRCS, os.path.join(HERE, "sanitize_driver.cpp"), "-o", exe],
                   check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=1", OMP_NUM_THREADS="4")
    r = subprocess.run([exe], capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"sanitize_check failed (exit {r.returncode}):\n{r.stdout}\n{r.stderr}")
    return r.stdout.strip()


if __name__ == "__main__":
    if "--sanitize" in sys.argv:
        print(sanitize())
    else:
        print(build(force="--if-stale" not in sys.argv))
