"""Build recipe for libflowwalker_hip.so and the flowwalker command-line tools (gfx950 only).

Run as a script (`python flowwalker-artifact_amd/build.py`) or call build_all().  hipcc cross-compiles
for gfx950 without a GPU present.  Outputs stay in-tree under flowwalker-artifact_amd/lib and bin.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIBDIR = os.path.join(PKG, "lib")
BINDIR = os.path.join(PKG, "bin")
OBJDIR = os.path.join(PKG, "build")
LIB = os.path.join(LIBDIR, "libflowwalker_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off / -fno-fast-math: the sampler's f32 products and sums must round exactly as written.
# packed-fp32 code generation is switched off for this target.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]

KERNEL_SOURCES = ["fw_walk_kernel.hip", "fw_ref_walk.hip", "fw_sampler_baselines.hip", "fw_api.hip", "fw_gen.hip", "fw_csr_io.hip"]
HOST_TOOLS = {"flowwalker": ["flowwalker_main.cpp"], "fw_gen": ["fw_gen_main.cpp"], "fw_convert": ["fw_convert_main.cpp"],
              "fw_sampler_bench": ["fw_sampler_bench_main.cpp"]}


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; that line is harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_library():
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    objs = [os.path.join(OBJDIR, s.replace(".hip", ".o")) for s in KERNEL_SOURCES]

    def compile_one(pair):
        src, obj = pair
        _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(compile_one, zip(KERNEL_SOURCES, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def build_tools():
    os.makedirs(BINDIR, exist_ok=True)
    built = []
    for name, srcs in HOST_TOOLS.items():
        paths = [os.path.join(HOST, s) for s in srcs]
        if not all(os.path.exists(p) for p in paths):
            continue
        out = os.path.join(BINDIR, name)
        _run(["g++", "-O2", "-std=c++17", "-Wall", "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-o", out]
             + paths + ["-L" + LIBDIR, "-lflowwalker_hip", "-Wl,-rpath,$ORIGIN/../lib"])
        built.append(out)
    return built


def build_oracle():
    """The CPU oracle is test infrastructure; building the checker is not using it."""
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "-B"])
    return os.path.join(ROOT, "oracle", "libfw_oracle.so")


def build_all():
    lib = build_library()
    tools = build_tools()
    orc = build_oracle()
    return [lib] + tools + [orc]


if __name__ == "__main__":
    for p in build_all():
        print("built", os.path.relpath(p, ROOT))
    sys.exit(0)
