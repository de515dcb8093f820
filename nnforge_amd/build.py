"""Build recipe: compiles the gfx950 library (hipcc) and the host-side C++ backend (g++) in-tree."""

import os
import shutil
import subprocess

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PACKAGE_DIR)
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")

HIP_LIBRARY = os.path.join(PACKAGE_DIR, "libnnforge_hip.so")
HIP_SOURCES = ["nnf_chain.hip", "nnf_softmax.hip", "nnf_pool.hip", "nnf_max.hip", "nnf_concat.hip", "nnf_stat.hip", "nnf_capi.hip"]

# -ffp-contract=off: every fp32 operation of the layer formulas rounds once, as the reference's
#   source states them. -packed-fp32-ops is switched off as a target feature (hipcc only).
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _run(cmd, cwd=None):
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def hipcc_path():
    for candidate in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc not found: the gfx950 library cannot be built")


def build_hip_library(verbose=False):
    """Compiles nnforge_amd/csrc/*.hip into nnforge_amd/libnnforge_hip.so (cross-compiles without a GPU): one
    object per source, a few sources at a time, then one link."""
    import concurrent.futures
    import tempfile

    hipcc = hipcc_path()
    compile_flags = [f for f in HIP_FLAGS if f != "-shared"] + ["-c"]
    with tempfile.TemporaryDirectory(prefix="nnforge_hip_build_") as tmp_dir:
        def compile_one(source):
            obj = os.path.join(tmp_dir, os.path.splitext(source)[0] + ".o")
            return obj, _run([hipcc] + compile_flags + ["-o", obj, os.path.join(CSRC_DIR, source)])

        with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
            results = list(pool.map(compile_one, HIP_SOURCES))
        tmp = HIP_LIBRARY + ".tmp"
        out = "".join(text for _, text in results)
        out += _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden", "-o", tmp] + [obj for obj, _ in results])
    os.replace(tmp, HIP_LIBRARY)
    if verbose and out.strip():
        print(out)
    return HIP_LIBRARY


HOST_DIR = os.path.join(PACKAGE_DIR, "host")
BACKEND_LIBRARY = os.path.join(PACKAGE_DIR, "libnnforge_hip_backend.so")
BACKEND_SOURCES = ["core.cpp", "layers.cpp", "schema.cpp", "propagation.cpp", "data_streams.cpp", "hip_testers.cpp",
                   "forward_propagation_hip.cpp", "backend_capi.cpp"]
# default symbol visibility: the C++ classes are the library's interface
BACKEND_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Wno-unused-parameter"]

USAGE_PROGRAM = os.path.join(REPO_ROOT, "tests", "cpp", "backend_usage")


def build_backend_library(verbose=False):
    """Compiles the host-side C++ backend (g++, no HIP headers) into libnnforge_hip_backend.so,
    linked against libnnforge_hip.so in the same directory."""
    if not os.path.exists(HIP_LIBRARY):
        raise RuntimeError("build the HIP library first: %s is missing" % HIP_LIBRARY)
    tmp = BACKEND_LIBRARY + ".tmp"
    cmd = (["g++"] + BACKEND_FLAGS + ["-I", os.path.join(REPO_ROOT, "include"), "-o", tmp]
           + [os.path.join(HOST_DIR, s) for s in BACKEND_SOURCES]
           + ["-L", PACKAGE_DIR, "-lnnforge_hip", "-Wl,-rpath,$ORIGIN"])
    out = _run(cmd)
    os.replace(tmp, BACKEND_LIBRARY)
    if verbose and out.strip():
        print(out)
    return BACKEND_LIBRARY


def build_usage_program(verbose=False):
    """Compiles tests/cpp/backend_usage.cpp: a C++ program that uses the backend the way an nnForge
    application uses one (run by the GPU tests)."""
    tmp = USAGE_PROGRAM + ".tmp"
    cmd = ["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-Wall", "-I", os.path.join(REPO_ROOT, "include"), "-o", tmp,
           USAGE_PROGRAM + ".cpp", "-L", PACKAGE_DIR, "-lnnforge_hip_backend", "-lnnforge_hip",
           "-Wl,-rpath,$ORIGIN/../../nnforge_amd"]
    out = _run(cmd)
    os.replace(tmp, USAGE_PROGRAM)
    if verbose and out.strip():
        print(out)
    return USAGE_PROGRAM


SANITIZED_PROGRAM_SOURCE = os.path.join(REPO_ROOT, "tests", "cpp", "host_sanitized.cpp")


def build_sanitized_host_program(output_path):
    """Compiles the backend's host sources together with tests/cpp/host_sanitized.cpp under AddressSanitizer and
    UndefinedBehaviorSanitizer (host code only: the program never touches a device). Used by the CPU tests."""
    if not os.path.exists(HIP_LIBRARY):
        raise RuntimeError("build the HIP library first: %s is missing" % HIP_LIBRARY)
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-Wall",
           "-I", os.path.join(REPO_ROOT, "include"), "-o", output_path, SANITIZED_PROGRAM_SOURCE]
    cmd += [os.path.join(HOST_DIR, s) for s in BACKEND_SOURCES]
    cmd += ["-L", PACKAGE_DIR, "-lnnforge_hip", "-Wl,-rpath," + PACKAGE_DIR]
    _run(cmd)
    return output_path


def build_all(verbose=False):
    built = [build_hip_library(verbose), build_backend_library(verbose), build_usage_program(verbose)]
    return built


if __name__ == "__main__":
    for path in build_all(verbose=True):
        print("built", path)
