"""Compiles the HIP sources under clusternet_amd/csrc into clusternet_amd/libcnhip.so (gfx950).

Usage: python -m clusternet_amd.build [--facade] | --host-asan
The library is built in-tree so that it travels with the source tree; nothing is installed.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
FACADE = os.path.join(HERE, "facade")
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libcnhip.so")
FACADE_LIB = os.path.join(HERE, "libclusternet.so")

ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions.
# -ffp-contract=off: the codec must round every operation exactly like the reference's kernels.
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument",
             # the direct-to-LDS loads set M0 inside their inline assembly and say so
             "-Wno-inline-asm"]
SOURCES = ["cn_runtime.cpp", "cn_encode_lut.cpp", "cn_gemm_plan.cpp", "cn_codec.hip", "cn_gemm.hip", "cn_gemm_w8_rows.hip", "cn_gemm_small.hip", "cn_gemm_c8c8.hip",
           "cn_layers.hip", "cn_update.hip", "cn_sparse.hip"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose=False):
    objs = []
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(objdir, src + ".o")
        cmd = [hipcc()] + HIP_FLAGS + ["-c", path, "-o", obj]
        out = _run(cmd)
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    _run([hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def build_facade(verbose=False):
    """The C++ ClusterNet / Matrix layer over the C-ABI, plus its test binary."""
    src = os.path.join(FACADE, "clusterNet.cpp")
    if not os.path.exists(src):
        return None
    cxx = shutil.which("g++") or "g++"
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + FACADE]
    _run([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-o", FACADE_LIB, src,
          os.path.join(FACADE, "basicOps.cpp"), os.path.join(FACADE, "util.cpp")] + inc +
         ["-L" + HERE, "-lcnhip", "-Wl,-rpath,$ORIGIN"])
    test_src = os.path.join(ROOT, "tests", "cpp", "facade_test.cpp")
    oracle_dir = os.path.join(ROOT, "oracle")
    if os.path.exists(test_src) and os.path.exists(os.path.join(oracle_dir, "liboracle.so")):
        # the test program (not the library) links the CPU checker to compare codes bit for bit
        _run([cxx, "-O2", "-std=c++17", "-Wall", "-o", os.path.join(ROOT, "tests", "cpp", "facade_test"),
              test_src] + inc + ["-L" + HERE, "-lclusternet", "-lcnhip", "-L" + oracle_dir, "-loracle",
                                 "-Wl,-rpath,$ORIGIN/../../clusternet_amd", "-Wl,-rpath,$ORIGIN/../../oracle"])
    return FACADE_LIB


def host_asan(verbose=True):
    """CPU only: the host code of the library and the CPU checker under AddressSanitizer + UndefinedBehavior-
    Sanitizer, and the CPU tests that exercise them run once against those builds.  Device code is compiled as
    usual (GPU sanitizers are not used); nothing here needs or touches a GPU."""
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
           "-fno-sanitize-recover=undefined", "-Xarch_host", "-fno-omit-frame-pointer", "-g"]
    objdir = os.path.join(HERE, "build", "asan")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    flags = [f for f in HIP_FLAGS if f != "-O3"] + ["-O1"]
    for src in SOURCES:
        obj = os.path.join(objdir, src + ".o")
        _run([hipcc()] + flags + san + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    lib = os.path.join(objdir, "libcnhip.so")
    _run([hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-fsanitize=address", "-fsanitize=undefined", "-shared-libasan",
          "-o", lib] + objs)
    facade = os.path.join(objdir, "libclusternet.so")
    _run([hipcc(), "-x", "c++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-fsanitize=address", "-fsanitize=undefined",
          "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-shared-libasan", "-o", facade,
          os.path.join(FACADE, "clusterNet.cpp"), os.path.join(FACADE, "basicOps.cpp"), os.path.join(FACADE, "util.cpp"),
          "-I" + os.path.join(ROOT, "include"), "-I" + FACADE, "-L" + objdir, "-lcnhip", "-Wl,-rpath,$ORIGIN"])
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-s", "asan"])
    clang_rt = subprocess.run([hipcc(), "-print-file-name=libclang_rt.asan-x86_64.so"], stdout=subprocess.PIPE, text=True).stdout.strip()
    gcc_rt = subprocess.run(["gcc", "-print-file-name=libasan.so"], stdout=subprocess.PIPE, text=True).stdout.strip()
    runs = (
        # the checker's own tests against the sanitized checker
        (gcc_rt, {"CN_ORACLE_LIB": os.path.join(ROOT, "oracle", "_asan", "liboracle.so")},
         ["tests/test_oracle_codec.py", "tests/test_oracle_gemm.py", "tests/test_oracle_sparse.py", "tests/test_oracle_update.py",
          "tests/test_codec_vectors.py"]),
        # the library's host logic (planner, encoder table, status codes, exports) and the facade's reader of the
        # reference's HDF5 files against the sanitized builds
        (clang_rt, {"CNHIP_LIB": lib, "CN_FACADE_LIB": facade, "CNHIP_NO_TORCH": "1"},
         ["tests/test_host_logic.py", "tests/test_hdf5_reader.py"]),
    )
    for runtime, extra, tests in runs:
        env = dict(os.environ)
        env.update(extra)
        before = env.get("LD_PRELOAD", "")
        env["LD_PRELOAD"] = runtime + (":" + before if before else "")  # the sanitizer runtime has to come first
        env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"  # the interpreter itself leaks by design
        env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
        cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + tests
        if verbose:
            print("LD_PRELOAD=%s %s %s" % (runtime, " ".join("%s=%s" % kv for kv in extra.items()), " ".join(cmd)), flush=True)
        subprocess.check_call(cmd, cwd=ROOT, env=env)
    return lib


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if argv == ["--host-asan"]:
        print(host_asan())
        return
    print(build_library(verbose=True))
    if "--facade" in argv:
        print(build_facade(verbose=True))
    if "--host-asan" in argv:
        print(host_asan())


if __name__ == "__main__":
    main()
