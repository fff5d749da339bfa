"""Builds the native libraries of the package, in-tree.

    libgern_hip.so        C ABI over hiprtc / hipModule (include/gern_hip.h)
    libgern.so            Gern's C++ front end, code generator and Runner
    libgern_pipelines.so  C ABI over the fused pipelines (include/gern_pipelines.h)

and ahead-of-time compiles every gernel header for gfx950 as a build check
(the kernels that actually run are instantiated by hiprtc from generated code).
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

CXXFLAGS = ["-std=c++20", "-O2", "-fPIC", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
            "-I" + os.path.join(HERE, "include"), "-I" + os.path.join(HERE, "include", "gern"),
            "-I" + HERE, "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROCM, "include")]
# Packed-FP32 instructions are kept out of every kernel.
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
            "-packed-fp32-ops", "-I" + HERE]


def run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_native():
    rpath = "-Wl,-rpath,$ORIGIN:" + os.path.join(ROCM, "lib")
    run(["g++"] + CXXFLAGS + ["-shared", os.path.join(HERE, "csrc", "gern_hip.cpp"),
                               "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lhiprtc", rpath,
                               "-o", os.path.join(HERE, "libgern_hip.so")])
    srcs = sorted(glob.glob(os.path.join(HERE, "src", "*.cpp")))
    run(["g++"] + CXXFLAGS + ["-shared"] + srcs + ["-L" + HERE, "-lgern_hip", "-ldl", rpath,
                                                  "-o", os.path.join(HERE, "libgern.so")])
    # The one file of the library with device code of its own (a device array): hipcc, linked in as an object.
    no_alloc = os.path.join(HERE, "csrc", "qk_no_alloc.o")
    run([os.path.join(ROCM, "bin", "hipcc")] + HIPFLAGS + ["-fPIC", "-I" + os.path.join(ROOT, "include"), "-c",
                                                          os.path.join(HERE, "csrc", "qk_no_alloc.hip"), "-o", no_alloc])
    run(["g++"] + CXXFLAGS + ["-shared", os.path.join(HERE, "csrc", "pipelines.cpp"), no_alloc, "-L" + HERE, "-lgern",
                               "-lgern_hip", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-ldl", rpath, "-o",
                               os.path.join(HERE, "libgern_pipelines.so")])


def build_gernel_check():
    """hipcc cross-compiles an instantiation of every gernel for gfx950."""
    src = os.path.join(HERE, "csrc", "gernel_check.hip")
    out = os.path.join(HERE, "csrc", "gernel_check.o")
    run([os.path.join(ROCM, "bin", "hipcc")] + HIPFLAGS + ["-c", "--cuda-device-only", src, "-o", out])


def build_cpp_tests():
    """The C++ front-end / lowering test programs (tests/cpp/*.cpp -> tests/cpp/bin/)."""
    tdir = os.path.join(ROOT, "tests", "cpp")
    bindir = os.path.join(tdir, "bin")
    os.makedirs(bindir, exist_ok=True)
    rpath = "-Wl,-rpath,$ORIGIN/../../../gern_amd:" + os.path.join(ROCM, "lib")
    for src in sorted(glob.glob(os.path.join(tdir, "test_*.cpp"))):
        exe = os.path.join(bindir, os.path.splitext(os.path.basename(src))[0])
        run(["g++", "-std=c++20", "-O1", "-I" + tdir] + [f for f in CXXFLAGS if f.startswith("-I") or f.startswith("-D")] +
            [src, "-L" + HERE, "-lgern", "-lgern_hip", rpath, "-o", exe])


def build_examples():
    """examples/*.c: hosts in plain C99 over the C ABI (examples/bin/)."""
    edir = os.path.join(ROOT, "examples")
    bindir = os.path.join(edir, "bin")
    os.makedirs(bindir, exist_ok=True)
    rpath = "-Wl,-rpath,$ORIGIN/../../gern_amd:" + os.path.join(ROCM, "lib")
    for src in sorted(glob.glob(os.path.join(edir, "*.c"))):
        exe = os.path.join(bindir, os.path.splitext(os.path.basename(src))[0])
        run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O2", "-ffp-contract=off",
             "-I" + os.path.join(ROOT, "include"), src, "-L" + HERE, "-lgern_pipelines", "-lgern", "-lgern_hip", rpath,
             "-o", exe])


def build_all():
    build_native()
    build_gernel_check()
    build_cpp_tests()
    build_examples()


def sanitize_check():
    """Host-side AddressSanitizer + UBSan run of the front end, the lowering and
    the pipelines' code generation, as the reference's CI does for its CPU tests
    (.github/workflows/main.yml:34-46).  Everything goes to build/sanitize/; the
    in-tree libraries are left alone.  Device code is not instrumented."""
    out = os.path.join(ROOT, "build", "sanitize")
    os.makedirs(out, exist_ok=True)
    san = ["-fsanitize=address,undefined", "-fno-omit-frame-pointer", "-g", "-O1"]
    flags = [f for f in CXXFLAGS if f != "-O2"] + san
    rpath = "-Wl,-rpath," + out + ":" + os.path.join(ROCM, "lib")
    run(["g++"] + flags + ["-shared", os.path.join(HERE, "csrc", "gern_hip.cpp"), "-L" + os.path.join(ROCM, "lib"),
                            "-lamdhip64", "-lhiprtc", rpath, "-o", os.path.join(out, "libgern_hip.so")])
    srcs = sorted(glob.glob(os.path.join(HERE, "src", "*.cpp")))
    run(["g++"] + flags + ["-shared"] + srcs + ["-L" + out, "-lgern_hip", "-ldl", rpath, "-o", os.path.join(out, "libgern.so")])
    run(["g++"] + flags + ["-shared", os.path.join(HERE, "csrc", "pipelines.cpp"), "-L" + out, "-lgern", "-lgern_hip", "-ldl",
                            rpath, "-o", os.path.join(out, "libgern_pipelines.so")])
    tdir = os.path.join(ROOT, "tests", "cpp")
    programs = []
    for src in sorted(glob.glob(os.path.join(tdir, "test_*.cpp"))) + [os.path.join(HERE, "csrc", "sanitize_pipelines.cpp")]:
        exe = os.path.join(out, os.path.splitext(os.path.basename(src))[0])
        run(["g++"] + flags + ["-I" + tdir, src, "-L" + out, "-lgern_pipelines", "-lgern", "-lgern_hip", rpath, "-o", exe])
        programs.append(exe)
    env = dict(os.environ)
    env.update({"GERN_TEST_LIBRARY": os.path.join(tdir, "library"), "GERN_TEST_PACKAGE": HERE,
                "GERN_TEST_TMP": out, "GERN_TEST_COMPILE_ONLY": "1", "GERN_PACKAGE_DIR": HERE,
                # libraries that other tools preload come before the sanitizer runtime; the JIT-compiled
                # host functions of the CPU lowering are not instrumented; hiprtc's own allocations are not ours
                "ASAN_OPTIONS": "verify_asan_link_order=0:detect_leaks=0:abort_on_error=0",
                "UBSAN_OPTIONS": "print_stacktrace=1:halt_on_error=1"})
    failed = []
    for exe in programs:
        print("+ " + exe, flush=True)
        p = subprocess.run([exe], cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        bad = p.returncode != 0 or "ERROR: AddressSanitizer" in p.stdout or "runtime error:" in p.stdout
        print(p.stdout[-3000:] if bad else "\n".join(p.stdout.splitlines()[-2:]))
        if bad:
            failed.append(os.path.basename(exe))
    if failed:
        raise SystemExit("sanitizer run failed: " + ", ".join(failed))
    print("sanitizer run clean: " + ", ".join(os.path.basename(e) for e in programs))


if __name__ == "__main__":
    if "--sanitize" in sys.argv[1:]:
        sanitize_check()
    else:
        build_all()
    print("build ok")
