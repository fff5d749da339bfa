"""Runs the C++ test programs of the front end and the lowering.

tests/cpp/test_frontend.cpp       expression nodes, call-site checks, pipeline legality, grid units
tests/cpp/test_cpu_lowering.cpp   programs lowered to host C++ by the Runner and executed
tests/cpp/test_gpu_lowering.cpp   programs lowered to one HIP kernel for gfx950; here they are
                                  generated and compiled with hiprtc only (no GPU), the gpu-marked
                                  test runs them on the device

Each program runs ONCE per session; every CASE(...) in its source becomes one pytest case that
looks its line up in the program's output.  The cases restate what the reference's own tests
specify (the reference files and lines are cited next to each case in the C++ sources).
"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
BIN = os.path.join(CPP, "bin")


def case_names(program):
    with open(os.path.join(CPP, program + ".cpp")) as f:
        return re.findall(r'^CASE\("([^"]+)"\)', f.read(), flags=re.M)


def run_program(program, tmp, extra_env=None):
    exe = os.path.join(BIN, program)
    if not os.path.exists(exe):
        pytest.fail("%s is missing: run `python gern_amd/build.py`" % exe)
    env = dict(os.environ)
    env.update({"GERN_TEST_LIBRARY": os.path.join(CPP, "library"), "GERN_TEST_PACKAGE": os.path.join(ROOT, "gern_amd"),
                "GERN_TEST_TMP": str(tmp)})
    env.update(extra_env or {})
    p = subprocess.run([exe], cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    results = {}
    for line in p.stdout.splitlines():
        m = re.match(r"\[\s*(ok|FAIL)\s*\] ([^:]+)(?:: (.*))?$", line)
        if m:
            results[m.group(2).strip()] = (m.group(1) == "ok", m.group(3) or "")
    return p.returncode, results, p.stdout


def check_case(run, name):
    rc, results, out = run
    assert name in results, "case %s did not run (exit code %d):\n%s" % (name, rc, out[-4000:])
    ok, msg = results[name]
    assert ok, msg


@pytest.fixture(scope="session")
def frontend_run(tmp_path_factory):
    return run_program("test_frontend", tmp_path_factory.mktemp("frontend"))


@pytest.fixture(scope="session")
def cpu_lowering_run(tmp_path_factory):
    return run_program("test_cpu_lowering", tmp_path_factory.mktemp("cpu_lowering"))


@pytest.fixture(scope="session")
def gpu_compile_run(tmp_path_factory):
    return run_program("test_gpu_lowering", tmp_path_factory.mktemp("gpu_compile"), {"GERN_TEST_COMPILE_ONLY": "1"})


@pytest.fixture(scope="session")
def gpu_lowering_run(tmp_path_factory):
    return run_program("test_gpu_lowering", tmp_path_factory.mktemp("gpu_lowering"), {"GERN_TEST_COMPILE_ONLY": "0"})


@pytest.mark.parametrize("name", case_names("test_frontend"))
def test_frontend(frontend_run, name):
    check_case(frontend_run, name)


@pytest.mark.parametrize("name", case_names("test_cpu_lowering"))
def test_cpu_lowering(cpu_lowering_run, name):
    check_case(cpu_lowering_run, name)


@pytest.mark.parametrize("name", case_names("test_gpu_lowering"))
def test_gpu_lowering_compiles_for_gfx950(gpu_compile_run, name):
    check_case(gpu_compile_run, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", case_names("test_gpu_lowering"))
def test_gpu_lowering_runs(gpu_lowering_run, name):
    check_case(gpu_lowering_run, name)
