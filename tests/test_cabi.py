"""The C ABI libraries load and export every symbol the headers declare, and
the pipelines generate HIP that compiles for gfx950.  No GPU, no compute."""
import ctypes as C
import os
import re

import pytest

import gern_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gern_[a-z0-9_]+)\s*\(", text)))


def test_runtime_abi_exports_every_declared_symbol():
    hip = gern_amd.hip_lib()
    names = _declared("gern_hip.h")
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(hip, n)]
    assert not missing, missing


def test_pipeline_abi_exports_every_declared_symbol():
    pipes = gern_amd.pipelines_lib()
    names = _declared("gern_pipelines.h")
    assert len(names) >= 10
    missing = [n for n in names if not hasattr(pipes, n)]
    assert not missing, missing


def test_blur_chain_generates_fused_kernel_with_inferred_halos():
    p = gern_amd.BlurChain("xyx", tile_rows=8, tile_cols=252, flags=gern_amd.COMPILE_ONLY)
    src = p.source
    assert p.kernel_name.endswith("<252, 8, 3, 64>")
    assert src.count("__global__") == 1 and "__launch_bounds__(64)" in src
    # input tile: (row + 2) x (col + 4); first temporary (row + 2) x (col + 2)
    assert "load_wave<((row + stride) - 1), ((((col + stride) - 1) + stride) - 1)>" in src
    assert "store_wave(" in src
    assert "allocate_wave_tile<((row + stride) - 1), ((col + stride) - 1)>" in src
    assert "allocate_wave_tile<row, ((col + stride) - 1)>" in src
    assert src.index("blur_x<stride>") < src.index("blur_y<stride>") < src.rindex("blur_x<stride>")
    assert "gern_block_x" in src  # XCD-aware workgroup order


def test_blur_chain_line_aligned_windows_by_default():
    # tiles of 224 columns (seven 128-byte lines) leave the 28 spare columns that
    # windows moved to line boundaries need: the default schedule
    p = gern_amd.BlurChain("xyx", tile_rows=6, flags=gern_amd.COMPILE_ONLY)
    assert p.kernel_name.endswith("<224, 6, 3, 64>")
    assert "load_wave_wide<((row + stride) - 1), ((((col + stride) - 1) + stride) - 1)>" in p.source
    assert "store_wave_lines(" in p.source
    # three x stages of five taps leave room for 192 columns only
    assert gern_amd.BlurChain("xxx", stride=5, flags=gern_amd.COMPILE_ONLY).kernel_name.split("<")[1].startswith("192,")
    # asked not to, or with a tile that is not whole lines wide, a tile stores its own columns
    for kw in ({"flags": gern_amd.COMPILE_ONLY | gern_amd.BLUR_PLAIN_STORES}, {"tile_cols": 228, "flags": gern_amd.COMPILE_ONLY},
               {"tile_cols": 240, "flags": gern_amd.COMPILE_ONLY}):
        src = gern_amd.BlurChain("xyx", **kw).source
        assert "store_wave(" in src and "store_wave_lines" not in src and "load_wave_wide" not in src


def test_blur_chain_wavefront_mapping_and_plain_order():
    p = gern_amd.BlurChain("xy", tile_rows=4, waves_per_block=4, flags=gern_amd.COMPILE_ONLY | gern_amd.NO_XCD_REMAP)
    src = p.source
    assert "(threadIdx.x / 64)" in src and "__launch_bounds__(256)" in src
    assert "gern_block_x" not in src and "blockIdx.x" in src


@pytest.mark.parametrize("ncol,load,threads", [(4096, "load_block8", 512), (2048, "load_block4", 256),
                                               (1024, "load_block2", 128), (1000, "load_wave", 64),
                                               (512, "load_wave", 64)])
def test_softmax_generates_one_pass_kernel(ncol, load, threads):
    # wide rows that divide into 256-column chunks are spread over the
    # wavefronts of a workgroup; the others stay in one wavefront
    p = gern_amd.Softmax(ncol, flags=gern_amd.COMPILE_ONLY)
    src = p.source
    for fn in ("max_row", "subtract_vec", "exp_matrix", "sum_row", "divide_vec"):
        assert "gernels::" + fn in src
    assert src.count(load) == 1  # the row is read once
    assert "__launch_bounds__(%d)" % threads in src


def test_bad_arguments_are_errors():
    with pytest.raises(gern_amd.GernError, match="pattern"):
        gern_amd.BlurChain("xz", flags=gern_amd.COMPILE_ONLY)
    with pytest.raises(gern_amd.GernError, match="tile_cols"):
        gern_amd.BlurChain("xyx", tile_cols=256, flags=gern_amd.COMPILE_ONLY)
    with pytest.raises(gern_amd.GernError):
        gern_amd.Softmax(100000, flags=gern_amd.COMPILE_ONLY)


def test_compile_only_pipeline_refuses_to_run():
    p = gern_amd.Softmax(256, flags=gern_amd.COMPILE_ONLY)
    rc = gern_amd.pipelines_lib().gern_softmax_run(p.h, C.c_void_p(16), C.c_void_p(16), 1, 256, None)
    assert rc != 0


def test_runtime_reports_compile_errors():
    hip = gern_amd.hip_lib()
    src = b"__global__ void broken( { }"
    names = (C.c_char_p * 1)(b"broken")
    size = C.c_size_t()
    rc = hip.gern_hip_compile_only(src, names, 1, None, 0, b"gfx950", C.byref(size))
    assert rc == 1
    buf = C.create_string_buffer(4096)
    hip.gern_hip_last_error(buf, 4096)
    assert b"error" in buf.value


def _kernel_notes(tmp_path, make_pipeline):
    """Compiles a pipeline with the run-time compiler (no GPU needed) and reads the resource
    usage the compiler recorded in the code object."""
    import shutil
    import subprocess
    readelf = shutil.which("llvm-readelf") or "/opt/rocm/llvm/bin/llvm-readelf"
    if not os.path.exists(readelf):
        pytest.skip("llvm-readelf not available")
    os.environ["GERN_HIP_KEEP_DIR"] = str(tmp_path)
    try:
        make_pipeline()
    finally:
        del os.environ["GERN_HIP_KEEP_DIR"]
    kernels = []
    for f in sorted(tmp_path.glob("*.hsaco")):
        out = subprocess.run([readelf, "--notes", str(f)], stdout=subprocess.PIPE, text=True, check=True).stdout
        cur = {}
        for line in out.splitlines():
            line = line.strip().lstrip("- ")
            for key in (".name", ".vgpr_count", ".agpr_count", ".vgpr_spill_count", ".private_segment_fixed_size"):
                if line.startswith(key + ":"):
                    val = line.split(":", 1)[1].strip()
                    cur[key] = val if key == ".name" else int(val)
            if ".name" in cur and ".vgpr_spill_count" in cur and ".private_segment_fixed_size" in cur and ".vgpr_count" in cur:
                kernels.append(cur)
                cur = {}
    assert kernels, "no kernel metadata found"
    return kernels


@pytest.mark.parametrize("name,make", [
    ("blur_xyx", lambda: gern_amd.BlurChain("xyx", tile_rows=4, flags=gern_amd.COMPILE_ONLY)),
    ("softmax_4096", lambda: gern_amd.Softmax(4096, flags=gern_amd.COMPILE_ONLY)),
    ("gemm_f32", lambda: gern_amd.Gemm("f32", overwrite=True, flags=gern_amd.COMPILE_ONLY)),
    ("gemm_f32_accumulate", lambda: gern_amd.Gemm("f32", flags=gern_amd.COMPILE_ONLY)),
    ("gemm_bf16", lambda: gern_amd.Gemm("bf16", overwrite=True, flags=gern_amd.COMPILE_ONLY)),
    ("gemm_bf16_accumulate", lambda: gern_amd.Gemm("bf16", flags=gern_amd.COMPILE_ONLY)),
    ("qk_softmax_4096", lambda: gern_amd.QKSoftmax(128, 4096, flags=gern_amd.COMPILE_ONLY)),
    ("qk_softmax_4096_row_blocks", lambda: gern_amd.QKSoftmax(128, 4096, flags=gern_amd.COMPILE_ONLY | gern_amd.QK_ROW_BLOCKS)),
])
def test_headline_kernels_use_no_scratch_memory(tmp_path, name, make):
    # A kernel that spills registers, or keeps an array on the stack, writes to
    # HBM on every iteration: once, that made the bf16 GEMM move 11x its result.
    for k in _kernel_notes(tmp_path, make):
        assert k[".vgpr_spill_count"] == 0, (name, k)
        assert k[".private_segment_fixed_size"] == 0, (name, k)


@pytest.mark.parametrize("variant", ["bf16", "f32"])
def test_whole_tile_gemm_reads_one_stage_while_the_other_fills(tmp_path, variant):
    # The whole-tile GEMMs load stage k+1 straight into LDS while they read
    # stage k.  The compiler keeps the two apart only while every LDS address is
    # a short pointer chain from its own static array; when it loses track it
    # waits for all outstanding loads (a bare "s_waitcnt vmcnt(0)") before the
    # first LDS read, which serialises fetch and compute (measured: +8 %).
    import shutil
    import subprocess
    objdump = shutil.which("llvm-objdump") or "/opt/rocm/llvm/bin/llvm-objdump"
    if not os.path.exists(objdump):
        pytest.skip("llvm-objdump not available")
    os.environ["GERN_HIP_KEEP_DIR"] = str(tmp_path)
    try:
        gern_amd.Gemm(variant, overwrite=True, flags=gern_amd.COMPILE_ONLY)
    finally:
        del os.environ["GERN_HIP_KEEP_DIR"]
    checked = 0
    for f in sorted(tmp_path.glob("*.hsaco")):
        text = subprocess.run([objdump, "-d", str(f)], stdout=subprocess.PIPE, text=True, check=True).stdout
        lines = [l.split("//")[0].strip() for l in text.splitlines()]
        to_lds = [i for i, l in enumerate(lines) if l.startswith("buffer_load_dwordx4") and l.endswith(" lds")]
        if not to_lds:
            continue  # the general (ragged) kernel stages through registers
        checked += 1
        first = to_lds[0]
        last = max(i for i, l in enumerate(lines) if l.startswith("v_mfma"))
        bare = [l for l in lines[first:last] if l.startswith("s_waitcnt") and "vmcnt(0)" in l and "lgkmcnt" not in l]
        assert not bare, bare
    assert checked == 1


@pytest.mark.parametrize("variant", ["f32", "bf16"])
def test_gemm_general_only_builds_one_kernel(tmp_path, variant):
    # without the flag a GEMM pipeline holds two kernels (the direct-to-LDS
    # matrix-core one with 512 threads, and the one for every shape); with it,
    # only the latter
    os.environ["GERN_HIP_KEEP_DIR"] = str(tmp_path)
    try:
        g = gern_amd.Gemm(variant, general_only=True, flags=gern_amd.COMPILE_ONLY)
    finally:
        del os.environ["GERN_HIP_KEEP_DIR"]
    assert len(list(tmp_path.glob("*.hsaco"))) == 1
    assert g.kernel_name.split("<")[1].split(",")[0].strip() != "512", g.kernel_name  # <lds bytes, threads, ...>
    both = gern_amd.Gemm(variant, flags=gern_amd.COMPILE_ONLY)
    assert both.kernel_name.split("<")[1].split(",")[0].strip() == "512", both.kernel_name


def test_pipelines_can_be_created_from_several_threads():
    # creation shares only an atomic name counter and per-thread error text
    import threading
    results = {}

    def make(i):
        try:
            p = gern_amd.Softmax(1024 * (i + 1), flags=gern_amd.COMPILE_ONLY) if i % 2 else \
                gern_amd.BlurChain("xy", tile_rows=4 + i, flags=gern_amd.COMPILE_ONLY)
            results[i] = (p.kernel_name, "__global__" in p.source)
        except Exception as e:  # noqa: BLE001
            results[i] = e

    threads = [threading.Thread(target=make, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert len(results) == 4
    for i, r in results.items():
        assert not isinstance(r, Exception), (i, r)
        assert r[1], (i, r)
    assert len({r[0].split("<")[0] for r in results.values()}) == 4  # four distinct generated kernels


def _compile_only(src, names, options):
    hip = gern_amd.hip_lib()
    size = C.c_size_t()
    arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
    opts = (C.c_char_p * len(options))(*[o.encode() for o in options])
    rc = hip.gern_hip_compile_only(src.encode(), arr, len(names), opts, len(options), b"gfx950", C.byref(size))
    return rc, size.value


def test_code_object_cache(tmp_path, monkeypatch):
    # GERN_HIP_CACHE_DIR: the second compile of the same inputs is a cache hit
    # (no compiler run); changing the source, a name expression, an option or
    # the content of an included header is a miss
    import time
    cache = tmp_path / "cache"
    inc = tmp_path / "inc"
    cache.mkdir()
    inc.mkdir()
    (inc / "scale.h").write_text("#define SCALE 2.0f\n")
    src = '#include "scale.h"\ntemplate<int N> __global__ void k(float *p) { p[threadIdx.x] *= SCALE * N; }\n'
    monkeypatch.setenv("GERN_HIP_CACHE_DIR", str(cache))
    opts = ["-I" + str(inc)]

    def entries():
        return sorted(p.name for p in cache.iterdir())

    t0 = time.time()
    rc, size = _compile_only(src, ["k<3>"], opts)
    cold = time.time() - t0
    assert rc == 0 and size > 0 and len(entries()) == 1
    t0 = time.time()
    rc, size2 = _compile_only(src, ["k<3>"], opts)
    warm = time.time() - t0
    assert rc == 0 and size2 == size and len(entries()) == 1
    assert warm < cold / 3, (cold, warm)
    # each change of an input makes a new entry
    assert _compile_only(src, ["k<4>"], opts)[0] == 0 and len(entries()) == 2
    assert _compile_only(src + "// changed\n", ["k<3>"], opts)[0] == 0 and len(entries()) == 3
    assert _compile_only(src, ["k<3>"], opts + ["-DUNUSED=1"])[0] == 0 and len(entries()) == 4
    (inc / "scale.h").write_text("#define SCALE 3.0f\n")
    assert _compile_only(src, ["k<3>"], opts)[0] == 0 and len(entries()) == 5
    # a damaged entry is a miss and gets rewritten
    first = cache / entries()[0]
    for p in cache.iterdir():
        p.write_bytes(b"gernhip1\nbroken")
    assert _compile_only(src, ["k<3>"], opts)[0] == 0
    assert any(p.stat().st_size > 100 for p in cache.iterdir())
    # compile errors are not cached and still reported
    before = entries()
    rc, _ = _compile_only("this is not HIP", ["k<3>"], opts)
    assert rc != 0 and entries() == before
    del first


def test_pipelines_use_the_code_object_cache(tmp_path, monkeypatch):
    import time
    monkeypatch.setenv("GERN_HIP_CACHE_DIR", str(tmp_path))
    t0 = time.time()
    a = gern_amd.Softmax(2048, flags=gern_amd.COMPILE_ONLY)
    cold = time.time() - t0
    n = len(list(tmp_path.iterdir()))
    assert n == 1
    t0 = time.time()
    b = gern_amd.Softmax(2048, flags=gern_amd.COMPILE_ONLY)
    warm = time.time() - t0
    # generated kernels are numbered, so the second pipeline's source differs in
    # its function name only if the generator numbers it differently
    assert len(list(tmp_path.iterdir())) in (1, 2)
    assert a.source and b.source
    del cold, warm


def _c_example(*args):
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "examples", "bin", "blur_c_host")
    if not os.path.exists(exe):
        pytest.fail("%s is missing: run `python gern_amd/build.py`" % exe)
    return subprocess.run([exe] + list(args), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)


def test_c_host_example_builds_the_pipeline_without_a_device():
    # examples/blur_c_host.c is strict C99 over include/*.h only
    p = _c_example("--compile-only")
    assert p.returncode == 0, p.stdout
    assert "kernel: function_" in p.stdout


@pytest.mark.gpu
def test_c_host_example_runs_bit_exact_on_the_device():
    p = _c_example()
    assert p.returncode == 0, p.stdout
    assert " 0 differ" in p.stdout, p.stdout
