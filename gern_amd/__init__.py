"""gern_amd: Gern's fused kernels on MI355X (gfx950).

This Python module is a thin ctypes view of the package's C ABI
(include/gern_hip.h, include/gern_pipelines.h) for tests, the smoke check and
the benchmark.  The product is the native code: Gern's C++ front end, the HIP
code generator and Runner (libgern.so), the hiprtc/hipModule runtime behind a C
ABI (libgern_hip.so), the hand-written gernels (gernels/*.h) and the composed
pipelines (libgern_pipelines.so).

There is no CPU fallback: every compute entry point raises if the native
libraries or a GPU are missing.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

COMPILE_ONLY = 1
NO_XCD_REMAP = 2
GEMM_OVERWRITE = 4
GEMM_GENERAL_ONLY = 8
BLUR_PLAIN_STORES = 16
QK_ROW_BLOCKS = 32
XCD_TILE_BLOCKS = 64

_libs = None


class GernError(RuntimeError):
    pass


def _load():
    """Loads the native libraries (built in-tree by gern_amd/build.py)."""
    global _libs
    if _libs is not None:
        return _libs
    # PyTorch ships its own HIP runtime under the same sonames.  Loading it
    # first makes the whole process share ONE runtime; two runtimes in one
    # process each open the device and the second one finds no GPU.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    paths = {n: os.path.join(_HERE, "lib%s.so" % n) for n in ("gern_hip", "gern", "gern_pipelines")}
    for n, p in paths.items():
        if not os.path.exists(p):
            raise GernError("%s is missing: run `python gern_amd/build.py` (or __graft_entry__.build())" % p)
    hip = C.CDLL(paths["gern_hip"], mode=C.RTLD_GLOBAL)
    C.CDLL(paths["gern"], mode=C.RTLD_GLOBAL)
    pipes = C.CDLL(paths["gern_pipelines"], mode=C.RTLD_GLOBAL)

    i64, vp, sz = C.c_int64, C.c_void_p, C.c_size_t
    hip.gern_hip_last_error.restype = sz
    hip.gern_hip_last_error.argtypes = [C.c_char_p, sz]
    pipes.gern_pipelines_last_error.restype = sz
    pipes.gern_pipelines_last_error.argtypes = [C.c_char_p, sz]
    pipes.gern_pipeline_source.restype = C.c_char_p
    pipes.gern_pipeline_source.argtypes = [vp]
    pipes.gern_pipeline_kernel_name.restype = C.c_char_p
    pipes.gern_pipeline_kernel_name.argtypes = [vp]
    pipes.gern_pipeline_destroy.argtypes = [vp]
    pipes.gern_pipeline_faults.argtypes = [vp, C.POINTER(i64)]
    pipes.gern_blur_chain_create.argtypes = [C.c_char_p, i64, i64, i64, C.c_int, C.c_int, C.POINTER(vp)]
    pipes.gern_blur_chain_run.argtypes = [vp, vp, i64, i64, i64, vp, i64, vp]
    pipes.gern_softmax_create.argtypes = [i64, i64, C.c_int, C.POINTER(vp)]
    pipes.gern_softmax_run.argtypes = [vp, vp, vp, i64, i64, vp]
    if hasattr(pipes, "gern_gemm_create"):
        pipes.gern_gemm_create.argtypes = [C.c_int, C.c_int, C.POINTER(vp)]
        pipes.gern_gemm_run.argtypes = [vp, vp, vp, vp, i64, i64, i64, vp]
    if hasattr(pipes, "gern_qk_softmax_create"):
        pipes.gern_qk_softmax_create.argtypes = [i64, i64, C.c_int, C.POINTER(vp)]
        pipes.gern_qk_softmax_run.argtypes = [vp, vp, vp, vp, i64, i64, C.c_float, vp]
        pipes.gern_qk_softmax_run_no_alloc.argtypes = [vp, vp, vp, vp, i64, i64, C.c_float, vp]
    pipes.gern_gemm_schedule_create.argtypes = [C.c_int, C.c_int, C.POINTER(vp)]
    pipes.gern_gemm_schedule_run.argtypes = [vp, vp, vp, vp, vp]
    cpp = C.POINTER(C.c_char_p)
    hip.gern_hip_compile.argtypes = [C.c_char_p, cpp, C.c_int, cpp, C.c_int, C.c_char_p, C.POINTER(vp)]
    hip.gern_hip_compile_only.argtypes = [C.c_char_p, cpp, C.c_int, cpp, C.c_int, C.c_char_p, C.POINTER(sz)]
    hip.gern_hip_get_kernel.argtypes = [vp, C.c_char_p, C.POINTER(vp)]
    hip.gern_hip_launch.argtypes = [vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32, C.POINTER(vp), vp]
    hip.gern_hip_event_create.argtypes = [C.POINTER(vp)]
    hip.gern_hip_event_record.argtypes = [vp, vp]
    hip.gern_hip_event_elapsed_ms.argtypes = [vp, vp, C.POINTER(C.c_float)]
    hip.gern_hip_event_destroy.argtypes = [vp]
    hip.gern_hip_stream_sync.argtypes = [vp]
    _libs = (hip, pipes)
    return _libs


def hip_lib():
    return _load()[0]


def pipelines_lib():
    return _load()[1]


def _pipe_error():
    n = pipelines_lib().gern_pipelines_last_error(None, 0)
    buf = C.create_string_buffer(n + 1)
    pipelines_lib().gern_pipelines_last_error(buf, n + 1)
    return buf.value.decode(errors="replace")


def _hip_error():
    n = hip_lib().gern_hip_last_error(None, 0)
    buf = C.create_string_buffer(n + 1)
    hip_lib().gern_hip_last_error(buf, n + 1)
    return buf.value.decode(errors="replace")


def _check(rc):
    if rc != 0:
        raise GernError(_pipe_error())


class Limits(C.Structure):
    _fields_ = [("wavefront_size", C.c_int32), ("max_threads_per_block", C.c_int32),
                ("max_block_dim", C.c_int32 * 3), ("max_grid_dim", C.c_int32 * 3),
                ("lds_bytes_per_block", C.c_int64), ("compute_units", C.c_int32), ("clock_khz", C.c_int32),
                ("hbm_bytes", C.c_int64), ("arch", C.c_char * 64)]


def device_limits():
    lim = Limits()
    if hip_lib().gern_hip_device_limits(C.byref(lim)) != 0:
        raise GernError(_hip_error())
    return lim


def device_count():
    n = C.c_int(0)
    hip_lib().gern_hip_device_count(C.byref(n))
    return n.value


class Event:
    """A HIP event recorded on the stream the kernels are launched on."""

    def __init__(self):
        self.h = C.c_void_p()
        if hip_lib().gern_hip_event_create(C.byref(self.h)) != 0:
            raise GernError(_hip_error())

    def record(self, stream=None):
        if hip_lib().gern_hip_event_record(self.h, stream) != 0:
            raise GernError(_hip_error())

    def elapsed_ms_until(self, stop):
        ms = C.c_float()
        if hip_lib().gern_hip_event_elapsed_ms(self.h, stop.h, C.byref(ms)) != 0:
            raise GernError(_hip_error())
        return ms.value

    def __del__(self):
        try:
            hip_lib().gern_hip_event_destroy(self.h)
        except Exception:
            pass


def _ptr(t):
    """Device pointer of a torch tensor (or a raw integer address)."""
    return C.c_void_p(t if isinstance(t, int) else t.data_ptr())


class _Pipeline:
    def __init__(self):
        self.h = C.c_void_p()

    @property
    def source(self):
        return pipelines_lib().gern_pipeline_source(self.h).decode()

    @property
    def kernel_name(self):
        return pipelines_lib().gern_pipeline_kernel_name(self.h).decode()

    def faults(self):
        """gern_pipeline_faults: waits for the device; what the kernels could only signal in their results
        (QK tile kernel: wavefronts that gave up waiting, rows whose logits did not fit), read and cleared."""
        n = C.c_int64(-1)
        _check(pipelines_lib().gern_pipeline_faults(self.h, C.byref(n)))
        return n.value

    def __del__(self):
        try:
            if self.h:
                pipelines_lib().gern_pipeline_destroy(self.h)
        except Exception:
            pass


class BlurChain(_Pipeline):
    """Fused separable box blur, e.g. BlurChain("xyx")."""

    def __init__(self, pattern, stride=3, tile_rows=4, tile_cols=None, waves_per_block=1, flags=0):
        super().__init__()
        nx = pattern.count("x")
        if tile_cols is None:
            # the widest tile that writes line-aligned windows (include/gern_pipelines.h)
            tile_cols = (256 - 28 - nx * (stride - 1)) // 32 * 32
        self.pattern, self.stride = pattern, stride
        self.nx, self.ny = nx, pattern.count("y")
        _check(pipelines_lib().gern_blur_chain_create(pattern.encode(), stride, tile_rows, tile_cols,
                                                      waves_per_block, flags, C.byref(self.h)))

    def out_shape(self, rows, cols):
        return rows - self.ny * (self.stride - 1), cols - self.nx * (self.stride - 1)

    def __call__(self, img, out, stream=None):
        """img, out: contiguous fp32 CUDA tensors; out has out_shape(*img.shape)."""
        rows, cols = img.shape
        assert tuple(out.shape) == self.out_shape(rows, cols)
        _check(pipelines_lib().gern_blur_chain_run(self.h, _ptr(img), rows, cols, img.stride(0), _ptr(out),
                                                   out.stride(0), stream))
        return out


class Softmax(_Pipeline):
    """Fused row softmax over matrices with `ncol` columns."""

    def __init__(self, ncol, rows_per_wave=1, flags=0):
        super().__init__()
        self.ncol = ncol
        _check(pipelines_lib().gern_softmax_create(ncol, rows_per_wave, flags, C.byref(self.h)))

    def __call__(self, x, out, stream=None):
        rows, cols = x.shape
        assert cols == self.ncol and tuple(out.shape) == (rows, cols) and x.stride(0) == out.stride(0)
        _check(pipelines_lib().gern_softmax_run(self.h, _ptr(x), _ptr(out), rows, x.stride(0), stream))
        return out


class Gemm(_Pipeline):
    """C += A @ B (or C = A @ B with overwrite=True).  variant "f32" or "bf16"
    (fp32 accumulate); general_only=True keeps shapes that the direct-to-LDS
    matrix-core kernels could take on the kernel for every shape."""

    def __init__(self, variant="f32", overwrite=False, general_only=False, flags=0):
        super().__init__()
        self.variant = variant
        if overwrite:
            flags |= GEMM_OVERWRITE
        if general_only:
            flags |= GEMM_GENERAL_ONLY
        _check(pipelines_lib().gern_gemm_create({"f32": 0, "bf16": 1}[variant], flags, C.byref(self.h)))

    def __call__(self, A, B, Cm, stream=None):
        M, K = A.shape
        N = B.shape[1]
        assert tuple(B.shape) == (K, N) and tuple(Cm.shape) == (M, N)
        assert A.is_contiguous() and B.is_contiguous() and Cm.is_contiguous()
        _check(pipelines_lib().gern_gemm_run(self.h, _ptr(A), _ptr(B), _ptr(Cm), M, N, K, stream))
        return Cm


class GemmSchedule(_Pipeline):
    """C += A @ B on 1024 x 1024 fp32 matrices through a schedule written at the level of Gern's API
    (the reference's gernels/mm/kernel_3.cu, kernel_6.cu or kernel_10.cu)."""

    SIZE = 1024

    def __init__(self, schedule, flags=0):
        super().__init__()
        self.schedule = schedule
        _check(pipelines_lib().gern_gemm_schedule_create(schedule, flags, C.byref(self.h)))

    def __call__(self, A, B, Cm, stream=None):
        n = self.SIZE
        assert tuple(A.shape) == (n, n) and tuple(B.shape) == (n, n) and tuple(Cm.shape) == (n, n)
        assert A.is_contiguous() and B.is_contiguous() and Cm.is_contiguous()
        _check(pipelines_lib().gern_gemm_schedule_run(self.h, _ptr(A), _ptr(B), _ptr(Cm), stream))
        return Cm


class QKSoftmax(_Pipeline):
    """S = softmax_rows(scale * Q @ K^T), Q and K in bf16, S in fp32."""

    def __init__(self, head_dim=128, max_keys=4096, flags=0):
        super().__init__()
        self.head_dim = head_dim
        _check(pipelines_lib().gern_qk_softmax_create(head_dim, max_keys, flags, C.byref(self.h)))

    def __call__(self, Q, K, S, scale, stream=None, no_alloc=False):
        """no_alloc=True: gern_qk_softmax_run_no_alloc (exchange memory from the library's device array)."""
        M, D = Q.shape
        N = K.shape[0]
        assert D == self.head_dim and K.shape[1] == D and tuple(S.shape) == (M, N)
        assert Q.is_contiguous() and K.is_contiguous() and S.is_contiguous()
        run = pipelines_lib().gern_qk_softmax_run_no_alloc if no_alloc else pipelines_lib().gern_qk_softmax_run
        _check(run(self.h, _ptr(Q), _ptr(K), _ptr(S), M, N, float(scale), stream))
        return S
