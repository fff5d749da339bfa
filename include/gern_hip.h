/*
 * gern_hip.h - the thin C ABI between Gern's host side and the HIP runtime.
 *
 * Everything the Runner (and any other host language) needs to turn one
 * generated device translation unit into launches on a gfx950 GPU: compile
 * with hiprtc, load with hipModule, look kernels up by C++ name expression,
 * launch, synchronise, move memory, read device limits, read the last error.
 *
 * Conventions: plain pointers and sizes only, no C++ types, no exceptions.
 * Every function returns 0 on success and a non-zero code on failure; the
 * message for the calling thread's last failure is read with
 * gern_hip_last_error().  Handles are opaque.
 *
 * Each entry point names the piece of the reference it replaces
 * (paths relative to the reference tree).
 */
#ifndef GERN_HIP_H
#define GERN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gern_hip_module_s *gern_hip_module;
typedef struct gern_hip_kernel_s *gern_hip_kernel;
typedef struct gern_hip_event_s *gern_hip_event;

enum {
    GERN_HIP_OK = 0,
    GERN_HIP_ERR_COMPILE = 1,   /* hiprtc rejected the source; log in last_error */
    GERN_HIP_ERR_RUNTIME = 2,   /* a HIP runtime call failed */
    GERN_HIP_ERR_ARGUMENT = 3,  /* bad argument (null handle, zero dimension, limit exceeded) */
    GERN_HIP_ERR_NO_DEVICE = 4  /* no usable GPU */
};

typedef struct {
    int32_t wavefront_size;        /* 64 on gfx950 */
    int32_t max_threads_per_block; /* 1024 */
    int32_t max_block_dim[3];
    int32_t max_grid_dim[3];
    int64_t lds_bytes_per_block;   /* 163840 on gfx950 */
    int32_t compute_units;
    int32_t clock_khz;
    int64_t hbm_bytes;
    char arch[64];                 /* e.g. "gfx950:sramecc+:xnack-" */
} gern_hip_limits;

/* Compiles one device translation unit for `arch` (NULL or "" = the arch of
 * device 0) and loads it.  `name_exprs` are C++ name expressions of the
 * __global__ templates to instantiate, e.g. "function_7<128, 8, 3>".
 * `options` are extra compiler options (e.g. "-I/path/to/gernels").
 * Replaces the `nvcc ... --shared` + dlopen step, src/codegen/runner.cpp:25-47.
 * With the environment variable GERN_HIP_CACHE_DIR naming an existing
 * directory, code objects are kept there under a key of the source, the name
 * expressions, the options, the arch, the compiler version and the content of
 * every header the source includes with quotes; a later compile of the same
 * inputs, in this or another process, loads the stored code object instead of
 * compiling (the reference compiles on every Runner::compile). */
int gern_hip_compile(const char *source, const char *const *name_exprs, int n_name_exprs,
                     const char *const *options, int n_options, const char *arch,
                     gern_hip_module *out);

/* Compile only (no GPU needed): returns the size of the code object, so that
 * generated code can be checked on a machine without a device. */
int gern_hip_compile_only(const char *source, const char *const *name_exprs, int n_name_exprs,
                          const char *const *options, int n_options, const char *arch,
                          size_t *code_size);

/* Looks a kernel up by the same name expression that was given to
 * gern_hip_compile.  Replaces dlsym of the hook, src/codegen/runner.cpp:49-52. */
int gern_hip_get_kernel(gern_hip_module module, const char *name_expr, gern_hip_kernel *out);

/* Registers spilled / used by a kernel, for reports. */
int gern_hip_kernel_info(gern_hip_kernel kernel, int32_t *vgprs, int32_t *sgprs,
                         int32_t *static_lds_bytes, int32_t *scratch_bytes);

/* Asynchronous launch on `stream` (NULL = the default stream).  params[i]
 * points at the i-th kernel argument (an aggregate passed by value or a
 * scalar), exactly the void** the reference hook receives.  Checks the launch
 * shape against the device limits first.  Replaces the <<<grid, block, smem>>>
 * launch, cudaFuncSetAttribute and the limit asserts:
 * src/codegen/codegen.cpp:576-611, src/codegen/codegen_printer.cpp:200-227,
 * include/gern/codegen/helpers/assert_device_properties.h:15-42. */
int gern_hip_launch(gern_hip_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t lds_bytes, void **params, void *stream);

/* hipDeviceSynchronize / hipStreamSynchronize. */
int gern_hip_sync(void);
int gern_hip_stream_sync(void *stream);

/* Non-blocking check for a pending asynchronous error.
 * Replaces include/gern/codegen/helpers/check_last_error.h:7-18. */
int gern_hip_check(void);

int gern_hip_module_unload(gern_hip_module module);

/* Address and size of a __device__ variable of the loaded code, by its
 * (unmangled) name.  *ptr is NULL, and the call succeeds, when the code has no
 * such variable.  No counterpart in the reference, whose generated code holds
 * no device variables. */
int gern_hip_module_global(gern_hip_module module, const char *name, void **ptr, size_t *bytes);

/* Device memory, for hosts that do not bring their own allocator (the
 * reference's data structures call cudaMalloc / cudaMemcpy themselves,
 * apps/common/impl/gpu-matrix-const.h:66-81,221-233). */
int gern_hip_malloc(void **ptr, size_t bytes);
int gern_hip_free(void *ptr);
int gern_hip_memcpy_h2d(void *dst, const void *src, size_t bytes);
int gern_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);
int gern_hip_memset(void *dst, int value, size_t bytes);

/* Events on a stream, for timing launches where they are issued. */
int gern_hip_event_create(gern_hip_event *out);
int gern_hip_event_record(gern_hip_event ev, void *stream);
int gern_hip_event_elapsed_ms(gern_hip_event start, gern_hip_event stop, float *ms);
int gern_hip_event_destroy(gern_hip_event ev);

/* Limits of device 0, cached after the first call. */
int gern_hip_device_limits(gern_hip_limits *out);
int gern_hip_device_count(int *count);

/* Copies the calling thread's last error message (NUL-terminated, possibly
 * truncated) into buf; returns the full length of the message. */
size_t gern_hip_last_error(char *buf, size_t buf_size);

#ifdef __cplusplus
}
#endif
#endif
