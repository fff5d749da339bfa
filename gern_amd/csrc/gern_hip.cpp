// Implementation of the C ABI declared in include/gern_hip.h: hiprtc compile,
// hipModule load, kernel lookup by name expression, checked launch, memory and
// event helpers.  Host code only; it links libamdhip64 and libhiprtc.
#include "gern_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char *what) {
    return fail(GERN_HIP_ERR_RUNTIME, std::string(what) + ": " + hipGetErrorString(e));
}

#define HIP_TRY(call)                           \
    do {                                        \
        hipError_t e_ = (call);                 \
        if (e_ != hipSuccess) {                 \
            return hip_fail(e_, #call);         \
        }                                       \
    } while (0)

// Limits of each device, read once per device: launches are checked against
// the limits of the device that is current in the calling thread.
std::mutex g_limits_mutex;
std::map<int, gern_hip_limits> g_limits_by_device;

int current_limits(gern_hip_limits &out) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        return fail(GERN_HIP_ERR_NO_DEVICE, "no HIP device is visible to this process");
    }
    std::lock_guard<std::mutex> lock(g_limits_mutex);
    auto it = g_limits_by_device.find(device);
    if (it != g_limits_by_device.end()) {
        out = it->second;
        return GERN_HIP_OK;
    }
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    gern_hip_limits limits;
    std::memset(&limits, 0, sizeof(limits));
    limits.wavefront_size = prop.warpSize;
    limits.max_threads_per_block = prop.maxThreadsPerBlock;
    for (int i = 0; i < 3; i++) {
        limits.max_block_dim[i] = prop.maxThreadsDim[i];
        limits.max_grid_dim[i] = prop.maxGridSize[i];
    }
    limits.lds_bytes_per_block = (int64_t)prop.sharedMemPerBlock;
    int optin = 0;
    if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, device) == hipSuccess &&
        optin > limits.lds_bytes_per_block) {
        limits.lds_bytes_per_block = optin;
    }
    limits.compute_units = prop.multiProcessorCount;
    limits.clock_khz = prop.clockRate;
    limits.hbm_bytes = (int64_t)prop.totalGlobalMem;
    std::snprintf(limits.arch, sizeof(limits.arch), "%.63s", prop.gcnArchName);
    g_limits_by_device[device] = limits;
    out = limits;
    return GERN_HIP_OK;
}

struct CompiledProgram {
    std::vector<char> code;
    std::map<std::string, std::string> lowered;  // name expression -> mangled name
};

// ---- optional on-disk cache of code objects (GERN_HIP_CACHE_DIR) ------------
// The reference recompiles on every Runner::compile (src/codegen/runner.cpp:25-40,
// seconds per pipeline).  With GERN_HIP_CACHE_DIR set, a code object is stored
// under a 128-bit key of everything that determines it: the source text, the
// name expressions, the options, the architecture, the hiprtc version, and the
// content of every header the source includes with quotes (the gernels are
// headers that the generated source includes).

struct KeyHash {
    uint64_t a = 0xcbf29ce484222325ull, b = 0x84222325cbf29ce4ull;
    void bytes(const void *p, size_t n) {
        const unsigned char *c = static_cast<const unsigned char *>(p);
        for (size_t i = 0; i < n; i++) {
            a = (a ^ c[i]) * 0x100000001b3ull;
            b = (b ^ c[i]) * 0x9e3779b97f4a7c15ull;
            b ^= b >> 29;
        }
    }
    void text(const std::string &t) {
        const uint64_t n = t.size();
        bytes(&n, sizeof n);  // length-prefixed: ("ab","c") and ("a","bc") differ
        bytes(t.data(), t.size());
    }
    std::string hex() const {
        char buf[40];
        std::snprintf(buf, sizeof buf, "%016llx%016llx", (unsigned long long)a, (unsigned long long)b);
        return buf;
    }
};

bool read_file(const std::string &path, std::vector<char> &out) {
    FILE *f = std::fopen(path.c_str(), "rb");
    if (f == nullptr) {
        return false;
    }
    std::fseek(f, 0, SEEK_END);
    const long n = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    out.resize(n > 0 ? (size_t)n : 0);
    const bool ok = n > 0 && std::fread(out.data(), 1, (size_t)n, f) == (size_t)n;
    std::fclose(f);
    return ok;
}

// Hashes the CONTENT of every file that `text` reaches through #include "..."
// lines, searched first beside the including file and then in the -I
// directories, as the compiler does.  Conditional compilation is ignored (a
// file behind a false #if is hashed too: more misses, never a stale hit);
// <...> headers belong to the toolchain, whose version is part of the key.
void hash_includes(const std::string &text, const std::string &self_dir, const std::vector<std::string> &dirs,
                   std::set<std::string> &seen, KeyHash &h, int depth) {
    size_t pos = 0;
    while (pos < text.size()) {
        size_t end = text.find('\n', pos);
        if (end == std::string::npos) {
            end = text.size();
        }
        size_t i = text.find_first_not_of(" \t", pos);
        if (i < end && text[i] == '#') {
            i = text.find_first_not_of(" \t", i + 1);
            if (i < end && text.compare(i, 7, "include") == 0) {
                i = text.find_first_not_of(" \t", i + 7);
                if (i < end && text[i] == '"') {
                    const size_t close = text.find('"', i + 1);
                    if (close != std::string::npos && close < end) {
                        const std::string name = text.substr(i + 1, close - i - 1);
                        std::vector<std::string> candidates;
                        if (!self_dir.empty()) {
                            candidates.push_back(self_dir + "/" + name);
                        }
                        for (const auto &d : dirs) {
                            candidates.push_back(d + "/" + name);
                        }
                        bool found = false;
                        for (const auto &path : candidates) {
                            std::vector<char> content;
                            if (!read_file(path, content)) {
                                continue;
                            }
                            found = true;
                            if (seen.insert(path).second) {
                                const std::string body(content.begin(), content.end());
                                h.text(name);
                                h.text(body);
                                if (depth < 32) {
                                    const size_t slash = path.rfind('/');
                                    hash_includes(body, slash == std::string::npos ? "" : path.substr(0, slash), dirs, seen, h,
                                                  depth + 1);
                                }
                            }
                            break;
                        }
                        if (!found) {
                            h.text("missing " + name);
                        }
                    }
                }
            }
        }
        pos = end + 1;
    }
}

std::string cache_key(const char *source, const char *const *name_exprs, int n_name_exprs,
                      const std::vector<std::string> &options, const std::string &arch) {
    KeyHash h;
    h.text(source);
    for (int i = 0; i < n_name_exprs; i++) {
        h.text(name_exprs[i]);
    }
    h.text(arch);
    int major = 0, minor = 0;
    hiprtcVersion(&major, &minor);
    const int version[3] = {major, minor, HIP_VERSION};
    h.bytes(version, sizeof version);
    std::vector<std::string> dirs;
    for (size_t i = 0; i < options.size(); i++) {
        h.text(options[i]);
        std::string dir;
        if (options[i] == "-I" && i + 1 < options.size()) {
            dir = options[i + 1];
        } else if (options[i].rfind("-I", 0) == 0 && options[i].size() > 2) {
            dir = options[i].substr(2);
            dir.erase(0, dir.find_first_not_of(' '));
        }
        if (!dir.empty()) {
            dirs.push_back(dir);
        }
    }
    std::set<std::string> seen;
    hash_includes(source, "", dirs, seen, h, 0);
    return h.hex();
}

// Entry file: "gernhip1\n", then per name expression "<expr>\n<lowered>\n",
// then "--code <size>\n" and the code object.  Anything unexpected is a miss.
bool cache_load(const std::string &path, const char *const *name_exprs, int n_name_exprs, CompiledProgram &out) {
    std::vector<char> blob;
    if (!read_file(path, blob)) {
        return false;
    }
    size_t pos = 0;
    auto line = [&](std::string &l) {
        const void *nl = std::memchr(blob.data() + pos, '\n', blob.size() - pos);
        if (nl == nullptr) {
            return false;
        }
        const size_t end = (const char *)nl - blob.data();
        l.assign(blob.data() + pos, end - pos);
        pos = end + 1;
        return true;
    };
    std::string l, lowered;
    if (!line(l) || l != "gernhip1") {
        return false;
    }
    std::map<std::string, std::string> names;
    for (;;) {
        if (!line(l)) {
            return false;
        }
        if (l.rfind("--code ", 0) == 0) {
            break;
        }
        if (!line(lowered)) {
            return false;
        }
        names[l] = lowered;
    }
    const size_t size = std::strtoull(l.c_str() + 7, nullptr, 10);
    if (size == 0 || blob.size() - pos != size || (int)names.size() > n_name_exprs) {
        return false;
    }
    for (int i = 0; i < n_name_exprs; i++) {
        if (names.find(name_exprs[i]) == names.end()) {
            return false;
        }
    }
    out.lowered = std::move(names);
    out.code.assign(blob.begin() + pos, blob.end());
    return true;
}

void cache_store(const std::string &path, const CompiledProgram &prog) {
    static std::atomic<int> serial{0};
    const std::string tmp = path + ".tmp" + std::to_string((long)getpid()) + "_" + std::to_string(serial++);
    FILE *f = std::fopen(tmp.c_str(), "wb");
    if (f == nullptr) {
        return;  // a cache that cannot be written is not an error
    }
    bool ok = std::fputs("gernhip1\n", f) >= 0;
    for (const auto &kv : prog.lowered) {
        ok = ok && std::fprintf(f, "%s\n%s\n", kv.first.c_str(), kv.second.c_str()) > 0;
    }
    ok = ok && std::fprintf(f, "--code %zu\n", prog.code.size()) > 0;
    ok = ok && std::fwrite(prog.code.data(), 1, prog.code.size(), f) == prog.code.size();
    ok = (std::fclose(f) == 0) && ok;
    if (!ok || std::rename(tmp.c_str(), path.c_str()) != 0) {  // rename: readers never see a partial entry
        std::remove(tmp.c_str());
    }
}

void keep_for_inspection(const char *source, const CompiledProgram &prog);

int compile_program(const char *source, const char *const *name_exprs, int n_name_exprs,
                    const char *const *options, int n_options, const char *arch,
                    CompiledProgram &out) {
    if (source == nullptr || (n_name_exprs > 0 && name_exprs == nullptr) ||
        (n_options > 0 && options == nullptr)) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_compile: null argument");
    }
    std::string arch_name = arch ? arch : "";
    if (arch_name.empty()) {
        gern_hip_limits limits;
        int rc = current_limits(limits);
        if (rc != GERN_HIP_OK) {
            return rc;
        }
        arch_name = limits.arch;
    }
    for (int i = 0; i < n_name_exprs; i++) {
        if (name_exprs[i] == nullptr || std::strchr(name_exprs[i], '\n') != nullptr) {
            return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_compile: a name expression is null or spans lines");
        }
    }
    std::string cache_path;
    if (const char *dir = std::getenv("GERN_HIP_CACHE_DIR")) {
        if (*dir != '\0') {
            std::vector<std::string> user_options;
            for (int i = 0; i < n_options; i++) {
                user_options.push_back(options[i] ? options[i] : "");
            }
            cache_path = std::string(dir) + "/" + cache_key(source, name_exprs, n_name_exprs, user_options, arch_name) + ".gernhip";
            if (cache_load(cache_path, name_exprs, n_name_exprs, out)) {
                keep_for_inspection(source, out);
                return GERN_HIP_OK;
            }
            out = CompiledProgram();
        }
    }
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, "gern_generated.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) {
        return fail(GERN_HIP_ERR_COMPILE, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
    }
    for (int i = 0; i < n_name_exprs; i++) {
        r = hiprtcAddNameExpression(prog, name_exprs[i]);
        if (r != HIPRTC_SUCCESS) {
            hiprtcDestroyProgram(&prog);
            return fail(GERN_HIP_ERR_COMPILE, std::string("hiprtcAddNameExpression(") + name_exprs[i] +
                                                  "): " + hiprtcGetErrorString(r));
        }
    }
    std::vector<std::string> opt_storage;
    opt_storage.push_back("--offload-arch=" + arch_name);
    opt_storage.push_back("-O3");
    opt_storage.push_back("-std=c++17");
    // Packed-FP32 instructions are kept out of every kernel.
    opt_storage.push_back("-Xclang");
    opt_storage.push_back("-target-feature");
    opt_storage.push_back("-Xclang");
    opt_storage.push_back("-packed-fp32-ops");
    for (int i = 0; i < n_options; i++) {
        opt_storage.push_back(options[i]);
    }
    std::vector<const char *> opts;
    for (const auto &o : opt_storage) {
        opts.push_back(o.c_str());
    }
    r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size > 0) {
            hiprtcGetProgramLog(prog, log.data());
        }
        hiprtcDestroyProgram(&prog);
        return fail(GERN_HIP_ERR_COMPILE, std::string("hiprtc: ") + hiprtcGetErrorString(r) + "\n" + log);
    }
    for (int i = 0; i < n_name_exprs; i++) {
        const char *lowered = nullptr;
        r = hiprtcGetLoweredName(prog, name_exprs[i], &lowered);
        if (r != HIPRTC_SUCCESS || lowered == nullptr) {
            hiprtcDestroyProgram(&prog);
            return fail(GERN_HIP_ERR_COMPILE, std::string("no kernel matches name expression ") + name_exprs[i]);
        }
        out.lowered[name_exprs[i]] = lowered;
    }
    size_t code_size = 0;
    r = hiprtcGetCodeSize(prog, &code_size);
    if (r != HIPRTC_SUCCESS || code_size == 0) {
        hiprtcDestroyProgram(&prog);
        return fail(GERN_HIP_ERR_COMPILE, "hiprtc produced no code object");
    }
    out.code.resize(code_size);
    hiprtcGetCode(prog, out.code.data());
    hiprtcDestroyProgram(&prog);
    if (!cache_path.empty()) {
        cache_store(cache_path, out);
    }
    keep_for_inspection(source, out);
    return GERN_HIP_OK;
}

// Like the reference Runner, which leaves its generated source and shared
// object in `prefix` (src/codegen/runner.cpp:20-35): with GERN_HIP_KEEP_DIR
// set, the source and the code object are kept there for inspection.
void keep_for_inspection(const char *source, const CompiledProgram &prog) {
    if (const char *dir = std::getenv("GERN_HIP_KEEP_DIR")) {
        static std::atomic<int> serial{0};
        const std::string base = std::string(dir) + "/gern_generated_" + std::to_string(serial++);
        if (FILE *f = std::fopen((base + ".hip").c_str(), "w")) {
            std::fputs(source, f);
            std::fclose(f);
        }
        if (FILE *f = std::fopen((base + ".hsaco").c_str(), "wb")) {
            std::fwrite(prog.code.data(), 1, prog.code.size(), f);
            std::fclose(f);
        }
    }
}

}  // namespace

struct gern_hip_module_s {
    hipModule_t module = nullptr;
    std::map<std::string, std::string> lowered;
    std::vector<gern_hip_kernel_s *> kernels;
};

struct gern_hip_kernel_s {
    hipFunction_t fn = nullptr;
    std::string name;
};

struct gern_hip_event_s {
    hipEvent_t ev = nullptr;
};

extern "C" {

int gern_hip_compile(const char *source, const char *const *name_exprs, int n_name_exprs,
                     const char *const *options, int n_options, const char *arch,
                     gern_hip_module *out) {
    if (out == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_compile: null output handle");
    }
    *out = nullptr;
    gern_hip_limits limits;
    int rc = current_limits(limits);
    if (rc != GERN_HIP_OK) {
        return rc;
    }
    CompiledProgram prog;
    rc = compile_program(source, name_exprs, n_name_exprs, options, n_options, arch, prog);
    if (rc != GERN_HIP_OK) {
        return rc;
    }
    auto *m = new gern_hip_module_s();
    hipError_t e = hipModuleLoadData(&m->module, prog.code.data());
    if (e != hipSuccess) {
        delete m;
        return hip_fail(e, "hipModuleLoadData");
    }
    m->lowered = std::move(prog.lowered);
    *out = m;
    return GERN_HIP_OK;
}

int gern_hip_compile_only(const char *source, const char *const *name_exprs, int n_name_exprs,
                          const char *const *options, int n_options, const char *arch,
                          size_t *code_size) {
    if (arch == nullptr || arch[0] == '\0') {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_compile_only needs an explicit arch");
    }
    CompiledProgram prog;
    int rc = compile_program(source, name_exprs, n_name_exprs, options, n_options, arch, prog);
    if (rc != GERN_HIP_OK) {
        return rc;
    }
    if (code_size) {
        *code_size = prog.code.size();
    }
    return GERN_HIP_OK;
}

int gern_hip_get_kernel(gern_hip_module module, const char *name_expr, gern_hip_kernel *out) {
    if (module == nullptr || name_expr == nullptr || out == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_get_kernel: null argument");
    }
    *out = nullptr;
    auto it = module->lowered.find(name_expr);
    // A plain (non-template) extern "C" kernel can be looked up directly.
    std::string symbol = (it != module->lowered.end()) ? it->second : std::string(name_expr);
    hipFunction_t fn = nullptr;
    hipError_t e = hipModuleGetFunction(&fn, module->module, symbol.c_str());
    if (e != hipSuccess) {
        return hip_fail(e, ("hipModuleGetFunction(" + symbol + ")").c_str());
    }
    auto *k = new gern_hip_kernel_s();
    k->fn = fn;
    k->name = name_expr;
    module->kernels.push_back(k);
    *out = k;
    return GERN_HIP_OK;
}

int gern_hip_kernel_info(gern_hip_kernel kernel, int32_t *vgprs, int32_t *sgprs,
                         int32_t *static_lds_bytes, int32_t *scratch_bytes) {
    if (kernel == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_kernel_info: null kernel");
    }
    int v = 0;
    if (vgprs) {
        HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, kernel->fn));
        *vgprs = v;
    }
    if (sgprs) {
        *sgprs = 0;
    }
    if (static_lds_bytes) {
        HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, kernel->fn));
        *static_lds_bytes = v;
    }
    if (scratch_bytes) {
        HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, kernel->fn));
        *scratch_bytes = v;
    }
    return GERN_HIP_OK;
}

int gern_hip_launch(gern_hip_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t lds_bytes, void **params, void *stream) {
    if (kernel == nullptr || grid == nullptr || block == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: null argument");
    }
    gern_hip_limits limits;
    int rc = current_limits(limits);
    if (rc != GERN_HIP_OK) {
        return rc;
    }
    uint64_t threads = 1;
    for (int i = 0; i < 3; i++) {
        if (grid[i] == 0 || block[i] == 0) {
            return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: zero-sized grid or block dimension");
        }
        if (block[i] > (uint32_t)limits.max_block_dim[i]) {
            return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: block dimension " + std::to_string(i) +
                                                   " = " + std::to_string(block[i]) + " exceeds the device limit");
        }
        if (grid[i] > (uint32_t)limits.max_grid_dim[i]) {
            return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: grid dimension " + std::to_string(i) +
                                                   " = " + std::to_string(grid[i]) + " exceeds the device limit");
        }
        threads *= block[i];
    }
    if (threads > (uint64_t)limits.max_threads_per_block) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: " + std::to_string(threads) +
                                               " threads per block exceeds the device limit of " +
                                               std::to_string(limits.max_threads_per_block));
    }
    if ((int64_t)lds_bytes > limits.lds_bytes_per_block) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_launch: " + std::to_string(lds_bytes) +
                                               " bytes of LDS exceeds the per-block limit of " +
                                               std::to_string(limits.lds_bytes_per_block));
    }
    HIP_TRY(hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                  lds_bytes, (hipStream_t)stream, params, nullptr));
    return GERN_HIP_OK;
}

int gern_hip_sync(void) {
    HIP_TRY(hipDeviceSynchronize());
    return GERN_HIP_OK;
}

int gern_hip_stream_sync(void *stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return GERN_HIP_OK;
}

int gern_hip_check(void) {
    HIP_TRY(hipPeekAtLastError());
    return GERN_HIP_OK;
}

int gern_hip_module_unload(gern_hip_module module) {
    if (module == nullptr) {
        return GERN_HIP_OK;
    }
    hipError_t e = hipModuleUnload(module->module);
    for (auto *k : module->kernels) {
        delete k;
    }
    delete module;
    if (e != hipSuccess) {
        return hip_fail(e, "hipModuleUnload");
    }
    return GERN_HIP_OK;
}

int gern_hip_module_global(gern_hip_module module, const char *name, void **ptr, size_t *bytes) {
    if (module == nullptr || name == nullptr || ptr == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_module_global: null argument");
    }
    *ptr = nullptr;
    hipDeviceptr_t at = nullptr;
    size_t size = 0;
    hipError_t e = hipModuleGetGlobal(&at, &size, module->module, name);
    if (e == hipErrorNotFound) {
        (void)hipGetLastError();
        return GERN_HIP_OK;
    }
    if (e != hipSuccess) {
        return hip_fail(e, (std::string("hipModuleGetGlobal(") + name + ")").c_str());
    }
    *ptr = at;
    if (bytes != nullptr) {
        *bytes = size;
    }
    return GERN_HIP_OK;
}

int gern_hip_malloc(void **ptr, size_t bytes) {
    if (ptr == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_malloc: null output pointer");
    }
    HIP_TRY(hipMalloc(ptr, bytes));
    return GERN_HIP_OK;
}

int gern_hip_free(void *ptr) {
    HIP_TRY(hipFree(ptr));
    return GERN_HIP_OK;
}

int gern_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return GERN_HIP_OK;
}

int gern_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return GERN_HIP_OK;
}

int gern_hip_memset(void *dst, int value, size_t bytes) {
    HIP_TRY(hipMemset(dst, value, bytes));
    return GERN_HIP_OK;
}

int gern_hip_event_create(gern_hip_event *out) {
    if (out == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_event_create: null output handle");
    }
    auto *ev = new gern_hip_event_s();
    hipError_t e = hipEventCreate(&ev->ev);
    if (e != hipSuccess) {
        delete ev;
        return hip_fail(e, "hipEventCreate");
    }
    *out = ev;
    return GERN_HIP_OK;
}

int gern_hip_event_record(gern_hip_event ev, void *stream) {
    if (ev == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_event_record: null event");
    }
    HIP_TRY(hipEventRecord(ev->ev, (hipStream_t)stream));
    return GERN_HIP_OK;
}

int gern_hip_event_elapsed_ms(gern_hip_event start, gern_hip_event stop, float *ms) {
    if (start == nullptr || stop == nullptr || ms == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_event_elapsed_ms: null argument");
    }
    HIP_TRY(hipEventSynchronize(stop->ev));
    HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
    return GERN_HIP_OK;
}

int gern_hip_event_destroy(gern_hip_event ev) {
    if (ev == nullptr) {
        return GERN_HIP_OK;
    }
    hipError_t e = hipEventDestroy(ev->ev);
    delete ev;
    if (e != hipSuccess) {
        return hip_fail(e, "hipEventDestroy");
    }
    return GERN_HIP_OK;
}

int gern_hip_device_limits(gern_hip_limits *out) {
    if (out == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_device_limits: null output");
    }
    return current_limits(*out);
}

int gern_hip_device_count(int *count) {
    if (count == nullptr) {
        return fail(GERN_HIP_ERR_ARGUMENT, "gern_hip_device_count: null output");
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    *count = (e == hipSuccess) ? n : 0;
    return GERN_HIP_OK;
}

size_t gern_hip_last_error(char *buf, size_t buf_size) {
    if (buf != nullptr && buf_size > 0) {
        size_t n = g_last_error.size() < buf_size - 1 ? g_last_error.size() : buf_size - 1;
        std::memcpy(buf, g_last_error.data(), n);
        buf[n] = '\0';
    }
    return g_last_error.size();
}

}  // extern "C"
