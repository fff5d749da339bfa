// Runner: lowers a composed program to source text, compiles it and runs it.
//
// A program wrapped in Global() becomes ONE HIP kernel for gfx950: the device
// translation unit is compiled in-process with hiprtc, loaded with hipModule,
// and launched through the C ABI in gern_hip.h; launch dimensions and host
// side assertions are evaluated by the Runner from the caller's objects.  Any
// other program is lowered to plain C++ loops, compiled with the host
// compiler and called through an extern "C" hook.
//
// Interface as in the reference (include/gern/compose/runner.h:12-46); the
// device path replaces src/codegen/runner.cpp:25-53.
#pragma once

#include "gern/core/composable.h"

#include <map>
#include <memory>
#include <optional>
#include <string>
#include <vector>

namespace gern {

using GernGenFuncPtr = void (*)(void **);

namespace codegen {
struct LaunchPlan;
}

class Runner {
public:
    Runner(Composable c, std::optional<std::vector<Parameter>> ordered_parameters = std::nullopt);
    ~Runner();

    struct Options {
        std::string filename;         // where the generated source is written (under prefix)
        std::string prefix = "/tmp";
        std::string cpp_std = "c++11";  // host pipelines only; device code is always C++17
        std::string include = "";     // "-I dir -I dir ..." for the gernel headers
        std::string ldflags = "";     // host pipelines only
        std::string arch = "";        // "" = the device that is present; else e.g. "gfx950"
        // Spread consecutive workgroups of one XCD over neighbouring tiles
        // (each of the 8 XCDs of an MI355X has its own L2).
        bool xcd_remap = true;
        // With xcd_remap: 0 gives each XCD ONE contiguous run of tiles (an eighth of
        // the grid); n > 0 deals bands of n rows of tiles (a row = gridDim.x tiles)
        // to the XCDs in turn, which keeps the halo sharing inside a band and lets
        // the eight XCDs stream through one window of memory together.
        int xcd_band_rows = 0;
        // Instead of that: the 32 workgroups that run on one XCD at a time take a
        // block of 4 x 8 tiles (x by y), for programs whose tiles share operands
        // along both grid axes (a GEMM: 12 operand panels per 32 tiles).  Applies
        // to launches whose grid is a multiple of 4 by 8 workgroups with a multiple
        // of 256 of them per z slice; other launches keep the plain order.
        bool xcd_tile_blocks = false;
        // Wavefronts per SIMD the kernel must leave room for (caps its
        // registers at 512 / n); 0 = the compiler decides.
        int min_waves_per_simd = 0;
        // HIP stream the kernel is launched on (NULL = default stream).
        void *stream = nullptr;
    };

    // Generates, writes and compiles the code.  Throws UserError
    // ("Compilation Failed") when the compiler rejects it.
    void compile(Options config);

    // args maps each parameter's name to the address of the caller's object
    // (a data-structure struct, or an int64_t / float for a variable).  A
    // device launch is asynchronous.
    void evaluate(std::map<std::string, void *> args);

    FunctionSignature getSignature() const;
    // The generated source text (after compile()).
    std::string getSource() const;
    // Names of the run-time parameters, in the order the generated function
    // takes them.
    std::vector<std::string> getArgumentOrder() const {
        return argument_order;
    }
    // Device launches: the instantiated kernel's name expression, and the HIP
    // stream later evaluate() calls launch on.
    std::string getKernelName() const;
    void setStream(void *s) {
        stream = s;
    }
    // Device launches: waits for the device (a kernel of this Runner may still
    // be running) and unloads the compiled code.  The destructor does NOT do
    // this, as the reference never closes its dlopen handle either; a caller
    // that creates Runners over and over calls release() when it is done with
    // one.  The Runner cannot evaluate afterwards.
    void release();
    // Device launches whose kernel uses the LDS allocator (gernels/lds_alloc.h):
    // waits for the device, then returns how many requests the allocator could
    // not meet since the code was loaded (results of such launches are wrong;
    // give the launch more dynamic LDS).  0 for every other kernel.
    int64_t ldsOverflows();

private:
    FunctionSignature signature;
    Composable c;
    GernGenFuncPtr fp = nullptr;
    std::vector<std::string> argument_order;
    bool compiled = false;
    std::optional<std::vector<Parameter>> ordered_parameters;
    std::string source;
    void *stream = nullptr;
    std::shared_ptr<codegen::LaunchPlan> plan;  // device launches only
    void *module = nullptr;                     // gern_hip_module
    void *kernel = nullptr;                     // gern_hip_kernel
};

void evaluate(Composable c, std::map<std::string, void *> args, Runner::Options config);

}  // namespace gern
