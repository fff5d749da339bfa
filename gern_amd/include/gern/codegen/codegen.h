// Code generation: lowered statement tree -> source text.
//
// Two targets.  A device launch becomes one HIP translation unit holding a
// single __global__ function template for gfx950, plus a LaunchPlan that tells
// the Runner how to size and launch it (there is no host hook in the text:
// hiprtc compiles device code only).  A host pipeline becomes a C++ function
// template of nested loops plus the extern "C" hook that unpacks void** and
// calls it.
//
// The index algebra that maps a loop onto a grid unit is the reference's
// (src/codegen/codegen.cpp:293-345): index = ((unit / inner_extent) %
// ceil(extent / step)) * step + start, and the launch dimension grows to
// inner_extent * ceil(...).  What is specific to this target: wavefront units
// divide a block dimension by 64, workgroup indices are re-ordered so that
// consecutive tiles land on the same XCD, and the kernel carries
// __launch_bounds__ whenever the block shape is known at generation time.
#pragma once

#include "gern/lower/lower.h"

#include <functional>
#include <optional>
#include <string>
#include <vector>

namespace gern {
namespace codegen {

// Everything the Runner needs to launch a generated kernel.
struct LaunchPlan {
    std::string function_name;             // function_<n>
    std::string name_expression;           // function_<n><v1, v2, ...> (or the plain name)
    std::vector<Variable> template_args;   // bound compile-time variables, in template order
    std::vector<Parameter> parameters;     // run-time parameters, in kernel order
    Expr grid[3];
    Expr block[3];
    Expr lds_bytes;                        // undefined = no dynamic LDS
    std::vector<Constraint> host_asserts;  // assumptions checked on the host before each launch
    bool device = false;
    // Device code that is not a launch: a __device__ function for another
    // generated kernel to call (FunctionPtr over gernels that occupy grid units).
    bool device_function = false;
};

// Values an expression is evaluated against on the host.
struct EvalEnv {
    std::function<bool(const std::string &name, int64_t &value)> variable;
    std::function<bool(const AbstractDataTypePtr &ds, const std::string &member, int64_t &value)> member;
};

// Integer evaluation; false when a leaf has no value in env.  Bound variables
// evaluate to their binding without consulting env.
bool evaluate(const Expr &e, const EvalEnv &env, int64_t &value);
bool evaluate(const Constraint &c, const EvalEnv &env, bool &value);

struct GeneratorOptions {
    bool xcd_remap = true;
    // With xcd_remap: rows of tiles per band (0 = one band per XCD); see Runner::Options.
    int xcd_band_rows = 0;
    // Instead: each XCD takes blocks of 4 x 8 tiles (see Runner::Options).
    bool xcd_tile_blocks = false;
    // Wavefronts per SIMD the kernel must leave room for (second argument of
    // __launch_bounds__): caps its registers at 512 / n.  0 = the compiler decides.
    int min_waves_per_simd = 0;
};

class CodeGenerator {
public:
    CodeGenerator(std::optional<std::vector<Parameter>> ordered_parameters = std::nullopt,
                  GeneratorOptions options = GeneratorOptions())
        : ordered_parameters(ordered_parameters), options(options) {
    }

    // Lowers and emits; returns the full source text.
    std::string generate_code(Composable c);

    std::string getName() const {
        return plan.function_name;
    }
    std::string getHookName() const {
        return "hook_" + plan.function_name;
    }
    std::vector<std::string> getArgumentOrder() const {
        return argument_order;
    }
    FunctionSignature getComputeFunctionSignature() const {
        return signature;
    }
    const LaunchPlan &getLaunchPlan() const {
        return plan;
    }
    std::vector<std::string> getHeaders() const {
        return std::vector<std::string>(headers.begin(), headers.end());
    }

private:
    std::optional<std::vector<Parameter>> ordered_parameters;
    GeneratorOptions options;
    LaunchPlan plan;
    FunctionSignature signature;
    std::vector<std::string> argument_order;
    std::set<std::string> headers;
};

}  // namespace codegen
}  // namespace gern
