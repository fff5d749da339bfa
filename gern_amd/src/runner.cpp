// Runner: generate, compile, launch (see gern/runtime/runner.h).
#include "gern/runtime/runner.h"

#include "gern/codegen/codegen.h"
#include "gern_hip.h"

#include <cstdlib>
#include <dlfcn.h>
#include <fstream>
#include <sstream>

namespace gern {

namespace {

std::string lastHipError() {
    std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
    gern_hip_last_error(msg.data(), msg.size());
    msg.resize(msg.size() - 1);
    return msg;
}

// "-I a -Ib  -I c" -> {"-Ia", "-Ib", "-Ic"}; anything else is passed through.
std::vector<std::string> splitIncludeFlags(const std::string &flags) {
    std::vector<std::string> out;
    std::istringstream in(flags);
    std::string tok;
    while (in >> tok) {
        if (tok == "-I") {
            std::string dir;
            if (in >> dir) {
                out.push_back("-I" + dir);
            }
        } else {
            out.push_back(tok);
        }
    }
    return out;
}

}  // namespace

Runner::Runner(Composable c, std::optional<std::vector<Parameter>> ordered_parameters)
    : c(c), ordered_parameters(ordered_parameters) {
}

int64_t Runner::ldsOverflows() {
    if (module == nullptr) {
        return 0;
    }
    void *at = nullptr;
    size_t bytes = 0;
    uint32_t count = 0;
    if (gern_hip_module_global(static_cast<gern_hip_module>(module), "gern_lds_overflows", &at, &bytes) != GERN_HIP_OK) {
        throw error::UserError("Cannot look up the LDS overflow count: " + lastHipError());
    }
    if (at == nullptr) {
        return 0;
    }
    if (bytes != sizeof(count) || gern_hip_sync() != GERN_HIP_OK || gern_hip_memcpy_d2h(&count, at, sizeof(count)) != GERN_HIP_OK) {
        throw error::UserError("Cannot read the LDS overflow count: " + lastHipError());
    }
    return count;
}

Runner::~Runner() {
    // The module stays loaded for the life of the process, like the
    // reference's dlopen handle: kernels may still be in flight.
}

void Runner::release() {
    if (module == nullptr) {
        return;
    }
    if (gern_hip_sync() == GERN_HIP_OK) {
        gern_hip_module_unload(static_cast<gern_hip_module>(module));
    }  // else: the device is in an error state; leave the module alone
    module = nullptr;
    kernel = nullptr;
    compiled = false;
}

void Runner::compile(Options config) {
    codegen::GeneratorOptions gen_options;
    gen_options.xcd_remap = config.xcd_remap;
    gen_options.xcd_tile_blocks = config.xcd_tile_blocks;
    gen_options.xcd_band_rows = config.xcd_band_rows;
    gen_options.min_waves_per_simd = config.min_waves_per_simd;
    codegen::CodeGenerator cg(ordered_parameters, gen_options);
    source = cg.generate_code(c);
    signature = cg.getComputeFunctionSignature();
    argument_order = cg.getArgumentOrder();
    stream = config.stream;

    const std::string file = config.prefix + "/" + config.filename;
    if (!config.filename.empty()) {
        std::ofstream out(file);
        out << source;
    }

    if (cg.getLaunchPlan().device_function) {
        // A __device__ function is only ever #included by another generated
        // kernel; the file written above is the whole product.
        if (config.filename.empty()) {
            throw error::UserError("Runner::Options::filename must be set for a device function: callers include that file");
        }
        compiled = false;  // it cannot be evaluated on its own
        return;
    }
    if (c.isDeviceLaunch()) {
        plan = std::make_shared<codegen::LaunchPlan>(cg.getLaunchPlan());
        std::vector<std::string> flags = splitIncludeFlags(config.include);
        // Device functions made by FunctionPtr are written under prefix.
        flags.push_back("-I" + config.prefix);
        std::vector<const char *> options;
        for (const auto &f : flags) {
            options.push_back(f.c_str());
        }
        const char *name_exprs[1] = {plan->name_expression.c_str()};
        gern_hip_module mod = nullptr;
        int rc = gern_hip_compile(source.c_str(), name_exprs, 1, options.data(), (int)options.size(),
                                  config.arch.empty() ? nullptr : config.arch.c_str(), &mod);
        if (rc == GERN_HIP_ERR_COMPILE) {
            throw error::UserError("Compilation Failed\n" + lastHipError());
        }
        if (rc != GERN_HIP_OK) {
            throw error::UserError("Cannot load the generated kernel: " + lastHipError());
        }
        gern_hip_kernel k = nullptr;
        rc = gern_hip_get_kernel(mod, plan->name_expression.c_str(), &k);
        if (rc != GERN_HIP_OK) {
            throw error::UserError("Error loading function: " + lastHipError());
        }
        module = mod;
        kernel = k;
        compiled = true;
        return;
    }

    const std::string shared_obj = config.prefix + "/" + getUniqueName("libGern") + ".so";
    const std::string cmd = "g++ -std=" + config.cpp_std + " -O2 -fPIC " + config.include + " --shared -o " +
                            shared_obj + " " + file + " " + config.ldflags + " 2>&1";
    if (config.filename.empty()) {
        throw error::UserError("Runner::Options::filename must be set for a host pipeline");
    }
    if (std::system(cmd.c_str()) != 0) {
        throw error::UserError("Compilation Failed");
    }
    void *handle = dlopen(shared_obj.c_str(), RTLD_LAZY);
    if (!handle) {
        throw error::UserError("Error loading library: " + std::string(dlerror()));
    }
    void *func = dlsym(handle, cg.getHookName().c_str());
    if (!func) {
        throw error::UserError("Error loading function: " + std::string(dlerror()));
    }
    fp = (GernGenFuncPtr)func;
    compiled = true;
}

void Runner::evaluate(std::map<std::string, void *> args) {
    if (!compiled) {
        throw error::UserError("Please compile the pipeline first");
    }
    const size_t num_args = argument_order.size();
    if (args.size() != num_args) {
        throw error::UserError("Incorrect number of args passed! Expecting " + std::to_string(num_args) + " args");
    }
    std::vector<void *> in_order;
    for (const auto &name : argument_order) {
        auto it = args.find(name);
        if (it == args.end()) {
            throw error::UserError("Argument " + name + "was not passed in");
        }
        in_order.push_back(it->second);
    }

    if (!c.isDeviceLaunch()) {
        fp(in_order.data());
        return;
    }

    // Host side of a device launch: read launch dimensions and assumptions
    // off the caller's objects, then hand the same void** to the kernel.
    std::map<std::string, Datatype> var_types;
    for (const auto &p : plan->parameters) {
        if (p.isExpr()) {
            var_types[p.getVar().getName()] = p.getVar().getDatatype();
        }
    }
    codegen::EvalEnv env;
    env.variable = [&](const std::string &name, int64_t &value) {
        auto it = args.find(name);
        auto ty = var_types.find(name);
        if (it == args.end() || ty == var_types.end() || !(ty->second == Datatype(Datatype::Int64))) {
            return false;
        }
        value = *static_cast<const int64_t *>(it->second);
        return true;
    };
    env.member = [&](const AbstractDataTypePtr &ds, const std::string &member, int64_t &value) {
        auto it = args.find(ds.getName());
        return it != args.end() && ds.readMember(it->second, member, value);
    };

    for (const auto &assumption : plan->host_asserts) {
        // The kernel was compiled to rely on every one of these, so one that cannot be checked
        // here refuses the launch just as one that fails.
        bool holds = true;
        if (!codegen::evaluate(assumption, env, holds)) {
            throw error::UserError("Cannot check the assumption " + assumption.str() +
                                   " on the host: a data structure whose members appear in an assumption of a "
                                   "device kernel must implement AbstractDataType::readMember");
        }
        if (!holds) {
            throw error::UserError("Assumption violated at launch: " + assumption.str());
        }
    }
    auto dimension = [&](const Expr &e, const char *what) -> uint32_t {
        int64_t v = 0;
        if (!codegen::evaluate(e, env, v)) {
            throw error::UserError(std::string("Cannot evaluate the ") + what + " " + e.str() +
                                   " on the host: a data structure whose members size the launch must implement "
                                   "AbstractDataType::readMember");
        }
        if (v <= 0 || v > 0x7fffffffLL) {
            throw error::UserError(std::string("The ") + what + " " + e.str() + " evaluates to " + std::to_string(v));
        }
        return (uint32_t)v;
    };
    uint32_t grid[3], block[3];
    for (int i = 0; i < 3; i++) {
        grid[i] = dimension(plan->grid[i], "grid dimension");
        block[i] = dimension(plan->block[i], "block dimension");
    }
    uint32_t lds = plan->lds_bytes.defined() ? dimension(plan->lds_bytes, "LDS size") : 0;

    int rc = gern_hip_launch((gern_hip_kernel)kernel, grid, block, lds, in_order.data(), stream);
    if (rc != GERN_HIP_OK) {
        throw error::UserError("Kernel launch failed: " + lastHipError());
    }
}

FunctionSignature Runner::getSignature() const {
    return signature;
}

std::string Runner::getSource() const {
    return source;
}

std::string Runner::getKernelName() const {
    return plan ? plan->name_expression : std::string();
}

void evaluate(Composable c, std::map<std::string, void *> args, Runner::Options config) {
    Runner runner(c);
    runner.compile(config);
    runner.evaluate(args);
}

}  // namespace gern
