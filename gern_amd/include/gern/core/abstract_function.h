// AbstractFunction: how a user function is introduced to the system (its
// annotation, its header, its signature), and how a call site is built from
// it.  FunctionPtr wraps an already-composed pipeline as such a function.
//
// Interface as in the reference (include/gern/annotations/abstract_function.h:22-92).
#pragma once

#include "gern/core/composable.h"
#include "gern/runtime/runner.h"

namespace gern {

class AbstractFunction {
public:
    // What an implementer supplies: the data-dependency annotation, the
    // signature that calls are printed from, and the headers that declare it.
    virtual FunctionSignature getFunction() = 0;
    virtual Annotation getAnnotation() = 0;
    virtual std::vector<std::string> getHeader() = 0;

    AbstractFunction() = default;
    virtual ~AbstractFunction() = default;

    // Binds annotation variables (by name) for the NEXT call site only.
    AbstractFunction &operator[](const std::map<std::string, Variable> &replacements) {
        bindings.insert(replacements.begin(), replacements.end());
        return *this;
    }

    template<typename... Args>
    Composable operator()(Args... args) {
        std::vector<Argument> arguments;
        addArguments(arguments, args...);
        if (sizeof...(Args) == 0 && getFunction().args.size() != 0) {
            throw error::UserError("Called FunctionSignature " + getFunction().name + " with 0 arguments");
        }
        return callSite(std::move(arguments));
    }

    template<typename FirstT, typename... Next>
    Composable construct(FirstT first, Next... remaining) {
        std::vector<Argument> arguments;
        addArguments(arguments, first, remaining...);
        return callSite(std::move(arguments));
    }

private:
    // Checks the arguments against the signature, renames the annotation's
    // variables apart, applies and clears the pending bindings.
    Composable callSite(std::vector<Argument> concrete);
    std::map<std::string, Variable> bindings;  // pending, for the next call site
};

class FunctionPtr : public AbstractFunction {
public:
    FunctionPtr(Composable function, Runner::Options options,
                std::optional<std::vector<Parameter>> ordered_parameters = std::nullopt);
    FunctionSignature getFunction() override;      // the compiled pipeline's own signature
    Annotation getAnnotation() override;           // the pipeline's annotation
    std::vector<std::string> getHeader() override; // the file the pipeline was written to

private:
    Composable pipeline;
    Runner::Options compile_options;
    FunctionSignature compiled_signature;
};

}  // namespace gern
