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
    AbstractFunction() = default;
    virtual ~AbstractFunction() = default;
    virtual Annotation getAnnotation() = 0;
    virtual std::vector<std::string> getHeader() = 0;
    virtual FunctionSignature getFunction() = 0;

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
        return constructComposableObject(arguments);
    }

    template<typename FirstT, typename... Next>
    Composable construct(FirstT first, Next... remaining) {
        std::vector<Argument> arguments;
        addArguments(arguments, first, remaining...);
        return constructComposableObject(arguments);
    }

private:
    Composable constructComposableObject(std::vector<Argument> concrete_arguments);
    std::map<std::string, Variable> bindings;
};

class FunctionPtr : public AbstractFunction {
public:
    FunctionPtr(Composable function, Runner::Options options,
                std::optional<std::vector<Parameter>> ordered_parameters = std::nullopt);
    Annotation getAnnotation() override;
    std::vector<std::string> getHeader() override;
    FunctionSignature getFunction() override;

private:
    Composable function;
    Runner::Options options;
    FunctionSignature signature;
};

}  // namespace gern
