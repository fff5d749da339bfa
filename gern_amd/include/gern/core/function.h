// Arguments, parameters, function signatures and function calls: the pieces a
// data structure or a compute function uses to tell the code generator what
// text to emit for "call this".
//
// Names and aggregate field order follow the reference
// (include/gern/annotations/argument.h:43-166, compose/compose.h:13-85,
// annotations/shared_memory_manager.h:14-45) because user code initialises
// these structs with designated initialisers.
#pragma once

#include "gern/core/lang.h"

#include <iostream>
#include <string>
#include <vector>

namespace gern {

// Either a data structure or an integer/float expression.
class Argument {
public:
    enum Kind { NONE, DATA, EXPR };

    Argument() = default;
    Argument(AbstractDataTypePtr ds)
        : kind(DATA), ds(ds) {
    }
    Argument(Expr e)
        : kind(e.defined() ? EXPR : NONE), e(e) {
    }

    bool defined() const {
        return kind != NONE;
    }
    bool isData() const {
        return kind == DATA;
    }
    bool isExpr() const {
        return kind == EXPR;
    }
    AbstractDataTypePtr getADTPtr() const {
        return ds;
    }
    Expr getExpr() const {
        return e;
    }
    Variable getVar() const {
        assert(isa<Variable>(e));
        return to<Variable>(e);
    }
    std::string str() const;
    // Both data structures, or both expressions.
    bool isSameTypeAs(Argument) const;
    // The C++ type this argument has in generated code ("void" when empty).
    std::string getType() const;

private:
    Kind kind = NONE;
    AbstractDataTypePtr ds;
    Expr e;
};

bool isSameArgument(Argument a, Argument b);
std::ostream &operator<<(std::ostream &, const Argument &);

// A formal parameter: a variable or a data structure, never a compound
// expression.
class Parameter : public Argument {
public:
    Parameter() = default;
    Parameter(Variable v)
        : Argument(Expr(v)) {
    }
    explicit Parameter(AbstractDataTypePtr ds)
        : Argument(ds) {
    }
};

// Same multiset of data structures (by name) and of variable names.
bool same_parameters(const std::vector<Parameter> &a, const std::vector<Parameter> &b);
std::vector<std::string> get_parameter_names(const std::vector<Parameter> &pars);

inline void addArgument(std::vector<Argument> &v, AbstractDataTypePtr ds) {
    v.push_back(Argument(ds));
}
inline void addArgument(std::vector<Argument> &v, Variable var) {
    v.push_back(Argument(Expr(var)));
}
inline void addArgument(std::vector<Argument> &v, Argument a) {
    if (!a.defined()) {
        throw error::UserError("Calling with an empty argument");
    }
    v.push_back(a);
}
inline void addArguments(std::vector<Argument> &) {
}
template<typename T, typename... Next>
inline void addArguments(std::vector<Argument> &v, T first, Next... next) {
    addArgument(v, first);
    addArguments(v, next...);
}

enum Access {
    HOST,
    GLOBAL,
    DEVICE,
};

struct LaunchArguments {
    Expr x = Expr();
    Expr y = Expr();
    Expr z = Expr();
    // Undefined components become 1.
    LaunchArguments constructDefaults() const;
};

// A concrete call: name, run-time arguments, template arguments, optional
// result, and (for a kernel) its launch shape.
struct FunctionCall {
    std::string name;
    std::vector<Argument> args;
    std::vector<Argument> template_args;
    Parameter output = Parameter();
    LaunchArguments grid;
    LaunchArguments block;
    Access access = HOST;
    Expr smem_size = Expr();

    FunctionCall replaceAllDS(std::map<AbstractDataTypePtr, AbstractDataTypePtr> replacement) const;
    std::vector<Argument> getAllArguments() const;
};

bool isSameFunctionCall(const FunctionCall &a, const FunctionCall &b);

struct MethodCall {
    AbstractDataTypePtr data;  // object the method is called on
    FunctionCall call;
};

// A declaration: name, formal parameters, template parameters (all int64_t),
// optional result.
struct FunctionSignature {
    std::string name;
    std::vector<Parameter> args = {};
    std::vector<Variable> template_args = {};
    Parameter output = Parameter();
    LaunchArguments grid = LaunchArguments();
    LaunchArguments block = LaunchArguments();
    Access access = HOST;
    bool device = false;
    Variable smem_size = Variable();

    FunctionCall constructCall() const;
};

std::ostream &operator<<(std::ostream &, const FunctionSignature &);
std::ostream &operator<<(std::ostream &, const FunctionCall &);
std::ostream &operator<<(std::ostream &, const MethodCall &);

namespace grid {

// Names the device function that initialises the dynamic-LDS allocator at the
// top of a kernel, and the header that declares the allocator.
class SharedMemoryManager {
public:
    SharedMemoryManager() = default;
    SharedMemoryManager(FunctionCall init, std::vector<std::string> headers = {})
        : init(init), headers(headers), initialized(true) {
    }
    FunctionCall getInit() const {
        return init;
    }
    std::vector<std::string> getHeaders() const {
        return headers;
    }
    bool isInitialized() const {
        return initialized;
    }

private:
    FunctionCall init{"", {}, {}, Parameter(), LaunchArguments(), LaunchArguments(), DEVICE, Expr()};
    std::vector<std::string> headers;
    bool initialized = false;
};

}  // namespace grid
}  // namespace gern
