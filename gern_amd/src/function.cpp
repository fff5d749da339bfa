// Arguments, calls, and the construction of a call site from an
// AbstractFunction (reference behaviour: src/annotations/abstract_function.cpp:74-171,
// src/annotations/argument.cpp).
#include "gern/core/abstract_function.h"

#include <sstream>

namespace gern {

std::string Argument::str() const {
    std::stringstream ss;
    ss << *this;
    return ss.str();
}

bool Argument::isSameTypeAs(Argument other) const {
    return defined() && kind == other.kind;
}

std::string Argument::getType() const {
    switch (kind) {
    case DATA:
        return ds.getType();
    case EXPR:
        return e.getType().str();
    default:
        return "void";
    }
}

bool isSameArgument(Argument a, Argument b) {
    if (!a.defined() && !b.defined()) {
        return true;
    }
    if (a.isData() && b.isData()) {
        return a.getADTPtr() == b.getADTPtr();
    }
    if (a.isExpr() && b.isExpr()) {
        return isSameExpr(a.getExpr(), b.getExpr());
    }
    return false;
}

std::ostream &operator<<(std::ostream &os, const Argument &a) {
    if (a.isData()) {
        os << a.getADTPtr();
    } else if (a.isExpr()) {
        os << a.getExpr();
    }
    return os;
}

bool same_parameters(const std::vector<Parameter> &a, const std::vector<Parameter> &b) {
    std::multiset<std::string> vars_a, vars_b, adts_a, adts_b;
    for (const auto &p : a) {
        (p.isExpr() ? vars_a : adts_a).insert(p.isExpr() ? p.getVar().getName() : p.getADTPtr().getName());
    }
    for (const auto &p : b) {
        (p.isExpr() ? vars_b : adts_b).insert(p.isExpr() ? p.getVar().getName() : p.getADTPtr().getName());
    }
    return vars_a == vars_b && adts_a == adts_b;
}

std::vector<std::string> get_parameter_names(const std::vector<Parameter> &pars) {
    std::vector<std::string> names;
    for (const auto &p : pars) {
        names.push_back(p.isExpr() ? p.getVar().getName() : p.getADTPtr().getName());
    }
    return names;
}

LaunchArguments LaunchArguments::constructDefaults() const {
    LaunchArguments out = *this;
    if (!out.x.defined()) out.x = Expr(1);
    if (!out.y.defined()) out.y = Expr(1);
    if (!out.z.defined()) out.z = Expr(1);
    return out;
}

FunctionCall FunctionCall::replaceAllDS(std::map<AbstractDataTypePtr, AbstractDataTypePtr> replacement) const {
    FunctionCall out = *this;  // keeps smem_size and the launch shape
    for (auto &arg : out.args) {
        if (arg.isData()) {
            auto it = replacement.find(arg.getADTPtr());
            if (it != replacement.end()) {
                arg = Argument(it->second);
            }
        }
    }
    return out;
}

std::vector<Argument> FunctionCall::getAllArguments() const {
    std::vector<Argument> all(args.begin(), args.end());
    all.insert(all.end(), template_args.begin(), template_args.end());
    return all;
}

bool isSameFunctionCall(const FunctionCall &a, const FunctionCall &b) {
    if (a.name != b.name || a.args.size() != b.args.size() || a.template_args.size() != b.template_args.size()) {
        return false;
    }
    for (size_t i = 0; i < a.args.size(); i++) {
        if (!isSameArgument(a.args[i], b.args[i])) {
            return false;
        }
    }
    for (size_t i = 0; i < a.template_args.size(); i++) {
        if (!isSameArgument(a.template_args[i], b.template_args[i])) {
            return false;
        }
    }
    return true;
}

FunctionCall FunctionSignature::constructCall() const {
    FunctionCall call;
    call.name = name;
    for (const auto &p : args) {
        call.args.push_back(p);
    }
    for (const auto &t : template_args) {
        call.template_args.push_back(Argument(Expr(t)));
    }
    call.output = output;
    call.grid = grid;
    call.block = block;
    call.access = access;
    call.smem_size = smem_size;
    return call;
}

static void printCallLike(std::ostream &os, const std::string &name, const std::vector<Argument> &targs,
                          const std::vector<Argument> &args) {
    os << name;
    if (!targs.empty()) {
        os << "<";
        for (size_t i = 0; i < targs.size(); i++) {
            os << (i ? ", " : "") << targs[i];
        }
        os << ">";
    }
    os << "(";
    for (size_t i = 0; i < args.size(); i++) {
        os << (i ? ", " : "") << args[i];
    }
    os << ")";
}

std::ostream &operator<<(std::ostream &os, const FunctionCall &f) {
    if (f.output.defined()) {
        os << f.output.getType() << " " << f.output << " = ";
    }
    printCallLike(os, f.name, f.template_args, f.args);
    return os;
}

std::ostream &operator<<(std::ostream &os, const FunctionSignature &f) {
    return os << f.constructCall();
}

std::ostream &operator<<(std::ostream &os, const MethodCall &m) {
    return os << m.data << "." << m.call;
}

// ---------------------------------------------------------------------------
// AbstractFunction
// ---------------------------------------------------------------------------
Composable AbstractFunction::callSite(std::vector<Argument> concrete) {
    FunctionSignature f = getFunction();
    if (concrete.size() != f.args.size()) {
        throw error::UserError("Size of both arguments should be the same");
    }

    Substitution rename;
    for (size_t i = 0; i < concrete.size(); i++) {
        const Argument &formal = f.args[i];
        const Argument &actual = concrete[i];
        if (!formal.isSameTypeAs(actual)) {
            throw error::UserError("Type of " + formal.str() + " and " + actual.str() + " is not the same");
        }
        if (formal.isData()) {
            rename.structures[formal.getADTPtr().getName()] = actual.getADTPtr();
        } else {
            if (!isa<Variable>(actual.getExpr())) {
                throw error::UserError("Only variables can be passed for scalar parameters, got " + actual.str());
            }
            rename.variables[formal.getVar().getName()] = actual.getExpr();
        }
    }

    // Every call site gets its own copy of the annotation's variables:
    // bound ones take the binding, argument variables take the caller's name,
    // all others get a fresh unique name.
    auto fresh = [&](const Variable &v, bool force_const) -> Expr {
        auto b = bindings.find(v.getName());
        if (b != bindings.end()) {
            return b->second;
        }
        return Variable(getUniqueName("_gern_" + v.getName()), v.getDatatype(), force_const || v.isConstExpr());
    };
    for (const auto &t : f.template_args) {
        rename.variables[t.getName()] = fresh(t, true);
    }
    Annotation annotation = getAnnotation();
    for (const auto &v : getVariables(annotation)) {
        if (bindings.count(v.getName())) {
            rename.variables[v.getName()] = bindings.at(v.getName());
        } else if (!rename.variables.count(v.getName())) {
            rename.variables[v.getName()] = fresh(v, false);
        }
    }
    bindings.clear();  // one use only

    FunctionCall call;
    call.name = f.name;
    call.args = concrete;
    for (const auto &t : f.template_args) {
        call.template_args.push_back(Argument(rename.variables.at(t.getName())));
    }
    call.output = f.output;
    call.grid = LaunchArguments{substitute(f.grid.x, rename), substitute(f.grid.y, rename), substitute(f.grid.z, rename)};
    call.block = LaunchArguments{substitute(f.block.x, rename), substitute(f.block.y, rename), substitute(f.block.z, rename)};
    call.access = f.access;
    call.smem_size = Expr();

    return Composable(new const ComputeFunctionCall(call, substitute(annotation, rename), getHeader()));
}

FunctionPtr::FunctionPtr(Composable function, Runner::Options options,
                         std::optional<std::vector<Parameter>> ordered_parameters)
    : pipeline(function), compile_options(options) {
    Runner runner(function, ordered_parameters);
    runner.compile(options);
    compiled_signature = runner.getSignature();
}

Annotation FunctionPtr::getAnnotation() {
    return pipeline.getAnnotation();
}

std::vector<std::string> FunctionPtr::getHeader() {
    return {compile_options.filename};
}

FunctionSignature FunctionPtr::getFunction() {
    return compiled_signature;
}

}  // namespace gern
