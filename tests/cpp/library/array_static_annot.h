// Annotations of array_static_host.h.
// Mirrors test/library/array/annot/cpu-array-template.h:11-114 of the reference.
#pragma once

#include "annotations/abstract_function.h"

namespace gern {
namespace annot {

template<int Size>
class ArrayCPUTemplate : public AbstractDataType {
public:
    ArrayCPUTemplate(const std::string &name = "test", bool temp = false)
        : name(name), temp(temp) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        // A temporary's length is only known where it is allocated.
        return temp ? "auto" : "gern::impl::ArrayCPUTemplate<" + std::to_string(Size) + ">";
    }
    std::vector<Variable> getFields() const override {
        return {x, len};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::temp_allocate", .template_args = {len}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "query", .args = {x}, .template_args = {len}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert", .args = {x}, .template_args = {len}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy", .args = {}};
    }
    bool insertQuery() const override {
        return true;
    }
    bool freeAlloc() const override {
        return false;
    }

protected:
    std::string name;
    bool temp;
    Variable x{"x"};
    Variable len{"len"};
};

class addStaticStore : public AbstractFunction {
public:
    addStaticStore()
        : input(new const ArrayCPUTemplate<10>("input")), output(new const ArrayCPUTemplate<10>("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        return annotate(Tileable(x = Expr(0), output["size"], step,
                                 Produces::Subset(output, {x, step}),
                                 Consumes::Subset(input, {x, step})));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add";
        f.args = {Parameter(input), Parameter(output)};
        f.template_args = {step};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"array_static_host.h"};
    }

protected:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable step{"step"};
};

}  // namespace annot
}  // namespace gern
