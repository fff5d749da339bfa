// Annotations of the host array library (array_host.h): the data structure and
// the functions, as the lowering tests introduce them to Gern.
//
// Mirrors the reference's test annotations
// (test/library/array/annot/cpu-array.h:12-203).
#pragma once

#include "annotations/abstract_function.h"

#include <string>
#include <vector>

namespace gern {
namespace annot {

class ArrayCPU : public AbstractDataType {
public:
    ArrayCPU(const std::string &name = "test")
        : name(name) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return "gern::impl::ArrayCPU";
    }
    std::vector<Variable> getFields() const override {
        return {x, len};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::ArrayCPU::allocate", .args = {x, len}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy", .args = {}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert", .args = {x, len}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "query", .args = {x, len}};
    }
    // The alternative names that Stage(...) tests swap in.
    FunctionSignature newStageFunction() const {
        return FunctionSignature{.name = "new_stage", .args = {x, len}};
    }
    FunctionSignature getNewInsertFunction() const {
        return FunctionSignature{.name = "new_insert", .args = {x, len}};
    }

protected:
    std::string name;
    Variable x{"x"};
    Variable len{"len"};
};

class add_1 : public AbstractFunction {
public:
    add_1()
        : input(new const ArrayCPU("input")), output(new const ArrayCPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        return annotate(Tileable(x = Expr(0), output["size"], step,
                                 Produces::Subset(output, {x, step}),
                                 Consumes::Subset(input, {x, step})));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add_1";
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"array_host.h"};
    }

protected:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable step{"step"};
};

class add_1_float : public add_1 {
public:
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add_1_float";
        f.args = {Parameter(input), Parameter(output), Parameter(float_val)};
        return f;
    }

protected:
    Variable float_val{"float_val", Datatype::Float32};
};

class add1Template : public add_1 {
public:
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add1Template";
        f.args = {Parameter(input), Parameter(output)};
        f.template_args = {step};
        return f;
    }
};

// Takes its step as a third argument; only call-site checks use it.
class addWithSize : public add_1 {
public:
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::addWithSize";
        f.args = {Parameter(input), Parameter(output), Parameter(step)};
        return f;
    }
};

// A reduction loop inside the consumes clause.
class reduction : public AbstractFunction {
public:
    reduction()
        : input(new const ArrayCPU("input")), output(new const ArrayCPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), r("r"), step("step"), reduce("reduce");
        return annotate(Tileable(x = Expr(0), output["size"], step,
                                 Computes(Produces::Subset(output, {x, step}),
                                          Consumes::Subsets(Reducible(r = Expr(0), k, reduce,
                                                                      SubsetObjMany{SubsetObj(input, {r, reduce})})))));
    }
    std::vector<std::string> getHeader() override {
        return {"array_host.h"};
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::reduction";
        f.args = {Parameter(input), Parameter(output), Parameter(k)};
        return f;
    }

protected:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable k{"k"};
};

}  // namespace annot
}  // namespace gern
