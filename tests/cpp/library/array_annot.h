// Annotations of the host array library (array_host.h): the data structure and
// the functions, as the lowering tests introduce them to Gern.
//
// Mirrors the reference's test annotations
// (test/library/array/annot/cpu-array.h:12-203).
#pragma once

#include "annot_table.h"

namespace gern {
namespace annot {

class ArrayCPU : public TableADT {
public:
    ArrayCPU(const std::string &name = "test")
        : TableADT(name, "gern::impl::ArrayCPU") {
        fields = {x, len};
        allocate_call = call("gern::impl::ArrayCPU::allocate", fields);
        query_call = call("query", fields);
        insert_call = call("insert", fields);
    }
    // The alternative names that Stage(...) tests swap in.
    FunctionSignature newStageFunction() const {
        return call("new_stage", fields);
    }
    FunctionSignature getNewInsertFunction() const {
        return call("new_insert", fields);
    }

protected:
    Variable x{"x"};
    Variable len{"len"};
};

struct add_1 : PiecewiseArrayFunction {
    explicit add_1(const std::string &function = "gern::impl::add_1")
        : PiecewiseArrayFunction(function, "array_host.h", AbstractDataTypePtr(new const ArrayCPU("input")),
                                 AbstractDataTypePtr(new const ArrayCPU("output"))) {
    }
};

struct add_1_float : add_1 {
    add_1_float()
        : add_1("gern::impl::add_1_float") {
    }

protected:
    std::vector<Variable> trailing_arguments() const override {
        return {float_val};
    }
    Variable float_val{"float_val", Datatype::Float32};
};

struct add1Template : add_1 {
    add1Template()
        : add_1("gern::impl::add1Template") {
    }

protected:
    bool step_is_a_template_argument() const override {
        return true;
    }
};

// Takes its step as a third argument; only call-site checks use it.
struct addWithSize : add_1 {
    addWithSize()
        : add_1("gern::impl::addWithSize") {
    }

protected:
    std::vector<Variable> trailing_arguments() const override {
        return {step};
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

// A data structure without index fields: one float.
class ScalarCPU : public TableADT {
public:
    ScalarCPU(const std::string &name = "scalar")
        : TableADT(name, "gern::impl::ScalarCPU") {
        allocate_call = call("gern::impl::ScalarCPU::allocate");
        query_call = call("open");
    }
};

// *output = input[0]: consumes the array's first element, produces the whole (field-less) scalar.
class first_element : public AbstractFunction {
public:
    first_element()
        : input(new const ArrayCPU("input")), output(new const ScalarCPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable one("one");
        return annotate(Computes(Produces::Subset(output, {}), Consumes::Subsets(SubsetObjMany{SubsetObj(input, {Expr(0), Expr(1)})})));
    }
    std::vector<std::string> getHeader() override {
        return {"array_host.h"};
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::first_element";
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }

protected:
    AbstractDataTypePtr input, output;
};

// output[x .. x+step) = input[x .. x+step) + *scalar
class add_scalar : public AbstractFunction {
public:
    add_scalar()
        : input(new const ArrayCPU("input")), scalar(new const ScalarCPU("scalar")), output(new const ArrayCPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), step("step");
        return annotate(Tileable(x = Expr(0), output["size"], step, Produces::Subset(output, {x, step}),
                                 Consumes::Subsets(SubsetObjMany{SubsetObj(input, {x, step}), SubsetObj(scalar, {})})));
    }
    std::vector<std::string> getHeader() override {
        return {"array_host.h"};
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add_scalar";
        f.args = {Parameter(input), Parameter(scalar), Parameter(output)};
        return f;
    }

protected:
    AbstractDataTypePtr input, scalar, output;
};

}  // namespace annot
}  // namespace gern
