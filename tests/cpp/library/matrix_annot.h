// Annotations of matrix_host.h.
// Mirrors test/library/matrix/annot/cpu-matrix.h:12-126,257-305 of the reference.
#pragma once

#include "annotations/abstract_function.h"

namespace gern {
namespace annot {

class MatrixCPU : public AbstractDataType {
public:
    MatrixCPU(const std::string &name = "test")
        : name(name) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return "gern::impl::MatrixCPU";
    }
    std::vector<Variable> getFields() const override {
        return {x, y, l_x, l_y};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::MatrixCPU::allocate", .args = {x, y, l_x, l_y}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy", .args = {}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert", .args = {x, y, l_x, l_y}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "query", .args = {x, y, l_x, l_y}};
    }
    bool insertQuery() const override {
        return true;
    }

protected:
    std::string name;
    Variable x{"x"}, y{"y"}, l_x{"l_x"}, l_y{"l_y"};
};

// A temporary that must start from zero (an accumulator).
class MatrixCPUZero : public MatrixCPU {
public:
    using MatrixCPU::MatrixCPU;
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::MatrixCPU::allocate_zero", .args = {x, y, l_x, l_y}};
    }
};

class MatrixAddCPU : public AbstractFunction {
public:
    MatrixAddCPU()
        : input(new const MatrixCPU("input")), output(new const MatrixCPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), y("y"), l_x("l_x"), l_y("l_y");
        return annotate(Tileable(x = Expr(0), output["row"], l_x,
                                 Tileable(y = Expr(0), output["col"], l_y,
                                          Produces::Subset(output, {x, y, l_x, l_y}),
                                          Consumes::Subset(input, {x, y, l_x, l_y}))));
    }
    std::vector<std::string> getHeader() override {
        return {"matrix_host.h"};
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add";
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }

protected:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

class MatrixMultiplyCPU : public AbstractFunction {
public:
    MatrixMultiplyCPU()
        : A(new const MatrixCPU("A")), B(new const MatrixCPU("B")), C(new const MatrixCPU("C")) {
    }
    Annotation getAnnotation() override {
        Variable i("i"), j("j"), k("k");
        Variable ti("ti", Datatype::Int64), tj("tj", Datatype::Int64), tk("tk", Datatype::Int64);
        return annotate(Tileable(i = Expr(0), ADTMember(C, "row", false), ti,
                                 Tileable(j = Expr(0), ADTMember(C, "col", false), tj,
                                          Produces::Subset(C, {i, j, ti, tj}),
                                          Consumes::Subsets(Reducible(k = Expr(0), k_dim, tk,
                                                                      SubsetObjMany({
                                                                          SubsetObj(A, {i, k, ti, tk}),
                                                                          SubsetObj(B, {k, j, tk, tj}),
                                                                      }))))));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::matrix_multiply";
        f.args = {Parameter(A), Parameter(B), Parameter(C), k_dim};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"matrix_host.h"};
    }

private:
    AbstractDataTypePtr A, B, C;
    Variable k_dim{"k_dim", Datatype::Int64};
};

}  // namespace annot
}  // namespace gern
