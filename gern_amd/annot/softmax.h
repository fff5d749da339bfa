// Annotations of the row-softmax gernels (gernels/softmax.h).
//
// Counterpart of the reference's apps/common/annot/functions.h:9-173.  Two
// things differ from the reference's text, both because its versions do not
// lower to working code (its only softmax test is commented out,
// test/test-cpu-matrix.cpp:69-148): a row reduction consumes the full row
// width through a variable `ncol` that the caller binds, and the element-wise
// functions are tileable over the columns of their output so that the caller
// fixes the tile width by tiling.
#pragma once

#include "annot/matrix.h"

namespace gern {
namespace annot {

// output[x .. x+l_x) = reduce over the columns of input rows [x .. x+l_x)
class MaxRow : public AbstractFunction {
public:
    MaxRow(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : input(input), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        Variable l_x("l_x", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "size", false), l_x,
                        Produces::Subset(output, {x, l_x}),
                        Consumes::Subset(input, {x, Expr(0), l_x, ncol}))
            .occupies({Grid::Unit::THREAD_X_IN_WRAPS});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = functionName();
        f.args = {Parameter(output), Parameter(input)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/softmax.h"};
    }

protected:
    virtual std::string functionName() {
        return "gernels::max_row";
    }
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable ncol{"ncol", Datatype::Int64, true};
};

class SumRow : public MaxRow {
public:
    SumRow(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : MaxRow(input, output) {
    }

protected:
    std::string functionName() override {
        return "gernels::sum_row";
    }
};

// output(x.., y..) = input(x.., y..) - vec[x..]
class SubtractVec : public AbstractFunction {
public:
    SubtractVec(AbstractDataTypePtr vec, AbstractDataTypePtr input, AbstractDataTypePtr output)
        : vec(vec), input(input), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        Variable y("y");
        Variable l_x("l_x", Datatype::Int64, true);
        Variable l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(output, "col", false), l_y,
                                 Produces::Subset(output, {x, y, l_x, l_y}),
                                 Consumes::Subsets(SubsetObjMany({
                                     SubsetObj(input, {x, y, l_x, l_y}),
                                     SubsetObj(vec, {x, l_x}),
                                 }))))
            .occupies({Grid::Unit::THREAD_X_IN_WRAPS});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = functionName();
        f.args = {Parameter(vec), Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/softmax.h"};
    }

protected:
    virtual std::string functionName() {
        return "gernels::subtract_vec";
    }
    AbstractDataTypePtr vec;
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

class DivideVec : public SubtractVec {
public:
    DivideVec(AbstractDataTypePtr vec, AbstractDataTypePtr input, AbstractDataTypePtr output)
        : SubtractVec(vec, input, output) {
    }

protected:
    std::string functionName() override {
        return "gernels::divide_vec";
    }
};

class ExpMatrix : public AbstractFunction {
public:
    ExpMatrix(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : input(input), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        Variable y("y");
        Variable l_x("l_x", Datatype::Int64, true);
        Variable l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(output, "col", false), l_y,
                                 Produces::Subset(output, {x, y, l_x, l_y}),
                                 Consumes::Subset(input, {x, y, l_x, l_y})))
            .occupies({Grid::Unit::THREAD_X_IN_WRAPS});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::exp_matrix";
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/softmax.h"};
    }

protected:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

// A row-major fp32 matrix whose subsets are rows spread over the `waves`
// wavefronts of a workgroup (gernels::BlockTile); the launch must give the
// workgroup exactly that many wavefronts.  Roles as for MatrixF32.
class BlockRowsF32 : public MatrixF32 {
public:
    BlockRowsF32(const std::string &name, Role role, int waves)
        : MatrixF32(name, role) {
        // the wavefront count is part of the gernel names: load_block8, ...
        const std::string n = std::to_string(waves);
        setCalls("gernels::allocate_block_tile" + n, (role == OUTPUT ? "template view_block" : "template load_block") + n,
                 "store_block");
    }
};

}  // namespace annot
}  // namespace gern
