// Annotations of the fused QK^T -> softmax gernels (gernels/qk_softmax.h).
// The softmax stages are the annotation classes of annot/softmax.h; only the
// data structures (a 16-row block of logits spread over a workgroup) and the
// logits producer are new.  Nothing in the reference corresponds to these.
#pragma once

#include "annot/mm.h"
#include "annot/softmax.h"

namespace gern {
namespace annot {

// Sixteen full rows of an fp32 matrix held in MFMA accumulators.
//   role OUTPUT : a window of the result matrix in HBM (stored on insert)
//   role TEMP   : registers only
class RowBlockF32 : public AbstractDataType {
public:
    enum Role { OUTPUT, TEMP };
    RowBlockF32(const std::string &name, Role role)
        : name(name), role(role) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return role == TEMP ? "auto" : "gernels::MatrixF32";
    }
    std::vector<Variable> getFields() const override {
        return {x, y, row, col};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{
            .name = "gernels::allocate_row_block",
            .template_args = {row, col},
        };
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{
            .name = "store_row_block",
            .args = {x, y},
        };
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{
            .name = "template view_row_block",
            .args = {x, y},
            .template_args = {row, col},
        };
    }
    bool insertQuery() const override {
        return role == OUTPUT;
    }
    bool freeAlloc() const override {
        return false;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        return MatrixF32("", MatrixF32::INPUT).readMember(object, member, value);
    }

private:
    std::string name;
    Role role;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// Per-row scalars of a row block.
class RowStat : public AbstractDataType {
public:
    explicit RowStat(const std::string &name)
        : name(name) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return "auto";
    }
    std::vector<Variable> getFields() const override {
        return {x, len};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{
            .name = "gernels::allocate_row_stat",
            .template_args = {len},
        };
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "unsupported_insert"};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "unsupported_query"};
    }
    bool freeAlloc() const override {
        return false;
    }

private:
    std::string name;
    Variable x{"x"};
    Variable len{"size", Datatype::Int64, true};
};

// logits(x.., y..) = scale * Q[x.., :] . K[y.., :]^T ; bind "d" to the head
// dimension.
class QKScaled : public AbstractFunction {
public:
    QKScaled(AbstractDataTypePtr Q, AbstractDataTypePtr K, AbstractDataTypePtr logits)
        : Q(Q), K(K), logits(logits) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), y("y");
        Variable l_x("l_x", Datatype::Int64, true), l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(logits, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(logits, "col", false), l_y,
                                 Produces::Subset(logits, {x, y, l_x, l_y}),
                                 Consumes::Subsets(SubsetObjMany({
                                     SubsetObj(Q, {x, Expr(0), l_x, d}),
                                     SubsetObj(K, {y, Expr(0), l_y, d}),
                                 }))))
            .occupies({Grid::Unit::THREAD_X});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::qk_scaled";
        f.args = {Parameter(Q), Parameter(K), Parameter(logits), Parameter(scale)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/qk_softmax.h"};
    }

private:
    AbstractDataTypePtr Q, K, logits;
    Variable d{"d", Datatype::Int64, true};
    Variable scale{"scale", Datatype::Float32};
};

// divide_vec for row blocks: a block spans ALL columns of its rows (the row
// statistics are those of whole rows), so the output may not be wider than
// one tile.  The launch is refused otherwise, and the generated kernel knows
// that its loop over column tiles runs once.
class DivideVecWholeRows : public DivideVec {
public:
    using DivideVec::DivideVec;
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
            .occupies({Grid::Unit::THREAD_X_IN_WRAPS})
            .assumes(Constraint(ADTMember(output, "col", false) <= l_y));
    }
};

}  // namespace annot
}  // namespace gern
