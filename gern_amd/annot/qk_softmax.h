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
        return {"gernels/qk_softmax.h", "gernels/qk_tiles.h"};
    }

private:
    AbstractDataTypePtr Q, K, logits;
    Variable d{"d", Datatype::Int64, true};
    Variable scale{"scale", Datatype::Float32};
};

// A 256 x 256 tile of scores spread over the eight wavefronts of a workgroup
// (gernels/qk_tiles.h).
//   role OUTPUT : a window of the result matrix in HBM (stored on insert)
//   role TEMP   : registers only
class ScoreTileF32 : public TableADT {
public:
    enum Role { OUTPUT, TEMP };
    ScoreTileF32(const std::string &name, Role role)
        : TableADT(name, role == TEMP ? "auto" : "gernels::MatrixF32") {
        fields = {x, y, row, col};
        allocate_call = call("gernels::allocate_score_tile", {}, {row, col});
        query_call = call("template view_score_tile", {x, y}, {row, col});
        insert_call = call("store_score_tile", {x, y});
        query_is_written_back = role == OUTPUT;
        temporaries_are_freed = false;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        return MatrixF32("", MatrixF32::INPUT).readMember(object, member, value);
    }

private:
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// Layout of the object handed to Runner::evaluate for a RowStatsExchange
// (gernels::RowStatsExchange): device memory, all zeros before its first use.
struct RowStatsExchangeLayout {
    void *entries;       // `capacity` entries of 8 bytes: rows (padded to the tile height) x pitch of them are used
    void *state;         // four 32-bit words: launch number, workgroups done, wavefronts that gave up, rows that did not fit
    int32_t pitch;       // entries per row: at least the number of column blocks
    int32_t spin_limit;  // polls before a wavefront gives up
    int64_t capacity;
};

// Where the workgroups of a row block meet (gernels/qk_tiles.h).  No fields and
// no subsets; its query opens the launch's session, which the code generator
// places at the top of the kernel because it depends on no loop.
class RowStatsExchange : public TableADT {
public:
    explicit RowStatsExchange(const std::string &name)
        : TableADT(name, "gernels::RowStatsExchange") {
        query_call = call("open");
        free_call = FunctionSignature{};
    }
};

// out = the softmax over WHOLE rows of the matrix that `input` is a tile of
// scaled products of; the tiles of a row block exchange their row statistics
// through `exchange` (gernels::softmax_rows_across_tiles).
class SoftmaxAcrossTiles : public AbstractFunction {
public:
    SoftmaxAcrossTiles(AbstractDataTypePtr input, AbstractDataTypePtr exchange, AbstractDataTypePtr output)
        : input(input), exchange(exchange), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), y("y");
        Variable l_x("l_x", Datatype::Int64, true), l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(output, "col", false), l_y,
                                 Produces::Subset(output, {x, y, l_x, l_y}),
                                 Consumes::Subsets(SubsetObjMany({
                                     SubsetObj(input, {x, y, l_x, l_y}),
                                     SubsetObj(exchange, {}),
                                 }))))
            .occupies({Grid::Unit::THREAD_X});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::softmax_rows_across_tiles";
        f.args = {Parameter(input), Parameter(exchange), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/qk_tiles.h"};
    }

private:
    AbstractDataTypePtr input, exchange, output;
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
