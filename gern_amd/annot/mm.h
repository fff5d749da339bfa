// Annotations of the block GEMM gernels (gernels/mm.h).
//
// The dependency pattern is the reference's (test/library/matrix/annot/cpu-matrix.h:258-303,
// gernels/mm/gern_annot/functions.h:7-100): to produce C[i..i+ti, j..j+tj] the
// function consumes, for every k step of a reducible loop over k_dim,
// A[i..i+ti, k..k+tk] and B[k..k+tk, j..j+tj].
#pragma once

#include "annot/matrix.h"

namespace gern {
namespace annot {

// A GEMM operand in HBM; its subsets are windows (no data movement).
class MatrixOperand : public AbstractDataType {
public:
    enum Element { F32, BF16 };
    // exact: the caller guarantees what gernels::GlobalView calls EXACT (one
    // dense allocation per matrix; rows of A 16-byte aligned whole numbers of
    // 16-byte pieces, i.e. a reduction extent that is a multiple of 8 for bf16
    // and of 4 for fp32; rows of B 4-byte aligned); the matrix-core gernels
    // then load both operands straight into LDS.
    MatrixOperand(const std::string &name, Element element, bool exact = false)
        : name(name), element(element), exact(exact) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return element == BF16 ? "gernels::MatrixBF16" : "gernels::MatrixF32";
    }
    std::vector<Variable> getFields() const override {
        return {x, y, row, col};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "unsupported_allocate"};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "unsupported_insert"};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{
            .name = exact ? "template view_exact" : "template view",
            .args = {x, y},
            .template_args = {row, col},
        };
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        // MatrixF32 and MatrixBF16 share their layout
        return MatrixF32("", MatrixF32::INPUT).readMember(object, member, value);
    }

private:
    std::string name;
    Element element;
    bool exact;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// The GEMM result in HBM; its subsets are block-distributed accumulator tiles
// that start at zero and are either ADDED to C when inserted (accumulate: the
// reference's C += A * B) or written over it (C = A * B; C is never read).
//   FMA    fp32 FMAs, 256 threads
//   MFMA4  matrix cores, four wavefronts (any shape)
//   MFMA8  matrix cores, eight wavefronts, 32 x 32 x 16 instruction
//   MFMA16 matrix cores, eight wavefronts, 16 x 16 x 32 instruction (the fast shape; operands must be
//          MatrixOperands that promise `exact`)
//   MFMA8_F32  fp32 operands on the matrix cores, eight wavefronts
class MatrixAccumulator : public AbstractDataType {
public:
    enum Engine { FMA, MFMA4, MFMA8, MFMA8_F32, MFMA16 };
    MatrixAccumulator(const std::string &name, Engine engine, bool accumulate = true)
        : name(name), engine(engine), accumulate(accumulate) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return "gernels::MatrixF32";
    }
    std::vector<Variable> getFields() const override {
        return {x, y, row, col};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "unsupported_allocate"};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{
            .name = accumulate ? "add_acc" : "store_acc",
            .args = {x, y},
        };
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{
            .name = engine == MFMA8_F32 ? "template load_acc_mfma8_f32" :
                    engine == MFMA8     ? "template load_acc_mfma8" :
                    engine == MFMA16    ? "template load_acc_mfma16" :
                    engine == MFMA4     ? "template load_acc_mfma" :
                                          "template load_acc_fma",
            .args = {x, y},
            .template_args = {row, col},
        };
    }
    bool insertQuery() const override {
        return true;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        return MatrixF32("", MatrixF32::INPUT).readMember(object, member, value);
    }

private:
    std::string name;
    Engine engine;
    bool accumulate;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// C += A * B on one workgroup.  Bind "k_dim" to the variable that holds the
// reduction extent, and Reduce over it.
class MatrixMultiply : public AbstractFunction {
public:
    MatrixMultiply(AbstractDataTypePtr A, AbstractDataTypePtr B, AbstractDataTypePtr C)
        : A(A), B(B), C(C) {
    }
    Annotation getAnnotation() override {
        Variable i("i"), j("j"), k("k");
        Variable ti("ti", Datatype::Int64, true), tj("tj", Datatype::Int64, true), tk("tk", Datatype::Int64, true);
        return Tileable(i = Expr(0), ADTMember(C, "row", false), ti,
                        Tileable(j = Expr(0), ADTMember(C, "col", false), tj,
                                 Produces::Subset(C, {i, j, ti, tj}),
                                 Consumes::Subsets(Reducible(k = Expr(0), k_dim, tk,
                                                             SubsetObjMany({
                                                                 SubsetObj(A, {i, k, ti, tk}),
                                                                 SubsetObj(B, {k, j, tk, tj}),
                                                             })))))
            // all threads of a workgroup cooperate
            .occupies({Grid::Unit::THREAD_X})
            // the matrix-core gernels address a tile with 32-bit byte offsets
            // (gernels/mm.h): row pitches up to 2^20 elements
            .assumes(Constraint(ADTMember(A, "lda", false) <= Expr((int64_t)1 << 20)),
                     Constraint(ADTMember(B, "lda", false) <= Expr((int64_t)1 << 20)));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::matrix_multiply";
        f.args = {Parameter(A), Parameter(B), Parameter(C)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/mm.h"};
    }

private:
    AbstractDataTypePtr A, B, C;
    Variable k_dim{"k_dim", Datatype::Int64};
};

}  // namespace annot
}  // namespace gern
