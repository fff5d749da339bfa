// Annotations of the user-schedule matrices (gernels/lds_matrix.h): one global
// matrix type whose subsets are, depending on the annotation class chosen,
// windows in place, per-thread register copies, or tiles staged into LDS by
// the workgroup; and the scalar matrix multiply over them.
//
// Mirrors the reference's gernels/mm/gern_annot/adt.h:8-234 and
// gernels/mm/gern_annot/functions.h:7-100 (same class names, same generated
// method names), so that its schedules (gernels/mm/kernel_3.cu, kernel_6.cu)
// can be written unchanged.
#pragma once

#include "annotations/abstract_function.h"
#include "annotations/shared_memory_manager.h"

namespace gern {

namespace hip {
// Host-side object of a gernels::GlobalMatrix<Row, Col, LDA>: one device pointer.
struct GlobalMatrixF32 {
    float *data;
};
}  // namespace hip

namespace annot {

// Base: subsets are per-thread register tiles (copied in, written back).
template<int Row, int Col>
class StaticMatrixGPU : public AbstractDataType {
public:
    StaticMatrixGPU(const std::string &name, bool temp)
        : name(name), temp(temp) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        if (temp) {
            return "auto";
        }
        return "gernels::GlobalMatrix<" + std::to_string(Row) + ", " + std::to_string(Col) + ", " + std::to_string(Col) + ">";
    }
    std::vector<Variable> getFields() const override {
        return {x, y, row, col};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gernels::allocate_static", .template_args = {row, col}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "free_smem"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "template insert_2_reg_no_vector", .args = {x, y}, .template_args = {row, col}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template query_2_reg_no_vector", .args = {x, y}, .template_args = {row, col}};
    }
    bool insertQuery() const override {
        return true;
    }
    bool freeAlloc() const override {
        return false;
    }
    // Extents are compile-time constants of the type.
    bool readMember(const void *, const std::string &member, int64_t &value) const override {
        if (member == "row") {
            value = Row;
        } else if (member == "col") {
            value = Col;
        } else {
            return false;
        }
        return true;
    }

protected:
    std::string name;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
    bool temp;
};

template<int Row, int Col>
using MatrixQueryRegNoVector = StaticMatrixGPU<Row, Col>;

// Subsets are windows onto the matrix itself.
template<int Row, int Col>
class MatrixGlobalToGlobal : public StaticMatrixGPU<Row, Col> {
public:
    using StaticMatrixGPU<Row, Col>::StaticMatrixGPU;
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template query_global_2_global", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "template insert_global_2_global", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    bool insertQuery() const override {
        return false;
    }
};

// Subsets are tiles staged into LDS by the whole workgroup.
template<int Row, int Col>
class MatrixGlobalToShared : public StaticMatrixGPU<Row, Col> {
public:
    using StaticMatrixGPU<Row, Col>::StaticMatrixGPU;
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template stage_into_smem", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "template insert_from_smem", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "free_smem"};
    }
    // For Stage(ds, getView(), body): a window of an already staged tile.
    FunctionSignature getView() const {
        return FunctionSignature{.name = "template get_view", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    FunctionSignature getViewVec() const {
        return FunctionSignature{.name = "template get_view_vec", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    // and a per-thread register copy of a piece of it
    FunctionSignature getRegisters() const {
        return FunctionSignature{.name = "template query_2_reg_no_vector", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    bool insertQuery() const override {
        return true;
    }
    bool freeQuery() const override {
        return true;
    }
    bool freeAlloc() const override {
        return true;
    }
};

// The same, staged 16 bytes per lane (gernels::GlobalMatrix::stage_into_smem_vec).
template<int Row, int Col>
class MatrixGlobalToSharedVec : public MatrixGlobalToShared<Row, Col> {
public:
    using MatrixGlobalToShared<Row, Col>::MatrixGlobalToShared;
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template stage_into_smem_vec", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
};

// The same, staged by loads that write LDS directly into a dense tile
// (gernels::GlobalMatrix::stage_into_smem_flat).
template<int Row, int Col>
class MatrixGlobalToSharedFlat : public MatrixGlobalToShared<Row, Col> {
public:
    using MatrixGlobalToShared<Row, Col>::MatrixGlobalToShared;
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template stage_into_smem_flat", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
};

// Subsets are per-thread float4 register tiles (the reference's gernels
// annot::MatrixGPU<Row, Col, Stride>, gernels/mm/gern_annot/adt.h:11-60).
template<int Row, int Col>
class MatrixGPUVec : public StaticMatrixGPU<Row, Col> {
public:
    using StaticMatrixGPU<Row, Col>::StaticMatrixGPU;
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gernels::allocate_static_vec", .template_args = {this->row, this->col}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template query", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "template insert", .args = {this->x, this->y}, .template_args = {this->row, this->col}};
    }
};

// C(i.., j..) += A(i.., k..) * B(k.., j..); bind "k_dim" to the reduction length.
class MatrixMultiplyScalar : public AbstractFunction {
public:
    MatrixMultiplyScalar(AbstractDataTypePtr A, AbstractDataTypePtr B, AbstractDataTypePtr C)
        : A(A), B(B), C(C) {
    }
    Annotation getAnnotation() override {
        Variable i("i"), j("j"), k("k");
        Variable ti("ti", Datatype::Int64, true), tj("tj", Datatype::Int64, true), tk("tk", Datatype::Int64, true);
        return Tileable(i = Expr(0), ADTMember(C, "row", true), ti,
                        Tileable(j = Expr(0), ADTMember(C, "col", true), tj,
                                 Produces::Subset(C, {i, j, ti, tj}),
                                 Consumes::Subsets(Reducible(k = Expr(0), k_dim, tk,
                                                             SubsetObjMany({
                                                                 SubsetObj(A, {i, k, ti, tk}),
                                                                 SubsetObj(B, {k, j, tk, tj}),
                                                             })))))
            .occupies({Grid::Unit::SCALAR_UNIT});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::matrix_multiply";
        f.args = {Parameter(A), Parameter(B), Parameter(C)};
        f.template_args = {k_dim};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/lds_matrix.h"};
    }

protected:
    AbstractDataTypePtr A, B, C;
    Variable k_dim{"k_dim", Datatype::Int64, true};
};

// The same on float4 register tiles (gernels::matrix_multiply_reg; the
// reference's annot::MatrixMultiplyReg, gernels/mm/gern_annot/functions.h:54-75).
class MatrixMultiplyReg : public MatrixMultiplyScalar {
public:
    using MatrixMultiplyScalar::MatrixMultiplyScalar;
    FunctionSignature getFunction() override {
        FunctionSignature f = MatrixMultiplyScalar::getFunction();
        f.name = "gernels::matrix_multiply_reg";
        return f;
    }
};

// The allocator's init call for Global(..., smem_size, LdsManager(smem_size)).
class LdsManager : public grid::SharedMemoryManager {
public:
    explicit LdsManager(Variable smem_size)
        : grid::SharedMemoryManager(
              FunctionCall{"gernels::lds_init", {smem_size}, {}, Parameter(), LaunchArguments(), LaunchArguments(), DEVICE},
              {"gernels/lds_alloc.h"}) {
    }
};

}  // namespace annot
}  // namespace gern
