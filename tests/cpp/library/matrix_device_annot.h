// Annotations of matrix_device.h.
// Mirrors test/library/matrix/annot/gpu-matrix.h:10-125 of the reference.
#pragma once

#include "library/matrix_annot.h"

namespace gern {
namespace annot {

struct MatrixGPULayout {
    float *data;
    int64_t row, col, lda;
};

class MatrixGPU : public MatrixCPU {
public:
    using MatrixCPU::MatrixCPU;
    std::string getType() const override {
        return "gern::impl::MatrixGPU";
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::MatrixGPU::allocate", .args = {x, y, l_x, l_y}};
    }
    bool insertQuery() const override {
        return false;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        const auto *m = static_cast<const MatrixGPULayout *>(object);
        if (member == "row") {
            value = m->row;
        } else if (member == "col") {
            value = m->col;
        } else if (member == "lda") {
            value = m->lda;
        } else {
            return false;
        }
        return true;
    }
};

// Queries copy the tile into LDS and inserts copy it back.
class MatrixGPUStageSmem : public MatrixGPU {
public:
    using MatrixGPU::MatrixGPU;
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "stage_into_smem", .args = {x, y, l_x, l_y}};
    }
    bool insertQuery() const override {
        return true;
    }
};

class MatrixAddGPU : public MatrixAddCPU {
public:
    Annotation getAnnotation() override {
        return resetUnit(MatrixAddCPU::getAnnotation(), {Grid::Unit::SCALAR_UNIT});
    }
    std::vector<std::string> getHeader() override {
        return {"matrix_device.h"};
    }
};

class MatrixAddGPUBlocks : public MatrixAddCPU {
public:
    Annotation getAnnotation() override {
        return resetUnit(MatrixAddCPU::getAnnotation(), {Grid::Unit::THREAD_X, Grid::Unit::THREAD_Y});
    }
    FunctionSignature getFunction() override {
        return FunctionSignature{.name = "gern::impl::add_smem", .args = {Parameter(input), Parameter(output)}};
    }
    std::vector<std::string> getHeader() override {
        return {"matrix_device.h"};
    }
};

}  // namespace annot
}  // namespace gern
