// Annotations (the code generator's view) of the gfx950 gernel data
// structures in gernels/wave_tile.h, and the host mirror of the device
// aggregate that callers fill in and pass to Runner::evaluate.
//
// Counterpart of the reference's apps/common/annot/adt.h:9-149.
#pragma once

#include "annotations/abstract_function.h"

#include <cstdint>
#include <string>

namespace gern {
namespace hip {

// Host mirror of gernels::MatrixF32 (same layout: pointer, three int64).
// `data` is a device pointer.
struct MatrixF32 {
    float *data;
    int64_t row;
    int64_t col;
    int64_t lda;
};

// Host mirror of gernels::MatrixBF16.
struct MatrixBF16 {
    uint16_t *data;
    int64_t row;
    int64_t col;
    int64_t lda;
};

}  // namespace hip

namespace annot {

// A row-major fp32 matrix in HBM whose subsets are wave-distributed register
// tiles.  Fields: (x, y) origin, (row, col) extent.
//   role INPUT  : query loads the tile (zero beyond the edges)
//   role OUTPUT : query only names the tile; the producer overwrites it and
//                 insert stores it (clipped to the matrix)
//   role TEMP   : never in memory; allocate makes a register tile
class MatrixF32 : public AbstractDataType {
public:
    enum Role { INPUT, OUTPUT, ACCUMULATE, TEMP };

    MatrixF32(const std::string &name, Role role)
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
            .name = "gernels::allocate_wave_tile",
            .template_args = {row, col},
        };
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{
            .name = "store_wave",
            .args = {x, y},
        };
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{
            .name = (role == OUTPUT) ? "template view_wave" : "template load_wave",
            .args = {x, y},
            .template_args = {row, col},
        };
    }
    bool insertQuery() const override {
        return role == OUTPUT || role == ACCUMULATE;
    }
    bool freeAlloc() const override {
        return false;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        const auto *m = static_cast<const hip::MatrixF32 *>(object);
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

protected:
    std::string name;
    Role role;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// Per-row scalars of a tile (row maxima, row sums); always a register
// temporary.  Fields: x origin, size.
class WaveVec : public AbstractDataType {
public:
    explicit WaveVec(const std::string &name)
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
            .name = "gernels::allocate_wave_vec",
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

}  // namespace annot
}  // namespace gern
