// Annotations (the code generator's view) of the gfx950 gernel data
// structures in gernels/wave_tile.h, and the host mirror of the device
// aggregate that callers fill in and pass to Runner::evaluate.
//
// Counterpart of the reference's apps/common/annot/adt.h:9-149.
#pragma once

#include "annot/table.h"

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
//   roles INPUT_WIDE / OUTPUT_LINES : a pair for a grid of one-chunk tiles
//                 whose width is a multiple of 32 columns: insert moves each
//                 tile's window to whole 128-byte lines of the result, and the
//                 query of the input loads the lanes past the tile's width that
//                 such a window needs (gernels/wave_tile.h, store_wave_lines)
class MatrixF32 : public TableADT {
public:
    enum Role { INPUT, OUTPUT, ACCUMULATE, TEMP, INPUT_WIDE, OUTPUT_LINES };

    MatrixF32(const std::string &name, Role role)
        : TableADT(name, role == TEMP ? "auto" : "gernels::MatrixF32"), role(role) {
        fields = {x, y, row, col};
        const bool written = role == OUTPUT || role == OUTPUT_LINES;
        setCalls("gernels::allocate_wave_tile",
                 written ? "template view_wave" : role == INPUT_WIDE ? "template load_wave_wide" : "template load_wave",
                 role == OUTPUT_LINES ? "store_wave_lines" : "store_wave");
        query_is_written_back = written || role == ACCUMULATE;
        temporaries_are_freed = false;
    }
    // Launch dimensions are computed on the host from the caller's object.
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        const auto *m = static_cast<const hip::MatrixF32 *>(object);
        const int64_t *found = member == "row" ? &m->row : member == "col" ? &m->col : member == "lda" ? &m->lda : nullptr;
        if (found != nullptr) {
            value = *found;
        }
        return found != nullptr;
    }

protected:
    // allocate<row, col>(), query<row, col>(x, y), insert(x, y, tile)
    void setCalls(const std::string &allocate, const std::string &query, const std::string &insert) {
        allocate_call = call(allocate, {}, {row, col});
        query_call = call(query, {x, y}, {row, col});
        insert_call = call(insert, {x, y});
    }
    Role role;
    Variable x{"x"};
    Variable y{"y"};
    Variable row{"row", Datatype::Int64, true};
    Variable col{"col", Datatype::Int64, true};
};

// Per-row scalars of a tile (row maxima, row sums); always a register
// temporary.  Fields: x origin, size.  It is never queried or inserted.
class WaveVec : public TableADT {
public:
    explicit WaveVec(const std::string &name)
        : TableADT(name, "auto") {
        fields = {x, len};
        allocate_call = call("gernels::allocate_wave_vec", {}, {len});
        query_call = call("unsupported_query");
        insert_call = call("unsupported_insert");
        temporaries_are_freed = false;
    }

private:
    Variable x{"x"};
    Variable len{"size", Datatype::Int64, true};
};

}  // namespace annot
}  // namespace gern
