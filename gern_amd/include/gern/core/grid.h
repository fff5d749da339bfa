// The launch-grid model: the units a loop can be distributed over, the launch
// dimensions those units consume, and the ordering of levels that decides
// which distributions are legal.
//
// Enumerators and free functions keep the reference's names
// (include/gern/annotations/grid.h:8-58, src/annotations/grid.cpp:113-254).
// What differs is the machine underneath: a "warp" here is a 64-lane CDNA
// wavefront, so WARP_* / THREAD_*_IN_WRAPS split a block dimension by 64.
#pragma once

#include <cstdint>
#include <ostream>
#include <set>

namespace gern {

namespace Grid {

enum Unit {
    UNDEFINED,  // not bound to the grid
    SCALAR_UNIT,

    THREAD_X_IN_WRAPS,  // lane index inside its wavefront
    THREAD_Y_IN_WRAPS,
    THREAD_Z_IN_WRAPS,

    THREAD_X,
    THREAD_Y,
    THREAD_Z,

    WARP_X,  // wavefront index along a block dimension
    WARP_Y,
    WARP_Z,

    BLOCK_X,
    BLOCK_Y,
    BLOCK_Z,
};

enum Dim {
    GRID_DIM_X,
    GRID_DIM_Y,
    GRID_DIM_Z,

    BLOCK_DIM_X,
    BLOCK_DIM_Y,
    BLOCK_DIM_Z,

    WARP_DIM_X,
    WARP_DIM_Y,
    WARP_DIM_Z,

    NULL_DIM,
};

enum Level {
    NULL_LEVEL = 0,
    SCALAR = 1,
    THREADS = 2,
    THREADS_WARPS = 3,
    WARPS = 4,
    BLOCK = 5,
    BLOCK_CLUSTER = 6,
    GRID = 7,
};

// Lanes per wavefront on gfx950.
constexpr int64_t kWavefrontSize = 64;

}  // namespace Grid

std::ostream &operator<<(std::ostream &, const Grid::Unit &);
std::ostream &operator<<(std::ostream &, const Grid::Dim &);
std::ostream &operator<<(std::ostream &, const Grid::Level &);

// True for every unit a loop can actually be mapped to (anything above
// SCALAR_UNIT).
bool isLegalUnit(const Grid::Unit &);
bool isLegalLevel(const Grid::Level &);

// A computation occupying `units` may be distributed over `over` only if
// `over` sits at or above the highest level already occupied.
bool legalToDistribute(const std::set<Grid::Unit> &units, const Grid::Unit &over);

Grid::Level getLevel(const Grid::Unit &);
Grid::Level getLevel(const std::set<Grid::Unit> &);
Grid::Level getLevel(const Grid::Dim &);
Grid::Level getLevel(const std::set<Grid::Dim> &);

// The launch dimension a unit consumes.
Grid::Dim getDim(const Grid::Unit &);
std::set<Grid::Dim> getDims(const std::set<Grid::Unit> &);

// Whether code occupying `dims` may fix or constrain `dim`: either it uses the
// dimension itself or the dimension belongs to a strictly lower level.
bool isDimInScope(const Grid::Dim &dim, const std::set<Grid::Dim> &dims);

}  // namespace gern
