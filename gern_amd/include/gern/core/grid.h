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

// Enumerator names and order are the reference API.
enum Unit {
    UNDEFINED,    // not bound to the grid
    SCALAR_UNIT,  // a sequential loop
    // lane index inside its wavefront, per block dimension
    THREAD_X_IN_WRAPS, THREAD_Y_IN_WRAPS, THREAD_Z_IN_WRAPS,
    // thread index inside its block
    THREAD_X, THREAD_Y, THREAD_Z,
    // wavefront index along a block dimension
    WARP_X, WARP_Y, WARP_Z,
    // block index inside the grid
    BLOCK_X, BLOCK_Y, BLOCK_Z,
};

// What a launch fixes: blocks per grid, threads per block, and the wavefront
// split of a block dimension.
enum Dim {
    GRID_DIM_X, GRID_DIM_Y, GRID_DIM_Z,
    BLOCK_DIM_X, BLOCK_DIM_Y, BLOCK_DIM_Z,
    WARP_DIM_X, WARP_DIM_Y, WARP_DIM_Z,
    NULL_DIM,
};

// Levels are ordered: a loop may only be distributed over a level at or above
// everything its body already occupies.
enum Level {
    NULL_LEVEL = 0, SCALAR = 1, THREADS = 2, THREADS_WARPS = 3, WARPS = 4, BLOCK = 5, BLOCK_CLUSTER = 6, GRID = 7,
};

// Lanes per wavefront on gfx950.
constexpr int64_t kWavefrontSize = 64;

}  // namespace Grid

// The launch dimension a unit consumes, and the level a unit or a dimension lives at.
Grid::Dim getDim(const Grid::Unit &);
std::set<Grid::Dim> getDims(const std::set<Grid::Unit> &);
Grid::Level getLevel(const Grid::Unit &);
Grid::Level getLevel(const Grid::Dim &);
Grid::Level getLevel(const std::set<Grid::Unit> &);  // the highest of the set
Grid::Level getLevel(const std::set<Grid::Dim> &);

// True for every unit a loop can actually be mapped to (anything above SCALAR_UNIT).
bool isLegalUnit(const Grid::Unit &);
bool isLegalLevel(const Grid::Level &);

// A computation occupying `units` may be distributed over `over` only if
// `over` sits at or above the highest level already occupied.
bool legalToDistribute(const std::set<Grid::Unit> &units, const Grid::Unit &over);

// Whether code occupying `dims` may fix or constrain `dim`: either it uses the
// dimension itself or the dimension belongs to a strictly lower level.
bool isDimInScope(const Grid::Dim &dim, const std::set<Grid::Dim> &dims);

std::ostream &operator<<(std::ostream &, const Grid::Unit &);
std::ostream &operator<<(std::ostream &, const Grid::Dim &);
std::ostream &operator<<(std::ostream &, const Grid::Level &);

}  // namespace gern
